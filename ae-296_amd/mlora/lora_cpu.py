"""Host-side mirror of the reference's ``Lora_CPU`` (``lightllm/models/lora_cpu.py``): the GPU side of
the CPU-assisted path, on which host workers compute the LoRA delta of the early layers while an
adapter is still being loaded into the pool.

This class is the transport -- shipping hidden states to the workers, waking them, and bringing their
results back.  The workers are any host code that follows the protocol below: the reference's
``lora_cpu/lora_shm_op/app.py`` processes, or the in-process thread pool of ``libmlora_cpu.so``
(``start_workers``), which computes the chunks with the package's own CPU kernel (``cpu_ops.py``).

Protocol (the reference's, ``lora_cpu.py:138-276`` and ``app.py:102-143``, with its result placement
restated from the arithmetic, because worker and collector of the reference only agree when a request
fits one chunk):

* ``x_slots [n_slots, slot_tokens, H]``: request ``b`` of a batch occupies slot ``b``, tokens from row 0.
* ``signals int16 [3, n_workers]``: worker ``w`` of projection ``q`` (q, k, v = 0, 1, 2) is woken with the
  code ``2 + 200 * q + w``; it serves request ``w // cpr``, chunk ``w % cpr`` with
  ``cpr = (tkn - 1) // token_per_lora + 1``, i.e. tokens ``[chunk * cap, min((chunk + 1) * cap, tkn))``,
  writes its rows to ``out[q][request, chunk * cap : ...]`` and stores 0 into its signal.
* ``tkn_len int32 [1]``: tokens per request of the batch in flight.

The buffers are pinned host memory mapped into the device address space (``mlora_host_alloc``); the
workers see them as numpy arrays (``np_x``, ``np_out``, ``np_signal``, ``np_tkn_len``).
"""
from __future__ import annotations

import ctypes as C
import time
from typing import List, Optional, Tuple

import numpy as np
import torch

from . import _ext, cpu_ops

PROMPT_MAX_LENGTH = 256          # tokens per request slot (lora_cpu.py:14)
SIGNAL_BASE, SIGNAL_STRIDE = 2, 200   # codes 2.., 202.., 402.. (lora_cpu.py:181-185, app.py:110-128)


def chunk_of(row_id: int, tkn_num: int, cap: int) -> Tuple[int, int, int]:
    """(request, first token, token count) of worker ``row_id`` (``app.py:133-135``)."""
    cpr = (tkn_num - 1) // cap + 1
    d0, d1 = row_id // cpr, row_id % cpr
    return d0, d1 * cap, min((d1 + 1) * cap, tkn_num) - d1 * cap


class _Mapped:
    """A pinned, device-mapped host allocation viewed as a numpy array."""

    def __init__(self, shape, dtype):
        self.shape, self.dtype = tuple(shape), np.dtype(dtype)
        nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        h, d = C.c_void_p(), C.c_void_p()
        _ext.check(_ext.lib().mlora_host_alloc(nbytes, C.byref(h), C.byref(d)))
        self.host_ptr, self.dev_ptr = h.value, d.value
        buf = (C.c_char * nbytes).from_address(self.host_ptr)
        self.array = np.frombuffer(buf, dtype=self.dtype).reshape(self.shape)

    def free(self):
        if self.host_ptr:
            self.array = None
            _ext.lib().mlora_host_free(C.c_void_p(self.host_ptr))
            self.host_ptr = self.dev_ptr = None


class Lora_CPU:
    def __init__(self, configJson, gpu_id: int = 0, device: str = "cuda"):
        self.batch_size = configJson["batch_size"]
        self.lora_num = configJson["lora_num"]                  # workers (= request slots) per projection
        self.tp_degree = configJson["tp_degree"]
        self.hidden_dim = configJson["hidden_dim"]
        self.lora_rank = configJson["lora_rank"]
        self.cpu_capacity = configJson["token_per_lora"]
        self.n_layers = configJson["n_layers"]
        self.gpu_id = gpu_id
        self.device = torch.device(device)
        self.out_size = self.hidden_dim // self.tp_degree
        if self.lora_num > SIGNAL_STRIDE:
            raise ValueError(f"at most {SIGNAL_STRIDE} workers per projection (signal codes are {SIGNAL_STRIDE} apart)")
        shape = (self.lora_num, PROMPT_MAX_LENGTH, self.hidden_dim)
        self._x = _Mapped(shape, np.uint16)
        self._out = [_Mapped(shape, np.uint16) for _ in range(3)]
        self._signal = _Mapped((3, self.lora_num), np.int16)
        self._tkn_len = _Mapped((1,), np.int32)
        self.np_x, self.np_out = self._x.array, [o.array for o in self._out]
        self.np_signal, self.np_tkn_len = self._signal.array, self._tkn_len.array
        self.active_cpu = 0
        self._dtype = torch.float16
        self._workers = None
        self._worker_pool = None

    # ------------------------------------------------------------------ in-process workers
    def start_workers(self, down, up, n_threads: int, slot_adapter=None) -> None:
        """Serve the slots from a pool of `n_threads` host threads inside this process (instead of the
        reference's one pinned process per request chunk and projection, ``runServerCPULoRA.py:74-90``):
        ``down[q] [N, H, r]`` / ``up[q] [N, r, H]`` (fp32 or binary16) are the q, k, v adapters,
        ``slot_adapter [lora_num]`` the adapter of the request in each slot (None: adapter 0).  fp16 only."""
        if self._workers is not None:
            raise RuntimeError("workers are already running")
        self._worker_pool = cpu_ops.CpuLoraPool(n_threads)
        self._workers = cpu_ops.AssistWorkers(self._worker_pool, self.np_x, self.np_out, self.np_signal, self.np_tkn_len,
                                              self.cpu_capacity, down, up, slot_adapter, SIGNAL_BASE, SIGNAL_STRIDE)

    def stop_workers(self):
        """Stop the in-process workers; returns (chunks served, codes rejected)."""
        out = (0, 0)
        if self._workers is not None:
            out = self._workers.stop()
            self._workers = None
        if self._worker_pool is not None:
            self._worker_pool.close()
            self._worker_pool = None
        return out

    def close(self):
        self.stop_workers()
        for m in [self._x, self._signal, self._tkn_len] + self._out:
            m.free()

    # ------------------------------------------------------------------ ship and wake
    def invoke_lora_async(self, hidden_states: torch.Tensor, tkn_num: int, layer_id: int = 0) -> None:
        """``hidden_states [B * tkn_num, H]`` (16-bit, on the device) to the request slots, then one wake-up
        code per worker of q, k and v.  Returns at once; everything is ordered on the current stream."""
        if hidden_states.dim() != 2 or hidden_states.shape[1] != self.hidden_dim or hidden_states.shape[0] % tkn_num:
            raise ValueError("hidden_states must be [B * tkn_num, hidden_dim]")
        if hidden_states.element_size() != 2 or not hidden_states.is_cuda or not hidden_states.is_contiguous():
            raise TypeError("hidden_states must be a contiguous 16-bit tensor on the device")
        batch = hidden_states.shape[0] // tkn_num
        cpr = (tkn_num - 1) // self.cpu_capacity + 1
        if batch * cpr > self.lora_num:
            raise ValueError(f"Not enough CPU LoRAs: {self.lora_num}/{batch * cpr}")            # lora_cpu.py:152-155
        self.active_cpu = batch * cpr
        self._dtype = hidden_states.dtype
        self.np_tkn_len[0] = tkn_num
        # guard value (lora_cpu.py:161-164): a collector that polls before the codes arrive must not
        # mistake the idle zeros for finished work; workers only react to codes > 1
        self.np_signal[:, :self.active_cpu] = 1
        rc = _ext.lib().mlora_assist_export(
            hidden_states.data_ptr(), batch, tkn_num, self.hidden_dim, self._x.dev_ptr, self.lora_num, PROMPT_MAX_LENGTH,
            self._signal.dev_ptr, 3, self.lora_num, self.cpu_capacity, SIGNAL_BASE, SIGNAL_STRIDE,
            _ext.current_stream_ptr())
        _ext.check(rc)

    # ------------------------------------------------------------------ collect
    def results_ready(self) -> bool:
        return not self.np_signal[:, :self.active_cpu].any()

    def collect_each(self, tkn_num: int, batch_size: int, timeout_s: Optional[float] = 60.0):
        """Yields ``(projection index, result [batch_size, tkn_num, out_size])`` for q, k and v, each as soon as all of
        its workers have reset their signals: that projection's rows come to the device (one launch) while the
        workers of the others are still computing -- the reference brings chunks back as they finish
        (``lora_cpu.py:219-270``)."""
        t0 = time.perf_counter()
        lib = _ext.lib()
        pending = [0, 1, 2]
        while pending:
            progressed = False
            for q in list(pending):
                if self.np_signal[q, :self.active_cpu].any():
                    continue
                res = torch.empty((batch_size, tkn_num, self.out_size), dtype=self._dtype, device=self.device)
                rp = (C.c_void_p * 4)(res.data_ptr(), None, None, None)
                op = (C.c_void_p * 4)(self._out[q].dev_ptr, None, None, None)
                _ext.check(lib.mlora_assist_import(1, rp, op, batch_size, tkn_num, self.hidden_dim, self.out_size,
                                                   self.out_size * self.gpu_id, self.lora_num, PROMPT_MAX_LENGTH,
                                                   _ext.current_stream_ptr()))
                pending.remove(q)
                progressed = True
                yield q, res
            if pending and not progressed and timeout_s is not None and time.perf_counter() - t0 > timeout_s:
                raise TimeoutError("CPU workers did not finish in time")

    def collect_qkv(self, tkn_num: int, batch_size: int, timeout_s: Optional[float] = 60.0) -> List[torch.Tensor]:
        """The q, k and v results of the batch in flight as ``[batch_size, tkn_num, out_size]`` tensors (the rank's
        column slice), each imported as soon as its projection's workers are done."""
        res: List[Optional[torch.Tensor]] = [None, None, None]
        for q, r in self.collect_each(tkn_num, batch_size, timeout_s):
            res[q] = r
        return res
