"""Host-side mirror of the reference's ``Lora_GPU`` (``lightllm/models/lora_gpu.py``) for the
apply path: same constructor keys, same pool attributes and shapes, same
``invoke_one_layer_{q,k,v}(x, layer_id, prefill)`` calls that
``LlamaTransformerLayerInfer._get_qkv`` makes
(``lightllm/models/llama/layer_infer/transformer_layer_infer.py:76-81,101-111``) -- with the
decode branch on the HIP BGMV kernel instead of ``punica.ops.add_lora_bgmv`` and the prefill
branch on the HIP SGMV kernels instead of ``torch.bmm(torch.bmm(...))`` plus two weight
transposes per call.

Left out on purpose (not part of the apply path): the zmq / CUDA-IPC sharing with the
swapper process (``lora_gpu.py:76-118,246-296``) and the progress polling (``:298-339``).
"""
from __future__ import annotations

import numpy as np
import torch

from . import ops


class Lora_GPU:
    def __init__(self, configJson, shared: bool = False, device: str = "cuda", seed: int = 0):
        self.device = torch.device(device)
        self.n_layers = configJson["n_layers"]
        self.batch_size = configJson["batch_size"]
        self.lora_rank = configJson["lora_rank"]
        self.in_size = configJson["hidden_dim"]
        self.output_size = configJson["hidden_dim"] // configJson["tp_degree"]
        self.tp_degree = configJson["tp_degree"]
        self.max_prefill_batch_size = configJson["max_prefill_batch_size"]
        self.dtype = configJson.get("dtype", torch.float16)
        self._gen = torch.Generator(device=self.device)
        self._gen.manual_seed(seed)

        # Decode pool, reference layout (lora_gpu.py:33-40): down [N, L, r, Hin], up [N, L, Hout, r].
        # The reference leaves these uninitialised (torch.empty); they are given small random values here.
        for name in ("q", "k", "v"):
            setattr(self, f"{name}_down", self._rand(self.batch_size, self.in_size, self.lora_rank))
            setattr(self, f"{name}_up", self._rand(self.batch_size, self.lora_rank, self.output_size))
            setattr(self, f"{name}_down_prefill", None)
            setattr(self, f"{name}_up_prefill", None)
        mode = configJson.get("mode", [])
        if shared or "aaas-cached" in mode or "aaas-gpu" in mode:
            self.prepare_lora_prefill(self.max_prefill_batch_size)

        # Per-batch-size index vectors (lora_gpu.py:120).  The reference draws from [0, 32) whatever the
        # pool size, which reads out of bounds when batch_size < 32; indices are kept inside the pool here.
        hi = min(32, self.batch_size)
        self.select_inds = [torch.randint(0, hi, (i + 1,), device=self.device, generator=self._gen)
                            for i in range(self.batch_size)]
        self._workspace = None

    def _rand(self, n, rows, cols):
        """[n, L, rows, cols] * 0.001, stored transposed and contiguous as the reference does."""
        w = torch.randn((n, self.n_layers, rows, cols), device=self.device, dtype=torch.float32,
                        generator=self._gen) * 0.001
        return w.to(self.dtype).transpose(-1, -2).contiguous()

    # ------------------------------------------------------------------ apply
    def _invoke(self, name, x, layer_id, prefill, lora_ids=None):
        bsz = x.shape[0]
        if prefill:
            down, up = getattr(self, f"{name}_down_prefill"), getattr(self, f"{name}_up_prefill")
            if down is None:
                raise RuntimeError("prefill adapters are not loaded (call prepare_lora_prefill)")
            if not x.is_contiguous():
                x = x.contiguous()
            need = ops._ext.lib().mlora_sgmv_workspace_bytes(bsz * x.shape[1], bsz)
            if self._workspace is None or self._workspace.numel() < need:
                self._workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
            return ops.lora_prefill_ref(x, down, up, layer_id, workspace=self._workspace)
        # The reference drops the request's adapter ids (``infer_state.lora_ids``, built at
        # pre_process.py:50,100) and applies a random stand-in; pass ``lora_ids`` to use the real ones.
        if lora_ids is None:
            cur_inds = self.select_inds[bsz - 1]
        else:
            if lora_ids.numel() != bsz:
                raise ValueError("lora_ids must hold one adapter slot per row of x")
            cur_inds = lora_ids.to(device=x.device, dtype=torch.int64)
        y = torch.zeros(bsz, self.output_size, device=x.device, dtype=x.dtype)
        ops.add_lora_bgmv(y, x, getattr(self, f"{name}_down"), getattr(self, f"{name}_up"), cur_inds, layer_id, 1)
        return y

    def invoke_one_layer_q(self, x, layer_id, prefill=False, lora_ids=None):
        return self._invoke("q", x, layer_id, prefill, lora_ids)

    def invoke_one_layer_k(self, x, layer_id, prefill=False, lora_ids=None):
        return self._invoke("k", x, layer_id, prefill, lora_ids)

    def invoke_one_layer_v(self, x, layer_id, prefill=False, lora_ids=None):
        return self._invoke("v", x, layer_id, prefill, lora_ids)

    # ------------------------------------------------------------------ slot management
    def prepare_lora_prefill(self, batch_size):
        """lora_gpu.py:190-200: fresh random prefill adapters, one slot per request."""
        for name in ("q", "k", "v"):
            setattr(self, f"{name}_down_prefill", self._rand(batch_size, self.in_size, self.lora_rank))
            setattr(self, f"{name}_up_prefill", self._rand(batch_size, self.lora_rank, self.output_size))

    def merge_lora_prefill(self, bsz, re_inds=None):
        """lora_gpu.py:202-217: copy the first bsz prefill slots into decode slots (random targets
        in the reference; pass re_inds to choose them)."""
        if re_inds is None:
            re_inds = np.random.randint(0, self.batch_size, size=bsz)
        for idx, re_ind in enumerate(re_inds):
            for name in ("q", "k", "v"):
                getattr(self, f"{name}_down")[re_ind].copy_(getattr(self, f"{name}_down_prefill")[idx])
                getattr(self, f"{name}_up")[re_ind].copy_(getattr(self, f"{name}_up_prefill")[idx])
        return re_inds

    def remove_lora(self, rm_ids, running_bsz, chosen=None):
        """lora_gpu.py:229-242 shifts slices of the *second* axis of [N, L, ...] tensors, i.e. layers, which
        looks unintended; the documented intent (drop the adapters of finished requests, closing the gap)
        is applied to the adapter axis here."""
        if running_bsz <= 0:
            return
        if chosen is None:
            chosen = np.random.randint(0, running_bsz, size=len(rm_ids))
        for rm_id in chosen:
            for name in ("q", "k", "v"):
                for side in ("down", "up"):
                    w = getattr(self, f"{name}_{side}")
                    w[rm_id:-1] = w[rm_id + 1:].clone()
