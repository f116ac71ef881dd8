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
        # Grouping of the current decode batch by adapter.  It is served again only for the very tensor object it was
        # made from (`_plan_src`, kept alive here so that neither its address nor its Python identity can pass to
        # another tensor) at the same torch version counter: a serving loop builds `lora_ids` afresh every step
        # (pre_process.py:50,100), and a new tensor of the same size often gets the freed one's address.
        self._plan = None
        self._plan_src = None
        self._plan_ver = None
        self._plan_gen = 0
        self._qkv = None           # q, k, v deltas of the last decode input ...
        self._qkv_x = None         # ... the input tensor itself (kept alive for the same reason) ...
        self._qkv_w = []           # ... the six weight tensors ...
        self._qkv_key = None       # ... and what else they were computed from

    def _rand(self, n, rows, cols):
        """[n, L, rows, cols] * 0.001, stored transposed and contiguous as the reference does."""
        w = torch.randn((n, self.n_layers, rows, cols), device=self.device, dtype=torch.float32,
                        generator=self._gen) * 0.001
        return w.to(self.dtype).transpose(-1, -2).contiguous()

    # ------------------------------------------------------------------ apply
    def _index_source(self, bsz, lora_ids):
        # The reference drops the request's adapter ids (``infer_state.lora_ids``, built at
        # pre_process.py:50,100) and applies a random stand-in; pass ``lora_ids`` to use the real ones.
        if lora_ids is None:
            return self.select_inds[bsz - 1]
        if lora_ids.numel() != bsz:
            raise ValueError("lora_ids must hold one adapter slot per row of x")
        return lora_ids

    def _indices(self, bsz, lora_ids, device):
        """The index vector as the kernels take it: int64 on the device (int32 ids, pre_process.py:100, are widened)."""
        src = self._index_source(bsz, lora_ids)
        if src.dtype == torch.int64 and src.device == device:
            return src
        return src.to(device=device, dtype=torch.int64)

    def plan_decode(self, bsz, lora_ids=None):
        """Group the decode batch by adapter (one gather launch): the step boundary.  A serving loop calls it once
        per step; ``invoke_one_layer_*`` call it themselves when they are handed another index tensor than the one
        the current plan was made from, or the same one after torch has written to it.  A tensor whose contents
        were changed behind torch's back (a raw kernel writing through its pointer) needs this call."""
        src = self._index_source(bsz, lora_ids)
        cur_inds = self._indices(bsz, lora_ids, self.q_down.device)
        reuse = self._plan if (self._plan is not None and self._plan.T == bsz) else None
        self._plan = ops.plan_decode_ref(cur_inds, self.batch_size, self.n_layers, self.lora_rank, out=reuse)
        self._plan_src, self._plan_ver = src, src._version
        self._plan_gen += 1
        self._qkv_key = None
        return self._plan

    def _plan_for(self, bsz, lora_ids):
        src = self._index_source(bsz, lora_ids)
        if self._plan is None or self._plan_src is not src or self._plan_ver != src._version or self._plan.T != bsz:
            self.plan_decode(bsz, lora_ids)
        return self._plan

    def invoke_one_layer_qkv(self, x, layer_id, lora_ids=None):
        """The q, k and v deltas of one decode layer in one call pair (the reference makes three
        ``add_lora_bgmv`` calls with a ``torch.zeros`` each, lora_gpu.py:137-138,149-150,161-162): returns
        ``(q_lora, k_lora, v_lora)``, each ``[bsz, hidden / tp]``."""
        bsz = x.shape[0]
        if not ops.ref_rank_supported(self.lora_rank):
            return tuple(self._invoke_single(n, x, layer_id, lora_ids) for n in "qkv")
        plan = self._plan_for(bsz, lora_ids)
        if not x.is_contiguous():
            x = x.contiguous()
        ys = [torch.empty(bsz, self.output_size, device=x.device, dtype=x.dtype) for _ in range(3)]
        ops.add_lora_bgmv_multi(ys, [x, x, x], [self.q_down, self.k_down, self.v_down], [self.q_up, self.k_up, self.v_up],
                                plan, layer_id, 1.0, accumulate=False)
        return tuple(ys)

    def _invoke_single(self, name, x, layer_id, lora_ids):
        bsz = x.shape[0]
        cur_inds = self._indices(bsz, lora_ids, x.device)
        y = torch.zeros(bsz, self.output_size, device=x.device, dtype=x.dtype)
        ops.add_lora_bgmv(y, x, getattr(self, f"{name}_down"), getattr(self, f"{name}_up"), cur_inds, layer_id, 1)
        return y

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
        if not ops.ref_rank_supported(self.lora_rank):
            return self._invoke_single(name, x, layer_id, lora_ids)
        # ``_get_qkv`` asks for q, k and v of the same input one after the other
        # (transformer_layer_infer.py:109-111): the first of the three calls computes all of them in one call pair,
        # the other two are answered from that result as long as it is the same input tensor object at the same
        # torch version, the same layer, the same plan and the same weight tensors at the same versions.
        self._plan_for(bsz, lora_ids)
        weights = [getattr(self, f"{n}_{side}") for n in "qkv" for side in ("down", "up")]
        key = (x._version, tuple(x.shape), layer_id, self._plan_gen, tuple(w._version for w in weights))
        fresh = (self._qkv_key != key or self._qkv_x is not x or name not in self._qkv
                 or any(a is not b for a, b in zip(self._qkv_w, weights)))
        if fresh:
            q, k, v = self.invoke_one_layer_qkv(x, layer_id, lora_ids)
            self._qkv, self._qkv_x, self._qkv_w, self._qkv_key = {"q": q, "k": k, "v": v}, x, weights, key
        return self._qkv.pop(name)

    def invoke_one_layer_q(self, x, layer_id, prefill=False, lora_ids=None):
        return self._invoke("q", x, layer_id, prefill, lora_ids)

    def invoke_one_layer_k(self, x, layer_id, prefill=False, lora_ids=None):
        return self._invoke("k", x, layer_id, prefill, lora_ids)

    def invoke_one_layer_v(self, x, layer_id, prefill=False, lora_ids=None):
        return self._invoke("v", x, layer_id, prefill, lora_ids)

    # ------------------------------------------------------------------ slot management
    def prepare_lora_prefill(self, batch_size):
        """lora_gpu.py:190-200: fresh random prefill adapters, one slot per request."""
        self._qkv_key = None
        for name in ("q", "k", "v"):
            setattr(self, f"{name}_down_prefill", self._rand(batch_size, self.in_size, self.lora_rank))
            setattr(self, f"{name}_up_prefill", self._rand(batch_size, self.lora_rank, self.output_size))

    def merge_lora_prefill(self, bsz, re_inds=None):
        """lora_gpu.py:202-217: copy the first bsz prefill slots into decode slots (random targets
        in the reference; pass re_inds to choose them)."""
        self._qkv_key = None                    # weights change: results computed from the old ones are not served again
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
        self._qkv_key = None
        if chosen is None:
            chosen = np.random.randint(0, running_bsz, size=len(rm_ids))
        for rm_id in chosen:
            for name in ("q", "k", "v"):
                for side in ("down", "up"):
                    w = getattr(self, f"{name}_{side}")
                    w[rm_id:-1] = w[rm_id + 1:].clone()
