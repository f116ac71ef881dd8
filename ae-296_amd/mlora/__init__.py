"""mlora: MI355X-native multi-LoRA batched apply (BGMV decode, SGMV prefill, adapter-pool gather).

Host layer in Python over ``libmlora_hip.so`` (hand-written gfx950 kernels behind the C ABI of
``include/mlora.h``).  Importing the package does not load the extension; the first call does,
and raises if it has not been built.
"""
from . import _ext, cpu_ops
from ._ext import MloraError
from .cold_start import ColdStartPrefill
from .loader import AdapterLoader, HostAdapter, LoadTicket, layer_order
from .lora_cpu import Lora_CPU
from .lora_gpu import Lora_GPU
from .ops import (DecodePlan, PrefillPlan, RefDecodePlan, SideStream, side_by_side, add_lora_bgmv, add_lora_bgmv_multi, plan_decode_ref, bgmv, gemm_lora, lora_apply, lora_prefill_ref, plan_decode,
                  plan_prefill, sgmv, sgmv_multi, sgmv_workspace)
from .pool import AdapterPool

__all__ = ["ColdStartPrefill", "AdapterLoader", "AdapterPool", "HostAdapter", "LoadTicket", "layer_order", "DecodePlan", "SideStream", "side_by_side", "Lora_CPU", "Lora_GPU", "MloraError", "RefDecodePlan", "add_lora_bgmv", "add_lora_bgmv_multi", "plan_decode_ref", "bgmv", "gemm_lora", "lora_apply",
           "lora_prefill_ref", "plan_decode", "plan_prefill", "PrefillPlan", "sgmv", "sgmv_multi", "sgmv_workspace", "_ext", "cpu_ops"]
