"""CPU-side checks of the C ABI: the library loads, exports every function include/mlora.h declares
with the arity the Python binding uses, and rejects bad arguments before touching the GPU."""
import ctypes as C
import os
import re

import pytest

from mlora import _ext

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "mlora.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(?:const\s+char\s*\*|int64_t|int)\s*(mlora_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args == "void" else len([a for a in args.split(",") if a.strip()])
    return out


def test_header_and_binding_agree():
    decl = _declared()
    assert set(decl) == set(_ext.SIGNATURES), (sorted(decl), sorted(_ext.SIGNATURES))
    for name, n in decl.items():
        assert len(_ext.SIGNATURES[name][1]) == n, name


def test_library_exports_every_symbol():
    lib = _ext.lib()
    for name in _declared():
        assert hasattr(lib, name), name
    assert lib.mlora_version() >= 100


def test_validation_errors_without_gpu():
    lib = _ext.lib()
    one = C.c_void_p(16)      # never dereferenced: every call below fails validation first
    P = (C.c_void_p * 8)(16, 16, 16, 16, 16, 16, 16, 16)
    H = (C.c_int32 * 8)(64, 64, 64, 64, 64, 64, 64, 64)

    def bgmv(**kw):
        a = dict(n_proj=1, hin=H, T=4, n_adapters=4, max_pages=8, page_rows=8, n_pages=10, max_rank=64, work=None,
                 group=1, dtype=0, y=P, ws=None, ws_bytes=0)
        a.update(kw)
        return lib.mlora_bgmv_multi(a["n_proj"], a["y"], P, P, P, a["hin"], H, one, a["T"], one, one, one,
                                    a["n_adapters"], a["max_pages"], a["page_rows"], a["n_pages"], a["max_rank"],
                                    a["work"], a["group"], a["ws"], a["ws_bytes"], a["dtype"], 1, None)

    assert bgmv(T=0) == _ext.MLORA_OK
    assert bgmv(dtype=7) == _ext.MLORA_EDTYPE
    assert b"dtype" in lib.mlora_last_error()
    assert bgmv(n_proj=9) == _ext.MLORA_ERANGE
    assert bgmv(max_rank=65) == _ext.MLORA_ERANGE
    assert bgmv(page_rows=3) == _ext.MLORA_EINVAL
    assert bgmv(ws=16, ws_bytes=1 << 20) == _ext.MLORA_EINVAL            # two-launch form without work records
    assert b"work records" in lib.mlora_last_error()
    assert bgmv(ws=16, ws_bytes=64, work=16, group=4) == _ext.MLORA_ENOSPACE
    assert lib.mlora_bgmv_workspace_bytes(4, 256, 4096, 16) == 4 * 256 * 2 * 16 * 4
    assert lib.mlora_bgmv_workspace_bytes(1, 10, 11008, 33) == 10 * 11 * 64 * 4
    assert bgmv(max_pages=1, page_rows=8, max_rank=16) == _ext.MLORA_ERANGE
    assert bgmv(hin=(C.c_int32 * 8)(60, 0, 0, 0, 0, 0, 0, 0)) == _ext.MLORA_EALIGN
    assert bgmv(y=(C.c_void_p * 8)(8, 0, 0, 0, 0, 0, 0, 0)) == _ext.MLORA_EALIGN
    assert bgmv(group=4) == _ext.MLORA_EINVAL          # grouped launch without work records
    assert bgmv(group=8, work=one, max_rank=64) == _ext.MLORA_ERANGE
    assert bgmv(group=3, work=one) == _ext.MLORA_EINVAL
    assert bgmv(T=-1) == _ext.MLORA_EINVAL
    with pytest.raises(_ext.MloraError) as e:
        _ext.check(bgmv(dtype=7))
    assert e.value.code == _ext.MLORA_EDTYPE

    # the allocation-free form: needs work records, and refuses a batch whose intermediate exceeds its fixed array
    def noalloc(T=4, work=one, n_proj=1, hin=H, max_rank=64):
        return lib.mlora_bgmv_multi_noalloc(n_proj, P, P, P, P, hin, H, one, T, one, one, one, 4, 8, 8, 10, max_rank,
                                            work, 4, 0, 1, None)
    assert noalloc(work=None) == _ext.MLORA_EINVAL
    assert b"work records" in lib.mlora_last_error()
    big = (C.c_int32 * 8)(*([11008] * 8))
    assert lib.mlora_bgmv_workspace_bytes(8, 8192, 11008, 64) > _ext.NOALLOC_SCRATCH_BYTES
    assert noalloc(T=8192, n_proj=8, hin=big) == _ext.MLORA_ENOSPACE
    assert b"allocation-free" in lib.mlora_last_error()
    assert noalloc(T=0) == _ext.MLORA_OK

    rc = lib.mlora_pool_gather(one, 9000, one, one, one, 4, 8, 8, 10, None, None, None, one, one, one, one, one, one, one, 4, one, one, None)
    assert rc == _ext.MLORA_ERANGE                     # more tokens than one gather call groups
    rc = lib.mlora_pool_gather(one, 10, one, one, one, 4, 8, 8, 10, None, None, None, one, None, one, one, one, one, one, 4, one, None, None)
    assert rc == _ext.MLORA_EINVAL                     # incomplete grouped view
    rc = lib.mlora_pool_gather(one, 10, one, one, one, 4, 8, 8, 10, None, None, None, one, one, one, one, one, one, one, 3, one, None, None)
    assert rc == _ext.MLORA_EINVAL                     # group not a power of two
    rc = lib.mlora_pool_gather(one, 10, one, one, one, 4, 8, 8, 0, None, None, None, one, one, one, one, one, one, one, 4, one, one, None)
    assert rc == _ext.MLORA_EINVAL                     # work records need the slab extent

    assert lib.mlora_sgmv_workspace_bytes(9089, 16) > 9089 * 64 * 4
    rc = lib.mlora_sgmv(one, one, one, one, one, one, one, 2, one, one, one, 100, 64, 64, 4, 8, 8, 10, 64, 1, 1,
                        one, 16, None)
    assert rc == _ext.MLORA_ENOSPACE
    rc = lib.mlora_bgmv_reflayout(one, one, one, one, one, 4, 8, 32, 16, 64, 64, 32, 1.0, 0, None)
    assert rc == _ext.MLORA_ERANGE                     # layer_idx == L
    # grouped reference-layout call: ranks 8 / 16 / 32 / 64 only, plan buffer and workspace sizes checked
    assert lib.mlora_reflayout_plan_bytes(256) == (7 * 256 + 8 + 256 * 80) * 4
    assert lib.mlora_reflayout_plan(one, 10, 8, 2, 12, 4, one, 1 << 20, None) == _ext.MLORA_ERANGE
    assert b"rank 8, 16, 32 or 64" in lib.mlora_last_error()
    assert lib.mlora_reflayout_plan(one, 10, 8, 2, 16, 4, one, 64, None) == _ext.MLORA_ENOSPACE
    assert lib.mlora_reflayout_plan(one, 10, 8, 2, 16, 8, one, 1 << 20, None) == _ext.MLORA_EINVAL
    rc = lib.mlora_bgmv_reflayout_multi(1, P, P, P, P, H, H, one, 10, 8, 2, 16, 2, 1.0, 4, 0, 1, one, 1 << 20, None)
    assert rc == _ext.MLORA_ERANGE                     # layer_idx == L
    rc = lib.mlora_bgmv_reflayout_multi(1, P, P, P, P, H, H, one, 10, 8, 2, 16, 1, 1.0, 4, 0, 1, one, 16, None)
    assert rc == _ext.MLORA_ENOSPACE
    rc = lib.mlora_prefill_reflayout(one, one, one, one, 2, 16, 4, 12, 64, 64, 0, 0, one, 1 << 30, None)
    assert rc == _ext.MLORA_ERANGE                     # rank not a multiple of 8
