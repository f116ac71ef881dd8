#!/usr/bin/env python3
"""Build-time check of what the compiler made of the kernels whose speed depends on it.

`python3 resource_usage.py` compiles the listed sources for gfx950 (device code only, no GPU needed) with
`-Rpass-analysis=kernel-resource-usage`, prints one line per kernel and exits with status 1 when a kernel leaves
the limits below.  The limits say what the kernels were designed around:

* no kernel of this library may use scratch memory (a spilled accumulator is a correct but several times slower
  kernel, which no parity test can see);
* `gemm_lora_kernel` keeps its 256 fp32 accumulators in AGPRs, runs one workgroup per compute unit and must not
  move accumulators between AGPRs and VGPRs inside the K loop (the epilogue reads each of them out: about a thousand
  moves over its unrolled paths; the K loop gone wrong adds more than that again);
* the decode shrink of a one-round launch needs at least four (rank <= 16) or three (rank 32) workgroups per
  compute unit, the expand three;
* M0 in `gemm_lora_kernel` is written only by the kernel's own LDS-bound loads: one `s_mov_b32 m0` per such load
  and no other instruction that names M0.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "--cuda-device-only", "-S", "-Rpass-analysis=kernel-resource-usage"]

# (source, regular expression on the demangled kernel name, {field: (min, max)})
LIMITS = [
    ("gemm_lora.hip", r"gemm_lora_kernel<", {"scratch": (0, 0), "vgpr_spill": (0, 0), "agprs": (256, 256), "vgprs": (0, 256),
                                             "occupancy": (1, 1), "lds": (0, 160 * 1024), "accvgpr_moves": (0, 1300)}),
    ("gemm_lora.hip", r".", {"scratch": (0, 0), "vgpr_spill": (0, 0)}),
    ("bgmv_split.hip", r".", {"scratch": (0, 0), "vgpr_spill": (0, 0)}),
    ("bgmv_split.hip", r"bgmv_shrink_kernel<\d, [124], 16, 256, false>", {"occupancy": (4, 8)}),
    ("bgmv_split.hip", r"bgmv_expand_kernel<\d, [124], 16, 256, 256, false>", {"occupancy": (3, 8)}),
    ("bgmv_split.hip", r"bgmv_shrink_kernel<\d, [124], 32, 128, false>", {"occupancy": (3, 8)}),
    ("bgmv_split.hip", r"bgmv_expand_kernel<\d, [124], 32, 128, 128, false>", {"occupancy": (3, 8)}),
    ("bgmv_decode.hip", r".", {"scratch": (0, 0), "vgpr_spill": (0, 0)}),
    ("sgmv_prefill.hip", r".", {"scratch": (0, 0), "vgpr_spill": (0, 0)}),
    ("sgmv_prefill.hip", r"sgmv_shrink_kernel<\d, (16|32)>", {"occupancy": (3, 8)}),
    ("sgmv_prefill.hip", r"sgmv_shrink_kernel<\d, 64>", {"occupancy": (2, 8)}),
]

FIELDS = {"TotalSGPRs": "sgprs", "VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch",
          "Occupancy [waves/SIMD]": "occupancy", "SGPRs Spill": "sgpr_spill", "VGPRs Spill": "vgpr_spill",
          "LDS Size [bytes/block]": "lds"}


def demangle(names):
    out = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True, check=True).stdout.split("\n")
    return dict(zip(names, out))


def parse_remarks(text: str):
    """{mangled kernel name: {field: int}} from the compiler's remarks."""
    kernels, cur = {}, None
    for line in text.splitlines():
        m = re.search(r"remark:\s+(.*?) \[-Rpass-analysis=kernel-resource-usage\]", line)
        if not m:
            continue
        body = m.group(1).strip()
        if body.startswith("Function Name:"):
            cur = kernels.setdefault(body.split(":", 1)[1].strip(), {})
        elif cur is not None and ":" in body:
            k, v = body.rsplit(":", 1)
            if k.strip() in FIELDS and v.strip().lstrip("-").isdigit():
                cur[FIELDS[k.strip()]] = int(v)
    return kernels


def parse_asm(text: str, kernels):
    """Adds per-kernel instruction counts taken from the assembly: AGPR <-> VGPR moves, M0 writes and other M0
    mentions, loads that land in LDS, scratch instructions."""
    for name, rec in kernels.items():
        m = re.search(r"^%s:" % re.escape(name), text, re.M)
        if not m:
            continue
        end = text.find(".Lfunc_end", m.end())
        body = [ln.split(";")[0] for ln in text[m.end():end].splitlines()]
        code = [ln.strip() for ln in body if ln.strip() and not ln.strip().startswith(".")]
        rec["accvgpr_moves"] = sum(1 for ln in code if ln.startswith("v_accvgpr_"))
        rec["scratch_insts"] = sum(1 for ln in code if ln.startswith("scratch_"))
        rec["lds_loads"] = sum(1 for ln in code if ln.startswith("buffer_load") and ln.endswith(" lds"))
        rec["m0_writes"] = sum(1 for ln in code if re.match(r"s_mov_b32 m0, ", ln))
        rec["m0_other"] = sum(1 for ln in code if re.search(r"\bm0\b", ln) and not re.match(r"s_mov_b32 m0, ", ln))
    return kernels


def compile_report(source: str, extra_flags=()):
    """Compile one source of this directory; returns {demangled name: fields}."""
    with tempfile.TemporaryDirectory() as tmp:
        asm = os.path.join(tmp, "k.s")
        r = subprocess.run([HIPCC, *FLAGS, *extra_flags, os.path.join(HERE, source), "-o", asm], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {source}:\n{r.stderr[-2000:]}")
        kernels = parse_remarks(r.stderr)
        with open(asm) as f:
            parse_asm(f.read(), kernels)
    names = demangle(list(kernels))
    return {re.sub(r"\(.*$", "", names[k]).replace("void ", "").replace("mlora::", ""): v for k, v in kernels.items()}


def violations(source: str, report):
    """List of strings, one per (kernel, field) outside LIMITS, plus the M0 rule of gemm_lora_kernel."""
    bad = []
    for src, pattern, limits in LIMITS:
        if src != source:
            continue
        hit = False
        for name, rec in report.items():
            if not re.search(pattern, name):
                continue
            hit = True
            for field, (lo, hi) in limits.items():
                v = rec.get(field)
                if v is None or not lo <= v <= hi:
                    bad.append(f"{source}: {name}: {field} = {v}, allowed {lo}..{hi}")
        if not hit:
            bad.append(f"{source}: no kernel matches {pattern!r}")
    if source == "gemm_lora.hip":
        for name, rec in report.items():
            if "gemm_lora_kernel<" in name:
                if rec.get("m0_other", 1) != 0 or rec.get("m0_writes", 0) != rec.get("lds_loads", -1):
                    bad.append(f"{source}: {name}: M0 is named by {rec.get('m0_other')} instructions besides its "
                               f"{rec.get('m0_writes')} writes, for {rec.get('lds_loads')} LDS-bound loads")
    return bad


def sources():
    return sorted({s for s, _, _ in LIMITS})


def main() -> int:
    bad = []
    for src in sources():
        rep = compile_report(src)
        for name, rec in sorted(rep.items()):
            print(f"{src:18s} {name[:66]:66s} vgpr {rec.get('vgprs', -1):3d} agpr {rec.get('agprs', -1):3d} "
                  f"sgpr {rec.get('sgprs', -1):3d} occ {rec.get('occupancy', -1)} scratch {rec.get('scratch', -1)} "
                  f"lds {rec.get('lds', -1):6d} acc-moves {rec.get('accvgpr_moves', -1)}")
        bad += violations(src, rep)
    for b in bad:
        print("VIOLATION:", b)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
