#!/usr/bin/env python3
"""Writes tests/golden/maf_trace_{128,256,512}.npy: the arrival times of the reference's trace files
(benchmark/traces/maf_trace_*_scale_0.4.txt, plain text, one time per line after a ===== line) as float64 arrays.
Data only; run in the container that holds /root/reference:  python tests/golden/make_traces.py"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "ae-296_amd"))
from mlora.trace_driver import parse_trace  # noqa: E402

SRC = "/root/reference/benchmark/traces"
for n in (128, 256, 512):
    t = parse_trace(os.path.join(SRC, f"maf_trace_{n}_scale_0.4.txt"))
    assert t.size > 0 and np.all(np.diff(t) >= 0)
    np.save(os.path.join(HERE, f"maf_trace_{n}.npy"), t)
    print(n, t.size, t[:4], t[-1])
