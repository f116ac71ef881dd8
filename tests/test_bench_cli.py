"""bench.py on a machine without a GPU: the contract's refusals and the arithmetic it reports."""
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_algorithmic_bytes_formula():
    """Per projection call: x + y read + y write + every touched adapter's rows once + indices
    (the worked figure for config 2 with 54 adapters touched is 20.4 MB per projection)."""
    sys.path.insert(0, ROOT)
    import bench
    one = bench.algorithmic_bytes(256, [(4096, 4096)], np.full(54, 16))
    assert one == 256 * 4096 * 2 + 2 * 256 * 4096 * 2 + 54 * 16 * 8192 * 2 + 4 * 256
    assert abs(one / 1e6 - 20.4) < 0.1
    four = bench.algorithmic_bytes(256, [(4096, 4096)] * 4, np.full(54, 16))
    assert four == 4 * one
    assert set(bench.DECODE) >= {"c1", "c2", "c3", "c5", "maf128", "maf256", "maf512"}
    for name, cfg in bench.DECODE.items():
        assert cfg["T"] > 0 and cfg["layers"] > 0 and all(p in bench._IN for p in cfg["projs"]), name


def test_traffic_figures_come_from_the_tracked_profiles():
    """`roofline.traffic` is not a constant in bench.py: it is the `hbm_bytes_...` line of the workload's summary
    under profiles/, which also states the counter commands and scale factors it came from."""
    import re
    sys.path.insert(0, ROOT)
    import bench
    for workload, (path, key) in bench.TRAFFIC_SOURCE.items():
        text = open(os.path.join(ROOT, path)).read()
        m = re.search(r"^\s*%s:\s*(\d+)\s*$" % re.escape(key), text, re.M)
        assert m, f"{path} has no `{key}:` line"
        value, source = bench.traffic_of(workload)
        assert value == float(m.group(1)) and path in source
        assert "rocprofv3 --pmc FETCH_SIZE" in text and "rocprofv3 --pmc WRITE_SIZE" in text and "FETCH_SIZE x" in text
        assert f"bench.py --workload {workload}" in text
    # every summary names the full command that produced it and runs committed files only
    for name in os.listdir(os.path.join(ROOT, "profiles")):
        text = open(os.path.join(ROOT, "profiles", name)).read()
        assert "command: rocprofv3 --kernel-trace --stats" in text and "python3 bench.py" in text, name
        assert "_work/" not in text, name
