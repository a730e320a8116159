"""Host-side checks of bench.py that need no GPU: its tables agree with the library's plan and with
the summaries under profiles/ they quote."""

import os
import re
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import bench  # noqa: E402
from custom_kernels import _l3lib  # noqa: E402


def test_measured_traffic_belongs_to_the_plan_the_library_makes():
    """roofline.traffic is reported only while the run's split plan is the profiled one: the table's
    plans must be what the library plans for a 256-unit device, or the key silently becomes null."""
    lib = _l3lib.load()
    B, HD, lengths, _ = bench.ATTN_WORKLOADS["c2"]
    for name in ("c2", "c3a", "c3b"):
        rec = bench.MEASURED_TRAFFIC[name]
        assert rec["flags"] == _l3lib.L3_ATTN_FLAG_WS_COUNTERS, "profiled with other flags than the default run uses"
        B, HD, lengths, _ = bench.ATTN_WORKLOADS[name]
        assert [lib.l3_attn_choose_splits(B, 8, S, HD, 256, rec["flags"]) for S in lengths] == rec["plan"]


def test_measured_traffic_quotes_its_profile():
    """Every entry names a summary under profiles/ that exists and holds the entry's figure in MB."""
    for name, rec in bench.MEASURED_TRAFFIC.items():
        path = os.path.join(ROOT, rec["profile"])
        assert os.path.isfile(path), f"{name}: {rec['profile']} is missing"
        text = open(path).read()
        mb = rec["bytes"] / 1e6
        figures = [float(x) for x in re.findall(r"\*\*(\d+\.\d+) MB", text)]
        assert any(abs(f - mb) < 0.02 for f in figures), f"{name}: {mb:.2f} MB not among {figures} in {rec['profile']}"


def test_more_than_one_gpu_is_refused():
    import subprocess

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)
