"""bench.py's host side: the traffic figure of every roofline line is the one its rocprofv3
summary under profiles/ holds, the workload list starts with the metric's configurations,
and a run on more than one GPU is refused.  No GPU work is issued."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_metric_configurations_come_first():
    assert bench.ALL_WORKLOADS[:2] == ["tbq_vgg19", "dgc_vgg19"]
    assert len(set(bench.ALL_WORKLOADS)) == len(bench.ALL_WORKLOADS)


@pytest.mark.parametrize("name", bench.ALL_WORKLOADS)
def test_traffic_is_read_from_the_committed_profile(name):
    w = bench.make_workload(name)
    path = os.path.join(ROOT, "profiles", name + ".md")
    traffic, source = bench.measured_traffic(name, w.dominant_kernel)
    if not os.path.exists(path) or "HBM traffic per dispatch" not in open(path).read():
        assert traffic is None
        return
    assert source == os.path.join("profiles", name + ".md")
    # the figure is the table's own: (2.0 x FETCH_SIZE + 1.0 x WRITE_SIZE) x 1024
    row = [l for l in open(path).read().split("HBM traffic per dispatch", 1)[1].splitlines() if w.dominant_kernel in l][0]
    cells = [c.strip() for c in row.split("|")]
    fetch_kib, write_kib = float(cells[3]), float(cells[4])
    assert abs(traffic - (2.0 * fetch_kib + write_kib) * 1024) <= 2048
    # and no more than a third above what the kernel must move
    launches = 1  # a very long accumulate pass is issued in equal parts; the table holds bytes per dispatch
    if w.dominant_kernel == "sparse_accum_kernel":
        launches = -(-sum(-(-n // 4096) for n in w.sizes) // 49152)
    algorithmic = w.dominant_bytes * w.elements / launches
    assert 0.9 * algorithmic <= traffic <= 1.35 * algorithmic, (traffic, algorithmic)


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "one GPU" in r.stderr
