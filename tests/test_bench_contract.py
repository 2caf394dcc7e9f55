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


@pytest.mark.parametrize("name", bench.ALL_WORKLOADS)
def test_kernel_duration_is_read_from_the_committed_profile(name):
    """roofline.frac is algorithmic bytes over the kernel's average duration in the committed
    rocprofv3 summary, so a reader can re-derive it from the table."""
    w = bench.make_workload(name)
    path = os.path.join(ROOT, "profiles", name + ".md")
    us, source = bench.profile_kernel_us(name, w.dominant_kernel)
    assert os.path.exists(path), "every bench workload has a committed summary"
    assert source == os.path.join("profiles", name + ".md")
    table = open(path).read().split("Kernel statistics", 1)[1].split("HBM traffic per dispatch", 1)[0]
    row = [l for l in table.splitlines() if w.dominant_kernel in l][0]
    assert us == float(row.split("|")[3])
    launches = bench.launches_per_step(w)
    bytes_per_launch = w.dominant_bytes * w.elements / launches
    roof = bench.roofline_of(name, w.dominant_kernel, bytes_per_launch, launches, events_ms=None)
    assert roof["kernel_ms_source"] == source and roof["kernel_ms_events"] is None
    assert roof["frac"] == pytest.approx(bytes_per_launch / (us * 1e-6) / 8e12, rel=1e-9)
    assert roof["achieved"] == pytest.approx(roof["frac"] * roof["peak"])
    if roof["traffic"] is not None:
        assert roof["traffic_ratio"] == pytest.approx(roof["traffic"] / bytes_per_launch)
    # the live duration is carried beside it and decides only where no summary exists
    live = bench.roofline_of(name, w.dominant_kernel, bytes_per_launch, launches, events_ms=us * 1.1e-3)
    assert live["frac"] == roof["frac"] and live["frac_events"] == pytest.approx(roof["frac"] / 1.1)
    none = bench.roofline_of("no_such_workload", w.dominant_kernel, bytes_per_launch, launches, events_ms=0.5)
    assert none["kernel_ms_source"] == "hipEvent" and none["frac"] == none["frac_events"]


def _canned(name, i):
    """A full per-workload record as bench.measure() returns it, with long numbers and a long
    CPU sample description."""
    w = bench.make_workload(name)
    launches = bench.launches_per_step(w)
    roof = bench.roofline_of(name, w.dominant_kernel, w.dominant_bytes * w.elements / launches, launches, 0.2650288507342339)
    return {"workload": name, "warmup_steps_run": 725 + i, "value": 1685.6654088812945 + i, "ms_per_step": 0.3409151999989035,
            "median_ms_per_step": 0.3430345058441162, "value_at_median": 1675.25, "elements": w.elements,
            "tensors": len(w.sizes), "algorithmic_bytes_per_element": 24.016549019804373,
            "pct_of_hbm_roofline": 86.91712264544175, "density": 0.0010343137377734827, "roofline": roof,
            "cpu_baseline": {"value": 0.6694913005727317, "unit": "GB/s", "cores": 1, "kind": "port",
                             "sample": "tbq encode+decode over the first <= 4,194,304 elements of 35 of the set's 38 tensors "
                                       "(25,165,824 elements per pass), 67 passes, 10.1 s, scalar C oracle (gcc -O3, one thread)",
                             "sample_short": "front of the same tensors, 25,165,824 elements/pass x 67 passes, 10.1 s, scalar C oracle",
                             "all_cores": {"value": 8.955231171352244, "unit": "GB/s", "cores": 16,
                                           "sample": "same sample, same source built with -fopenmp, 445 passes, 5.0 s"}}}


def test_the_printed_line_is_compact_and_complete():
    """The line the driver parses: one JSON object below 4 KB with the headline's roofline and
    CPU baseline, whatever the number of workloads measured beside it."""
    import json

    records = [_canned(name, i) for i, name in enumerate(bench.ALL_WORKLOADS)]
    line = bench.compact_line(records[0], records[1:], 20, 5)
    text = json.dumps(line, separators=(",", ":"))
    assert "\n" not in text and len(text) < bench.MAX_LINE_BYTES == 4096, len(text)
    back = json.loads(text)
    assert back["metric"] == bench.METRIC and back["unit"] == "GB/s" and back["n_gpus"] == 1
    assert back["steps"] == 20 and back["warmup"] == 5 and back["higher_is_better"] is True
    assert back["config"]["workload"] == "tbq_vgg19" and back["vs_baseline"] is None and back["dtype"] == "f32"
    assert back["value"] == pytest.approx(records[0]["value"], rel=1e-5)
    assert back["ms_per_step"] == pytest.approx(records[0]["ms_per_step"], rel=1e-5)
    roof = back["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert roof["kernel"] == "tbq_encode_kernel" and 0 < roof["frac"] < 1
    assert roof["frac"] == pytest.approx(roof["achieved"] / roof["peak"], rel=2e-3)
    assert roof["traffic"] > 0 and roof["traffic_ratio"] == pytest.approx(roof["traffic"] / roof["algorithmic_bytes_per_launch"], rel=1e-3)
    assert roof["kernel_ms_profile"] > 0 and roof["kernel_ms_events"] > 0
    cpu = back["cpu_baseline"]
    assert cpu["value"] > 0 and cpu["cores"] == 1 and cpu["kind"] == "port" and len(cpu["sample"]) <= 120
    assert cpu["all_cores"]["cores"] == 16
    assert back["others_cpu_cores"] == {"cpu1": 1, "cpuN": 16}
    assert [o["workload"] for o in back["others"]] == bench.ALL_WORKLOADS[1:]
    for o in back["others"]:
        assert set(o) == {"workload", "value", "ms_per_step", "pct", "frac", "cpu1", "cpuN"}
        assert o["frac"] is not None and o["cpu1"] is not None


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "one GPU" in r.stderr
