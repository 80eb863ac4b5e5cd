"""Host-side pieces of bench.py that need no GPU: the argument contract and the power-sensor reader."""
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "one GPU" in r.stderr


def test_median():
    assert bench._median([3.0, 1.0, 2.0]) == 2.0
    assert bench._median([4.0, 1.0, 2.0, 3.0]) == 2.5


def test_power_sampler_reads_microwatts_and_drops_the_ramp(tmp_path):
    power, cap = tmp_path / "power1_input", tmp_path / "power1_cap"
    power.write_text("250000000\n")
    cap.write_text("1400000000\n")
    ps = bench.PowerSampler()
    ps.path, ps.cap_path = str(power), str(cap)
    with ps:
        time.sleep(0.15)
        power.write_text("1380000000\n")
        time.sleep(0.3)
    rep = ps.report()
    assert rep["cap_w"] == 1400.0
    assert rep["max_w"] == 1380.0
    assert rep["avg_w"] > 1000.0  # the first two fifths of the samples are not counted
    assert rep["samples"] >= 5


def test_power_sampler_without_a_sensor_reports_nothing(tmp_path):
    ps = bench.PowerSampler()
    ps.path, ps.cap_path = str(tmp_path / "missing"), None
    with ps:
        time.sleep(0.05)
    assert ps.report() is None


def test_traffic_table_names_files_that_exist():
    for (workload, instance), (nbytes, path) in bench.MEASURED_TRAFFIC.items():
        assert workload in bench.SHAPES
        assert nbytes > 0
        full = os.path.join(ROOT, path)
        assert os.path.isfile(full), path
        text = open(full).read()
        assert instance in text
        # the file shows the figure itself, as megabytes or written out
        assert f"{nbytes:,}".replace(",", " ") in text, (path, nbytes)
        assert bench.measured_traffic(workload, instance)[0] == nbytes
    assert bench.measured_traffic("c2a", "no_such_instance")[0] is None


def test_graph_of_a_launch_bound_configuration_never_holds_fewer_than_100_launches():
    # the driver's "--steps 20 --warmup 5" reaches other_configs as 20 steps in 20 groups
    assert bench.graph_plan(20, 20) == (100, 20)
    assert bench.graph_plan(1, 20) == (100, 1)
    assert bench.graph_plan(200, 20) == (100, 20)
    # more steps than 100 per group: the graph grows, the number of replays stays the number of groups
    assert bench.graph_plan(4000, 20) == (200, 20)
    assert bench.graph_plan(4001, 20) == (201, 20)
    assert bench.graph_plan(60, 1) == (100, 1)


class _FakeTorch:
    """Just enough of torch.cuda for timed_region's direct-launch path: events count the steps issued so far."""

    class cuda:
        issued = 0

        @staticmethod
        def synchronize():
            pass

        class Event:
            def __init__(self, enable_timing=True):
                self.at = None

            def record(self):
                self.at = _FakeTorch.cuda.issued

            def elapsed_time(self, other):
                return float(other.at - self.at)


def test_timed_region_runs_settle_and_warmup_untimed_and_times_exactly_k_steps():
    calls = []

    def step(i):
        _FakeTorch.cuda.issued += 1
        calls.append(i)

    _FakeTorch.cuda.issued = 0
    r = bench.timed_region(_FakeTorch, step, 20, 5, settle=300)
    assert len(calls) == 300 + 5 + 20
    # the driver's 20 steps make two groups of ten: no event between single launches
    assert r["steps"] == 20 and r["settle_launches"] == 300 and r["groups"] == 2
    assert r["event_ms_per_launch"] == 1.0 and r["median_ms_per_launch"] == 1.0  # one "ms" per fake launch
    assert bench.SETTLE_LAUNCHES >= 300
