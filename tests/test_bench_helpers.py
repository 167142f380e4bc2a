"""Host logic of bench.py that needs no GPU: the per-call distribution, the rotation over operand sets, and the figures read
from the committed profiles.  A stand-in for torch.cuda supplies a stream clock that advances by a known amount per call
and per event, so the arithmetic of the helpers can be checked against closed forms."""
import os
import sys
import types

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


class _Clock:
    def __init__(self, marker_us):
        self.us = 0.0
        self.marker_us = marker_us


def _fake_torch(clock):
    class Event:
        def __init__(self, enable_timing=False):
            self.t = None

        def record(self, stream=None):
            clock.us += clock.marker_us
            self.t = clock.us

        def elapsed_time(self, other):  # milliseconds, like torch
            return (other.t - self.t) * 1e-3

    cuda = types.SimpleNamespace(Event=Event, synchronize=lambda: None, empty_cache=lambda: None)
    return types.SimpleNamespace(cuda=cuda)


def _bench(clock, plain=False):
    b = bench.Bench.__new__(bench.Bench)
    b.args = types.SimpleNamespace(plain=plain, steps=20, warmup=5)
    b.torch = _fake_torch(clock)
    b.stream = object()
    b.settle = lambda fn, seconds=0.0: fn()
    return b


def test_per_launch_distribution_and_marker_cost():
    clock = _Clock(marker_us=3.5)
    b = _bench(clock)
    calls = []

    def fn():
        calls.append(1)
        clock.us += 60.0 if len(calls) % 7 else 67.0  # every seventh call is slower

    d = b.per_launch(fn, n=60, group=5)
    assert d["launches"] == 300 and d["intervals"] == 60 and d["calls_per_interval"] == 5
    # an interval holds five calls and one marker: 5 x 60 + 3.5 = 303.5 us without a slow call
    assert d["min"] == pytest.approx(303.5 / 5) and d["max"] >= d["median"] >= d["min"]
    assert d["max"] == pytest.approx((303.5 + 7.0) / 5)
    assert d["marker_us_per_call"] == pytest.approx(3.5 / 5, abs=0.05)
    assert d["mean_without_markers"] == pytest.approx(61.0, abs=0.1) and d["mean"] == pytest.approx(61.7, abs=0.1)
    assert len(calls) == 1 + 300 + 300  # the settle call, the marker-free pass, the pass with markers


def test_plain_mode_skips_the_extras():
    clock = _Clock(marker_us=1.0)
    b = _bench(clock, plain=True)
    assert b.per_launch(lambda: None) is None and b.clocked(lambda: None) is None and b.matrix_core_ceiling(0) is None
    roof = {"bound": "mfma", "peak": 5000.0}
    assert bench.rotating_figures(b, [lambda: None], 1.0, roof, 1) is None


def test_rotating_takes_every_set_in_turn():
    clock = _Clock(marker_us=0.0)
    b = _bench(clock)
    hits = [0, 0, 0, 0, 0]

    def make(i):
        def fn():
            hits[i] += 1
            clock.us += 50.0
        return fn

    roof = {"bound": "mfma", "peak": 5000.0}
    r = bench.rotating_figures(b, [make(i) for i in range(5)], 137.4e9, roof, 64 << 20)
    assert r["sets"] == 5 and r["bytes_cycled"] == 5 * (64 << 20)
    assert max(hits) - min(hits) <= 1 and min(hits) > 50
    assert r["kernel_ms"] == pytest.approx(0.05) and r["achieved"] == pytest.approx(137.4e9 / 50e-6 / 1e12, rel=1e-3)
    assert r["frac"] == pytest.approx(r["achieved"] / 5000.0, abs=1e-4)
    assert r["per_launch_us"]["median"] == pytest.approx(50.0)


def test_number_of_sets_exceeds_the_memory_side_cache():
    for set_bytes in (64 << 20, 51 << 20, 40 << 20, 400 << 20):
        assert bench.n_sets(set_bytes) >= 2 and bench.n_sets(set_bytes) * set_bytes >= bench.ROTATE_BYTES > (256 << 20)


def test_profile_figures_follow_from_the_committed_profiles():
    """Every workload's profile names a traced kernel time and the bytes moved; the fraction bench.py prints beside its own
    is that time's, recomputed here from the file's text."""
    import re
    work = {"c2": 2.0 * 4096 ** 3, "c3": 2.0 * 64 * 56 * 56 * 64 * 64 * 9, "c5": 2.0 * 4 * 2048 * 14336 * 4096, "cast_fp8_143": 5.0 * 2 ** 28}
    peak = {"c2": 5e15, "c3": 2.5e15, "c5": 5e15, "cast_fp8_143": 8e12}
    for name in bench.PROFILE_FILE:
        path = os.path.join(ROOT, "profiles", bench.PROFILE_FILE[name])
        assert os.path.exists(path), path
        fig = bench.profile_figures(name, work.get(name, 1.0), peak.get(name, 1.0))
        assert fig is not None and fig["file"].endswith(bench.PROFILE_FILE[name]) and fig["kernel_us"] > 0
        text = open(path).read()
        us = float(re.search(r"kernel_us=([0-9.]+)", text).group(1))
        assert fig["kernel_us"] == us
        if name in work:
            assert fig["frac"] == pytest.approx(work[name] / (us * 1e-6) / peak[name], abs=1e-4)
            assert 0.05 < fig["frac"] < 1.0
        assert fig.get("traffic", 1.0) > 0
    roof = {"bound": "mfma", "peak": 5000.0, "work_per_launch": work["c2"]}
    bench.attach_profile(roof, "c2")
    assert roof["profile"]["frac"] == pytest.approx(work["c2"] / (roof["profile"]["kernel_us"] * 1e-6) / 5e15, abs=1e-4)
    assert roof["traffic"] == roof["profile"]["traffic"]
    assert bench.profile_figures("no such workload", 1.0, 1.0) is None
