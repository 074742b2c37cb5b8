"""bench.py's clip-length and graph-launch arithmetic, without a GPU: every section must fit the
clip it builds for itself for any (steps, warmup) a caller passes, and exactly `steps` frames
are timed."""
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


CASES = [(20, 5), (8, 0), (200, 20), (7, 3), (1, 0), (13, 1), (64, 16), (9, 9)]


@pytest.mark.parametrize("steps,warmup", CASES)
def test_launch_plan_times_exactly_the_requested_frames(bench, steps, warmup):
    p = bench.launch_plan(steps, warmup)
    assert 1 <= p["unroll"] <= bench.UNROLL
    assert p["timed_main"] * p["unroll"] + p["tail"] == steps
    assert 0 <= p["tail"] < p["unroll"]
    assert p["warm_frames"] >= warmup
    assert p["warm_frames"] == p["warm_main"] * p["unroll"] + p["warm_tail"] * p["tail"]
    assert (p["warm_tail"] == 1) == (p["tail"] > 0)   # the tail graph has run once before the clock starts
    assert p["frames_after_start"] == p["warm_frames"] + steps
    if steps >= bench.UNROLL:
        assert p["unroll"] == bench.UNROLL            # never falls back to one frame per launch


@pytest.mark.parametrize("steps,warmup", CASES)
def test_headline_clip_holds_every_frame_the_graphs_touch(bench, steps, warmup):
    """Replays the frame positions time_graph visits (delta path starts at frame 2, the dense
    model at frame 1) against the clip length main() builds."""
    clip = bench.clip_frames(steps, warmup)
    p = bench.launch_plan(steps, warmup)
    for start in (1, 2):
        pos = start + p["warm_main"] * p["unroll"]
        if p["tail"]:
            pos += p["tail"]
        last = pos + p["timed_main"] * p["unroll"] + p["tail"]  # one past the last frame read
        assert last == start + p["frames_after_start"]
        assert last <= clip
    assert clip >= 4  # the kernel trace reads frames 0..3


def test_launch_plan_rejects_nonsense(bench):
    with pytest.raises(ValueError):
        bench.launch_plan(0, 0)
    with pytest.raises(ValueError):
        bench.launch_plan(8, -1)


@pytest.mark.parametrize("batch", [1, 8, 32])
@pytest.mark.parametrize("steps,warmup", [(64, 16), (32, 8), (4, 0), (6, 3)])
def test_streams_clip_is_sized_from_its_own_arguments(bench, batch, steps, warmup):
    u, stride = bench.STREAM_UNROLL, bench.STREAM_STRIDE
    eff = max(u, steps - steps % u)
    clip = bench.streams_clip_frames(batch, eff, warmup)
    last_stream_start = (batch - 1) * stride
    frames_read = 2 + -(-warmup // u) * u + (eff // u) * u
    assert last_stream_start + frames_read <= clip


def test_more_than_one_gpu_is_refused(bench, monkeypatch, capsys):
    monkeypatch.setattr("sys.argv", ["bench.py", "--gpus", "2"])
    with pytest.raises(SystemExit) as e:
        bench.main()
    assert e.value.code == 2
    assert "ONE GPU" in capsys.readouterr().err
