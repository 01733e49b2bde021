"""CPU checks of bench.py's contract: more than one GPU is refused with a message, the traffic
figures it quotes come out of the committed counter summaries, and its byte models are the
formulas the design states (per seed and per sampled edge)."""
import glob
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr + r.stdout and "--gpus 2" in r.stderr + r.stdout
    assert not r.stdout.strip().startswith("{")  # no bench line


def test_every_counter_summary_holds_a_traffic_figure_the_bench_can_read():
    paths = sorted(glob.glob(os.path.join(ROOT, "profiles", "*_hbm_counters.txt")))
    assert paths
    read = 0
    for path in paths:
        m = re.match(r"(.+)_(rmat-[^_]+)_hbm_counters\.txt$", os.path.basename(path))
        assert m, path
        text = open(path).read()
        assert "rocprofv3 --pmc FETCH_SIZE" in text and "WRITE_SIZE" in text, path  # the command is there
        got = bench.traffic_from_profile(m.group(1), m.group(2))
        if "traffic_bytes_per_launch" in text:
            assert isinstance(got, int) and got > 0, path
            read += 1
        else:
            assert got is None
    assert read >= 4  # the three launch sites of the minibatch on both graphs and the super-batch sampler
    assert bench.traffic_from_profile("layer_sample", "no-such-workload") is None


def test_byte_models_are_the_stated_formulas():
    S, E, U = 1000, 9000, 7000
    # fused slice + sample: 28 B per seed + 8 B per sampled edge at 4-byte ids, + 8 B per edge
    # with a weight read and written
    assert bench.sample_bytes(4, 0, S, E, U) == 28 * S + 8 * E
    assert bench.sample_bytes(4, 8, S, E, U) == 28 * S + 16 * E
    assert bench.sample_bytes(8, 0, S, E, U) == 32 * S + 16 * E
    assert bench.insert_bytes(4, 0, S, E, U) == 24 * (S + E)
    assert bench.compact_bytes(4, 0, S, E, U) == 20 * (S + E) + 4 * U
    # the published peak the fractions are taken against
    assert bench.HBM_PEAK_GBS == 8000.0


def test_a_failing_secondary_leg_is_recorded_and_does_not_raise():
    assert bench.leg(lambda: {"value": 1}) == {"value": 1}
    got = bench.leg(lambda: [][1])
    assert set(got) == {"error"} and got["error"].startswith("IndexError")
