"""bench.py's command line where no GPU is needed: more than one GPU is refused with a message."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and "shard by weight rows" in r.stderr
    assert r.stdout.strip() == ""  # no bench line


def test_traffic_figures_come_from_the_tracked_summaries():
    """`roofline.traffic` of the default decode steps is read from the counter summaries under profiles/, which
    state the commands that made them; the figure has to sit within a few percent of the algorithmic bytes."""
    sys.path.insert(0, ROOT)
    import bench

    C, H = 4096, 14336
    for quant, per_weight, per_block, block in (("int8", 1.0, 4, 128), ("nf4", 0.5, 2, 64)):
        traffic = bench.read_traffic(quant)
        assert isinstance(traffic, int) and traffic > 0
        weights = 5 * C * C + 2 * C * H + C * C  # one layer, 4 launches
        algorithmic = weights * (per_weight + per_block / block) / 4
        assert 0.98 < traffic / algorithmic < 1.05, (quant, traffic, algorithmic)
    assert bench.read_traffic("no-such-format") is None


def test_rnn_iter_cuts_runs_like_the_reference():
    """Known answers of the run cutter (src/runtime/infer/rnn.rs:280-335): chunk 256 with three prompts, then
    decode; run lengths above 32 are rounded down to multiples of 32."""
    sys.path.insert(0, ROOT)
    import bench

    state = [[False, 300], [False, 40], [False, 5]]
    lens = bench.rnn_iter_next(state, 256)
    assert sum(lens) == 256 and lens[2] == 5 and lens[1] == 40 and lens[0] == 211
    assert state == [[False, 89], [True, 0], [True, 0]]
    # 89 tokens left on slot 0, one token each on the two generating slots: 91 -> 64 after rounding
    lens = bench.rnn_iter_next(state, 256)
    assert sum(lens) == 64 and lens[1] == 1 and lens[2] == 1 and lens[0] == 62
