"""Host-side logic of bench.py that needs no GPU: how weight copies are rotated so that every timed launch reads HBM, the
byte counts behind the GB/s figures, and the refusal of more than one GPU."""
import math
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def reuse_distance(steps, copies, graphs, replays):
    """Smallest number of other launches between two reads of one buffer when `graphs` graphs of `steps` launches are
    replayed in turn."""
    seq = [(r * steps + i) % copies for r in range(replays) for i in range(steps)]
    last, best = {}, None
    for n, b in enumerate(seq):
        if b in last:
            d = n - last[b] - 1
            best = d if best is None else min(best, d)
        last[b] = n
    return best


def test_rotation_never_reuses_a_buffer_too_early():
    for steps in (1, 2, 5, 7, 20, 100, 500, 2000):
        for copies in (2, 3, 10, 19, 20, 21, 61, 96):
            for needed in (2, 3, 10, 11, 20):
                needed = min(needed, copies)
                c, g = bench.rotation(steps, copies, needed)
                assert needed <= c <= copies and g == c // math.gcd(steps, c)
                # replaying the g graphs in turn continues one sequence 0, 1, ..., c - 1, 0, ... without a seam
                assert (g * steps) % c == 0
                d = reuse_distance(steps, c, g, 3 * g + 2)
                assert d is None or d >= c - 1 >= needed - 1, (steps, copies, needed, c, g, d)


def test_rotating_needs_more_than_the_last_level_cache():
    r = bench.Rotating(lambda c, s: None, 96, 28311552)          # the headline matrix: 11 copies pass 1.1 x 256 MB
    assert r.needed == math.ceil(1.1 * bench.LLC_BYTES / 28311552) and r.needed * 28311552 > bench.LLC_BYTES
    assert bench.Rotating(lambda c, s: None, 3, 510504960).needed == 2        # the 510 MB head: never fewer than two
    assert bench.Rotating(lambda c, s: None, 5, 1 << 20).needed == 5          # capped by what exists


def test_algorithmic_bytes():
    # Q4_K 12288 x 4096, one token: weights + x + out
    assert bench.gemv_bytes(28311552, 4096, 12288, 1) == 28311552 + 4 * 4096 + 4 * 12288 == 28377088
    assert bench.gemv_bytes(28311552, 4096, 12288, 8) == 28311552 + 8 * 4 * (4096 + 12288)


def test_more_than_one_gpu_is_refused():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode != 0 and "one GPU" in (p.stderr + p.stdout)
