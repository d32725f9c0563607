"""The tile walk and cache-hint switches of the step change where data is found, never a bit:
sum of squares (two loops, changeover at any tile), update walking forward or backward, with
non-temporal hints or without.  Each setting runs in a process of its own (the library reads its
switches once unless told to read them again), and all settings that share a grid must print the same digests."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

CHILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "switch_child.py")


FLAT_CHILD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "flat_switch_child.py")


def run_child(child=CHILD, counts=False, **switches):
    env = {k: v for k, v in os.environ.items() if not k.startswith("ANNI_")}
    env.update({k: str(v) for k, v in switches.items()})
    r = subprocess.run([sys.executable, child], env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    line = [ln for ln in r.stdout.splitlines() if ln.startswith("DIGEST ")][-1]
    if counts:
        c = [ln for ln in r.stdout.splitlines() if ln.startswith("COUNTS ")][-1]
        return json.loads(line[7:]), json.loads(c[7:])
    return json.loads(line[7:])


def test_default_grid(gpu):
    want = run_child()
    for gt in ("0", "1", "2"):
        assert [row[1] for row in want[gt]].count(1) >= 1          # at least one clipped step
        assert not any(row[6] for row in want[gt])                   # gradients cleared
    assert run_child(ANNI_REVERSE=0, ANNI_KEEP_MB=0) == want
    assert run_child(ANNI_NT=0, ANNI_PIPE=0) == want
    assert run_child(ANNI_TILES_PER_WG=0) == want            # the resident grid
    assert run_child(ANNI_TILES_PER_WG=3, ANNI_PIPE=2) == want
    # the norm's second stage taking the partials over with fences instead of atomic accesses:
    # the same sum of squares (it is in the digests) and the same state, bit for bit
    assert run_child(ANNI_FOLD="fence") == want


def test_one_workgroup_per_cu_changeover_inside_every_workgroup(gpu):
    """256 workgroups over ~2200 tiles: each one takes 8 or 9 tiles, and with 5 MiB kept the
    changeover from streaming to ordinary loads falls inside every workgroup's run (after one round
    of the grid for fp8 codes)."""
    want = run_child(ANNI_BLOCKS_PER_CU=1, ANNI_SUMSQ_PER_CU=1, ANNI_KEEP_MB=0)
    assert run_child(ANNI_BLOCKS_PER_CU=1, ANNI_SUMSQ_PER_CU=1, ANNI_KEEP_MB=5) == want
    assert run_child(ANNI_BLOCKS_PER_CU=1, ANNI_SUMSQ_PER_CU=1, ANNI_KEEP_MB=3, ANNI_REVERSE=0) == want
    assert run_child(ANNI_BLOCKS_PER_CU=1, ANNI_SUMSQ_PER_CU=1, ANNI_KEEP_MB=100000) == want


def test_what_the_backend_does_ahead_of_time_for_the_flat_caller_changes_no_bit(gpu):
    """The call order of lang/lm_adam.c on the flat entry points, nine steps: with the sum begun at
    the first upload and the vectors updated and read back first (both in use from the fourth
    step on, as the counters must show), with either switched off, with both off, and without
    the batching of small copies -- the same sums of squares, the same vectors handed back, the same
    p, m, v and twins at every step."""
    want, counts = run_child(FLAT_CHILD, counts=True)
    found = counts.pop("second_stream") != 0         # 0: no stream runs beside the compute stream in that process
    if found:
        assert counts["early"] >= 5 and counts["dropped"] == 0, counts
        assert counts["split_steps"] >= 5 and counts["served"] == 7 * counts["split_steps"], counts
    assert not any(row[6] for row in want["rows"])               # gradients cleared by every step
    got, c = run_child(FLAT_CHILD, counts=True, ANNI_EARLY_SUM=0)
    assert got == want and c["early"] == 0 and (c["split_steps"] >= 5 or c["second_stream"] == 0)
    got, c = run_child(FLAT_CHILD, counts=True, ANNI_VECTORS_FIRST=0)
    assert got == want and c["split_steps"] == 0 and (c["early"] >= 5 or c["second_stream"] == 0)
    nothing = {"early": 0, "dropped": 0, "split_steps": 0, "served": 0, "second_stream": -1}
    got, c = run_child(FLAT_CHILD, counts=True, ANNI_EARLY_SUM=0, ANNI_VECTORS_FIRST=0)
    assert got == want and c == nothing
    got, c = run_child(FLAT_CHILD, counts=True, ANNI_SMALL_COPY_BATCH=0)
    assert got == want and c == nothing
