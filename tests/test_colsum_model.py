"""Host-side model of colsum_add_kernel's control flow (anni_amd/csrc/util_kernels.hip): the
kernel's eight wavefronts pass their barriers at different places of the same loop, which is
correct -- and free of hangs -- only while every wavefront passes the same NUMBER of barriers and
every chunk of 64 rows is added exactly once, in order, by the wavefront that holds it complete.
The model walks each wavefront through the kernel's statements for every row count from 0 to a
little more than four rounds of the workgroup; an edit of the kernel's loop that breaks the count
has to break this walk too (keep the two in step).  CPU only."""
import re
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "anni_amd", "csrc", "util_kernels.hip")


def constants():
    text = open(SRC).read()
    waves = int(re.search(r"struct CsWaves \{ static constexpr int n = (\d+); \}", text).group(1))
    rows = int(re.search(r"struct CsRows \{ static constexpr int n = (\d+); \}", text).group(1))
    return waves, rows


def walk(wave, rows, W, R, prod):
    """Events of one wavefront: ('bar',), ('fetch', chunk, first_row, count), ('mul',),
    ('add', chunk, rows_added) in program order."""
    ev = []
    n_chunks = (rows + R - 1) // R
    done = 0

    def fetch(chunk, first, count):
        if chunk * R < rows:                       # colsum_fetch returns at once past the end
            ev.append(("fetch", chunk, first, count))
    fetch(wave, 0, R)
    if prod:
        ev.append(("mul",))
    ev.append(("bar",))                            # the barrier behind the first fetch
    k = 0
    while k < wave and done < n_chunks:
        ev.append(("bar",))
        done += 1
        k += 1
    while done < n_chunks:
        left = rows - done * R
        ev.append(("add", done, min(left, R)))
        ev.append(("bar",))
        done += 1
        if done >= n_chunks:
            break
        q = R // 4
        stop = False
        for part in range(4):
            fetch(done - 1 - part + W, part * q, q)
            ev.append(("bar",))
            done += 1
            if done >= n_chunks:
                stop = True
                break
        if stop:
            break
        k = 5
        while k < W - 1 and done < n_chunks:
            ev.append(("bar",))
            done += 1
            k += 1
        if done >= n_chunks:
            break
        if prod:
            ev.append(("mul",))
        ev.append(("bar",))
        done += 1
    return ev


@pytest.mark.parametrize("prod", [False, True])
def test_every_wavefront_passes_the_same_barriers_and_every_chunk_is_added_once(prod):
    W, R = constants()
    assert W >= 7 and R % 4 == 0                   # the cycle: own turn, four fetch turns, W - 6 idle, multiply
    for rows in range(0, 4 * R * W + 4):
        n_chunks = (rows + R - 1) // R
        walks = [walk(w, rows, W, R, prod) for w in range(W)]
        bars = [sum(1 for e in ev if e[0] == "bar") for ev in walks]
        assert len(set(bars)) == 1 and bars[0] == n_chunks + 1, (rows, bars)
        added = {}
        for w, ev in enumerate(walks):
            passed = 0                              # barriers passed so far, the first one included
            held = {}                               # chunk -> rows fetched so far (by quarter)
            multiplied = None
            for e in ev:
                if e[0] == "bar":
                    passed += 1
                elif e[0] == "fetch":
                    held.setdefault(e[1], set()).update(range(e[2], e[2] + e[3]))
                    multiplied = None
                elif e[0] == "mul":
                    multiplied = max(held) if held else None
                else:
                    _, chunk, cnt = e
                    assert chunk not in added, (rows, chunk)
                    assert chunk % W == w                               # the wavefront whose turn it is
                    assert passed == chunk + 1, (rows, w, chunk, passed)  # chunks 0 .. chunk-1 were added before
                    assert held.get(chunk) == set(range(R)), (rows, w, chunk)   # fetched completely
                    assert not prod or multiplied == chunk
                    assert cnt == min(R, rows - chunk * R) and cnt > 0
                    added[chunk] = w
        assert sorted(added) == list(range(n_chunks)), rows
