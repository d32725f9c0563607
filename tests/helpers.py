"""Shared pieces of the parity tests."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
GOLDEN_CASES = ["cfg1_noclip", "cfg2_clip_sched", "rig_gradscale", "defaults"]


def load_golden(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"))


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32 if a.dtype == np.float32 else a.dtype)


def same_bits(a, b):
    return a.shape == b.shape and bool((bits(a) == bits(b)).all())


CHUNK = 1 << 26          # elements per pass of the full-size comparisons (keeps temporaries small)


def rel_err(a, b):
    """max |a-b| / max(|b|, rms(b)), in double.

    Used only where the two sides were computed under clip norms that differ in their last
    bits (different summation order).  m = b1*m + (1-b1)*g cancels for some elements, and there
    ANY perturbation of the gradient scale -- the 1e-5 the norm itself is allowed included --
    is amplified without bound relative to the tiny result, and one float ulp of m carried into
    the next step does the same.  Errors are therefore measured against max(|b|, rms(b)): relative
    for ordinary elements, against the array's own scale for cancelling ones.  Where both sides
    use the same norm the tests ask for identical bits instead.
    """
    if not a.size:
        return 0.0
    a, b = a.reshape(-1), b.reshape(-1)
    ss = 0.0
    for at in range(0, b.size, CHUNK):
        y = b[at:at + CHUNK].astype(np.float64)
        ss += float(np.dot(y, y))
    floor = float(np.sqrt(ss / b.size)) + 1e-300
    worst = 0.0
    for at in range(0, b.size, CHUNK):
        x = a[at:at + CHUNK].astype(np.float64)
        y = b[at:at + CHUNK].astype(np.float64)
        worst = max(worst, float(np.max(np.abs(x - y) / np.maximum(np.abs(y), floor))))
    return worst


def strict_misses(a, b, tol):
    """The letter of "within tol relative": how many elements have |a-b| > tol*|b|, and the
    largest |b| among them (0.0 when there is none).  See rel_err for why some must exist when the
    two sides used clip norms that differ in their last bits: they are the cancelling ones."""
    a, b = a.reshape(-1), b.reshape(-1)
    count, biggest = 0, 0.0
    for at in range(0, b.size, CHUNK):
        x = a[at:at + CHUNK].astype(np.float64)
        y = np.abs(b[at:at + CHUNK].astype(np.float64))
        bad = np.abs(x - b[at:at + CHUNK].astype(np.float64)) > tol * y
        k = int(np.count_nonzero(bad))
        if k:
            count += k
            biggest = max(biggest, float(y[bad].max()))
    return count, biggest


def bf16_ulp_diff(a_u16, b_u16):
    """Distance in bf16 units of last place between two uint16 bit patterns (same-sign aware)."""
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7fff), u & 0x7fff)
    return int(np.max(np.abs(key(a_u16) - key(b_u16)))) if a_u16.size else 0
