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


def rel_err(a, b):
    """max |a-b| / max(|b|, tiny) over finite entries, in double."""
    a = a.astype(np.float64)
    b = b.astype(np.float64)
    den = np.maximum(np.abs(b), 1e-30)
    return float(np.max(np.abs(a - b) / den)) if a.size else 0.0


def bf16_ulp_diff(a_u16, b_u16):
    """Distance in bf16 units of last place between two uint16 bit patterns (same-sign aware)."""
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7fff), u & 0x7fff)
    return int(np.max(np.abs(key(a_u16) - key(b_u16)))) if a_u16.size else 0
