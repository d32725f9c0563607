"""Child process of test_gpu_switches.py: the call order of lang/lm_adam.c:452-515 on the flat
entry points -- a synchronisation, small uploads of vectors and their gradients, gpu_grad_sumsq,
the norm on the host, gpu_adam_step_dev_bf16, small read-backs, gpu_stream_sync -- for nine steps,
printed as digests.  What the backend does ahead of time for such a caller (small copies in
batches, the sum begun at the first upload, the vectors updated and read back first) is switched
by the environment, which the library reads once per process."""
import ctypes as C
import hashlib
import json
import math
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from anni_amd import lib                      # noqa: E402
from anni_amd.lm_adam import DeviceBuffer     # noqa: E402

N = 4096 * 1500 + 777
VECS = [(100, 1024), (4096 * 10 + 5, 1024), (4096 * 400, 4096), (4096 * 401, 4096), (4096 * 900 - 100, 300),
        (N - 777, 777), (3000000, 100000)]


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()[:24]


def main():
    L = lib.require_gpu()
    rng = np.random.default_rng(5)
    L.gpu_set_compute_prec(1)
    p, g, m, v = (DeviceBuffer(4 * N) for _ in range(4))
    tw = DeviceBuffer(2 * N)
    host_p = (rng.standard_normal(N) * 0.02).astype(np.float32)
    p.upload(host_p)
    assert L.gpu_memset(m.ptr, 0, 4 * N) == 0 and L.gpu_memset(v.ptr, 0, 4 * N) == 0
    assert L.gpu_adam_seed_bf16_flat(tw.ptr, p.ptr, N) == 0
    L.gpu_adam_set_bf16_flat(tw.ptr, p.ptr, N)
    vec_p = [host_p[o:o + c].copy() for o, c in VECS]      # the caller's host-resident vectors
    rows = []
    for t in range(1, 10):
        g.upload((rng.standard_normal(N) * 1e-3).astype(np.float32))      # "the backward pass"
        L.gpu_device_sync()
        for (o, c), hp in zip(VECS, vec_p):                # gather: parameters and fresh gradients go up
            hg = (rng.standard_normal(c) * 1e-3).astype(np.float32)
            assert L.gpu_memcpy_h2d(p.ptr + 4 * o, hp.ctypes.data, 4 * c) == 0
            assert L.gpu_memcpy_h2d(g.ptr + 4 * o, hg.ctypes.data, 4 * c) == 0
        ss = C.c_double(0)
        assert L.gpu_grad_sumsq(g.ptr, N, C.byref(ss)) == 0
        gs = 1.0 / (math.sqrt(N) * 1e-3) * (1.7 if t % 2 else 0.6)
        norm = math.sqrt(ss.value) * gs
        if norm > 1.0:
            gs *= 1.0 / norm
        L.gpu_adam_set_weight_decay(0.1)
        assert L.gpu_adam_step_dev_bf16(p.ptr, tw.ptr, g.ptr, m.ptr, v.ptr, N, 1e-3 / t, 0.9, 0.95, 1e-8,
                                        t, gs) == 0
        for (o, c), hp in zip(VECS, vec_p):                # scatter: the vectors come back
            assert L.gpu_memcpy_d2h_async(hp.ctypes.data, p.ptr + 4 * o, 4 * c) == 0
        assert L.gpu_stream_sync() == 0
        rows.append([float(ss.value).hex(), digest(np.concatenate(vec_p)), digest(p.download(np.float32, N)),
                     digest(m.download(np.float32, N)), digest(v.download(np.float32, N)),
                     digest(tw.download(np.uint16, N)), bool(g.download(np.float32, N).any())])
    early, dropped, steps, served = (C.c_long(0) for _ in range(4))
    L.anni_early_sum_stats(C.byref(early), C.byref(dropped))
    L.anni_vectors_first_stats(C.byref(steps), C.byref(served))
    print("DIGEST " + json.dumps({"rows": rows}))
    print("COUNTS " + json.dumps({"early": early.value, "dropped": dropped.value, "split_steps": steps.value,
                                  "served": served.value, "second_stream": L.anni_second_stream_state()}))


if __name__ == "__main__":
    main()
