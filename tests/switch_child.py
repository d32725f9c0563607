"""Child process of test_gpu_switches.py: three steps in each gradient storage type on a ragged
tensor list, printed as digests.  The library reads its environment switches once per process,
so every setting needs a process of its own."""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from anni_amd import lib                      # noqa: E402
from anni_amd.lm_adam import LmAdam           # noqa: E402

SIZES = [(4096 * 700 + 5, 3), (1536, 0), (4096 * 600, 3), (1, 0), (4096 * 897 + 4095, 3), (777, 1)]


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()[:24]


def main():
    lib.require_gpu()
    out = {}
    for gt in (0, 1, 2):
        rng = np.random.default_rng(100 + gt)
        opt = LmAdam(SIZES, grad_type=gt, moment_type=1 if gt == 1 else 0, twins=True,
                     skip_nonfinite=True, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
        n = opt.n
        opt.upload("param", (rng.standard_normal(n) * 0.02).astype(np.float32))
        opt.seed_twins()
        rows = []
        for s in range(3):
            g = (rng.standard_normal(n) * (3e-4 if s == 1 else 2e-3)).astype(np.float32)
            if gt == 0:
                opt.upload("grad", g)
            elif gt == 1:
                opt.upload("grad", (g.view(np.uint32) >> 16).astype(np.uint16))
            else:
                q = rng.integers(0, 256, n, dtype=np.uint8)
                q[(q & 0x7f) == 0x7f] = 0x3c              # no NaN codes
                opt.upload("grad", q)
                opt.upload("gscale", (rng.random(len(SIZES)) * 1e-5 + 1e-6).astype(np.float32))
            opt.step_scaled(1e-3)
            st = opt.sync_stats()
            rows.append([float(st.last_sumsq).hex(), int(st.last_clipped), digest(opt.download("param")),
                         digest(opt.download("m")), digest(opt.download("v")),
                         digest(opt.download("twin")), bool(opt.download("grad").any())])
        out[str(gt)] = rows
        opt.free()
    print("DIGEST " + json.dumps(out))


if __name__ == "__main__":
    main()
