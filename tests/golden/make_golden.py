"""Writes the golden vectors of the optimizer step from the reference's OWN compiled code.

Run in a container that holds the reference tree (oracle/Makefile builds
oracle/_ref/libanni_ref.so from the reference's sources where they lie):

    python tests/golden/make_golden.py            # everything
    python tests/golden/make_golden.py ln_colsum  # only the named fixtures

Each fixture holds seeded inputs (p0, one gradient per step, hyper-parameters,
the per-step lr and grad_scale) and what the reference's lm_adam_step_scaled host
path (lang/lm_adam.c:559-606) produced after every step (p, m, v).  The learning
rates come from the reference's lm_train_step_lr (lang/lm_train.c:98-124).
ln_colsum holds the bias / LayerNorm gradient sums: dgamma and dbeta as the reference's
host layernorm_backward (lang/layernorm.c:312-376) accumulates them over seeded dy and x_hat.
Fixtures are data only; the GPU box re-checks the oracle and the HIP path
against them without the reference being present.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import binding as ob  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
STEPS = 10

CASES = {
    # benchmark configuration 1: constant lr 3e-4, no clip, wd 0.1, beta2 0.95
    "cfg1_noclip": dict(n=1531, seed=11, base_lr=3e-4, sched=None, wd=0.1, clip=0.0,
                        beta2=0.95, gmul=[1.0] * STEPS, grad_scale=1.0),
    # benchmark configuration 2: clip 1.0 with about half the steps clipping, warmup 100 + cosine
    "cfg2_clip_sched": dict(n=1531, seed=12, base_lr=3e-4, sched=(100, 1000, "cosine"),
                            wd=0.1, clip=1.0, beta2=0.95,
                            gmul=[13.0, 40.0, 20.0, 70.0, 8.0, 33.0, 52.0, 18.0, 25.0, 61.0],
                            grad_scale=1.0),
    # the reference's test rig constants (tests/test_gpu.c:67-84,175): lr 1e-3, grad_scale 1/(B(T-1))
    "rig_gradscale": dict(n=777, seed=13, base_lr=1e-3, sched=None, wd=0.1, clip=1.0,
                          beta2=0.95, gmul=[100.0, 3000.0, 500.0, 9000.0, 200.0, 50.0, 7000.0,
                                            1000.0, 250.0, 4000.0],
                          grad_scale=1.0 / (4 * 63)),
    # defaults of lm_adam_create (beta2 0.999, no decay, no clip)
    "defaults": dict(n=515, seed=14, base_lr=1e-3, sched=None, wd=0.0, clip=0.0,
                     beta2=0.999, gmul=[1.0] * STEPS, grad_scale=1.0),
}


def ln_colsum():
    """Inputs whose float column sums depend on the order of the additions: magnitudes spread
    over eight decades, exact cancellations, signed zeros, accumulators that do not start at 0."""
    rng = np.random.default_rng(21)
    T, d = 19, 1024
    dy = (rng.standard_normal((T, d)) * 10.0 ** rng.integers(-4, 4, (T, d))).astype(np.float32)
    xh = rng.standard_normal((T, d)).astype(np.float32)
    dy[0, :8] = 1e8
    dy[1, :8] = 1.0
    dy[2, :8] = -1e8                       # (1e8 + 1) - 1e8 = 0 in float, 1 in any other order
    dy[:, 8] = -0.0                        # a column of -0: the sum stays -0 from a -0 start
    xh[:, 9] = 0.0
    dgamma0 = (rng.standard_normal(d) * 1e-2).astype(np.float32)
    dbeta0 = (rng.standard_normal(d) * 1e-2).astype(np.float32)
    dbeta0[8] = -0.0
    dgamma, dbeta = dgamma0.copy(), dbeta0.copy()
    ob.ref_ln_backward_grads(dy, xh, dgamma, dbeta)
    np.savez_compressed(os.path.join(HERE, "ln_colsum.npz"), dy=dy, x_hat=xh, dgamma0=dgamma0,
                        dbeta0=dbeta0, dgamma=dgamma, dbeta=dbeta)
    print("wrote ln_colsum", T, d)


def main(only=()):
    if not ob.ref_available():
        raise SystemExit("oracle/_ref/libanni_ref.so is missing: run `make -C oracle` "
                         "where the reference tree is present")
    if not only or "ln_colsum" in only:
        ln_colsum()
    for name, c in CASES.items():
        if only and name not in only:
            continue
        rng = np.random.default_rng(c["seed"])
        n = c["n"]
        p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
        grads = np.stack([(rng.standard_normal(n) * 1e-3 * c["gmul"][s]).astype(np.float32)
                          for s in range(STEPS)])
        # a few awkward values: zeros, a denormal-producing tiny gradient, a large one
        grads[:, 0] = 0.0
        grads[:, 1] = 1e-22
        grads[3, 2] = 0.5
        p = p0.copy()
        g = np.zeros(n, np.float32)
        R = ob.RefAdam(p, g, beta2=c["beta2"], weight_decay=c["wd"], grad_clip=c["clip"])
        lrs = []
        P, M, V = [], [], []
        for s in range(STEPS):
            g[:] = grads[s]
            if c["sched"]:
                w, d, k = c["sched"]
                lr = ob.ref_lr(c["base_lr"], s, w, d, k)   # called with t before the increment
            else:
                lr = c["base_lr"]
            lrs.append(lr)
            t = R.step(lr, c["grad_scale"])
            assert t == s + 1 and not g.any()
            m, v = R.moments()
            P.append(p.copy())
            M.append(m)
            V.append(v)
        R.close()
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"), p0=p0, grads=grads,
            lr=np.array(lrs, np.float64), grad_scale=np.float64(c["grad_scale"]),
            beta1=np.float64(0.9), beta2=np.float64(c["beta2"]), eps=np.float64(1e-8),
            wd=np.float64(c["wd"]), clip=np.float64(c["clip"]),
            p=np.stack(P), m=np.stack(M), v=np.stack(V))
        print("wrote", name, n)
    if only and "lr_table" not in only:
        return
    # learning-rate table straight from lm_train_step_lr
    steps = np.array([0, 1, 9, 50, 98, 99, 100, 101, 350, 600, 1099, 1100, 1101, 5000], np.int32)
    rows = []
    for (w, d, k, frm) in [(100, 1000, "cosine", 0), (100, 1000, "linear", 0), (0, 1000, "cosine", 0),
                           (100, 0, "cosine", 0), (100, 1000, "none", 0), (100, 1000, "cosine", 40),
                           (1000, 20000, "cosine", 0)]:
        rows.append([ob.ref_lr(3e-4, int(s), w, d, k, frm) for s in steps])
    np.savez_compressed(os.path.join(HERE, "lr_table.npz"), steps=steps,
                        lr=np.array(rows, np.float64),
                        cases=np.array(["100,1000,cosine,0", "100,1000,linear,0", "0,1000,cosine,0",
                                        "100,0,cosine,0", "100,1000,none,0", "100,1000,cosine,40",
                                        "1000,20000,cosine,0"]))
    print("wrote lr_table")


if __name__ == "__main__":
    main(tuple(sys.argv[1:]))
