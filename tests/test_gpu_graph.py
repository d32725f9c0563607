"""The arena step inside a captured HIP graph: it allocates nothing, synchronises nothing and
clears memory with kernels only, so a caller may record it once and replay it.  Every replay is
checked against the eager arithmetic (the oracle under the device's own sum of squares), with
eager work and synchronisations between the replays."""
import ctypes as C

import numpy as np
import pytest

from helpers import same_bits

pytestmark = pytest.mark.gpu

FP8TWIN = 4


def hip_runtime():
    try:
        return C.CDLL("libamdhip64.so")
    except OSError:
        pytest.skip("libamdhip64.so not found")


def ok(rc, what):
    assert rc == 0, "%s: hipError %d" % (what, rc)


@pytest.mark.parametrize("derived", [False, True])
def test_step_replays_from_a_captured_graph(gpu, oracle, derived):
    from anni_amd.lm_adam import LmAdam
    hip = hip_runtime()
    tensors = [(5000, 3 | (FP8TWIN if derived else 0)), (3, 0), (4096 * 3, 3 | (FP8TWIN if derived else 0)),
               (8191, 1), (40000, 3), (1023, 0)]
    opt = LmAdam(tensors, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True)
    n = opt.n
    rng = np.random.default_rng(5)
    P = (rng.standard_normal(n) * 0.02).astype(np.float32)
    M, V = np.zeros(n, np.float32), np.zeros(n, np.float32)
    opt.upload("param", P)
    if derived:
        opt.enable_derived([(2, 4096, 0, 4096)], 4096 * 3)
    opt.seed_twins()
    segs = [(opt.offsets[i], t[0], t[1] & 1, 1.0) for i, t in enumerate(tensors)]
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True,
                      tensors=segs, threads=2)
    unit = 1.0 / (np.sqrt(n) * 1e-3)

    def new_grad(k):
        g = (rng.standard_normal(n) * 1e-3 * unit * (1.8 if k % 2 else 0.5)).astype(np.float32)
        opt.upload("grad", g)
        return g

    def check(g, t_before, lr):
        st = opt.sync_stats()
        O.o.t = t_before                              # the recorded step carries its own t
        O.step(P, g.copy(), M, V, lr, sumsq_override=st.last_sumsq)
        assert st.last_clipped == O.o.last_clipped
        assert same_bits(opt.download("param"), P) and same_bits(opt.download("m"), M)
        assert same_bits(opt.download("v"), V) and not opt.download("grad").any()
        if derived:
            q0, s0 = oracle.fp8_quantize(P[:5000])
            assert (opt.download("fp8twin", 5000) == q0).all()
            assert opt.download("wscale")[0] == s0
            off = opt.offsets[2]
            assert (opt.download("pack") == oracle.bf16_rne(P[off:off + 4096 * 3])).all()

    stream = C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(stream)), "hipStreamCreate")
    gpu.anni_gpu_set_stream(stream)
    try:
        g = new_grad(0)
        assert opt.step_scaled(1e-3) == 0             # eager, on the new stream: t = 1
        check(g, 0, 1e-3)
        new_grad(1)
        graph, gexec = C.c_void_p(), C.c_void_p()
        ok(hip.hipStreamBeginCapture(stream, 2), "hipStreamBeginCapture")       # relaxed mode
        rc = opt.step_scaled(2e-3)                    # recorded, not run: t = 2
        ok(hip.hipStreamEndCapture(stream, C.byref(graph)), "hipStreamEndCapture")
        assert rc == 0 and graph.value
        hip.hipGraphInstantiate.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        ok(hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0), "hipGraphInstantiate")
        assert opt.t == 2
        assert opt.download("grad").any()             # nothing ran during the capture
        for k in range(1, 5):
            g = opt.download("grad") if k == 1 else new_grad(k)
            ok(hip.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            ok(hip.hipStreamSynchronize(stream), "hipStreamSynchronize")
            check(g, 1, 2e-3)                         # every replay is the step recorded at t = 2
        g = new_grad(5)
        assert opt.step_scaled(1e-3) == 0             # and eager steps carry on afterwards: t = 3
        check(g, 2, 1e-3)
        ok(hip.hipGraphExecDestroy(gexec), "hipGraphExecDestroy")
        ok(hip.hipGraphDestroy(graph), "hipGraphDestroy")
    finally:
        gpu.gpu_device_sync()
        gpu.anni_gpu_set_stream(None)
        hip.hipStreamDestroy(stream)
        opt.free()
