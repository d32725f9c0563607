"""Parity of the flat drop-in ABI (the num/gpu.h entry points lang/lm_adam.c calls) against the
CPU oracle, through the C ABI.  Bit-exact where the arithmetic is identical by construction;
required tolerances (1e-6 relative on p/m/v, 1 bf16 ulp on twins, 1e-5 on the norm) where the
summation order of the norm differs."""
import ctypes as C
import math
import os

import numpy as np
import pytest

from helpers import GOLDEN_CASES, load_golden, same_bits, rel_err, bf16_ulp_diff

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL_STATE = 1e-6     # required: FP32 master/m/v within 1e-6 relative per step
TOL_NORM = 1e-5      # required: clip norm within 1e-5 relative


def dev(gpu, arr):
    from anni_amd.lm_adam import DeviceBuffer
    arr = np.ascontiguousarray(arr)
    b = DeviceBuffer(max(arr.nbytes, 16))
    if arr.nbytes:
        b.upload(arr)
    return b


def needs_second_stream(gpu):
    """What the backend begins ahead of time runs on a second stream of its own; when none of the
    runtime's streams runs beside the compute stream in this process (the library measures it) it
    never happens, results are the same, and the counters stay at zero: nothing to count then."""
    if gpu.anni_second_stream_state() == 0:
        pytest.skip("no stream runs beside the compute stream in this process: nothing is begun ahead of time")


def test_device_is_gfx950_backend(gpu):
    assert gpu.gpu_available() == 1
    assert gpu.gpu_backend_name() == b"hip-gfx950"
    f, t = C.c_size_t(0), C.c_size_t(0)
    assert gpu.gpu_mem_info(C.byref(f), C.byref(t)) == 0 and 0 < f.value <= t.value
    assert gpu.gpu_debug_last_error() == b""


def test_memory_primitives(gpu):
    from anni_amd.lm_adam import DeviceBuffer
    rng = np.random.default_rng(1)
    x = rng.integers(0, 255, 100003, dtype=np.uint8)
    a = dev(gpu, x)
    b = DeviceBuffer(x.nbytes)
    assert gpu.gpu_memcpy_d2d(b.ptr, a.ptr, x.nbytes) == 0
    assert (b.download(np.uint8, x.size) == x).all()
    # byte fill on awkward offsets / lengths, neighbours untouched
    for off, ln, val in ((0, 100003, 0), (1, 17, 0xab), (3, 4099, 0x5c), (15, 1, 1), (16, 64, 0xff),
                         (7, 99990, 0x11)):
        assert gpu.gpu_memcpy_d2d(b.ptr, a.ptr, x.nbytes) == 0
        assert gpu.gpu_memset(b.ptr + off, val, ln) == 0
        want = x.copy()
        want[off:off + ln] = val
        assert (b.download(np.uint8, x.size) == want).all(), (off, ln)
    # asynchronous copy lands by the stream sync (lm_adam.c:407-413,500)
    host = np.zeros(x.size, np.uint8)
    assert gpu.gpu_host_pin(host.ctypes.data, host.nbytes) == 0
    assert gpu.gpu_host_pin(host.ctypes.data, host.nbytes) == 0
    assert gpu.gpu_memcpy_d2h_async(host.ctypes.data, a.ptr, x.nbytes) == 0
    assert gpu.gpu_stream_sync() == 0
    assert (host == x).all()
    gpu.gpu_host_forget(host.ctypes.data)
    # argument checks as gpu_cuda.cu:2964-3029
    assert gpu.gpu_memcpy_h2d(None, x.ctypes.data, 4) == -1
    assert gpu.gpu_memcpy_d2h(x.ctypes.data, a.ptr, 0) == -1
    assert gpu.gpu_memset(None, 0, 4) == -1
    assert gpu.gpu_malloc(0) is None
    hp = gpu.gpu_host_alloc(4096)
    assert hp
    gpu.gpu_host_free(hp)
    gpu.gpu_device_sync()


@pytest.mark.parametrize("n", [1, 3, 255, 4096, 4097, 65536 + 5, 3000017])
def test_grad_sumsq(gpu, oracle, n):
    rng = np.random.default_rng(n)
    g = (rng.standard_normal(n) * 3e-2).astype(np.float32)
    d = dev(gpu, g)
    out = C.c_double(0)
    assert gpu.gpu_grad_sumsq(d.ptr, n, C.byref(out)) == 0
    want = oracle.sumsq(g)
    assert abs(out.value - want) <= 1e-11 * want      # the serial sum itself carries ~sqrt(n) ulp
    first = out.value
    for _ in range(3):                      # run-to-run deterministic
        assert gpu.gpu_grad_sumsq(d.ptr, n, C.byref(out)) == 0 and out.value == first
    # arguments (gpu_cuda.cu:8488-8489)
    assert gpu.gpu_grad_sumsq(None, n, C.byref(out)) == -1
    assert gpu.gpu_grad_sumsq(d.ptr, 0, C.byref(out)) == -1
    assert gpu.gpu_grad_sumsq(d.ptr, n, None) == -1


def test_grad_sumsq_unaligned_and_nonfinite(gpu, oracle):
    rng = np.random.default_rng(77)
    g = rng.standard_normal(20001).astype(np.float32)
    d = dev(gpu, g)
    out = C.c_double(0)
    assert gpu.gpu_grad_sumsq(d.ptr + 4, 20000, C.byref(out)) == 0      # 4-byte aligned only
    want = oracle.sumsq(g[1:])
    assert abs(out.value - want) <= 1e-11 * want      # the serial sum itself carries ~sqrt(n) ulp
    for bad in (np.nan, np.inf):
        g2 = g.copy()
        g2[12345] = bad
        d2 = dev(gpu, g2)
        assert gpu.gpu_grad_sumsq(d2.ptr, g2.size, C.byref(out)) == 0
        assert not math.isfinite(out.value)


def test_grad_sumsq_back_to_back_on_changing_inputs(gpu, oracle):
    """The second stage of the sum runs inside the same launch: the last workgroup to finish
    folds the partials of all the others.  Launches back to back on inputs of different content and
    size must each return their own sum, to the bit, every time -- a partial left over from the
    launch before, or one not yet visible, would show."""
    rng = np.random.default_rng(2048)
    cases = []
    for n, scale in ((4096 * 2075 + 17, 3e-2), (3000017, 1.0), (4096 * 2048, 1e-3), (5, 2.0)):
        g = (rng.standard_normal(n) * scale).astype(np.float32)
        want = oracle.sumsq(g)
        cases.append((dev(gpu, g), n, want))
    out = C.c_double(0)
    first = []
    for d, n, want in cases:
        assert gpu.gpu_grad_sumsq(d.ptr, n, C.byref(out)) == 0
        assert abs(out.value - want) <= 1e-11 * want
        first.append(out.value)
    order = rng.integers(0, len(cases), 1500)
    for k in order:
        d, n, _want = cases[k]
        assert gpu.gpu_grad_sumsq(d.ptr, n, C.byref(out)) == 0
        assert out.value == first[k], (k, out.value, first[k])


class FlatState:
    """p/g/m/v/twin on the device + the same on the host for the oracle."""

    def __init__(self, gpu, n, seed, twin=True):
        rng = np.random.default_rng(seed)
        self.gpu, self.n, self.rng = gpu, n, rng
        self.p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        self.m = np.zeros(n, np.float32)
        self.v = np.zeros(n, np.float32)
        self.g = np.zeros(n, np.float32)
        self.twin = np.zeros(n, np.uint16) if twin else None
        self.dp, self.dm, self.dv = dev(gpu, self.p), dev(gpu, self.m), dev(gpu, self.v)
        self.dg = dev(gpu, self.g)
        self.dt = dev(gpu, np.zeros(n, np.uint16))

    def new_grad(self, scale):
        g = (self.rng.standard_normal(self.n) * scale).astype(np.float32)
        self.g[:] = g
        self.dg.upload(g)

    def fetch(self):
        f32 = np.float32
        return (self.dp.download(f32, self.n), self.dm.download(f32, self.n),
                self.dv.download(f32, self.n), self.dg.download(f32, self.n),
                self.dt.download(np.uint16, self.n))


@pytest.mark.parametrize("n,wd", [(1000003, 0.1), (4096 * 3, 0.0), (5, 0.1)])
def test_flat_step_bit_exact_over_ten_steps(gpu, oracle, n, wd):
    """gpu_adam_step_dev_bf16 with the grad_scale given: identical arithmetic -> identical bits."""
    S = FlatState(gpu, n, seed=n)
    O = oracle.Oracle(n, beta2=0.95, weight_decay=wd, threads=8)
    gpu.gpu_set_compute_prec(1)
    gpu.gpu_adam_set_weight_decay(wd)
    for t in range(1, 11):
        S.new_grad(1e-3 * (1 + (t % 4)))
        lr = oracle.lr(3e-4, t - 1, 100, 1000, "cosine")
        gs = 1.0 / (1 + t)
        assert gpu.gpu_adam_step_dev_bf16(S.dp.ptr, S.dt.ptr, S.dg.ptr, S.dm.ptr, S.dv.ptr, n, lr,
                                          0.9, 0.95, 1e-8, t, gs) == 0
        O.step(S.p, S.g, S.m, S.v, lr, gs, twin=S.twin)
        p, m, v, g, tw = S.fetch()
        assert same_bits(p, S.p), t
        assert same_bits(m, S.m) and same_bits(v, S.v), t
        assert not g.any()                          # d_grad is zeroed by the step (gpu.h:125-127)
        assert (tw == S.twin).all()
        assert (tw == oracle.bf16_rne(p)).all()     # twin = RNE of the final p
    gpu.gpu_set_compute_prec(0)
    gpu.gpu_adam_set_weight_decay(0.0)


def test_flat_step_without_bf16_precision_leaves_twins_alone(gpu, oracle):
    n = 10000
    S = FlatState(gpu, n, seed=3)
    S.dt.upload(np.full(n, 0x1234, np.uint16))
    gpu.gpu_set_compute_prec(0)                     # twins only when prec == BF16 (gpu_cuda.cu:8687,8704)
    S.new_grad(1e-3)
    assert gpu.gpu_adam_step_dev_bf16(S.dp.ptr, S.dt.ptr, S.dg.ptr, S.dm.ptr, S.dv.ptr, n, 1e-3,
                                      0.9, 0.999, 1e-8, 1, 1.0) == 0
    assert (S.dt.download(np.uint16, n) == 0x1234).all()
    O = oracle.Oracle(n)
    O.step(S.p, S.g, S.m, S.v, 1e-3)
    assert same_bits(S.dp.download(np.float32, n), S.p)
    # NULL twin pointer with BF16 precision is fine too
    gpu.gpu_set_compute_prec(1)
    S.new_grad(1e-3)
    assert gpu.gpu_adam_step_dev_bf16(S.dp.ptr, None, S.dg.ptr, S.dm.ptr, S.dv.ptr, n, 1e-3,
                                      0.9, 0.999, 1e-8, 2, 1.0) == 0
    O.step(S.p, S.g, S.m, S.v, 1e-3)
    assert same_bits(S.dp.download(np.float32, n), S.p)
    gpu.gpu_set_compute_prec(0)


def test_flat_step_unaligned_pointers(gpu, oracle):
    """Pointers that are only 4-byte aligned take the element-wise path; same results."""
    n = 9001
    S = FlatState(gpu, n + 1, seed=21)
    S.new_grad(1e-3)
    gpu.gpu_set_compute_prec(1)
    gpu.gpu_adam_set_weight_decay(0.1)
    assert gpu.gpu_adam_step_dev_bf16(S.dp.ptr + 4, S.dt.ptr + 2, S.dg.ptr + 4, S.dm.ptr + 4,
                                      S.dv.ptr + 4, n, 1e-3, 0.9, 0.95, 1e-8, 1, 0.5) == 0
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1)
    p, g, m, v, tw = S.p[1:].copy(), S.g[1:].copy(), S.m[1:].copy(), S.v[1:].copy(), S.twin[1:].copy()
    O.step(p, g, m, v, 1e-3, 0.5, twin=tw)
    dp, dm, dv, dg, dt = S.fetch()
    assert same_bits(dp[1:], p) and same_bits(dm[1:], m) and same_bits(dv[1:], v)
    assert (dt[1:] == tw).all() and not dg[1:].any()
    assert dp[0] == S.p[0] and dg[0] == S.g[0] and dt[0] == 0      # element before the range untouched
    gpu.gpu_set_compute_prec(0)
    gpu.gpu_adam_set_weight_decay(0.0)


def test_flat_step_argument_checks(gpu):
    """gpu_cuda.cu:8675-8682."""
    S = FlatState(gpu, 64, seed=1)
    ok = (S.dp.ptr, S.dt.ptr, S.dg.ptr, S.dm.ptr, S.dv.ptr)
    f = gpu.gpu_adam_step_dev_bf16
    assert f(None, ok[1], ok[2], ok[3], ok[4], 64, 1e-3, 0.9, 0.95, 1e-8, 1, 1.0) == -1
    assert f(ok[0], ok[1], None, ok[3], ok[4], 64, 1e-3, 0.9, 0.95, 1e-8, 1, 1.0) == -1
    assert f(ok[0], ok[1], ok[2], None, ok[4], 64, 1e-3, 0.9, 0.95, 1e-8, 1, 1.0) == -1
    assert f(ok[0], ok[1], ok[2], ok[3], None, 64, 1e-3, 0.9, 0.95, 1e-8, 1, 1.0) == -1
    assert f(*ok, 0, 1e-3, 0.9, 0.95, 1e-8, 1, 1.0) == -1
    assert f(*ok, 64, 0.0, 0.9, 0.95, 1e-8, 1, 1.0) == -1
    assert f(*ok, 64, 1e-3, 0.9, 0.95, 1e-8, 0, 1.0) == -1
    assert f(*ok, 64, 1e-3, 1.0, 0.95, 1e-8, 1, 1.0) == -1         # 1 - beta1^t == 0
    p = S.dp.download(np.float32, 64)
    assert same_bits(p, S.p)                                        # nothing ran
    gpu.gpu_adam_set_weight_decay(-3.0)                             # negatives clamp to 0


def reference_device_flow(gpu, S, t, lr, grad_scale, clip, wd):
    """The control flow of adam_step_gpu (lang/lm_adam.c:466-495) on the flat ABI."""
    ss = C.c_double(0)
    assert gpu.gpu_grad_sumsq(S.dg.ptr, S.n, C.byref(ss)) == 0
    norm = math.sqrt(ss.value) * abs(grad_scale)
    if not math.isfinite(norm):
        assert gpu.gpu_memset(S.dg.ptr, 0, S.n * 4) == 0
        return norm, True
    if clip > 0 and norm > clip:
        grad_scale *= clip / norm
    gpu.gpu_adam_set_weight_decay(wd)
    assert gpu.gpu_adam_step_dev_bf16(S.dp.ptr, S.dt.ptr, S.dg.ptr, S.dm.ptr, S.dv.ptr, S.n, lr,
                                      0.9, 0.95, 1e-8, t, grad_scale) == 0
    assert gpu.gpu_stream_sync() == 0
    gpu.gpu_half_wt_invalidate(None)
    return norm, False


def test_unchanged_caller_flow_matches_cpu_path(gpu, oracle):
    """What lang/lm_adam.c does with this backend vs its own host loop: required tolerances.
    (The caller's device branch scales by clip/norm, its host loop by clip/(norm+1e-12).)"""
    n = 300007
    S = FlatState(gpu, n, seed=5)
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, threads=8)
    gpu.gpu_set_compute_prec(1)
    e0 = gpu.gpu_param_epoch()
    clipped = 0
    for t in range(1, 11):
        S.new_grad(1e-3 * (1.0 if t % 2 else 4.0))      # sqrt(n)*1e-3 = 0.55 -> every other step clips
        lr = oracle.lr(3e-4, t - 1, 100, 1000, "cosine")
        norm, skipped = reference_device_flow(gpu, S, t, lr, 1.0, 1.0, 0.1)
        O.step(S.p, S.g, S.m, S.v, lr, 1.0, twin=S.twin)
        assert not skipped
        assert abs(norm - O.o.last_grad_norm) <= TOL_NORM * O.o.last_grad_norm
        clipped += O.o.last_clipped
        p, m, v, g, tw = S.fetch()
        assert rel_err(p, S.p) <= TOL_STATE and rel_err(m, S.m) <= TOL_STATE
        assert rel_err(v, S.v) <= TOL_STATE
        assert bf16_ulp_diff(tw, S.twin) <= 1 and not g.any()
    assert clipped == 5 and gpu.gpu_param_epoch() == e0 + 10
    gpu.gpu_set_compute_prec(0)
    gpu.gpu_adam_set_weight_decay(0.0)


def test_unchanged_caller_flow_skips_nonfinite(gpu):
    n = 5000
    S = FlatState(gpu, n, seed=6)
    S.new_grad(1e-3)
    g = S.g.copy()
    g[77] = np.nan
    S.dg.upload(g)
    norm, skipped = reference_device_flow(gpu, S, 1, 1e-3, 1.0, 1.0, 0.1)
    assert skipped and math.isnan(norm)
    p, m, v, gg, _tw = S.fetch()
    assert same_bits(p, S.p) and not m.any() and not v.any() and not gg.any()


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_golden_vectors_through_flat_abi(gpu, name):
    """The reference's own outputs (written by its compiled host loop) vs this backend."""
    G = load_golden(name)
    n = G["p0"].size
    S = FlatState(gpu, n, seed=0)
    S.dp.upload(G["p0"])
    clip, wd, gs0 = float(G["clip"]), float(G["wd"]), float(G["grad_scale"])
    gpu.gpu_set_compute_prec(1)
    for s in range(G["grads"].shape[0]):
        S.dg.upload(G["grads"][s])
        if clip > 0:
            reference_device_flow(gpu, S, s + 1, float(G["lr"][s]), gs0, clip, wd)
        else:
            gpu.gpu_adam_set_weight_decay(wd)
            assert gpu.gpu_adam_step_dev_bf16(S.dp.ptr, S.dt.ptr, S.dg.ptr, S.dm.ptr, S.dv.ptr, n,
                                              float(G["lr"][s]), float(G["beta1"]),
                                              float(G["beta2"]), float(G["eps"]), s + 1, gs0) == 0
        p, m, v, g, _tw = S.fetch()
        if clip > 0:
            assert rel_err(p, G["p"][s]) <= TOL_STATE and rel_err(m, G["m"][s]) <= TOL_STATE
            assert rel_err(v, G["v"][s]) <= TOL_STATE
        else:
            assert same_bits(p, G["p"][s]) and same_bits(m, G["m"][s]) and same_bits(v, G["v"][s])
        assert not g.any()
    gpu.gpu_set_compute_prec(0)
    gpu.gpu_adam_set_weight_decay(0.0)


def test_seed_bf16_flat(gpu, oracle):
    for n in (1, 7, 4096, 100003):
        x = (np.random.default_rng(n).standard_normal(n) * 0.02).astype(np.float32)
        d = dev(gpu, x)
        o = dev(gpu, np.zeros(n, np.uint16))
        gpu.gpu_adam_set_bf16_flat(o.ptr, d.ptr, n)
        assert gpu.gpu_adam_seed_bf16_flat(o.ptr, d.ptr, n) == 0
        assert (o.download(np.uint16, n) == oracle.bf16_rne(x)).all()
        gpu.gpu_adam_set_bf16_flat(None, None, 0)
    assert gpu.gpu_adam_seed_bf16_flat(None, None, 5) == -1


def test_twin_flat_is_served_and_checked(gpu, oracle, capfd):
    """anni_gpu_bf16_twin_of: slices of the registered flat are served from the twin flat, anything
    else and everything after gpu_free / a cleared registration gets NULL; with ANN_TWIN_CHECK=1
    (read once per process: a child) a stale slice is reported as the reference reports it."""
    import subprocess
    import sys
    n = 10000
    x = (np.random.default_rng(9).standard_normal(n) * 0.02).astype(np.float32)
    d, o = dev(gpu, x), dev(gpu, np.zeros(n, np.uint16))
    assert gpu.anni_gpu_bf16_twin_of(d.ptr, n) is None               # nothing registered
    gpu.gpu_adam_set_bf16_flat(o.ptr, d.ptr, n)
    assert gpu.gpu_adam_seed_bf16_flat(o.ptr, d.ptr, n) == 0
    assert gpu.anni_gpu_bf16_twin_of(d.ptr, n) == o.ptr
    assert gpu.anni_gpu_bf16_twin_of(d.ptr + 4 * 100, 50) == o.ptr + 2 * 100
    assert gpu.anni_gpu_bf16_twin_of(d.ptr + 4 * (n - 1), 1) == o.ptr + 2 * (n - 1)
    assert gpu.anni_gpu_bf16_twin_of(d.ptr + 4 * (n - 1), 2) is None  # one element too far
    assert gpu.anni_gpu_bf16_twin_of(d.ptr, 0) is None and gpu.anni_gpu_bf16_twin_of(None, 4) is None
    assert gpu.anni_gpu_bf16_twin_of(o.ptr, 4) is None               # not an fp32 slice of the flat
    gpu.gpu_adam_set_bf16_flat(None, None, 0)
    assert gpu.anni_gpu_bf16_twin_of(d.ptr, n) is None
    gpu.gpu_adam_set_bf16_flat(o.ptr, d.ptr, n)
    o.free()                                                         # gpu_free forgets the registration
    assert gpu.anni_gpu_bf16_twin_of(d.ptr, n) is None
    d.free()
    child = (
        "import sys, numpy as np\n"
        "sys.path.insert(0, %r)\n"
        "from anni_amd import lib\n"
        "from anni_amd.lm_adam import DeviceBuffer\n"
        "L = lib.require_gpu()\n"
        "n = 5000\n"
        "x = np.linspace(-1, 1, n).astype(np.float32)\n"
        "d, o = DeviceBuffer(4 * n), DeviceBuffer(2 * n)\n"
        "d.upload(x)\n"
        "L.gpu_adam_set_bf16_flat(o.ptr, d.ptr, n)\n"
        "assert L.gpu_adam_seed_bf16_flat(o.ptr, d.ptr, n) == 0\n"
        "assert L.anni_gpu_bf16_twin_of(d.ptr, n) == o.ptr\n"
        "print('FRESH-DONE', flush=True)\n"
        "d.upload((x * 3).astype(np.float32))\n"          # weights change behind the twins' back
        "assert L.anni_gpu_bf16_twin_of(d.ptr + 400, 1000) == o.ptr + 200\n"
        "L.gpu_adam_set_bf16_flat(None, None, 0)\n"
    ) % ROOT
    env = dict(os.environ, ANN_TWIN_CHECK="1")
    r = subprocess.run([sys.executable, "-c", child], env=env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-1500:]
    stale = [ln for ln in r.stderr.splitlines() if ln.startswith("[twin] STALE flat")]
    assert len(stale) == 1 and "n=1000" in stale[0], r.stderr[-1500:]


def test_the_unchanged_reference_caller_on_this_backend(gpu, oracle):
    """lang/lm_adam.c itself, compiled from the reference tree and linked against
    libanni_gpu_hip.so instead of its CPU stub (oracle/_ref/libanni_ref_hip.so): its device path
    (lm_adam.c:452-515) runs on this backend and must give what its own host path gives."""
    if not oracle.ref_hip_available():
        pytest.skip("oracle/_ref/libanni_ref_hip.so not built (reference tree absent at build time)")
    rng = np.random.default_rng(2024)
    n = 200003
    p = (rng.standard_normal(n) * 0.02).astype(np.float32)
    g = np.zeros(n, np.float32)
    P, M, V = p.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    gpu.gpu_set_compute_prec(1)
    e0 = gpu.gpu_param_epoch()
    R = oracle.RefAdamOnBackend(p, g, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1)            # clip applied by hand below
    Ocpu = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    Pc, Mc, Vc = p.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    unit = 1.0 / (math.sqrt(n) * 1e-3)
    for t in range(1, 11):
        gg = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        g[:] = gg
        lr = oracle.lr(3e-4, t - 1, 100, 1000, "cosine")
        gs = unit * (1.7 if t % 2 else 0.6)
        assert R.step(lr, gs) == t and R.on_device
        # the caller's own device-branch arithmetic: norm = sqrt(ss)*|gs|, scale *= clip/norm
        norm = R.last_grad_norm
        eff = gs * (1.0 / norm) if norm > 1.0 else gs
        O.step(P, gg.copy(), M, V, lr, eff)
        m, v = R.moments()
        assert same_bits(p, P) and same_bits(m, M) and same_bits(v, V), t
        assert not g.any()                                          # vec_zero after the scatter
        # ... and against the caller's HOST path (clip/(norm+1e-12), serial norm): tolerances
        Ocpu.step(Pc, gg.copy(), Mc, Vc, lr, gs)
        assert abs(norm - Ocpu.o.last_grad_norm) <= TOL_NORM * norm
        assert rel_err(p, Pc) <= TOL_STATE and rel_err(m, Mc) <= TOL_STATE
        assert rel_err(v, Vc) <= TOL_STATE
    assert gpu.gpu_param_epoch() >= e0 + 10
    R.close()
    gpu.gpu_set_compute_prec(0)
    gpu.gpu_adam_set_weight_decay(0.0)


def test_large_allocations_are_dealt_to_two_pools(gpu):
    """gpu_malloc deals blocks of 256 MiB and more to two pools of chunks, each block to the pool
    with fewer live bytes: the caller's p, g, twin, m, v (lm_adam.c:222-229,295-297) end up as
    p, twin, v | g, m, and the second pool's chunk is looked for in another section of device
    memory.  Freed blocks are reused, empty chunks stay reserved and count as free."""
    from anni_amd.lm_adam import LmAdam
    opt = LmAdam([(4096, 3)])                            # creating an arena returns idle chunks first
    opt.free()
    fr0, tt = C.c_size_t(0), C.c_size_t(0)
    assert gpu.gpu_mem_info(C.byref(fr0), C.byref(tt)) == 0
    n = 160 * 1000 * 1000                                # every block >= 256 MiB
    sizes = [4 * n, 4 * n, 2 * n, 4 * n, 4 * n]
    ptrs = [gpu.gpu_malloc(sz) for sz in sizes]
    assert all(ptrs)
    chunk = 4 * (-(-4 * n // (2 << 20)) * (2 << 20))     # four times the request that opened it
    a, b = ptrs[0], ptrs[1]                              # first block of each pool = start of its chunk

    def pool_of(p):
        return 0 if a <= p < a + chunk else 1 if b <= p < b + chunk else None
    assert [pool_of(p) for p in ptrs] == [0, 1, 0, 1, 0]
    assert not (a <= b < a + chunk) and not (b <= a < b + chunk)
    assert all(p % (2 << 20) == 0 for p in ptrs)
    small = gpu.gpu_malloc(1 << 20)                      # small blocks are ordinary allocations
    assert small and pool_of(small) is None
    gpu.gpu_debug_last_error()
    gpu.gpu_free(ptrs[1] + 4096)                         # not the start of a block: refused, nothing freed
    assert b"not the start of a block" in gpu.gpu_debug_last_error()
    gpu.gpu_free(ptrs[1])
    again = gpu.gpu_malloc(4 * n)                        # a freed block is reused (first fit)
    assert again == ptrs[1]
    # the memory is usable: fill and read back the ends of one block
    assert gpu.gpu_memset(ptrs[3], 0x5a, 4 * n) == 0
    tail = np.zeros(16, np.uint8)
    assert gpu.gpu_memcpy_d2h(tail.ctypes.data, ptrs[3] + 4 * n - 16, 16) == 0 and (tail == 0x5a).all()
    head = np.zeros(16, np.uint8)
    assert gpu.gpu_memset(ptrs[4], 0x33, 4 * n) == 0     # the neighbour in the other pool's chunk is untouched
    assert gpu.gpu_memcpy_d2h(head.ctypes.data, ptrs[3], 16) == 0 and (head == 0x5a).all()
    fr_live = C.c_size_t(0)
    assert gpu.gpu_mem_info(C.byref(fr_live), C.byref(tt)) == 0
    # what the pools hold without a block in it counts as free: in use are the five blocks, no more
    live = sum(-(-sz // (2 << 20)) * (2 << 20) for sz in sizes)
    assert abs((fr0.value - fr_live.value) - live) <= (64 << 20)
    for p in [ptrs[0], again, ptrs[2], ptrs[3], ptrs[4], small]:
        gpu.gpu_free(p)
    # everything returned: the chunks stay reserved for the next large request, are reported as
    # free memory, and go back to the driver when an arena is created
    fr_idle = C.c_size_t(0)
    assert gpu.gpu_mem_info(C.byref(fr_idle), C.byref(tt)) == 0
    assert abs(fr_idle.value - fr0.value) <= (64 << 20)
    fresh = gpu.gpu_malloc(4 * n)
    assert fresh == a                                    # merged back into one free block
    gpu.gpu_free(fresh)
    opt = LmAdam([(4096, 3)])
    opt.free()
    again2 = gpu.gpu_malloc(4 * n)                       # new chunks after the release
    assert again2
    gpu.gpu_free(again2)


def test_small_copies_are_batched_in_order(gpu):
    """Small gpu_memcpy_h2d / gpu_memcpy_d2h_async calls (the bias / LayerNorm traffic of
    lm_adam.c:372-377,407-413) go through the staging rings: contents, ordering against other
    stream work, reuse of the caller's buffer after return, and ring overflow."""
    from anni_amd.lm_adam import DeviceBuffer
    rng = np.random.default_rng(3)
    nseg, seg = 500, 40000                               # 500 x 40 kB = 20 MB: overflows the 16 MiB ring
    d = DeviceBuffer(nseg * seg)
    assert gpu.gpu_memset(d.ptr, 0xee, nseg * seg) == 0
    want = np.empty(nseg * seg, np.uint8)
    scratch = np.empty(seg, np.uint8)
    for i in range(nseg):
        scratch[:] = rng.integers(0, 255, seg, dtype=np.uint8)
        want[i * seg:(i + 1) * seg] = scratch
        assert gpu.gpu_memcpy_h2d(d.ptr + i * seg, scratch.ctypes.data, seg) == 0
        scratch[:] = 0                                   # the caller may reuse its buffer at once
    assert (d.download(np.uint8, nseg * seg) == want).all()
    # h2d batch, then a fill of part of it, then more h2d: order on the stream is kept
    a = np.full(1000, 7, np.uint8)
    assert gpu.gpu_memcpy_h2d(d.ptr, a.ctypes.data, 1000) == 0
    assert gpu.gpu_memset(d.ptr + 500, 9, 1000) == 0
    b = np.full(100, 3, np.uint8)
    assert gpu.gpu_memcpy_h2d(d.ptr + 1400, b.ctypes.data, 100) == 0
    got = d.download(np.uint8, 2000)
    assert (got[:500] == 7).all() and (got[500:1400] == 9).all() and (got[1400:1500] == 3).all()
    assert (got[1500:] == want[1500:2000]).all()
    # async d2h of many pieces, visible after the stream sync; odd sizes and offsets
    outs = []
    for i in range(200):
        off, ln = 12345 * i + (i % 7), 1 + (i * 37) % 5000
        o = np.zeros(ln, np.uint8)
        assert gpu.gpu_memcpy_d2h_async(o.ctypes.data, d.ptr + off, ln) == 0
        outs.append((off, ln, o))
    assert gpu.gpu_memset(d.ptr, 0, nseg * seg) == 0     # later work must not reach the copies
    assert gpu.gpu_stream_sync() == 0
    ref = want.copy()
    ref[:500] = 7
    ref[500:1400] = 9
    ref[1400:1500] = 3
    for off, ln, o in outs:
        assert (o == ref[off:off + ln]).all(), (off, ln)
    assert not d.download(np.uint8, 4096).any()


def test_small_uploads_that_overlap_keep_the_callers_order(gpu):
    """The pieces of one batch are copied in no particular order, so an upload that overlaps one
    still waiting must go into a later launch: as with separate copies, the later one wins.
    Checked with no synchronisation between the uploads: the same bytes many times, ranges that
    overlap in part, neighbours that only touch (which may share a launch), and more uploads
    waiting than the list of waiting ranges holds."""
    from anni_amd.lm_adam import DeviceBuffer
    rng = np.random.default_rng(8)
    size = 1 << 20
    d = DeviceBuffer(size)
    want = np.zeros(size, np.uint8)
    assert gpu.gpu_memset(d.ptr, 0, size) == 0
    keep = []                                            # the host buffers may be reused, but keep them anyway

    def up(off, values):
        a = np.ascontiguousarray(values, dtype=np.uint8)
        keep.append(a)
        want[off:off + a.size] = a
        assert gpu.gpu_memcpy_h2d(d.ptr + off, a.ctypes.data, a.size) == 0
    for k in range(300):                                 # the same four bytes, 300 times
        up(1000, np.full(4, k % 251, np.uint8))
    for k in range(200):                                 # sliding windows, each overlapping the last
        up(5000 + 37 * k, rng.integers(0, 255, 100, dtype=np.uint8))
    for k in range(100):                                 # neighbours that only touch
        up(40000 + 64 * k, np.full(64, k, np.uint8))
    for k in range(700):                                 # many disjoint bytes, then all of them again
        up(100000 + 16 * k, [k % 256])
    for k in range(700):
        up(100000 + 16 * k, [(k * 7 + 1) % 256])
    up(0, rng.integers(0, 255, 300000, dtype=np.uint8))  # a large one over everything so far ...
    up(999, np.full(10, 77, np.uint8))                   # ... and a small one on top of it
    assert (d.download(np.uint8, size) == want).all()
    d.free()


def test_batched_copies_and_the_librarys_own_syncs(gpu):
    """A small gpu_memcpy_d2h_async is complete after ANY synchronising call of the library, the
    arena's included, and anni_gpu_flush puts a pending small upload on the stream for work the
    caller enqueues on the stream handle itself."""
    from anni_amd.lm_adam import DeviceBuffer, LmAdam
    d = DeviceBuffer(4096)
    src = np.arange(4096, dtype=np.uint8)
    d.upload(src)
    opt = LmAdam([(4096, 3)])
    out = np.zeros(1000, np.uint8)
    assert gpu.gpu_memcpy_d2h_async(out.ctypes.data, d.ptr + 96, 1000) == 0
    opt.sync_stats()                                     # not one of the gpu_* syncs
    assert (out == src[96:1096]).all()
    # a pending small upload reaches the stream on request
    up = np.full(512, 0xab, np.uint8)
    assert gpu.gpu_memcpy_h2d(d.ptr, up.ctypes.data, 512) == 0
    gpu.anni_gpu_flush()
    up[:] = 0                                            # staged at call time
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    assert hip.hipStreamSynchronize(gpu.anni_gpu_stream()) == 0       # the caller's own wait
    got = np.zeros(512, np.uint8)
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    assert hip.hipMemcpy(got.ctypes.data, d.ptr, 512, 2) == 0          # 2 = device to host
    assert (got == 0xab).all()
    opt.free()
    d.free()


def test_malloc_and_free_from_many_threads(gpu):
    """gpu_malloc / gpu_free are called from OpenMP threads in the reference (gpu_cuda.cu:2644-2645):
    eight threads allocate, fill, check and free blocks of mixed sizes, the large ones out of the
    two pools; afterwards the device holds what it held before."""
    import threading
    fr0, tt = C.c_size_t(0), C.c_size_t(0)
    hold = gpu.gpu_malloc(300 << 20)                 # keeps one chunk alive while the threads churn
    assert hold
    gpu.gpu_device_sync()
    assert gpu.gpu_mem_info(C.byref(fr0), C.byref(tt)) == 0
    errors = []

    def worker(k):
        try:
            rng = np.random.default_rng(k)
            for i in range(25):
                nbytes = int(rng.choice([64, 4096, 1 << 20, 300 << 20])) + 16 * int(rng.integers(0, 8))
                p = gpu.gpu_malloc(nbytes)
                if not p:
                    raise MemoryError(nbytes)
                val = (k * 25 + i) % 251 + 1
                if gpu.gpu_memset(p, val, min(nbytes, 1 << 16)) != 0:
                    raise RuntimeError("memset")
                out = np.zeros(64, np.uint8)
                if gpu.gpu_memcpy_d2h(out.ctypes.data, p, 64) != 0 or not (out == val).all():
                    raise RuntimeError("thread %d block %d read back %r" % (k, i, out[:4]))
                gpu.gpu_free(p)
        except Exception as e:                       # noqa: BLE001 - reported below
            errors.append(repr(e))
    threads = [threading.Thread(target=worker, args=(k,)) for k in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    gpu.gpu_device_sync()
    fr1 = C.c_size_t(0)
    assert gpu.gpu_mem_info(C.byref(fr1), C.byref(tt)) == 0
    assert abs(fr1.value - fr0.value) <= 64 << 20    # the runtime's own pools may have grown a little
    gpu.gpu_free(hold)


def test_grad_sumsq_from_two_threads_is_right_or_refused(gpu, oracle):
    """gpu_grad_sumsq has one result slot per process (as the reference's static accumulator,
    num/gpu_cuda.cu:8485-8486) and is meant for one thread.  A second call that arrives while one
    is between its launch and its read-back is turned away with -1 -- it never returns the other
    call's sum."""
    import threading
    from anni_amd.lm_adam import DeviceBuffer
    rng = np.random.default_rng(77)
    n = 6 * 1000 * 1000
    xs = [(rng.standard_normal(n) * (k + 1)).astype(np.float32) for k in range(2)]
    want = [oracle.sumsq(x, threads=4) for x in xs]
    bufs = [DeviceBuffer(4 * n) for _ in xs]
    for b, x in zip(bufs, xs):
        b.upload(x)
    results = [[], []]

    def work(k):
        out = C.c_double(0)
        good = 0
        for _ in range(200000):                            # until 60 calls got in (the other thread is in the way)
            rc = gpu.gpu_grad_sumsq(bufs[k].ptr, n, C.byref(out))
            results[k].append((rc, out.value))
            good += rc == 0
            if good == 60:
                break
    th = [threading.Thread(target=work, args=(k,)) for k in range(2)]
    for t in th:
        t.start()
    for t in th:
        t.join()
    refused = 0
    for k in range(2):
        done = 0
        for rc, val in results[k]:
            assert rc in (0, -1)
            if rc == 0:
                assert abs(val - want[k]) <= 1e-10 * want[k], (k, val, want[k])
                done += 1
            else:
                refused += 1
        assert done == 60, (k, done, len(results[k]))
    print("calls refused while the other thread was inside: %d" % refused, flush=True)
    out = C.c_double(0)
    assert gpu.gpu_grad_sumsq(bufs[0].ptr, n, C.byref(out)) == 0      # and the flag is free afterwards
    assert abs(out.value - want[0]) <= 1e-10 * want[0]
    for b in bufs:
        b.free()


def test_sum_begun_early_gives_the_same_bits_and_is_dropped_when_anything_intervenes(gpu, oracle):
    """The caller's pattern (lang/lm_adam.c:462-470): a synchronisation, small uploads of vectors
    into the parameter and gradient flats, then gpu_grad_sumsq of the gradient flat.  After the
    pattern has been shown twice the backend begins the sum at the first upload and repairs the
    chunks written afterwards.  The result must have the bits of a sum taken from the start, the
    counters must show the early sum in use, and anything else that reaches the stream between
    its launch and the call -- a fill, a device-to-device copy, another flat -- must make the
    backend drop it and still answer right."""
    from anni_amd.lm_adam import DeviceBuffer
    rng = np.random.default_rng(314)
    n = 3 * 1000 * 1000 + 17
    p, g = DeviceBuffer(4 * n), DeviceBuffer(4 * n)
    tw, other = DeviceBuffer(2 * n), DeviceBuffer(4 * n)
    host = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    g.upload(host)
    other.upload(host[::-1].copy())
    p.upload(np.zeros(n, np.float32))
    gpu.gpu_adam_set_bf16_flat(tw.ptr, p.ptr, n)
    vecs = [(5, 1000), (4096 * 3 - 7, 4100), (n - 70000, 70000), (1234567, 1), (2000000, 16384)]
    used0, dropped0 = C.c_long(0), C.c_long(0)
    gpu.anni_early_sum_stats(C.byref(used0), C.byref(dropped0))

    def gather():
        """What seg_gather does for the vector segments: parameters and fresh gradients go up."""
        gpu.gpu_device_sync()
        for off, cnt in vecs:
            fresh = (rng.standard_normal(cnt) * 1e-3).astype(np.float32)
            host[off:off + cnt] = fresh
            assert gpu.gpu_memcpy_h2d(p.ptr + 4 * off, fresh.ctypes.data, 4 * cnt) == 0
            assert gpu.gpu_memcpy_h2d(g.ptr + 4 * off, fresh.ctypes.data, 4 * cnt) == 0

    def sumsq(buf):
        out = C.c_double(0)
        assert gpu.gpu_grad_sumsq(buf.ptr, n, C.byref(out)) == 0
        return out.value

    def counters():
        u, d = C.c_long(0), C.c_long(0)
        gpu.anni_early_sum_stats(C.byref(u), C.byref(d))
        return u.value - used0.value, d.value - dropped0.value
    def learn():
        """The pattern twice, each sum checked against the host's."""
        for _ in range(2):
            gather()
            got = sumsq(g)
            want = oracle.sumsq(host, threads=4)
            assert abs(got - want) <= 1e-10 * want
    for rnd in range(3):
        learn()
        gather()                                          # third time: the sum begins at the first upload
        got = sumsq(g)
        needs_second_stream(gpu)
        assert counters() == (rnd + 1, 0)
        again = sumsq(g)                                  # no uploads before it: taken from the start
        want = oracle.sumsq(host, threads=4)              # (and a call that does not fit: the count starts again)
        assert got == again, rnd
        assert abs(got - want) <= 1e-10 * want, rnd
    used = 3
    # something else reaches the stream after the early sum was launched: it must be dropped
    learn()
    gather()
    assert gpu.gpu_memset(g.ptr + 4 * 777, 0, 4 * 100) == 0
    host[777:877] = 0.0
    got = sumsq(g)
    assert counters() == (used, 1)
    assert abs(got - oracle.sumsq(host, threads=4)) <= 1e-10 * got and got == sumsq(g)
    # the pattern has to be shown twice again before the next guess
    gather()
    assert sumsq(g) > 0 and counters() == (used, 1)
    gather()
    assert sumsq(g) > 0 and counters() == (used, 1)
    gather()
    got = sumsq(g)
    assert counters() == (used + 1, 1) and got == sumsq(g)
    assert abs(got - oracle.sumsq(host, threads=4)) <= 1e-10 * got
    # the sum of another flat is asked for after the early sum of g was launched: dropped, right answer
    learn()
    gather()
    got = sumsq(other)
    assert counters() == (used + 1, 2)
    back = other.download(np.float32, n)
    want = oracle.sumsq(back, threads=4)
    assert abs(got - want) <= 1e-10 * want and got == sumsq(other)
    gpu.gpu_adam_set_bf16_flat(None, None, 0)
    for b in (p, g, tw, other):
        b.free()


def test_sum_begun_early_with_more_rewritten_chunks_than_one_launch_takes(gpu, oracle):
    """The last stage of the flat sum is one launch that also recomputes the chunks the caller
    rewrote after the early sum began, their list travelling in the kernel's arguments (768 at
    most); longer lists go through the separate kernels.  Both must give the bits of a sum taken
    from the start, and the self-check that holds the one launch against the separate kernels on
    first use must have run without a mismatch."""
    from anni_amd.lm_adam import DeviceBuffer
    rng = np.random.default_rng(2718)
    n = 20 * 1000 * 1000 + 3                              # 4883 chunks of 4096 floats
    p, g = DeviceBuffer(4 * n), DeviceBuffer(4 * n)
    host = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    g.upload(host)
    p.upload(np.zeros(n, np.float32))
    used0, dropped0 = C.c_long(0), C.c_long(0)
    gpu.anni_early_sum_stats(C.byref(used0), C.byref(dropped0))

    def step(count):
        """`count` single floats, one per chunk, in falling order (the list is sorted by the backend)."""
        gpu.gpu_device_sync()
        for k in reversed(range(count)):
            off = 4096 * (5 * k + 1) + 11
            fresh = (rng.standard_normal(1) * 1e-3).astype(np.float32)
            host[off] = fresh[0]
            assert gpu.gpu_memcpy_h2d(g.ptr + 4 * off, fresh.ctypes.data, 4) == 0
        out = C.c_double(0)
        assert gpu.gpu_grad_sumsq(g.ptr, n, C.byref(out)) == 0
        return out.value

    def fresh_sum():
        out = C.c_double(0)
        assert gpu.gpu_grad_sumsq(g.ptr, n, C.byref(out)) == 0
        return out.value
    for rnd, count in enumerate((700, 900)):
        for _ in range(3 if rnd == 0 else 2):             # the pattern, twice with the flat known
            got = step(count)
            assert abs(got - oracle.sumsq(host, threads=4)) <= 1e-10 * got
        got = step(count)                                 # begun early
        needs_second_stream(gpu)
        u, d = C.c_long(0), C.c_long(0)
        gpu.anni_early_sum_stats(C.byref(u), C.byref(d))
        assert (u.value - used0.value, d.value - dropped0.value) == (rnd + 1, 0)
        assert got == fresh_sum(), count
        assert abs(got - oracle.sumsq(host, threads=4)) <= 1e-10 * got
    runs, bad = C.c_int(0), C.c_int(0)
    gpu.anni_fold_guard_stats(C.byref(runs), C.byref(bad))
    assert runs.value >= 1 and bad.value == 0
    p.free()
    g.free()


def test_vectors_first_split_update_serves_the_read_backs_and_leaves_no_tile_out(gpu, oracle):
    """lang/lm_adam.c reads its bias / LayerNorm vectors back after every update, one small
    gpu_memcpy_d2h_async each, then synchronises (lm_adam.c:407-413,500).  Once the same list has
    followed two updates the backend updates the tiles that hold those vectors in a launch of their
    own beside the large one and copies them out ahead of it.  Every step, split or not, must
    leave p, m, v, g and the twins with the oracle's bits over the WHOLE flat (no tile twice, none
    left out) and hand the caller the vectors' new values; a request that departs from the list,
    an operation between the update and a read-back, and an update on a stream that was not
    idle must all give the ordinary result."""
    n = 4096 * 700 + 1234                                   # 701 tiles, the last one ragged
    S = FlatState(gpu, n, seed=99)
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, threads=8)
    gpu.gpu_set_compute_prec(1)
    vecs = [(7, 1000), (4096 * 5 - 3, 10), (4096 * 300, 4096), (4096 * 699 + 100, 2000), (n - 1234, 1234),
            (1500000, 70000)]
    def vf_stats():
        a, b = C.c_long(0), C.c_long(0)
        assert gpu.anni_vectors_first_stats(C.byref(a), C.byref(b)) == 0
        return a.value, b.value
    steps0, served0 = vf_stats()
    t = [0]

    def one_step(ranges, between=None, dirty_stream=False):
        """Sum, norm on the host, update, read-backs, synchronisation: adam_step_gpu's order of calls."""
        t[0] += 1
        S.new_grad(1e-3 * (1 + t[0] % 3))
        ss = C.c_double(0)
        assert gpu.gpu_grad_sumsq(S.dg.ptr, n, C.byref(ss)) == 0
        gs = 0.5 if t[0] % 2 else 1.0
        lr = 1e-3 / t[0]
        if dirty_stream:                                    # something small is still waiting to go up
            one = np.float32([0.25])
            S.p[11] = one[0]
            assert gpu.gpu_memcpy_h2d(S.dp.ptr + 4 * 11, one.ctypes.data, 4) == 0
        gpu.gpu_adam_set_weight_decay(0.1)
        assert gpu.gpu_adam_step_dev_bf16(S.dp.ptr, S.dt.ptr, S.dg.ptr, S.dm.ptr, S.dv.ptr, n, lr,
                                          0.9, 0.95, 1e-8, t[0], gs) == 0
        O.step(S.p, S.g, S.m, S.v, lr, gs, twin=S.twin)
        if between:
            between()
        got = [np.full(cnt, np.nan, np.float32) for _off, cnt in ranges]
        for (off, cnt), out in zip(ranges, got):
            assert gpu.gpu_memcpy_d2h_async(out.ctypes.data, S.dp.ptr + 4 * off, 4 * cnt) == 0
        assert gpu.gpu_stream_sync() == 0
        for (off, cnt), out in zip(ranges, got):
            assert same_bits(out, S.p[off:off + cnt]), (t[0], off)
        p, m, v, g, tw = S.fetch()
        assert same_bits(p, S.p) and same_bits(m, S.m) and same_bits(v, S.v), t[0]
        assert not g.any() and (tw == S.twin).all(), t[0]

    def counters():
        a, b = vf_stats()
        return a - steps0, b - served0
    one_step(vecs)
    one_step(vecs)
    assert counters() == (0, 0)                             # shown twice: from now on the update is split
    one_step(vecs)
    one_step(vecs)
    needs_second_stream(gpu)
    assert counters() == (2, 2 * len(vecs))
    # the fourth request departs from the list: the first three are served, the rest copied the ordinary way
    other = vecs[:3] + [(4096 * 20 + 5, 333)] + vecs[4:]
    one_step(other)
    assert counters() == (3, 2 * len(vecs) + 3)
    one_step(other)                                         # the new list, shown for the second time
    assert counters() == (3, 2 * len(vecs) + 3)
    one_step(other)
    assert counters() == (4, 2 * len(vecs) + 3 + len(other))

    # an operation between the update and the read-backs: they must see its result
    def clear_some():
        assert gpu.gpu_memset(S.dp.ptr + 4 * 7, 0, 4 * 500) == 0
        S.p[7:507] = 0.0
    one_step(other, between=clear_some)
    assert counters() == (4, 2 * len(vecs) + 3 + len(other))
    one_step(other)                                         # (the pattern has to be shown twice again)
    one_step(other)
    assert counters()[0] == 4
    one_step(other)
    assert counters()[0] == 5
    # the stream is not idle at the update (a small upload is waiting): no split, same results
    one_step(other, dirty_stream=True)
    assert counters()[0] == 5
    gpu.gpu_set_compute_prec(0)
    gpu.gpu_adam_set_weight_decay(0.0)


@pytest.mark.parametrize("seed", list(range(1, 11)))
def test_random_call_sequences_against_a_host_model(gpu, oracle, seed):
    """The flat entry points under call sequences nobody wrote by hand: the caller's regular step
    (which, repeated, brings in the sum begun early and the split update) mixed at random with
    everything that must make the backend drop what it began -- large and small uploads, fills,
    read-backs of other places, extra sums, extra synchronisations, uploads that overlap -- against
    a model kept on the host: every sum within 1e-10 of the exact one and equal to a second call's,
    every read-back equal to the model at the time it was asked for, and p, g, m, v and the twins
    equal to the model's bits after every round."""
    rng = np.random.default_rng(1000 + seed)
    n = 4096 * 290 + 1000 + seed
    S = FlatState(gpu, n, seed=seed)
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, threads=8)
    gpu.gpu_set_compute_prec(1)
    gpu.gpu_adam_set_bf16_flat(S.dt.ptr, S.dp.ptr, n)
    S.twin[:] = oracle.bf16_rne(S.p)
    assert gpu.gpu_adam_seed_bf16_flat(S.dt.ptr, S.dp.ptr, n) == 0
    flats = {"p": (S.dp, S.p), "g": (S.dg, S.g), "m": (S.dm, S.m), "v": (S.dv, S.v)}
    vecs = [(int(o), int(c)) for o, c in zip(rng.integers(0, n - 5000, 9), rng.integers(1, 5000, 9))]
    pending = []                                         # read-backs asked for: (buffer, expected)
    keep = []
    t = [0]

    def upload(name, off, values):
        buf, host = flats[name]
        a = np.ascontiguousarray(values, dtype=np.float32)
        keep.append(a)
        host[off:off + a.size] = a
        assert gpu.gpu_memcpy_h2d(buf.ptr + 4 * off, a.ctypes.data, 4 * a.size) == 0

    def read_back(name, off, cnt):
        buf, host = flats[name]
        out = np.full(cnt, np.nan, np.float32)
        assert gpu.gpu_memcpy_d2h_async(out.ctypes.data, buf.ptr + 4 * off, 4 * cnt) == 0
        pending.append((out, host[off:off + cnt].copy()))

    def sync(which):
        if which:
            assert gpu.gpu_stream_sync() == 0
        else:
            gpu.gpu_device_sync()
        for out, want in pending:
            assert same_bits(out, want)
        pending.clear()

    def sumsq():
        out = C.c_double(0)
        assert gpu.gpu_grad_sumsq(S.dg.ptr, n, C.byref(out)) == 0
        for o, want in pending:                          # the call implies a synchronisation
            assert same_bits(o, want)
        pending.clear()
        want = oracle.sumsq(S.g, threads=4)
        assert abs(out.value - want) <= 1e-10 * want, (out.value, want)
        return out.value

    def update(gs):
        t[0] += 1
        lr = 1e-3 / t[0]
        gpu.gpu_adam_set_weight_decay(0.1)
        assert gpu.gpu_adam_step_dev_bf16(S.dp.ptr, S.dt.ptr, S.dg.ptr, S.dm.ptr, S.dv.ptr, n, lr,
                                          0.9, 0.95, 1e-8, t[0], gs) == 0
        O.step(S.p, S.g, S.m, S.v, lr, gs, twin=S.twin)

    def disturbance():
        k = int(rng.integers(0, 12))
        if k == 0:
            off = int(rng.integers(0, n - 400000))
            upload("g", off, rng.standard_normal(300000) * 1e-3)          # more than 1 MiB: an ordinary copy
        elif k == 1:
            off, cnt = int(rng.integers(0, n - 3000)), int(rng.integers(1, 3000))
            name = "pg"[int(rng.integers(0, 2))]
            assert gpu.gpu_memset(flats[name][0].ptr + 4 * off, 0, 4 * cnt) == 0
            flats[name][1][off:off + cnt] = 0.0
        elif k == 2:
            read_back("pgmv"[int(rng.integers(0, 4))], int(rng.integers(0, n - 2000)), int(rng.integers(1, 2000)))
        elif k == 3:
            assert sumsq() == sumsq()
        elif k == 4:
            sync(int(rng.integers(0, 2)))
        elif k == 5:
            off = int(rng.integers(0, n - 300))
            for _ in range(3):                           # the same place three times: the last one wins
                upload("pg"[int(rng.integers(0, 2))], off, rng.standard_normal(200) * 1e-3)
        elif k == 6:
            update(float(rng.random()) + 0.1)            # an update nobody announced
        elif k == 7:
            out = np.empty(1000, np.float32)
            off = int(rng.integers(0, n - 1000))
            assert gpu.gpu_memcpy_d2h(out.ctypes.data, S.dp.ptr + 4 * off, 4000) == 0
            assert same_bits(out, S.p[off:off + 1000])
            for o, want in pending:
                assert same_bits(o, want)
            pending.clear()
        elif k == 8:
            out = C.c_double(0)                          # the sum of another flat
            assert gpu.gpu_grad_sumsq(S.dp.ptr, n, C.byref(out)) == 0
            want = oracle.sumsq(S.p, threads=4)
            assert abs(out.value - want) <= 1e-10 * want
            for o, w in pending:
                assert same_bits(o, w)
            pending.clear()
        elif k == 9:
            gpu.anni_gpu_flush()                         # a caller announcing work of its own on the stream
        elif k == 10 and not pending:
            S.dg.free()                                  # the gradient flat freed and allocated anew
            S.dg = dev(gpu, S.g)                         # (the driver may hand out the same address)
            flats["g"] = (S.dg, S.g)

    def regular_step(noise):
        """adam_step_gpu's order of calls; `noise` = chance of a disturbance at each of its joints."""
        S.new_grad(1e-3 * (1 + t[0] % 3))                # "the backward pass": a large upload
        sync(0)
        for off, cnt in vecs:
            if rng.random() < noise:
                disturbance()
            upload("p", off, S.p[off:off + cnt] * np.float32(1.0))
            upload("g", off, rng.standard_normal(cnt) * 1e-3)
        if rng.random() < noise:
            disturbance()
        ss = sumsq()
        if rng.random() < noise:
            disturbance()
        gs = 1.0 / (math.sqrt(n) * 1e-3) * (1.7 if t[0] % 2 else 0.6)
        norm = math.sqrt(oracle.sumsq(S.g, threads=4)) * gs if noise else math.sqrt(ss) * gs
        update(gs / norm if norm > 1.0 else gs)
        for off, cnt in vecs:
            if rng.random() < noise:
                disturbance()
            read_back("p", off, cnt)
        sync(1)
        p, m, v, g, tw = S.fetch()
        assert same_bits(p, S.p) and same_bits(m, S.m) and same_bits(v, S.v) and same_bits(g, S.g), t[0]
        assert (tw == S.twin).all(), t[0]
    for rnd in range(6):
        for _ in range(4):
            regular_step(0.0)                            # long enough for both patterns to be learned and used
        for _ in range(4):
            regular_step(0.3 if rnd % 3 == 2 else 0.08)
    early, dropped = C.c_long(0), C.c_long(0)
    gpu.anni_early_sum_stats(C.byref(early), C.byref(dropped))
    assert early.value > 0 or gpu.anni_second_stream_state() == 0
    gpu.gpu_adam_set_bf16_flat(None, None, 0)
    gpu.gpu_set_compute_prec(0)
    gpu.gpu_adam_set_weight_decay(0.0)
