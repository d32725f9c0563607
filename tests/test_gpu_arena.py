"""Parity of the multi-tensor arena step (include/anni_adam.h) against the CPU oracle, through the
C ABI: the benchmark configurations at reduced size, ragged tensor lists, every storage mode, the
non-finite skip, and the golden vectors of the reference."""
import numpy as np
import pytest

from helpers import GOLDEN_CASES, load_golden, same_bits, rel_err, bf16_ulp_diff

pytestmark = pytest.mark.gpu

TOL_STATE = 1e-6     # required: FP32 master/m/v within 1e-6 relative per step
TOL_NORM = 1e-5      # required: clip norm within 1e-5 relative

F32, BF16, FP8 = 0, 1, 2
DECAY, TWIN = 1, 2

RAGGED = [(5000, 3), (3, 0), (4096, 3), (1, 2), (0, 3), (8191, 1), (12288, 3), (7, 0), (4097, 3),
          (2, 1), (40000, 3), (1023, 0)]


def oracle_tensors(opt, gscales=None):
    return [(opt.offsets[i], opt.sizes[i], 1 if (f & DECAY) else 0,
             1.0 if gscales is None else float(gscales[i]))
            for i, f in enumerate(opt._flags)]


def make(gpu, tensors, **kw):
    from anni_amd.lm_adam import LmAdam
    opt = LmAdam(tensors, **kw)
    opt._flags = [t[-1] for t in tensors]
    return opt


def twin_mask(opt):
    mask = np.zeros(opt.n, bool)
    for off, n, f in zip(opt.offsets, opt.sizes, opt._flags):
        if f & TWIN:
            mask[off:off + n] = True
    return mask


def run_fp32_case(gpu, oracle, tensors, steps, clip, wd, gmul, grad_scale=1.0, seed=0,
                  sched=(100, 1000, "cosine"), layout=0):
    """Ten steps on the arena vs the oracle twice: against the oracle's own (serial) norm with the
    required tolerances, and bit for bit when the oracle is handed the device's sum of squares."""
    from anni_amd import lm_adam
    rng = np.random.default_rng(seed)
    opt = make(gpu, tensors, beta2=0.95, weight_decay=wd, grad_clip=clip, layout=layout)
    n = opt.n
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    opt.upload("param", p0)
    opt.seed_twins()
    A = dict(p=p0.copy(), m=np.zeros(n, np.float32), v=np.zeros(n, np.float32))   # own norm
    B = dict(p=p0.copy(), m=np.zeros(n, np.float32), v=np.zeros(n, np.float32))   # device norm
    twinB = oracle.bf16_rne(p0)
    segs = oracle_tensors(opt)
    OA = oracle.Oracle(n, beta2=0.95, weight_decay=wd, grad_clip=clip, tensors=segs, threads=4)
    OB = oracle.Oracle(n, beta2=0.95, weight_decay=wd, grad_clip=clip, tensors=segs, threads=4)
    mask = twin_mask(opt)
    n_clipped = 0
    for s in range(steps):
        g = (rng.standard_normal(n) * 1e-3 * gmul[s % len(gmul)]).astype(np.float32)
        opt.upload("grad", g)
        lr = lm_adam.step_lr(3e-4, opt.t, *sched)
        assert lr == oracle.lr(3e-4, s, *sched)
        assert opt.step_scaled(lr, grad_scale) == 0
        st = opt.sync_stats()
        assert opt.t == s + 1
        gA, gB = g.copy(), g.copy()
        OA.step(A["p"], gA, A["m"], A["v"], lr, grad_scale)
        p, m, v = opt.download("param"), opt.download("m"), opt.download("v")
        tw, gd = opt.download("twin"), opt.download("grad")
        if clip > 0:
            assert abs(st.last_grad_norm - OA.o.last_grad_norm) <= TOL_NORM * OA.o.last_grad_norm
            assert st.last_clipped == OA.o.last_clipped and st.last_skipped == 0
            n_clipped += st.last_clipped
        assert rel_err(p, A["p"]) <= TOL_STATE, s
        assert rel_err(m, A["m"]) <= TOL_STATE and rel_err(v, A["v"]) <= TOL_STATE, s
        assert bf16_ulp_diff(tw[mask], oracle.bf16_rne(A["p"])[mask]) <= 1
        assert not gd.any()
        OB.step(B["p"], gB, B["m"], B["v"], lr, grad_scale, twin=twinB,
                sumsq_override=st.last_sumsq if clip > 0 else None)
        assert same_bits(p, B["p"]) and same_bits(m, B["m"]) and same_bits(v, B["v"]), s
        assert (tw[mask] == twinB[mask]).all()
        assert (tw[~mask] == oracle.bf16_rne(p0)[~mask]).all()       # unflagged tensors keep the seed
        if clip > 0:
            assert st.last_grad_scale == OB.o.last_grad_scale
    opt.free()
    return n_clipped


def test_split_layout_gives_the_same_results(gpu, oracle):
    """Two allocations (p, m, tables | v, twins, gradient slots) instead of one."""
    from anni_amd import lib
    opt = make(gpu, RAGGED, layout=lib.LAYOUT_SPLIT, grad_slots=2)
    n = opt.n
    assert opt.split and opt.grad_slot(1) - opt.grad_slot(0) >= 4 * n
    assert opt.o.d_m - opt.o.d_param >= 4 * n                     # first block: p, m
    assert opt.o.d_param_bf16 - opt.o.d_v >= 4 * n                # second block: v, twins, slots
    assert opt.grad_slot(0) - opt.o.d_param_bf16 >= 2 * n
    assert not (opt.o.d_param <= opt.o.d_v < opt.o.d_param + 8 * n)
    assert opt.arena_bytes >= opt.resident_bytes + 4 * n          # the second slot
    assert opt.arena_bytes <= opt.resident_bytes + 4 * n + (16 << 20)   # nothing reserved beyond the contents
    assert opt.apart_ratio == 1.0                                 # too small to be placed by measurement
    assert opt.grad_slot(2) is None
    opt.free()
    base = 1.0 / (np.sqrt(n) * 1e-3)
    assert run_fp32_case(gpu, oracle, RAGGED, 4, clip=1.0, wd=0.1, gmul=[0.5 * base, 2.0 * base],
                         layout=lib.LAYOUT_SPLIT) == 2


def test_config1_no_clip_ragged(gpu, oracle):
    """benchmark configuration 1 hyper-parameters (constant lr, no clip, decay on flagged tensors)."""
    run_fp32_case(gpu, oracle, RAGGED, 10, clip=0.0, wd=0.1, gmul=[1.0], sched=(0, 0, "none"))


def test_config2_clip_half_the_steps_ragged(gpu, oracle):
    """benchmark configuration 2: clip 1.0 with about half the steps clipping, warmup 100 + cosine."""
    n = sum(t[0] for t in RAGGED)
    base = 1.0 / (np.sqrt(n) * 1e-3)                       # gmul = base -> norm ~ 1
    k = run_fp32_case(gpu, oracle, RAGGED, 10, clip=1.0, wd=0.1,
                      gmul=[0.5 * base, 2.0 * base, 0.7 * base, 1.5 * base])
    assert k == 5


def test_tiny_model_layout_with_grad_scale(gpu, oracle):
    """The reference's 64-wide test model and rig constants (tests/test_gpu.c:30-34,67-84)."""
    from anni_amd import layout
    t = layout.tensors("tiny", "reference")
    k = run_fp32_case(gpu, oracle, t, 4, clip=1.0, wd=0.1, gmul=[300.0, 90000.0],
                      grad_scale=1.0 / (4 * 63), sched=(0, 0, "none"), seed=1234)
    assert k == 2


def test_single_tensor_and_unit_sizes(gpu, oracle):
    for tensors in ([(1, 3)], [(4095, 3)], [(4096, 3)], [(4097, 1)], [(1, 0)] * 9, [(0, 3), (5, 3), (0, 0)]):
        run_fp32_case(gpu, oracle, tensors, 3, clip=1.0, wd=0.1, gmul=[1e3, 1.0], seed=len(tensors))


def test_golden_vectors_through_arena(gpu, oracle):
    """The reference's own outputs vs the fused device step (CPU-form clip, device norm)."""
    from anni_amd.lm_adam import LmAdam
    for name in GOLDEN_CASES:
        G = load_golden(name)
        n = G["p0"].size
        opt = LmAdam([(n, 3)], beta1=float(G["beta1"]), beta2=float(G["beta2"]),
                     eps=float(G["eps"]), weight_decay=float(G["wd"]), grad_clip=float(G["clip"]))
        opt.upload("param", G["p0"])
        exact = 0
        for s in range(G["grads"].shape[0]):
            opt.upload("grad", G["grads"][s])
            assert opt.step_scaled(float(G["lr"][s]), float(G["grad_scale"])) == 0
            p, m, v = opt.download("param"), opt.download("m"), opt.download("v")
            assert rel_err(p, G["p"][s]) <= TOL_STATE and rel_err(m, G["m"][s]) <= TOL_STATE
            assert rel_err(v, G["v"][s]) <= TOL_STATE
            exact += same_bits(p, G["p"][s]) and same_bits(m, G["m"][s]) and same_bits(v, G["v"][s])
            assert not opt.download("grad").any()
        if float(G["clip"]) == 0.0:
            assert exact == G["grads"].shape[0]              # no norm involved: bit for bit
        opt.free()


def test_lr_nonpositive_is_a_noop(gpu):
    opt = make(gpu, [(100, 3)])
    opt.upload("grad", np.ones(100, np.float32))
    e0 = gpu.gpu_param_epoch()
    assert opt.step_scaled(0.0) == 1 and opt.t == 0          # lm_adam.c:531-532
    assert opt.step_scaled(-1.0) == 1 and opt.t == 0
    assert opt.download("grad").all() and not opt.download("param").any()
    assert gpu.gpu_param_epoch() == e0                        # nothing moved
    assert opt.step_scaled(1e-3) == 0 and opt.t == 1
    assert gpu.gpu_param_epoch() == e0 + 1                    # lm_adam.c:547: the weight epoch moves
    opt.free()


@pytest.mark.parametrize("bad,where", [(np.nan, 0), (np.inf, 5000 + 3 + 17), (-np.inf, -1)])
def test_nonfinite_skip_leaves_state_bit_identical(gpu, oracle, bad, where, capfd):
    rng = np.random.default_rng(31)
    opt = make(gpu, RAGGED, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True)
    n = opt.n
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    opt.upload("param", p0)
    opt.seed_twins()
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True,
                      tensors=oracle_tensors(opt), threads=4)
    P, M, V = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for s in range(4):
        g = (rng.standard_normal(n) * 3e-3).astype(np.float32)
        if s == 2:
            g[where] = bad
        before = [opt.download(k) for k in ("param", "m", "v", "twin")]
        opt.upload("grad", g)
        assert opt.step_scaled(1e-3) == 0
        st = opt.sync_stats()
        gg = g.copy()
        O.step(P, gg, M, V, 1e-3, sumsq_override=st.last_sumsq if s != 2 else None)
        assert st.last_skipped == O.o.last_skipped == (1 if s == 2 else 0)     # decision matches exactly
        assert opt.t == O.t == s + 1                                            # t advances on a skip
        after = [opt.download(k) for k in ("param", "m", "v", "twin")]
        if s == 2:
            for a, b in zip(before, after):
                assert same_bits(a, b) if a.dtype == np.float32 else (a == b).all()
        assert same_bits(after[0], P) and same_bits(after[1], M) and same_bits(after[2], V)
        assert not opt.download("grad").any()
        opt.sync_stats()                                 # a second read of the same step prints nothing more
    # the reference's message for the skipped step (lm_adam.c:479-480), once
    err = capfd.readouterr().err
    lines = [ln for ln in err.splitlines() if ln.startswith("[adam] step ")]
    assert len(lines) == 1 and lines[0].startswith("[adam] step 3 skipped: grad norm "), err
    assert lines[0].split()[-1] in ("nan", "-nan", "inf")
    opt.free()


def test_without_skip_flag_nonfinite_poisons_like_the_cpu_path(gpu, oracle):
    """The reference's host loop has no skip: a NaN gradient reaches the state (lm_adam.c:571-598)."""
    opt = make(gpu, [(4096, 3)], grad_clip=1.0)
    g = np.full(4096, 1e-3, np.float32)
    g[5] = np.nan
    opt.upload("grad", g)
    opt.step_scaled(1e-3)
    st = opt.sync_stats()
    assert st.last_skipped == 0 and np.isnan(st.last_grad_norm)
    assert np.isnan(opt.download("param")[5])
    opt.free()


def test_bf16_moments_and_grads(gpu, oracle):
    """benchmark configuration 4 at reduced size, long tail included (parity unpinned by the reference:
    the oracle defines the rounding points)."""
    rng = np.random.default_rng(44)
    opt = make(gpu, RAGGED, grad_type=BF16, moment_type=BF16, beta2=0.95, weight_decay=0.1,
               grad_clip=1.0)
    n = opt.n
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    opt.upload("param", p0)
    P = p0.copy()
    M = np.zeros(n, np.uint16)
    V = np.zeros(n, np.uint16)
    twin = oracle.bf16_rne(p0)
    opt.seed_twins()
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, grad_type=oracle.BF16,
                      moment_type=oracle.BF16, tensors=oracle_tensors(opt), threads=4)
    mask = twin_mask(opt)
    base = 1.0 / (np.sqrt(n) * 1e-3)
    for s in range(10):
        g = oracle.bf16_rne((rng.standard_normal(n) * 1e-3 * base * (0.6 if s % 2 else 1.7))
                            .astype(np.float32))
        opt.upload("grad", g)
        lr = oracle.lr(3e-4, s, 100, 1000, "cosine")
        opt.step_scaled(lr)
        st = opt.sync_stats()
        own = oracle.sumsq(g, oracle.BF16)
        assert abs(st.last_sumsq - own) <= 1e-11 * own
        gg = g.copy()
        O.step(P, gg, M, V, lr, twin=twin, sumsq_override=st.last_sumsq)
        assert st.last_clipped == O.o.last_clipped == (0 if s % 2 else 1)
        assert same_bits(opt.download("param"), P)
        assert (opt.download("m") == M).all() and (opt.download("v") == V).all()
        assert (opt.download("twin")[mask] == twin[mask]).all()
        assert not opt.download("grad").any()
    opt.free()


def test_fp8_gradients_with_per_tensor_scale_and_skip(gpu, oracle):
    """benchmark configuration 5 at reduced size: device quantisation, in-kernel unscale, NaN skip."""
    rng = np.random.default_rng(55)
    tensors = [(6000, 3), (64, 0), (4096, 3), (8192 + 3, 3), (1, 0), (20000, 3)]
    opt = make(gpu, tensors, grad_type=FP8, beta2=0.95, weight_decay=0.1, grad_clip=1.0,
               skip_nonfinite=True)
    n = opt.n
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    opt.upload("param", p0)
    opt.seed_twins()
    P, M, V = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    twin = oracle.bf16_rne(p0)
    mask = twin_mask(opt)
    from anni_amd.lm_adam import DeviceBuffer
    stage = DeviceBuffer(n * 4)
    for s in range(6):
        g32 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        for i, (off, cnt) in enumerate(zip(opt.offsets, opt.sizes)):
            g32[off:off + cnt] *= 1.0 + i                   # different amax per tensor
        g32 *= np.float32((0.5 if s % 2 else 2.0) / np.linalg.norm(g32.astype(np.float64)))
        if s == 3:
            g32[opt.offsets[3] + 11] = np.nan               # one tensor carries a NaN
        stage.upload(g32)
        q_want = np.empty(n, np.uint8)
        scales = np.empty(len(tensors), np.float32)
        for i, (off, cnt) in enumerate(zip(opt.offsets, opt.sizes)):
            assert gpu.anni_fp8_quantize(opt.o.d_grad + off, opt.o.d_gscale + 4 * i,
                                         stage.ptr + 4 * off, cnt) == 0
            q_want[off:off + cnt], scales[i] = oracle.fp8_quantize(g32[off:off + cnt])
        assert gpu.gpu_stream_sync() == 0
        q = opt.download("grad")
        assert (q == q_want).all()                          # device quantiser == oracle quantiser
        assert same_bits(opt.download("gscale"), scales)
        O = None
        lr = oracle.lr(3e-4, s, 100, 1000, "cosine")
        opt.step_scaled(lr)
        st = opt.sync_stats()
        if O is None:
            O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True,
                              grad_type=oracle.FP8, tensors=oracle_tensors(opt, scales), threads=4)
            O.o.t = s
        qq = q.copy()
        O.step(P, qq, M, V, lr, twin=twin, sumsq_override=None if s == 3 else st.last_sumsq)
        assert st.last_skipped == O.o.last_skipped == (1 if s == 3 else 0)
        if s != 3:
            own = oracle.sumsq(q, oracle.FP8, oracle_tensors(opt, scales))
            assert abs(st.last_sumsq - own) <= 1e-11 * own
            assert st.last_clipped == O.o.last_clipped == (0 if s % 2 else 1)
        assert same_bits(opt.download("param"), P) and same_bits(opt.download("m"), M)
        assert same_bits(opt.download("v"), V)
        assert (opt.download("twin")[mask] == twin[mask]).all()
        assert not opt.download("grad").any()
        assert opt.t == s + 1
    opt.free()


def test_multi_tensor_gradient_quantiser_equals_the_per_tensor_one(gpu, oracle):
    """anni_adam_quantize_grads: the whole float gradient flat into E4M3 codes and per-tensor scales
    in four launches -- identical, code for code and scale for scale, to the oracle's quantiser on
    each tensor (which the per-tensor device quantiser equals): tensors that share tiles, single
    elements, an all-zero tensor, values up to the saturation point, a NaN, and a step after it."""
    from anni_amd.lm_adam import DeviceBuffer
    rng = np.random.default_rng(808)
    tensors = [(6000, 3), (64, 0), (4096, 3), (8192 + 3, 3), (1, 0), (20000, 3), (3, 0),
               (4096 * 5, 3), (777, 1), (2, 0)]
    opt = make(gpu, tensors, grad_type=FP8, beta2=0.95, weight_decay=0.1, grad_clip=1.0,
               skip_nonfinite=True)
    n = opt.n
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    opt.upload("param", p0)
    opt.seed_twins()
    src = DeviceBuffer(n * 4)
    for case in range(3):
        g32 = (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 2, n)).astype(np.float32)
        for i, (off, cnt) in enumerate(zip(opt.offsets, opt.sizes)):
            g32[off:off + cnt] *= np.float32(1.0 + 3 * i)
        o2, c2 = opt.offsets[2], opt.sizes[2]
        g32[o2:o2 + c2] = 0.0                                  # amax 0: scale 1e-12, codes 0
        g32[opt.offsets[6]] = -0.0
        if case == 1:
            g32[opt.offsets[3] + 4100] = np.nan                # the NaN becomes the NaN code
        src.upload(g32)
        assert gpu.anni_adam_quantize_grads(opt.h, src.ptr) == 0
        assert gpu.gpu_stream_sync() == 0
        q = opt.download("grad")
        sc = opt.download("gscale")
        for i, (off, cnt) in enumerate(zip(opt.offsets, opt.sizes)):
            qw, sw = oracle.fp8_quantize(g32[off:off + cnt])
            assert (q[off:off + cnt] == qw).all(), (case, i)
            assert np.float32(sc[i]).view(np.uint32) == np.float32(sw).view(np.uint32), (case, i)
        # and the step takes them: skipped with the NaN, bit for bit otherwise
        P, M, V = opt.download("param"), opt.download("m"), opt.download("v")
        t0 = opt.t
        opt.step_scaled(1e-3)
        st = opt.sync_stats()
        assert st.last_skipped == (1 if case == 1 else 0)
        O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True,
                          grad_type=oracle.FP8, tensors=oracle_tensors(opt, sc), threads=4)
        O.o.t = t0
        O.step(P, q.copy(), M, V, 1e-3, sumsq_override=None if case == 1 else st.last_sumsq)
        assert same_bits(opt.download("param"), P) and same_bits(opt.download("m"), M)
        assert same_bits(opt.download("v"), V)
    # refusals: not an fp8 arena, no source, unaligned source
    assert gpu.anni_adam_quantize_grads(opt.h, None) == -1
    assert gpu.anni_adam_quantize_grads(opt.h, src.ptr + 4) == -1
    other = make(gpu, [(100, 0)])
    assert gpu.anni_adam_quantize_grads(other.h, src.ptr) == -1
    other.free()
    src.free()
    opt.free()


@pytest.mark.parametrize("gt,mt", [(F32, BF16), (BF16, BF16), (FP8, F32)])
def test_moment_overflow_follows_the_host_loop(gpu, oracle, gt, mt):
    """A gradient so large that v overflows to infinity in float: the host loop then divides by
    infinity and leaves p where it was (lm_adam.c:590-593), and so must the narrow storage modes,
    whose division by the step constants is a reciprocal multiply with a residual (inf - inf)."""
    n = 4096 * 3 + 5
    rng = np.random.default_rng(5)
    opt = make(gpu, [(n, 3)], grad_type=gt, moment_type=mt, beta2=0.95, weight_decay=0.1)
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    opt.upload("param", p0)
    g32 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    big = rng.choice(n, 200, replace=False)
    g32[big] = np.float32(1e20) * np.sign(g32[big])
    segs = [(0, n, 1, 1.0)]
    if gt == F32:
        g_dev, g_or = g32, g32.copy()
    elif gt == BF16:
        g_dev = oracle.bf16_rne(g32)
        g_or = g_dev.copy()
    else:
        g_dev, sc = oracle.fp8_quantize(g32)
        g_or = g_dev.copy()
        opt.upload("gscale", np.array([sc], np.float32))
        segs = [(0, n, 1, float(sc))]
    opt.upload("grad", g_dev)
    P = p0.copy()
    M = np.zeros(n, np.float32 if mt == F32 else np.uint16)
    V = np.zeros(n, np.float32 if mt == F32 else np.uint16)
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_type=gt, moment_type=mt, tensors=segs)
    for step in range(2):
        if step:
            opt.upload("grad", g_dev)
            g_or = g_dev.copy()
        opt.step_scaled(1e-3)
        O.step(P, g_or, M, V, 1e-3)
        got_v = opt.download("v")
        vf = oracle.bf16_widen(got_v) if mt == BF16 else got_v
        assert np.isinf(vf[big]).all()                           # the case is what it claims to be
        assert same_bits(opt.download("param"), P), (gt, mt, step)
        assert (opt.download("m").view(M.dtype) == M).all() and (got_v.view(V.dtype) == V).all()
    assert np.isfinite(opt.download("param")).all()
    opt.free()


def test_fp8_decode_all_codes_on_device(gpu, oracle):
    """Every E4M3 byte through the kernel's decoder: with m = v = 0 and t = 1, m = (1-b1) * g."""
    opt = make(gpu, [(256, 0)], grad_type=FP8, beta1=0.5, beta2=0.5)
    q = np.arange(256, dtype=np.uint8)
    opt.upload("grad", q)
    opt.upload("gscale", np.array([0.25], np.float32))
    opt.step_scaled(1e-3)
    m = opt.download("m")
    want = 0.5 * 0.0 + (oracle.fp8_decode_table() * np.float32(0.25)).astype(np.float64) * 0.5
    nan = np.isnan(want)
    assert (np.isnan(m) == nan).all() and nan.sum() == 2
    assert same_bits(m[~nan], want[~nan].astype(np.float32)), np.flatnonzero(
        m[~nan].view(np.uint32) != want[~nan].astype(np.float32).view(np.uint32))
    opt.free()


def test_device_normal_generator_and_bf16_convert(gpu, oracle):
    from anni_amd.lm_adam import DeviceBuffer
    n = 1 << 20
    a = DeviceBuffer(n * 4)
    b = DeviceBuffer(n * 4)
    assert gpu.anni_fill_normal_f32(a.ptr, n, 7, 3, 0.0, 1e-3) == 0
    assert gpu.anni_fill_normal_f32(b.ptr, n, 7, 3, 0.0, 1e-3) == 0
    x, y = a.download(np.float32, n), b.download(np.float32, n)
    assert same_bits(x, y) and np.isfinite(x).all()
    assert abs(x.mean()) < 5e-6 and abs(x.std() - 1e-3) < 1e-5
    assert gpu.anni_fill_normal_f32(b.ptr, n, 7, 4, 0.0, 1e-3) == 0
    assert not same_bits(x, b.download(np.float32, n))
    h = DeviceBuffer(n * 2)
    assert gpu.anni_f32_to_bf16(h.ptr, a.ptr, n) == 0
    assert (h.download(np.uint16, n) == oracle.bf16_rne(x)).all()


def test_steps_back_to_back_equal_steps_with_a_sync_between(gpu):
    """Eight steps queued in one go (sum of squares, second stage in its last workgroup, update,
    again and again with nothing in between) against the same eight steps with a host
    synchronisation after each: a second stage that read a partial too early, or one left from the
    step before, would change the clip scale and with it every element."""
    import ctypes as C
    tensors = [(4096 * 1500 + 7, 3), (1536, 0), (4096 * 700, 3), (3, 1)]
    rng = np.random.default_rng(31)
    steps = 8
    runs = []
    p0 = grads = None
    for mode in ("queued", "synced"):
        opt = make(gpu, tensors, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True,
                   grad_slots=steps)
        n = opt.n
        if p0 is None:
            p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
            # norms 0.3 .. 2.4 around the clip at 1.0
            grads = [(rng.standard_normal(n) * ((0.3 + 0.3 * k) / np.sqrt(n))).astype(np.float32)
                     for k in range(steps)]
        opt.upload("param", p0)
        opt.seed_twins()
        slots = [opt.grad_slot(k) for k in range(steps)]
        for k in range(steps):
            assert gpu.gpu_memcpy_h2d(slots[k], grads[k].ctypes.data, grads[k].nbytes) == 0
        assert gpu.gpu_stream_sync() == 0
        lrs = [1e-3 * (k + 1) for k in range(steps)]
        if mode == "queued":
            ms = C.c_float(0)
            assert gpu.anni_adam_time_steps(opt.h, steps, (C.c_void_p * steps)(*slots), steps,
                                            (C.c_double * steps)(*lrs),
                                            (C.c_double * steps)(*[1.0] * steps), C.byref(ms),
                                            None, None) == 0
        else:
            for k in range(steps):
                opt.bind_grad(slots[k])
                opt.step_scaled(lrs[k])
                st = opt.sync_stats()
                assert st.last_clipped == (1 if 0.3 + 0.3 * k > 1.0 else 0), k
        st = opt.sync_stats()
        runs.append((opt.download("param"), opt.download("m"), opt.download("v"),
                     opt.download("twin"), st.last_sumsq, opt.t))
        opt.free()
    a, b = runs
    assert a[4] == b[4] and a[5] == b[5] == steps
    for x, y in zip(a[:4], b[:4]):
        assert same_bits(x, y)


def test_two_optimizers_side_by_side(gpu, oracle):
    """Two arenas with different storage modes stepping in turn share the stream and the
    library's state and do not disturb each other."""
    rng = np.random.default_rng(77)
    a = make(gpu, RAGGED, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True)
    b = make(gpu, [(9000, 3), (17, 0)], grad_type=BF16, moment_type=BF16, beta2=0.99,
             weight_decay=0.01, grad_clip=0.5)
    st = {}
    for opt, name in ((a, "a"), (b, "b")):
        n = opt.n
        p = (rng.standard_normal(n) * 0.02).astype(np.float32)
        opt.upload("param", p)
        opt.seed_twins()
        bf = name == "b"
        st[name] = dict(P=p.copy(), M=np.zeros(n, np.uint16 if bf else np.float32),
                        V=np.zeros(n, np.uint16 if bf else np.float32),
                        O=oracle.Oracle(n, beta2=0.99 if bf else 0.95,
                                        weight_decay=0.01 if bf else 0.1,
                                        grad_clip=0.5 if bf else 1.0, skip_nonfinite=not bf,
                                        grad_type=oracle.BF16 if bf else oracle.F32,
                                        moment_type=oracle.BF16 if bf else oracle.F32,
                                        tensors=oracle_tensors(opt), threads=2))
    for s in range(4):
        grads = {}
        for opt, name in ((a, "a"), (b, "b")):
            g = (rng.standard_normal(opt.n) * (3e-2 if s % 2 else 1e-4)).astype(np.float32)
            grads[name] = oracle.bf16_rne(g) if name == "b" else g
            opt.upload("grad", grads[name])
        assert a.step_scaled(1e-3) == 0 and b.step_scaled(2e-3) == 0       # both queued, then read
        for opt, name, lr in ((a, "a", 1e-3), (b, "b", 2e-3)):
            stats = opt.sync_stats()
            S = st[name]
            S["O"].step(S["P"], grads[name].copy(), S["M"], S["V"], lr,
                        sumsq_override=stats.last_sumsq)
            assert stats.last_clipped == S["O"].o.last_clipped == s % 2
            assert same_bits(opt.download("param"), S["P"]), (name, s)
            assert (opt.download("m") == S["M"]).all() and (opt.download("v") == S["V"]).all()
    a.free()
    b.free()


def test_fp8_quantizer_on_every_rounding_boundary(gpu, oracle):
    """The device quantiser against the oracle's (pinned to torch's float8_e4m3fn cast) on a tensor
    whose amax is exactly 448, so the scale is 1 and the bytes are the plain encoding of the
    inputs: for every binade of the format, both signs and every half step of its 3-bit mantissa,
    the tie itself and its two float neighbours; the subnormal grid; 448 and just below; signed
    zeros; float denormals; and two million random values."""
    from anni_amd.lm_adam import DeviceBuffer
    vals = [448.0, 0.0, -0.0, 1e-45, -1e-45, 1e-39, 2.0 ** -10, 2.0 ** -9, 3 * 2.0 ** -10,
            447.99997, 432.0, 464.0 - 32.0, 2.0 ** -6, 2.0 ** -7, 0.0146484375]
    for e in range(-12, 9):
        for k in range(0, 32):                         # 1.k/16 * 2^e: grid points and ties
            c = np.float32((1.0 + k / 16.0) * 2.0 ** e)
            if c > 448:
                continue
            for v in (c, np.nextafter(c, np.float32(0)), np.nextafter(c, np.float32(1e9))):
                if v <= 448:
                    vals += [float(v), -float(v)]
    rng = np.random.default_rng(123)
    rnd = (rng.standard_normal(2000000) * 10.0 ** rng.integers(-6, 3, 2000000)).astype(np.float32)
    x = np.concatenate([np.array(vals, np.float32), np.clip(rnd, -448, 448)])
    assert np.abs(x).max() == 448.0
    src, q, sc = DeviceBuffer(x.nbytes), DeviceBuffer(x.size), DeviceBuffer(4)
    src.upload(x)
    assert gpu.anni_fp8_quantize(q.ptr, sc.ptr, src.ptr, x.size) == 0
    assert gpu.gpu_stream_sync() == 0
    want, scale = oracle.fp8_quantize(x)
    assert scale == 1.0 and sc.download(np.float32, 1)[0] == 1.0
    got = q.download(np.uint8, x.size)
    bad = np.flatnonzero(got != want)
    assert bad.size == 0, [(float(x[i]), int(got[i]), int(want[i])) for i in bad[:8]]
    # non-finite inputs: the amax is then taken as 1e-8 (scale 1e-8/448), NaN stays NaN, infinities saturate
    y = np.array([np.nan, -np.nan, np.inf, -np.inf, 1e-9, -3e-9, 0.0], np.float32)
    src.upload(y)
    assert gpu.anni_fp8_quantize(q.ptr, sc.ptr, src.ptr, y.size) == 0
    assert gpu.gpu_stream_sync() == 0
    want, scale = oracle.fp8_quantize(y)
    assert (q.download(np.uint8, y.size) == want).all() and sc.download(np.float32, 1)[0] == scale


def test_bf16_conversion_on_all_float_patterns(gpu, oracle):
    """The twins and bf16 moments are rounded by the gfx950 conversion instruction: all 2^32 float
    bit patterns (every NaN, denormal and tie among them) give the bits of the oracle's
    round-to-nearest-even routine, which is pinned against torch's bfloat16 cast."""
    from anni_amd.lm_adam import DeviceBuffer
    ch = 1 << 28
    src, dst = DeviceBuffer(ch * 4), DeviceBuffer(ch * 2)
    for c in range(16):
        bits = np.arange(c * ch, (c + 1) * ch, dtype=np.uint64).astype(np.uint32)
        x = bits.view(np.float32)
        src.upload(x)
        assert gpu.anni_f32_to_bf16(dst.ptr, src.ptr, ch) == 0
        got = dst.download(np.uint16, ch)
        bad = np.flatnonzero(got != oracle.bf16_rne(x))
        assert bad.size == 0, [(hex(int(bits[i])), hex(int(got[i]))) for i in bad[:4]]
    src.free()
    dst.free()


@pytest.mark.parametrize("mode", ["f32", "bf16"])
def test_moments_offloaded_between_steps(gpu, oracle, mode):
    """anni_adam_set_offload (lm_adam_set_offload, lang/lm_adam.c:211-214,295-334): after every step
    m and v leave the device for page-locked host memory and their blocks are given back, the next
    step brings them back first.  Same bits as the oracle at every step; the moments really are
    gone in between (NULL pointers, and device memory in use reads the same after every step);
    the checkpoint calls still see them; switching it off brings them back for good."""
    import ctypes as C
    narrow = 1 if mode == "bf16" else 0
    tensors = [(80 * 1000 * 1000, 3), (4097, 0), (12288, 3), (3, 1)]      # flats of 160 - 320 MB: pooled blocks
    opt = make(gpu, tensors, grad_type=0, moment_type=narrow, beta2=0.95, weight_decay=0.1,
               grad_clip=1.0, skip_nonfinite=True)
    n = opt.n
    rng = np.random.default_rng(11)
    P = (rng.standard_normal(n) * 0.02).astype(np.float32)
    opt.upload("param", P)
    opt.seed_twins()
    mt = oracle.BF16 if narrow else oracle.F32
    M, V = (np.zeros(n, np.uint16), np.zeros(n, np.uint16)) if narrow else \
        (np.zeros(n, np.float32), np.zeros(n, np.float32))
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True,
                      moment_type=mt, tensors=oracle_tensors(opt), threads=8)
    unit = 1.0 / (np.sqrt(n) * 1e-3)

    def one_step(s):
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        opt.upload("grad", g)
        gs = unit * (1.7 if s % 2 else 0.6)
        assert opt.step_scaled(1e-3, gs) == 0
        st = opt.sync_stats()
        O.step(P, g, M, V, 1e-3, gs, sumsq_override=st.last_sumsq)
        assert st.last_clipped == s % 2
        assert same_bits(opt.download("param"), P), s
        assert (opt.download("twin")[twin_mask(opt)] == oracle.bf16_rne(P)[twin_mask(opt)]).all()

    one_step(0)                                              # a step before the switch: m, v non-zero
    old = (opt.o.d_param, opt.o.d_m)
    assert gpu.anni_adam_mv_on_device(opt.h) == 1
    assert gpu.anni_adam_set_offload(opt.h, 1) == 0, gpu.gpu_debug_last_error()
    assert gpu.anni_adam_mv_on_device(opt.h) == 0 and not opt.o.d_m and not opt.o.d_v
    assert opt.o.d_param and opt.o.d_param != old[0]         # the arena was re-housed without m and v
    fr0, tt = C.c_size_t(0), C.c_size_t(0)
    assert gpu.gpu_mem_info(C.byref(fr0), C.byref(tt)) == 0
    for s in range(1, 4):
        one_step(s)
        assert gpu.anni_adam_mv_on_device(opt.h) == 0
        fr = C.c_size_t(0)
        assert gpu.gpu_mem_info(C.byref(fr), C.byref(tt)) == 0
        assert fr.value == fr0.value, "device memory in use moved between steps"
    pairs = opt.export_mv(0, 5000)                           # brings them back, sends them away again
    wide = (lambda a: oracle.bf16_widen(a)) if narrow else (lambda a: a)
    assert same_bits(pairs[:, 0].copy(), wide(M[:5000])) and same_bits(pairs[:, 1].copy(), wide(V[:5000]))
    assert gpu.anni_adam_mv_on_device(opt.h) == 0
    assert gpu.anni_adam_set_offload(opt.h, 0) == 0
    assert gpu.anni_adam_mv_on_device(opt.h) == 1 and opt.o.d_m and opt.o.d_v
    got_m, got_v = opt.download("m"), opt.download("v")
    assert (got_m.view(M.dtype) == M).all() if narrow else same_bits(got_m, M)
    assert (got_v.view(V.dtype) == V).all() if narrow else same_bits(got_v, V)
    one_step(4)                                              # and on it goes, moments resident again
    assert gpu.anni_adam_mv_on_device(opt.h) == 1
    opt.free()


def test_sum_of_squares_self_check_runs_once_and_agrees(gpu, oracle):
    """The first sum of squares with a second stage compares its atomic hand-over of the partials
    with the fenced one on the caller's own gradients (two extra launches, one wait); so does the
    first one after the switches were read again.  The two never disagree here, and the fenced
    form selected by hand gives the same bits as the default."""
    import ctypes as C
    import os
    runs0, bad0 = C.c_int(0), C.c_int(0)
    opt = make(gpu, [(4096 * 2300 + 77, 3), (513, 0)], beta2=0.95, grad_clip=1.0, skip_nonfinite=True)
    n = opt.n
    rng = np.random.default_rng(12)
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    opt.upload("grad", g)
    assert opt.step_scaled(1e-3) == 0
    st = opt.sync_stats()
    want = st.last_sumsq
    assert gpu.anni_fold_guard_stats(C.byref(runs0), C.byref(bad0)) == 0
    assert runs0.value >= 1 and bad0.value == 0
    opt.upload("grad", g)
    assert opt.step_scaled(1e-3) == 0                       # no second check
    runs1, bad1 = C.c_int(0), C.c_int(0)
    gpu.anni_fold_guard_stats(C.byref(runs1), C.byref(bad1))
    assert runs1.value == runs0.value and opt.sync_stats().last_sumsq == want
    try:
        os.environ["ANNI_FOLD"] = "fence"
        gpu.anni_gpu_reload_switches()
        opt.upload("grad", g)
        assert opt.step_scaled(1e-3) == 0
        assert opt.sync_stats().last_sumsq == want          # the fenced form, same bits
        gpu.anni_fold_guard_stats(C.byref(runs1), C.byref(bad1))
        assert runs1.value == runs0.value                   # nothing to check it against
    finally:
        os.environ.pop("ANNI_FOLD", None)
        gpu.anni_gpu_reload_switches()
    opt.upload("grad", g)
    assert opt.step_scaled(1e-3) == 0                       # read again: checked again
    gpu.anni_fold_guard_stats(C.byref(runs1), C.byref(bad1))
    assert runs1.value == runs0.value + 1 and bad1.value == 0
    assert opt.sync_stats().last_sumsq == want
    assert abs(want - oracle.sumsq(g, threads=4)) <= 1e-10 * want
    opt.free()


def test_gnorm_every_alone_computes_and_prints_the_norm(gpu):
    """lm_adam.c:466,484-487: with ANN_GNORM_EVERY=N the norm is computed and printed every N steps
    also when nothing clips and nothing skips (the switch is read once per process: a child)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    child = (
        "import sys; sys.path.insert(0, %r)\n"
        "import numpy as np\n"
        "from anni_amd.lm_adam import LmAdam\n"
        "opt = LmAdam([(5000, 3), (77, 0)])\n"
        "for s in range(4):\n"
        "    opt.upload('grad', np.full(opt.n, 0.5, np.float32))\n"
        "    opt.step_scaled(1e-3)\n"
        "    st = opt.sync_stats()\n"
        "    print('NORM %%d %%r %%d' %% (opt.t, st.last_grad_norm, st.last_clipped))\n"
    ) % root
    env = dict(os.environ, ANN_GNORM_EVERY="2")
    r = subprocess.run([sys.executable, "-c", child], env=env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-1500:]
    want = float(np.sqrt(5077 * 0.25))
    norms = [ln.split() for ln in r.stdout.splitlines() if ln.startswith("NORM ")]
    assert len(norms) == 4 and all(abs(float(x[2]) - want) < 1e-9 * want and x[3] == "0" for x in norms)
    said = [ln for ln in r.stderr.splitlines() if ln.startswith("[adam] step ")]
    assert said == ["[adam] step 2 grad norm %.4g" % want, "[adam] step 4 grad norm %.4g" % want], r.stderr


def test_op_prof_times_the_arena_steps_launches(gpu):
    """ANN_OP_PROF=1 (num/gpu_cuda.cu:3205-3409, lang/lm_adam.c:541): every launch of the optimizer
    step is bracketed by an event pair and the table is printed after each step, on the arena path as
    on the flat entry points (the switch is read once per process: a child)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    child = (
        "import sys; sys.path.insert(0, %r)\n"
        "import numpy as np\n"
        "from anni_amd.lm_adam import LmAdam\n"
        "opt = LmAdam([(300000, 3), (77, 0)], grad_clip=1.0)\n"
        "for s in range(3):\n"
        "    opt.upload('grad', np.full(opt.n, 0.5, np.float32))\n"
        "    opt.step_scaled(1e-3)\n"
        "    opt.sync_stats()\n"
    ) % root
    env = dict(os.environ, ANN_OP_PROF="1")
    r = subprocess.run([sys.executable, "-c", child], env=env, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-1500:]
    rows = [ln.split() for ln in r.stderr.splitlines() if ln.startswith("[op-prof] ")]
    per = {}
    for w in rows:                                        # [op-prof] name ms "ms" calls "calls"
        per.setdefault(w[1], []).append((float(w[2]), int(w[4])))
    assert set(per) == {"grad_sumsq", "adam_step"}, r.stderr
    for name, got in per.items():
        assert sum(c for _ms, c in got) == 3, (name, got)
        assert all(0.0 < ms < 50.0 for ms, _c in got), (name, got)


@pytest.mark.parametrize("seed,mode", [(1, "f32"), (2, "bf16"), (3, "f32"), (4, "bf16"), (5, "f32"), (6, "bf16")])
def test_random_sequences_of_arena_calls_against_the_oracle(gpu, oracle, seed, mode):
    """The arena's entry points in an order nobody wrote by hand: steps (clipped and not, with a NaN
    now and then), the moments sent to the host and brought back, gradient slots switched, the
    gradients cleared, slices of the optimizer block exported and imported -- against the oracle,
    bit for bit under the device's sum, after every call that changes state."""
    narrow = mode == "bf16"
    rng = np.random.default_rng(7000 + seed)
    tensors = [(4096 * 70 + 13, 3), (333, 0), (4096 * 20, 3), (1, 1), (50000, 2), (4096 * 45 + 4000, 3), (77, 0)]
    opt = make(gpu, tensors, grad_type=0, moment_type=1 if narrow else 0, grad_slots=2, beta2=0.95,
               weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True)
    n = opt.n
    P = (rng.standard_normal(n) * 0.02).astype(np.float32)
    opt.upload("param", P)
    opt.seed_twins()
    TW = oracle.bf16_rne(P)
    M = np.zeros(n, np.uint16 if narrow else np.float32)
    V = np.zeros(n, np.uint16 if narrow else np.float32)
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True,
                      moment_type=oracle.BF16 if narrow else oracle.F32, tensors=oracle_tensors(opt), threads=8)
    wide = (lambda a: oracle.bf16_widen(a)) if narrow else (lambda a: a)
    mask = twin_mask(opt)
    unit = 1.0 / (np.sqrt(n) * 1e-3)
    parked = [False]
    slot = [0]
    G = [np.zeros(n, np.float32), np.zeros(n, np.float32)]     # what each gradient slot holds

    def check_state():
        assert same_bits(opt.download("param"), P)
        assert (opt.download("twin")[mask] == TW[mask]).all()
        assert same_bits(opt.download("grad"), G[slot[0]])
        if parked[0]:
            assert gpu.anni_adam_mv_on_device(opt.h) == 0
            first = int(rng.integers(0, n - 3000))
            pairs = opt.export_mv(first, 3000)
            assert same_bits(pairs[:, 0].copy(), wide(M[first:first + 3000]))
            assert same_bits(pairs[:, 1].copy(), wide(V[first:first + 3000]))
        else:
            gm, gv = opt.download("m"), opt.download("v")
            assert (gm.view(M.dtype) == M).all() and (gv.view(V.dtype) == V).all()

    def step(kind):
        g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
        if kind == "nan":
            g[int(rng.integers(0, n))] = np.nan
        if kind != "cleared":
            opt.upload("grad", g)
            G[slot[0]][:] = g
        gs = unit * (1.7 if rng.random() < 0.5 else 0.6)
        lr = 1e-3 * float(rng.random() + 0.1)
        assert opt.step_scaled(lr, gs) == 0
        st = opt.sync_stats()
        assert st.last_skipped == (1 if kind == "nan" else 0)
        O.step(P, G[slot[0]], M, V, lr, gs, twin=TW, sumsq_override=st.last_sumsq)
    for _ in range(40):
        k = int(rng.integers(0, 10))
        if k <= 3:
            step("plain")
        elif k == 4:
            step("nan")
        elif k == 5:
            parked[0] = not parked[0]
            assert gpu.anni_adam_set_offload(opt.h, 1 if parked[0] else 0) == 0, gpu.gpu_debug_last_error()
        elif k == 6:
            slot[0] ^= 1
            opt.bind_grad(opt.grad_slot(slot[0]))
        elif k == 7:
            assert opt.zero_grad() in (0, None)
            G[slot[0]][:] = 0.0
            step("cleared")
        elif k == 8:
            first, cnt = int(rng.integers(0, n - 5000)), int(rng.integers(1, 5000))
            pairs = (rng.standard_normal((cnt, 2)) * 1e-4).astype(np.float32)
            pairs[:, 1] = np.abs(pairs[:, 1])
            opt.import_mv(pairs, first)
            M[first:first + cnt] = oracle.bf16_rne(pairs[:, 0].copy()) if narrow else pairs[:, 0]
            V[first:first + cnt] = oracle.bf16_rne(pairs[:, 1].copy()) if narrow else pairs[:, 1]
        else:
            first, cnt = int(rng.integers(0, n - 5000)), int(rng.integers(1, 5000))
            pairs = opt.export_mv(first, cnt)
            assert same_bits(pairs[:, 0].copy(), wide(M[first:first + cnt]))
            assert same_bits(pairs[:, 1].copy(), wide(V[first:first + cnt]))
        check_state()
    opt.free()
