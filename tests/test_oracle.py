"""The CPU oracle pinned: against the reference's compiled optimizer, the golden vectors it
wrote, the reference's own known answers, closed forms and independent codecs.  CPU only."""
import math

import numpy as np
import pytest

from helpers import GOLDEN_CASES, load_golden, same_bits, bits


# ---- against the reference's own compiled code (present only in the build container) ----

@pytest.mark.parametrize("wd,clip,gs,gmul", [
    (0.0, 0.0, 1.0, 1.0), (0.1, 0.0, 1.0, 1.0), (0.1, 1.0, 1.0, 5.0),
    (0.1, 1.0, 0.37, 0.5), (0.1, 1.0, 1 / 252.0, 300.0), (0.0, 0.5, 2.0, 9.0)])
def test_oracle_equals_compiled_reference(oracle, wd, clip, gs, gmul):
    if not oracle.ref_available():
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(int(1000 * (wd + clip + gs + gmul)))
    n = 40009
    p = (rng.standard_normal(n) * 0.02).astype(np.float32)
    p2 = p.copy()
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    g = np.empty(n, np.float32)
    g2 = np.empty(n, np.float32)
    R = oracle.RefAdam(p2, g2, beta2=0.95, weight_decay=wd, grad_clip=clip)
    O = oracle.Oracle(n, beta2=0.95, weight_decay=wd, grad_clip=clip)
    for t in range(1, 11):
        gg = (rng.standard_normal(n) * 1e-3 * gmul * (1 + t % 3)).astype(np.float32)
        g[:] = gg
        g2[:] = gg
        lr = oracle.lr(3e-4, t - 1, 100, 1000, "cosine")
        assert lr == oracle.ref_lr(3e-4, t - 1, 100, 1000, "cosine")
        assert O.step(p, g, m, v, lr, gs) == 0
        assert R.step(lr, gs) == t == O.t
        rm, rv = R.moments()
        assert same_bits(p, p2) and same_bits(m, rm) and same_bits(v, rv)
        assert not g.any() and not g2.any()
    R.close()


def test_oracle_lr_nonpositive_is_a_noop(oracle):
    n = 16
    p = np.ones(n, np.float32)
    g = np.ones(n, np.float32)
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    O = oracle.Oracle(n)
    assert O.step(p, g, m, v, 0.0) == 1 and O.t == 0      # lm_adam.c:531-532
    assert O.step(p, g, m, v, -1.0) == 1 and O.t == 0
    assert g.all() and (p == 1).all()
    if oracle.ref_available():
        R = oracle.RefAdam(p.copy(), g.copy())
        assert R.step(0.0) == 0
        R.close()


# ---- against the committed golden vectors (written by the compiled reference) ----

@pytest.mark.parametrize("name", GOLDEN_CASES)
@pytest.mark.parametrize("threads", [1, 3])
def test_oracle_matches_golden(oracle, name, threads):
    G = load_golden(name)
    n = G["p0"].size
    p = G["p0"].copy()
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    O = oracle.Oracle(n, beta1=float(G["beta1"]), beta2=float(G["beta2"]), eps=float(G["eps"]),
                      weight_decay=float(G["wd"]), grad_clip=float(G["clip"]), threads=threads)
    for s in range(G["grads"].shape[0]):
        g = G["grads"][s].copy()
        O.step(p, g, m, v, float(G["lr"][s]), float(G["grad_scale"]))
        assert same_bits(p, G["p"][s]), (name, s)
        assert same_bits(m, G["m"][s]) and same_bits(v, G["v"][s])
        assert not g.any()


@pytest.mark.parametrize("simd", ["avx2", "avx512"])
def test_vectorised_build_is_bit_identical(oracle, simd):
    """The -O3 auto-vectorised build of the same source (CPU timing leg) vs the reference-flags build."""
    if simd == "avx512" and oracle.cpu_simd() != "avx512":
        pytest.skip("CPU without AVX-512")
    if simd == "avx2" and oracle.cpu_simd() == "none":
        pytest.skip("CPU without AVX2")
    rng = np.random.default_rng(17)
    n = 300007
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    A = dict(p=p0.copy(), m=np.zeros(n, np.float32), v=np.zeros(n, np.float32))
    B = dict(p=p0.copy(), m=np.zeros(n, np.float32), v=np.zeros(n, np.float32))
    OA = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    OB = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, threads=4, simd=simd)
    for s in range(5):
        g = (rng.standard_normal(n) * 1e-3 * (1 + 3 * (s % 2))).astype(np.float32)
        ga, gb = g.copy(), g.copy()
        OA.step(A["p"], ga, A["m"], A["v"], 3e-4)
        OB.step(B["p"], gb, B["m"], B["v"], 3e-4)
        assert OA.o.last_sumsq == OB.o.last_sumsq        # serial norm in both
        for k in "pmv":
            assert same_bits(A[k], B[k]), (simd, s, k)


def test_golden_lr_table(oracle):
    T = np.load(__import__("os").path.join(__import__("helpers").GOLDEN, "lr_table.npz"))
    for row, case in zip(T["lr"], T["cases"]):
        w, d, k, frm = str(case).split(",")
        for s, want in zip(T["steps"], row):
            assert oracle.lr(3e-4, int(s), int(w), int(d), k, int(frm)) == want


# ---- the reference's own known answers ----

def test_lr_known_answers_of_the_reference_test(oracle):
    """tests/test_ann.c:866-879 (test_lr_sched_from)."""
    lr = oracle.lr
    assert abs(lr(1.0, 29000, 100, 1000, "cosine", 0) - 0.0) < 1e-12
    assert abs(lr(1.0, 29000, 100, 1000, "cosine", 29000) - 0.01) < 1e-12
    assert abs(lr(1.0, 29099, 100, 1000, "cosine", 29000) - 1.0) < 1e-12
    assert abs(lr(1.0, 29600, 100, 1000, "cosine", 29000) - 0.5) < 1e-12
    assert abs(lr(1.0, 31000, 100, 1000, "cosine", 29000) - 0.0) < 1e-12
    assert abs(lr(1.0, 10, 100, 1000, "cosine", 29000) - 0.01) < 1e-12
    assert lr(0.25, 12345, 0, 0, "none", 0) == 0.25


def test_lr_warmup_is_lr_times_t_over_warmup(oracle):
    # optimizer steps t = 1..10 use schedule steps 0..9 (lm_train.c:1336 passes t before t++)
    for t in range(1, 11):
        assert oracle.lr(3e-4, t - 1, 100, 1000, "cosine") == 3e-4 * float(t) / 100.0


# ---- closed forms ----

def test_first_step_closed_form(oracle):
    """t=1, m=v=0: m=(1-b1)g, v=(1-b2)g^2, mhat=g, vhat=g^2 -> dp = -lr*g/(|g|+eps), then decay."""
    rng = np.random.default_rng(5)
    n = 5000
    g0 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    for wd in (0.0, 0.1):
        p, g = p0.copy(), g0.copy()
        m = np.zeros(n, np.float32)
        v = np.zeros(n, np.float32)
        O = oracle.Oracle(n, beta2=0.95, weight_decay=wd)
        O.step(p, g, m, v, 3e-4)
        gd = g0.astype(np.float64)
        want = p0.astype(np.float64) - 3e-4 * gd / (np.abs(gd) + 1e-8)
        want = want * (1.0 - 3e-4 * wd)
        # m, v round to float first, so mhat/vhat differ from g, g^2 by float rounding only
        # two float roundings of p (step, decay) plus the float rounding of m and v
        assert np.all(np.abs(p - want) <= 1.5 * np.spacing(np.abs(p)) + 3e-4 * 1e-6)
        assert np.allclose(m, 0.1 * gd, rtol=1e-6, atol=0)
        assert np.allclose(v, 0.05 * gd * gd, rtol=1e-6, atol=1e-45)
        # worked example of docs/adam-lm-weights.md:107-111 (w=0.01, g=0.1, defaults): |dw| = lr
    p = np.array([0.01], np.float32)
    g = np.array([0.1], np.float32)
    m = np.zeros(1, np.float32)
    v = np.zeros(1, np.float32)
    oracle.Oracle(1).step(p, g, m, v, 1e-3)
    assert abs((0.01 - float(p[0])) - 1e-3) < 1e-8


def test_zero_gradient_is_pure_decay(oracle):
    n = 64
    p0 = np.linspace(-1, 1, n).astype(np.float32)
    p = p0.copy()
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    O = oracle.Oracle(n, weight_decay=0.1)
    for _ in range(5):
        g = np.zeros(n, np.float32)
        O.step(p, g, m, v, 1e-2)
    want = p0.astype(np.float64) * (1 - 1e-2 * 0.1) ** 5
    assert np.allclose(p, want, rtol=5e-7, atol=0)
    assert not m.any() and not v.any()


def test_constant_gradient_emas(oracle):
    n = 8
    c = 0.25
    p = np.zeros(n, np.float32)
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    O = oracle.Oracle(n, beta1=0.9, beta2=0.95)
    for k in range(1, 8):
        g = np.full(n, c, np.float32)
        O.step(p, g, m, v, 1e-3)
        assert np.allclose(m, c * (1 - 0.9 ** k), rtol=1e-6)
        assert np.allclose(v, c * c * (1 - 0.95 ** k), rtol=1e-6)
    # mhat = c, vhat = c^2 at every step: p moves by lr*c/(c+eps) each time
    assert np.allclose(p, -7 * 1e-3 * c / (c + 1e-8), rtol=1e-5)


def test_decay_only_where_flagged(oracle):
    n = 100
    p = np.ones(n, np.float32)
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    g = np.zeros(n, np.float32)
    O = oracle.Oracle(n, weight_decay=0.5, tensors=[(0, 60, 1, 1.0), (60, 40, 0, 1.0)])
    O.step(p, g, m, v, 0.1)
    assert np.allclose(p[:60], 0.95) and (p[60:] == 1.0).all()


def test_clip_invariant(oracle):
    rng = np.random.default_rng(9)
    n = 30000
    g0 = rng.standard_normal(n).astype(np.float32)
    for gs, should_clip in ((1.0, True), (1e-4, False)):
        p = np.zeros(n, np.float32)
        m = np.zeros(n, np.float32)
        v = np.zeros(n, np.float32)
        g = g0.copy()
        O = oracle.Oracle(n, grad_clip=1.0)
        O.step(p, g, m, v, 1e-3, gs)
        norm = math.sqrt(math.fsum((float(x) * gs) ** 2 for x in g0))
        assert abs(O.o.last_grad_norm - norm) <= 1e-12 * norm
        assert bool(O.o.last_clipped) == should_clip
        eff = O.o.last_grad_scale
        if should_clip:
            assert abs(norm / gs * eff - 1.0) < 1e-9     # ||g * eff|| == clip
        else:
            assert eff == gs
        # m after one step is (1-b1) * g * eff
        assert np.allclose(m, 0.1 * g0.astype(np.float64) * eff, rtol=1e-6, atol=1e-45)


def test_sumsq_against_exact_sum(oracle):
    rng = np.random.default_rng(3)
    g = (rng.standard_normal(20011) * 3).astype(np.float32)
    exact = math.fsum(float(x) * float(x) for x in g)
    for threads in (1, 4):
        got = oracle.sumsq(g, threads=threads)
        assert abs(got - exact) <= 1e-12 * exact
    s = 0.0
    for x in g:                      # the reference's order: one running double
        s += float(x) * float(x)
    assert oracle.sumsq(g, threads=1) == s


def test_nonfinite_skip_keeps_state(oracle):
    rng = np.random.default_rng(4)
    n = 1000
    p = rng.standard_normal(n).astype(np.float32)
    m = rng.standard_normal(n).astype(np.float32)
    v = np.abs(rng.standard_normal(n)).astype(np.float32)
    for bad in (np.nan, np.inf, -np.inf):
        g = rng.standard_normal(n).astype(np.float32)
        g[n // 2] = bad
        p2, m2, v2 = p.copy(), m.copy(), v.copy()
        O = oracle.Oracle(n, grad_clip=1.0, skip_nonfinite=True)
        assert O.step(p2, g, m2, v2, 1e-3) == 0
        assert O.o.last_skipped == 1 and O.t == 1          # t still advances (lm_adam.c:533)
        assert same_bits(p, p2) and same_bits(m, m2) and same_bits(v, v2)
        assert not g.any()


# ---- codecs against independent implementations ----

def test_bf16_rne_against_torch(oracle):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(8)
    x = np.concatenate([
        (rng.standard_normal(200000) * 0.02).astype(np.float32),
        np.array([0.0, -0.0, 1.0, -1.0, 3.4e38, -3.4e38, 1e-40, -1e-40, np.inf, -np.inf],
                 np.float32),
        # exact ties: mantissa low half = 0x8000 with even / odd upper part
        np.array([0x3f808000, 0x3f818000, 0xbf808000, 0x3f807fff, 0x3f808001, 0x7f7f8000],
                 np.uint32).view(np.float32)])
    got = oracle.bf16_rne(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert (got == want).all()
    assert oracle.bf16_rne(np.array([np.nan], np.float32))[0] & 0x7fc0 == 0x7fc0
    assert same_bits(oracle.bf16_widen(got[:1000]).astype(np.float32),
                     torch.from_numpy(x[:1000]).to(torch.bfloat16).float().numpy())


def test_fp8_e4m3_codec_against_torch(oracle):
    torch = pytest.importorskip("torch")
    if not hasattr(torch, "float8_e4m3fn"):
        pytest.skip("torch without float8_e4m3fn")
    table = oracle.fp8_decode_table()
    want = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    nan = np.isnan(want)
    assert (np.isnan(table) == nan).all() and nan.sum() == 2
    assert same_bits(table[~nan], want[~nan])
    assert table[0x7e] == 448.0 and table[0x01] == 2.0 ** -9 and table[0x08] == 2.0 ** -6
    # encode: round to nearest even inside the finite range, saturate outside
    L = oracle.lib()
    rng = np.random.default_rng(2)
    xs = np.concatenate([(rng.standard_normal(50000) * s).astype(np.float32)
                         for s in (1e-3, 0.05, 1.0, 30.0, 200.0)])
    xs = xs[np.abs(xs) <= 448.0]
    got = np.array([L.oracle_fp8_encode(float(x)) for x in xs], np.uint8)
    want = torch.from_numpy(xs).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert (got == want).all()
    # every code that is not NaN survives decode -> encode (negative zero included)
    for q in range(256):
        if not nan[q]:
            assert L.oracle_fp8_encode(float(table[q])) == q
    assert L.oracle_fp8_encode(1e9) == 0x7e and L.oracle_fp8_encode(-1e9) == 0xfe
    assert L.oracle_fp8_encode(float("inf")) == 0x7e
    assert L.oracle_fp8_encode(float("nan")) & 0x7f == 0x7f
    # midpoints between neighbours go to the even mantissa
    assert L.oracle_fp8_encode(17.0) == L.oracle_fp8_encode(16.0)      # 16 | 18: tie -> 16
    assert L.oracle_fp8_encode(19.0) == L.oracle_fp8_encode(20.0)      # 18 | 20: tie -> 20


def test_fp8_scale_convention(oracle):
    """num/gpu_cuda.cu:927-938: scale = max(amax/448, 1e-12); amax <= 0 or non-finite -> 1e-8/448."""
    L = oracle.lib()
    f = np.float32
    assert L.oracle_fp8_scale_from_amax(448.0) == 1.0
    assert f(L.oracle_fp8_scale_from_amax(1.0)) == f(1.0) / f(448.0)
    assert f(L.oracle_fp8_scale_from_amax(0.0)) == f(1e-8) / f(448.0)
    assert f(L.oracle_fp8_scale_from_amax(float("inf"))) == f(1e-8) / f(448.0)
    assert f(L.oracle_fp8_scale_from_amax(1e-20)) == f(1e-12)
    x = (np.random.default_rng(1).standard_normal(4096) * 1e-3).astype(np.float32)
    q, s = oracle.fp8_quantize(x)
    deq = oracle.fp8_decode_table()[q] * s
    assert np.max(np.abs(deq - x)) <= np.max(np.abs(x)) / 448.0 * 16 + 1e-12   # half a step of the top binade
    assert np.abs(deq).max() == np.abs(x).max() or abs(np.abs(deq).max() - np.abs(x).max()) < 1e-6


def test_storage_modes_round_where_documented(oracle):
    """bf16 moments: computed as the fp32 path from the widened value, RNE on store (unpinned by the reference)."""
    rng = np.random.default_rng(6)
    n = 4096
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    g32 = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    g16 = oracle.bf16_rne(g32)
    m16 = oracle.bf16_rne((rng.standard_normal(n) * 1e-4).astype(np.float32))
    v16 = oracle.bf16_rne((np.abs(rng.standard_normal(n)) * 1e-7).astype(np.float32))
    # fp32 run on the widened inputs
    p_a = p0.copy()
    g_a = oracle.bf16_widen(g16).copy()
    m_a = oracle.bf16_widen(m16).copy()
    v_a = oracle.bf16_widen(v16).copy()
    A = oracle.Oracle(n, beta2=0.95, weight_decay=0.1)
    A.o.t = 4
    A.step(p_a, g_a, m_a, v_a, 3e-4)
    # bf16 storage run
    p_b, g_b, m_b, v_b = p0.copy(), g16.copy(), m16.copy(), v16.copy()
    B = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_type=oracle.BF16,
                      moment_type=oracle.BF16)
    B.o.t = 4
    B.step(p_b, g_b, m_b, v_b, 3e-4)
    assert same_bits(p_a, p_b)                       # p sees the unrounded fp32 moments
    assert (m_b == oracle.bf16_rne(m_a)).all() and (v_b == oracle.bf16_rne(v_a)).all()
    assert not g_b.any()
    # fp8 gradients: g = decode(q) * scale in float, then the fp32 path
    q, s = oracle.fp8_quantize(g32)
    p_c = p0.copy()
    m_c = np.zeros(n, np.float32)
    v_c = np.zeros(n, np.float32)
    Cc = oracle.Oracle(n, beta2=0.95, grad_type=oracle.FP8, tensors=[(0, n, 1, float(s))])
    qq = q.copy()
    Cc.step(p_c, qq, m_c, v_c, 3e-4)
    p_d = p0.copy()
    m_d = np.zeros(n, np.float32)
    v_d = np.zeros(n, np.float32)
    g_d = (oracle.fp8_decode_table()[q] * s).astype(np.float32)
    oracle.Oracle(n, beta2=0.95).step(p_d, g_d, m_d, v_d, 3e-4)
    assert same_bits(p_c, p_d) and same_bits(m_c, m_d) and same_bits(v_c, v_d) and not qq.any()


# ---- the FP8 norm's value and the slot-layout loop (the last two functions nothing pinned) ----

def _fp8_direct_sumsq(q, tensors, gs, table):
    """Brute force of what the update consumes: g_i = float32(decode(q_i) * scale_t), then
    (double(g_i) * gs)^2 summed exactly."""
    terms = []
    for off, cnt, _wd, sc in tensors:
        g = (table[q[off:off + cnt]] * np.float32(sc)).astype(np.float32)
        terms.extend((float(x) * gs) ** 2 for x in g)
    return math.fsum(terms)


def _fp8_case(rng, sizes):
    tensors, off = [], 0
    for cnt in sizes:
        tensors.append([off, cnt, 1, float(np.float32(rng.uniform(1e-6, 3e-3)))])
        off += cnt
    q = rng.integers(0, 256, off).astype(np.uint8)
    q[(q & 0x7f) == 0x7f] = 0x3a                    # no NaN codes in the value test
    return q, tensors


@pytest.mark.parametrize("sizes", [
    [5000, 1, 3000, 4096, 777],                     # tensors sharing a 4096-element tile, one element
    [1, 1, 1], [4096, 4096], [8191, 3, 12289]])
def test_fp8_sumsq_value_against_brute_force(oracle, sizes):
    """oracle_sumsq's FP8 branch (the factored form) against the direct form, <= 1e-7 relative."""
    rng = np.random.default_rng(sum(sizes))
    table = oracle.fp8_decode_table()
    q, tensors = _fp8_case(rng, sizes)
    if len(sizes) == 5:
        q[tensors[2][0]:tensors[2][0] + tensors[2][1]] = 0      # an all-zero tensor
    for gs in (1.0, 0.37, 1 / 252.0):
        want = _fp8_direct_sumsq(q, tensors, gs, table)
        for threads in (1, 4):
            got = oracle.sumsq(q, oracle.FP8, [tuple(t) for t in tensors], gs, threads)
            assert abs(got - want) <= 1e-7 * want, (sizes, gs, threads, got, want)


def test_fp8_sumsq_invariants(oracle):
    """What a wrong factoring breaks: a tensor's share scales with the square of ITS scale only,
    one element gives the closed form, the order of codes inside a tensor is irrelevant."""
    rng = np.random.default_rng(11)
    table = oracle.fp8_decode_table()
    q, tensors = _fp8_case(rng, [3000, 500, 4096])
    T = [tuple(t) for t in tensors]
    base = oracle.sumsq(q, oracle.FP8, T, 0.5)
    # share of tensor 1 alone (the other scales zeroed: exact zeros)
    only1 = [(o, c, w, sc if i == 1 else 0.0) for i, (o, c, w, sc) in enumerate(T)]
    share1 = oracle.sumsq(q, oracle.FP8, only1, 0.5)
    rest = [(o, c, w, 0.0 if i == 1 else sc) for i, (o, c, w, sc) in enumerate(T)]
    share_rest = oracle.sumsq(q, oracle.FP8, rest, 0.5)
    assert abs(base - (share1 + share_rest)) <= 4e-16 * base
    doubled = [(o, c, w, sc * 2 if i == 1 else sc) for i, (o, c, w, sc) in enumerate(T)]
    got = oracle.sumsq(q, oracle.FP8, doubled, 0.5)
    assert abs(got - (4.0 * share1 + share_rest)) <= 4e-16 * got        # x2 is exact, so is x4
    # one element: (decode(q) * scale * gs)^2 up to the two roundings of the factored product
    for code in (0x01, 0x38, 0x7e, 0xc5):
        one = np.array([code], np.uint8)
        sc = float(np.float32(7.25e-4))
        want = (float(table[code]) * sc * 0.37) ** 2
        got = oracle.sumsq(one, oracle.FP8, [(0, 1, 1, sc)], 0.37)
        assert abs(got - want) <= 1e-15 * want
    # permuting the codes inside each tensor changes nothing, bit for bit
    qp = q.copy()
    for o, c, _w, _s in T:
        qp[o:o + c] = rng.permutation(qp[o:o + c])
    assert oracle.sumsq(qp, oracle.FP8, T, 0.5) == base
    # a NaN code anywhere makes the sum NaN (the skip decision of the step rests on it)
    qn = q.copy()
    qn[3100] = 0x7f
    assert math.isnan(oracle.sumsq(qn, oracle.FP8, T, 0.5))


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_slot_loop_matches_golden(oracle, name):
    """oracle_adam_step_slots (the reference's 24-byte-slot layout, the serial timing leg of the
    bench) bit for bit against the vectors the compiled reference wrote."""
    import ctypes as C
    G = load_golden(name)
    n = G["p0"].size
    p = G["p0"].copy()
    g = np.zeros(n, np.float32)
    slots = np.zeros(n, dtype=[("param", np.uint64), ("grad", np.uint64), ("m", np.float32),
                               ("v", np.float32)])
    assert slots.itemsize == 24
    slots["param"] = p.ctypes.data + 4 * np.arange(n, dtype=np.uint64)
    slots["grad"] = g.ctypes.data + 4 * np.arange(n, dtype=np.uint64)
    L = oracle.lib()
    L.oracle_adam_step_slots.argtypes = [C.c_void_p, C.c_int64, C.c_int] + [C.c_double] * 7
    L.oracle_adam_step_slots.restype = None
    for s in range(G["grads"].shape[0]):
        g[:] = G["grads"][s]
        L.oracle_adam_step_slots(slots.ctypes.data, n, s + 1, float(G["beta1"]), float(G["beta2"]),
                                 float(G["eps"]), float(G["wd"]), float(G["clip"]),
                                 float(G["lr"][s]), float(G["grad_scale"]))
        assert same_bits(p, G["p"][s]), (name, s)
        assert same_bits(np.ascontiguousarray(slots["m"]), G["m"][s])
        assert same_bits(np.ascontiguousarray(slots["v"]), G["v"][s])
        assert not g.any()


# ---- bias / LayerNorm gradient column sums ---------------------------------------------------

def test_colsum_matches_golden_of_the_reference(oracle):
    """dgamma / dbeta written by the reference's compiled host layernorm_backward."""
    G = load_golden("ln_colsum")
    dbeta = oracle.colsum_add(G["dbeta0"].copy(), G["dy"])
    dgamma = oracle.colsum_add(G["dgamma0"].copy(), G["dy"], G["x_hat"])
    assert same_bits(dbeta, G["dbeta"]) and same_bits(dgamma, G["dgamma"])
    assert np.signbit(G["dbeta"][8]) and G["dbeta"][8] == 0.0        # -0 + (-0) ... stays -0


def test_colsum_equals_compiled_reference(oracle):
    if not oracle.ref_available():
        pytest.skip("compiled reference absent")
    rng = np.random.default_rng(8)
    for T in (1, 2, 63, 130):
        dy = (rng.standard_normal((T, 1024)) * 10.0 ** rng.integers(-3, 3, (T, 1024))).astype(np.float32)
        xh = rng.standard_normal((T, 1024)).astype(np.float32)
        g0 = rng.standard_normal(1024).astype(np.float32)
        b0 = rng.standard_normal(1024).astype(np.float32)
        g, b = g0.copy(), b0.copy()
        oracle.ref_ln_backward_grads(dy, xh, g, b)
        assert same_bits(oracle.colsum_add(b0.copy(), dy), b)
        assert same_bits(oracle.colsum_add(g0.copy(), dy, xh), g)


def test_colsum_order_and_rounding_known_answers(oracle):
    """Cases where another order, a wider accumulator or a fused multiply-add gives another
    float: the answers below follow from IEEE single arithmetic alone."""
    x = np.array([[1e8], [1.0], [-1e8], [1.0]], np.float32)
    assert oracle.colsum_add(np.zeros(1, np.float32), x)[0] == 1.0      # ((0+1e8)+1)-1e8 = 0, +1
    assert oracle.colsum_add(np.ones(1, np.float32), x[::-1].copy())[0] == 0.0   # (((1+1)-1e8)+1)+1e8
    # 2^24 + 1 + 1 = 2^24 serially (each 1 is lost); a double accumulator would give 2^24 + 2
    x = np.array([[1.0], [1.0]], np.float32)
    assert oracle.colsum_add(np.array([2.0 ** 24], np.float32), x)[0] == 2.0 ** 24
    # the product is rounded to float before it is added: a = 1 + 2^-12, a*a = 1 + 2^-11 + 2^-24
    # rounds to 1 + 2^-11; adding -(1 + 2^-11) gives exactly 0, a fused multiply-add 2^-24
    a = np.float32(1.0 + 2.0 ** -12)
    x = np.array([[a]], np.float32)
    acc = np.array([-(1.0 + 2.0 ** -11)], np.float32)
    assert oracle.colsum_add(acc, x, x.copy())[0] == 0.0
    # zero rows: nothing is added, a -0 accumulator keeps its sign
    acc = np.array([-0.0, 3.0], np.float32)
    out = oracle.colsum_add(acc, np.zeros((0, 2), np.float32))
    assert np.signbit(out[0]) and out[1] == 3.0
