"""Outputs derived from the new weights inside the step (anni_adam_enable_derived): the E4M3
weight twins with their per-tensor scales and the packed [Wq | Wk | Wv] bf16 operand, against the
oracle's restatement of the reference's producers (num/gpu_cuda.cu:826-851,927-938,1090-1115 and
:6456-6470) applied to the oracle's new weights."""
import numpy as np
import pytest

from helpers import same_bits

pytestmark = pytest.mark.gpu

F32, BF16, FP8 = 0, 1, 2
DECAY, TWIN, FP8TWIN = 1, 2, 4


def make(tensors, **kw):
    from anni_amd.lm_adam import LmAdam
    opt = LmAdam(tensors, **kw)
    opt._flags = [t[-1] for t in tensors]
    return opt


def oracle_tensors(opt):
    return [(opt.offsets[i], opt.sizes[i], 1 if (f & DECAY) else 0, 1.0)
            for i, f in enumerate(opt._flags)]


def want_fp8(oracle, opt, P, q_prev, s_prev):
    """Codes and scales of the flagged tensors from P; the rest keep what they had."""
    q, sc = q_prev.copy(), s_prev.copy()
    for i, (off, cnt, f) in enumerate(zip(opt.offsets, opt.sizes, opt._flags)):
        if f & FP8TWIN and cnt:
            q[off:off + cnt], sc[i] = oracle.fp8_quantize(P[off:off + cnt])
        elif f & FP8TWIN:
            sc[i] = oracle.fp8_quantize(np.zeros(0, np.float32))[1]
    return q, sc


def want_pack(oracle, opt, P, packs, pack_elems, prev):
    out = prev.copy()
    h = oracle.bf16_rne(P)
    for tensor, cols, dst, stride in packs:
        off, cnt = opt.offsets[tensor], opt.sizes[tensor]
        rows = cnt // cols
        idx = dst + np.arange(rows)[:, None] * stride + np.arange(cols)[None, :]
        out[idx.ravel()] = h[off:off + cnt]
    return out


def test_tiny_model_qkv_pack_and_fp8_twins(gpu, oracle):
    """The reference's 64-wide model: every matrix keeps an E4M3 twin, every block a [D][3D]
    packed QKV.  Checked after the seed, over clipped and unclipped steps, across a skipped step
    (both stay as they were) and on the step after it."""
    from anni_amd import layout
    d = layout.SIZES["tiny"][0]
    tensors = [(name, n, f | (FP8TWIN if f & TWIN else 0))
               for name, n, f in layout.tensors("tiny", "reference")]
    names = [t[0] for t in tensors]
    packs, pack_elems = [], 0
    for b in range(layout.SIZES["tiny"][3]):
        for k, w in enumerate(("wq", "wk", "wv")):
            packs.append((names.index("blk%d.%s" % (b, w)), d, pack_elems + k * d, 3 * d))
        pack_elems += 3 * d * d
    opt = make(tensors, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True)
    n = opt.n
    rng = np.random.default_rng(77)
    P = (rng.standard_normal(n) * 0.02).astype(np.float32)
    M, V = np.zeros(n, np.float32), np.zeros(n, np.float32)
    opt.upload("param", P)
    opt.enable_derived(packs, pack_elems)
    assert opt.o.d_param_fp8 and opt.o.d_wscale and opt.o.d_pack_bf16
    opt.seed_twins()
    q, sc = want_fp8(oracle, opt, P, np.zeros(n, np.uint8), np.ones(len(tensors), np.float32))
    pk = want_pack(oracle, opt, P, packs, pack_elems, np.zeros(pack_elems, np.uint16))
    assert (opt.download("fp8twin") == q).all() and same_bits(opt.download("wscale"), sc)
    assert (opt.download("pack") == pk).all()
    # the packed operand is what the reference's kernel builds from the three twins
    h = oracle.bf16_rne(P)
    blk0 = [h[opt.offsets[names.index("blk0." + w)]:][:d * d].reshape(d, d) for w in ("wq", "wk", "wv")]
    assert (pk[:3 * d * d].reshape(d, 3 * d) == np.concatenate(blk0, axis=1)).all()
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True,
                      tensors=oracle_tensors(opt), threads=2)
    base = 1.0 / (np.sqrt(n) * 1e-3)
    for s in range(6):
        g = (rng.standard_normal(n) * 1e-3 * base * (2.0 if s % 2 else 0.5)).astype(np.float32)
        if s == 3:
            g[opt.offsets[5] + 3] = np.inf
        opt.upload("grad", g)
        assert opt.step_scaled(1e-2) == 0
        st = opt.sync_stats()
        O.step(P, g.copy(), M, V, 1e-2, sumsq_override=None if s == 3 else st.last_sumsq)
        assert st.last_skipped == (1 if s == 3 else 0)
        assert same_bits(opt.download("param"), P)
        if s != 3:
            q, sc = want_fp8(oracle, opt, P, q, sc)
            pk = want_pack(oracle, opt, P, packs, pack_elems, pk)
        assert (opt.download("fp8twin") == q).all(), s
        assert same_bits(opt.download("wscale"), sc), s
        assert (opt.download("pack") == pk).all(), s
        assert (opt.download("twin")[:opt.sizes[0]] == oracle.bf16_rne(P)[:opt.sizes[0]]).all()
    opt.free()


RAGGED = [(5000, 3 | FP8TWIN), (3, FP8TWIN), (4096, 3), (1, 2 | FP8TWIN), (0, FP8TWIN),
          (8190, 1 | FP8TWIN), (12288, 3 | FP8TWIN), (7, 0), (4097 * 3, 3), (6 * 1022, 1 | FP8TWIN),
          (40000, 3 | FP8TWIN), (1023, 0)]
# odd widths, a target that is not 8-byte aligned, rows that straddle tiles, a one-column matrix
RAGGED_PACKS = [(0, 50, 3, 61), (8, 3, 7000, 5), (9, 1022, 80000, 1022), (2, 4096, 100000, 4096),
                (7, 1, 30000, 2), (5, 8190, 6200000, 8190)]
RAGGED_PACK_ELEMS = 6200000 + 8190


@pytest.mark.parametrize("mode", ["f32", "bf16", "fp8"])
def test_ragged_tensors_odd_widths_every_storage_mode(gpu, oracle, mode):
    gt = {"f32": F32, "bf16": BF16, "fp8": FP8}[mode]
    mt = BF16 if mode == "bf16" else F32
    opt = make(RAGGED, grad_type=gt, moment_type=mt, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    n = opt.n
    rng = np.random.default_rng(5)
    P = (rng.standard_normal(n) * 0.02).astype(np.float32)
    P[opt.offsets[6]:opt.offsets[6] + opt.sizes[6]] = 0.0          # an all-zero tensor: amax 0
    P[opt.offsets[10] + 9] = 3.0e38                                  # a huge amax
    opt.upload("param", P)
    opt.enable_derived(RAGGED_PACKS, RAGGED_PACK_ELEMS)
    opt.seed_twins()
    q, sc = want_fp8(oracle, opt, P, np.zeros(n, np.uint8), np.ones(len(RAGGED), np.float32))
    pk = want_pack(oracle, opt, P, RAGGED_PACKS, RAGGED_PACK_ELEMS,
                   np.zeros(RAGGED_PACK_ELEMS, np.uint16))
    assert (opt.download("fp8twin") == q).all() and same_bits(opt.download("wscale"), sc)
    assert (opt.download("pack") == pk).all()
    ot = {"f32": oracle.F32, "bf16": oracle.BF16, "fp8": oracle.FP8}[mode]
    gsc = np.linspace(0.5, 2.0, len(RAGGED)).astype(np.float32)
    segs = [(o, c, w, float(gsc[i]) if mode == "fp8" else 1.0)
            for i, (o, c, w, _x) in enumerate(oracle_tensors(opt))]
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, grad_type=ot,
                      moment_type=oracle.BF16 if mode == "bf16" else oracle.F32, tensors=segs,
                      threads=2)
    if mode == "fp8":
        opt.upload("gscale", gsc)
    mdt = np.uint16 if mode == "bf16" else np.float32
    M, V = np.zeros(n, mdt), np.zeros(n, mdt)
    for s in range(3):
        g32 = (rng.standard_normal(n) * (3e-3 if s == 1 else 1e-5)).astype(np.float32)
        if mode == "f32":
            g = g32
        elif mode == "bf16":
            g = oracle.bf16_rne(g32)
        else:
            g = oracle.fp8_quantize(g32 / np.float32(3e-3) * 100)[0]
        opt.upload("grad", g)
        assert opt.step_scaled(1e-3) == 0
        st = opt.sync_stats()
        O.step(P, g.copy(), M, V, 1e-3, sumsq_override=st.last_sumsq)
        assert same_bits(opt.download("param"), P), s
        q, sc = want_fp8(oracle, opt, P, q, sc)
        pk = want_pack(oracle, opt, P, RAGGED_PACKS, RAGGED_PACK_ELEMS, pk)
        assert (opt.download("fp8twin") == q).all(), s
        assert same_bits(opt.download("wscale"), sc), s
        assert (opt.download("pack") == pk).all(), s
    opt.free()


def test_fp8_twins_alone_and_pack_alone(gpu, oracle):
    rng = np.random.default_rng(9)
    for tensors, packs, elems in (([(9000, 3 | FP8TWIN), (100, 0)], [], 0),
                                  ([(9000, 3), (100, 0)], [(0, 90, 10, 100)], 10010)):
        opt = make(tensors, grad_clip=0.0, weight_decay=0.01)
        n = opt.n
        P = (rng.standard_normal(n) * 0.02).astype(np.float32)
        opt.upload("param", P)
        opt.enable_derived(packs, elems)
        assert bool(opt.o.d_param_fp8) == (not packs) and bool(opt.o.d_pack_bf16) == bool(packs)
        opt.seed_twins()
        M, V = np.zeros(n, np.float32), np.zeros(n, np.float32)
        O = oracle.Oracle(n, weight_decay=0.01, tensors=oracle_tensors(opt))
        q, sc = np.zeros(n, np.uint8), np.ones(2, np.float32)
        pk = np.zeros(max(elems, 1), np.uint16)
        for s in range(2):
            g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
            opt.upload("grad", g)
            opt.step_scaled(1e-3)
            O.step(P, g.copy(), M, V, 1e-3)
            assert same_bits(opt.download("param"), P)
            if packs:
                pk = want_pack(oracle, opt, P, packs, elems, pk)
                assert (opt.download("pack") == pk).all()
            else:
                q, sc = want_fp8(oracle, opt, P, q, sc)
                assert (opt.download("fp8twin") == q).all()
                assert same_bits(opt.download("wscale"), sc)
        opt.free()


def test_refusals(gpu):
    from anni_amd import lib as L
    opt = make([(4096, 3), (100, 0)])
    Pk = L.Pack
    def enable(packs, elems):
        arr = (Pk * max(len(packs), 1))(*[Pk(*p) for p in packs])
        return gpu.anni_adam_enable_derived(opt.h, arr if packs else None, len(packs), elems)
    assert enable([], 0) == -1                                    # nothing flagged, nothing packed
    assert enable([(2, 64, 0, 64)], 4096) == -1                   # no such tensor
    assert enable([(0, 100, 0, 100)], 4096) == -1                 # 4096 is not a multiple of 100
    assert enable([(0, 64, 0, 32)], 4096) == -1                   # rows would overlap
    assert enable([(0, 64, 1, 64)], 4096) == -1                   # runs past the packed flat
    assert enable([(0, 64, 0, 64), (0, 64, 0, 64)], 8192) == -1   # two homes for one tensor
    assert enable([(0, 64, 0, 64)], 0) == -1
    assert not opt.o.d_pack_bf16 and not opt.o.d_param_fp8
    assert enable([(0, 64, 0, 64)], 4096) == 0
    assert enable([(0, 64, 0, 64)], 4096) == -1                   # once only
    opt.free()


def test_185m_reference_layout_full_size(gpu, oracle):
    """The reference's own model size (separate Wq, Wk, Wv of 1024 x 1024, 12 blocks): E4M3 twins of
    all 74 matrices and the 12 packed [1024][3072] operands over two steps, one of them clipped,
    every element compared."""
    import math
    import os
    from anni_amd import layout
    threads = max(1, min(16, len(os.sched_getaffinity(0))))
    d, _h, _ff, blocks, _v = layout.SIZES["185m"]
    tensors = [(name, n, f | (FP8TWIN if f & TWIN else 0))
               for name, n, f in layout.tensors("185m", "reference")]
    names = [t[0] for t in tensors]
    packs, pack_elems = [], 0
    for b in range(blocks):
        for k, w in enumerate(("wq", "wk", "wv")):
            packs.append((names.index("blk%d.%s" % (b, w)), d, pack_elems + k * d, 3 * d))
        pack_elems += 3 * d * d
    opt = make(tensors, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True)
    n = opt.n
    assert gpu.anni_fill_normal_f32(opt.o.d_param, n, 4, 1, 0.0, 0.02) == 0
    opt.enable_derived(packs, pack_elems)
    opt.seed_twins()
    P = opt.download("param")
    M, V = np.zeros(n, np.float32), np.zeros(n, np.float32)
    q, sc = want_fp8(oracle, opt, P, np.zeros(n, np.uint8), np.ones(len(tensors), np.float32))
    pk = want_pack(oracle, opt, P, packs, pack_elems, np.zeros(pack_elems, np.uint16))
    assert (opt.download("fp8twin") == q).all() and same_bits(opt.download("wscale"), sc)
    assert (opt.download("pack") == pk).all()
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, skip_nonfinite=True,
                      tensors=oracle_tensors(opt), threads=threads, simd=oracle.cpu_simd())
    unit = 1.0 / (math.sqrt(n) * 1e-3)
    for s, mult in enumerate((1.7, 0.6)):
        assert gpu.anni_fill_normal_f32(opt.o.d_grad, n, 4, 50 + s, 0.0, 1e-3) == 0
        g = opt.download("grad")
        assert opt.step_scaled(3e-4, unit * mult) == 0
        st = opt.sync_stats()
        assert st.last_clipped == (mult > 1)
        O.step(P, g, M, V, 3e-4, unit * mult, sumsq_override=st.last_sumsq)
        assert same_bits(opt.download("param"), P)
        q, sc = want_fp8(oracle, opt, P, q, sc)
        pk = want_pack(oracle, opt, P, packs, pack_elems, pk)
        assert (opt.download("fp8twin") == q).all(), s
        assert same_bits(opt.download("wscale"), sc), s
        assert (opt.download("pack") == pk).all(), s
        print("185m derived step %d ok" % (s + 1), flush=True)
    opt.free()


def test_hardware_encode_on_every_rounding_boundary(gpu, oracle):
    """The E4M3 twins of whole tiles are made with the gfx950 conversion instruction, the ragged
    ends with the bit-level encoder: both against the oracle's encoder (pinned to torch's
    float8_e4m3fn cast) on tensors whose max |p| is exactly 448, so scale = 1 and the bytes are the
    plain encoding: every binade, both signs, every half step of the 3-bit mantissa with its two
    float neighbours, the subnormal grid, signed zeros, float denormals, NaNs of both signs,
    and random values."""
    vals = [448.0, 0.0, -0.0, 1e-45, -1e-45, 1e-39, 2.0 ** -10, 2.0 ** -9, 3 * 2.0 ** -10,
            447.99997, 432.0, 2.0 ** -6, 2.0 ** -7, 0.0146484375, np.nan, -np.nan]
    for e in range(-12, 9):
        for k in range(0, 32):
            c = np.float32((1.0 + k / 16.0) * 2.0 ** e)
            if c > 448:
                continue
            for v in (c, np.nextafter(c, np.float32(0)), np.nextafter(c, np.float32(1e9))):
                if v <= 448:
                    vals += [float(v), -float(v)]
    rng = np.random.default_rng(321)
    n_big = 4096 * 40
    rnd = (rng.standard_normal(n_big) * 10.0 ** rng.integers(-6, 3, n_big)).astype(np.float32)
    big = np.clip(rnd, -448, 448)
    special = np.array(vals, np.float32)
    big[:special.size] = special                       # whole tiles: the hardware path
    big = big[rng.permutation(n_big)]
    tail = np.concatenate([special, np.float32([448.0])])[:4095]     # a ragged tensor: the bit-level path
    opt = make([(n_big, FP8TWIN), (tail.size, FP8TWIN)], twins=False)
    opt.upload("param", np.concatenate([big, tail]))
    opt.enable_derived()
    opt.seed_twins()
    got, sc = opt.download("fp8twin"), opt.download("wscale")
    assert sc[0] == 1.0 and sc[1] == 1.0
    for off, x in ((0, big), (n_big, tail)):
        want, scale = oracle.fp8_quantize(x)
        assert scale == 1.0
        g = got[off:off + x.size]
        bad = np.flatnonzero(g != want)
        assert bad.size == 0, [(float(x[i]), int(g[i]), int(want[i])) for i in bad[:8]]
    opt.free()
