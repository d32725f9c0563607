"""Bias / LayerNorm gradient column sums on the device (anni_colsum_add) against the oracle's
restatement of the reference's host loops (lang/ffn.c:301-305,358-362, lang/layernorm.c:368-372)
and against dgamma / dbeta written by the compiled reference: identical bits, any shape."""
import numpy as np
import pytest

from helpers import load_golden, same_bits

pytestmark = pytest.mark.gpu


def wide(rng, shape):
    """Magnitudes over six decades, so that a float sum depends on the order of the additions."""
    return (rng.standard_normal(shape) * 10.0 ** rng.integers(-3, 3, shape)).astype(np.float32)


def device_colsum(gpu, acc, x, y=None):
    from anni_amd.lm_adam import DeviceBuffer
    rows, cols = x.shape
    d_acc = DeviceBuffer(acc.nbytes)
    d_acc.upload(acc)
    d_x = DeviceBuffer(max(x.nbytes, 4))
    if x.size:
        d_x.upload(x)
    d_y = None
    if y is not None:
        d_y = DeviceBuffer(max(y.nbytes, 4))
        if y.size:
            d_y.upload(y)
    assert gpu.anni_colsum_add(d_acc.ptr, d_x.ptr, d_y.ptr if d_y else None, rows, cols) == 0
    out = d_acc.download(np.float32, cols)
    for b in (d_acc, d_x, d_y):
        if b:
            b.free()
    return out


def test_golden_of_the_reference(gpu):
    G = load_golden("ln_colsum")
    assert same_bits(device_colsum(gpu, G["dbeta0"], G["dy"]), G["dbeta"])
    assert same_bits(device_colsum(gpu, G["dgamma0"], G["dy"], G["x_hat"]), G["dgamma"])


@pytest.mark.parametrize("cols", [1, 63, 64, 65, 1000, 1536])
def test_shapes_against_the_oracle(gpu, oracle, cols):
    rng = np.random.default_rng(cols)
    for rows in (0, 1, 2, 15, 16, 17, 127, 128, 129, 255, 256, 257, 1000):
        x, y = wide(rng, (rows, cols)), rng.standard_normal((rows, cols)).astype(np.float32)
        a0 = wide(rng, cols)
        a0[0] = -0.0
        if rows:
            x[:, 0] = -0.0
        assert same_bits(device_colsum(gpu, a0, x), oracle.colsum_add(a0.copy(), x)), rows
        assert same_bits(device_colsum(gpu, a0, x, y), oracle.colsum_add(a0.copy(), x, y)), rows


def test_order_dependent_known_answers(gpu):
    x = np.array([[1e8], [1.0], [-1e8], [1.0]], np.float32)
    assert device_colsum(gpu, np.zeros(1, np.float32), x)[0] == 1.0
    assert device_colsum(gpu, np.ones(1, np.float32), x[::-1].copy())[0] == 0.0
    a = np.float32(1.0 + 2.0 ** -12)                     # product rounded before the add: no fma
    x = np.array([[a]], np.float32)
    assert device_colsum(gpu, np.array([-(1.0 + 2.0 ** -11)], np.float32), x, x.copy())[0] == 0.0
    nan = device_colsum(gpu, np.zeros(3, np.float32),
                        np.array([[1.0, np.inf, np.nan], [2.0, -np.inf, 1.0]], np.float32))
    assert nan[0] == 3.0 and np.isnan(nan[1]) and np.isnan(nan[2])


def test_ffn_and_layernorm_shapes_at_full_size(gpu, oracle):
    """db1 of the 555M model (16384 token rows x 6272) and dgamma at 1536 wide, every column."""
    from anni_amd.lm_adam import DeviceBuffer
    rows = 16384
    for cols, prod in ((6272, False), (1536, True)):
        d_x, d_y = DeviceBuffer(rows * cols * 4), DeviceBuffer(rows * cols * 4)
        assert gpu.anni_fill_normal_f32(d_x.ptr, rows * cols, 3, cols, 0.0, 1e-2) == 0
        assert gpu.anni_fill_normal_f32(d_y.ptr, rows * cols, 3, cols + 1, 0.0, 1.0) == 0
        x = d_x.download(np.float32, rows * cols).reshape(rows, cols)
        y = d_y.download(np.float32, rows * cols).reshape(rows, cols) if prod else None
        a0 = np.linspace(-1, 1, cols).astype(np.float32)
        d_a = DeviceBuffer(cols * 4)
        d_a.upload(a0)
        assert gpu.anni_colsum_add(d_a.ptr, d_x.ptr, d_y.ptr if prod else None, rows, cols) == 0
        assert same_bits(d_a.download(np.float32, cols), oracle.colsum_add(a0.copy(), x, y))
        # twice more on top: the accumulator carries over
        assert gpu.anni_colsum_add(d_a.ptr, d_x.ptr, d_y.ptr if prod else None, rows, cols) == 0
        want = oracle.colsum_add(oracle.colsum_add(a0.copy(), x, y), x, y)
        assert same_bits(d_a.download(np.float32, cols), want)
        for b in (d_x, d_y, d_a):
            b.free()


def test_bias_gradient_lands_in_the_flat_and_the_step_uses_it(gpu, oracle):
    """The producer writes into the bias tensor's slice of the gradient flat; the step then
    sees exactly the gradient the host loops would have produced."""
    from anni_amd.lm_adam import LmAdam, DeviceBuffer
    rng = np.random.default_rng(12)
    tensors = [(4096 * 3, 3), (1000, 0), (5000, 3), (64, 0)]
    opt = LmAdam(tensors, beta2=0.95, weight_decay=0.1, grad_clip=1.0)
    n = opt.n
    P = (rng.standard_normal(n) * 0.02).astype(np.float32)
    opt.upload("param", P)
    g = (rng.standard_normal(n) * 1e-3).astype(np.float32)
    g[opt.offsets[1]:opt.offsets[1] + 1000] = 0.0          # the step left the bias gradients at zero
    g[opt.offsets[3]:opt.offsets[3] + 64] = 0.0
    opt.upload("grad", g)
    for i, (rows, cols) in ((1, (300, 1000)), (3, (77, 64))):
        for _micro in range(2):                             # two microbatches accumulate
            dout = wide(rng, (rows, cols)) * np.float32(1e-3)
            d = DeviceBuffer(dout.nbytes)
            d.upload(dout)
            assert gpu.anni_colsum_add(opt.o.d_grad + 4 * opt.offsets[i], d.ptr, None, rows, cols) == 0
            assert gpu.gpu_stream_sync() == 0
            d.free()
            oracle.colsum_add(g[opt.offsets[i]:opt.offsets[i] + cols], dout)
    assert same_bits(opt.download("grad"), g)
    opt.step_scaled(1e-3)
    st = opt.sync_stats()
    M, V = np.zeros(n, np.float32), np.zeros(n, np.float32)
    segs = [(opt.offsets[i], t[0], t[1] & 1, 1.0) for i, t in enumerate(tensors)]
    O = oracle.Oracle(n, beta2=0.95, weight_decay=0.1, grad_clip=1.0, tensors=segs)
    O.step(P, g, M, V, 1e-3, sumsq_override=st.last_sumsq)
    assert same_bits(opt.download("param"), P) and same_bits(opt.download("m"), M)
    assert same_bits(opt.download("v"), V)
    opt.free()


def test_batch_equals_one_call_per_job(gpu, oracle):
    """The bias and LayerNorm gradients of a block in one call: plain and product sums mixed,
    widths that do not fill their last workgroup, a job without rows."""
    from anni_amd import lib
    from anni_amd.lm_adam import DeviceBuffer
    rng = np.random.default_rng(99)
    shapes = [(300, 6272, False), (300, 1536, False), (77, 1536, True), (300, 1, False),
              (0, 64, False), (129, 1000, True), (64, 65, False), (1, 63, True)]
    keep, jobs, want = [], [], []
    for rows, cols, prod in shapes:
        x, y, a0 = wide(rng, (rows, cols)), wide(rng, (rows, cols)), wide(rng, cols)
        bufs = [DeviceBuffer(cols * 4), DeviceBuffer(max(x.nbytes, 4)), DeviceBuffer(max(y.nbytes, 4))]
        bufs[0].upload(a0)
        if rows:
            bufs[1].upload(x)
            bufs[2].upload(y)
        keep.append(bufs)
        jobs.append(lib.Colsum(bufs[0].ptr, bufs[1].ptr, bufs[2].ptr if prod else None, rows, cols))
        want.append(oracle.colsum_add(a0.copy(), x, y if prod else None))
    arr = (lib.Colsum * len(jobs))(*jobs)
    assert gpu.anni_colsum_add_batch(arr, len(jobs)) == 0
    for bufs, w in zip(keep, want):
        assert same_bits(bufs[0].download(np.float32, w.size), w)
    assert gpu.anni_colsum_add_batch(arr, 0) == -1
    assert gpu.anni_colsum_add_batch(None, 1) == -1
    assert gpu.anni_colsum_add_batch((lib.Colsum * 17)(*([jobs[0]] * 17)), 17) == -1
    for bufs in keep:
        for b in bufs:
            b.free()


def test_argument_checks(gpu):
    from anni_amd.lm_adam import DeviceBuffer
    d = DeviceBuffer(1024)
    assert gpu.anni_colsum_add(None, d.ptr, None, 4, 4) == -1
    assert gpu.anni_colsum_add(d.ptr, None, None, 4, 4) == -1
    assert gpu.anni_colsum_add(d.ptr, d.ptr, None, -1, 4) == -1
    assert gpu.anni_colsum_add(d.ptr, d.ptr, None, 4, 0) == -1
    assert gpu.anni_colsum_add(d.ptr, d.ptr, None, 4, (1 << 24) + 1) == -1
    assert gpu.anni_colsum_add(d.ptr, d.ptr, None, 0, 4) == 0
    d.free()


def test_the_references_own_entry_point(gpu, oracle):
    """gpu_mat_col_sum_add (num/gpu.h:195-199), the call of lang/ffn.c:298,355: a device matrix is
    summed into the caller's HOST bias gradient with the host loop's bits, over several calls
    (gradient accumulation: the vector is not zero at the second call); a host matrix is declined,
    and the caller's own loop runs."""
    import ctypes as C
    from anni_amd.lm_adam import DeviceBuffer
    gpu.gpu_mat_col_sum_add.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int]
    gpu.gpu_mat_col_sum_add.restype = C.c_int
    rng = np.random.default_rng(77)
    for rows, cols in ((1, 1), (130, 257), (1000, 1536), (64, 6272)):
        db = wide(rng, cols)
        want = db.copy()
        for _call in range(3):
            x = wide(rng, (rows, cols))
            d_x = DeviceBuffer(x.nbytes)
            d_x.upload(x)
            assert gpu.gpu_mat_col_sum_add(db.ctypes.data, d_x.ptr, rows, cols) == 0
            oracle.colsum_add(want, x)
            assert same_bits(db, want), (rows, cols, _call)
            d_x.free()
    x = wide(rng, (8, 16))
    db = np.zeros(16, np.float32)
    assert gpu.gpu_mat_col_sum_add(db.ctypes.data, x.ctypes.data, 8, 16) == -1      # host matrix
    assert not db.any()
    assert gpu.gpu_mat_col_sum_add(None, x.ctypes.data, 8, 16) == -1
    assert gpu.gpu_mat_col_sum_add(db.ctypes.data, x.ctypes.data, 0, 16) == -1
    assert gpu.gpu_debug_last_error() == b""             # declining is not an error
