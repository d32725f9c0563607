"""anni_adam_quantize_grads_static, the entry point that allocates nothing: the gradient quantiser
with its work area in a fixed device array instead of a block allocated at the first call.  Its
codes and scales must equal those of anni_adam_quantize_grads bit for bit -- on two calls in a
row, the second on a smaller optimizer, so that what the first call left in the shared array is
in the way -- and the oracle's quantiser on each tensor."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

FP8 = 2


def _case(gpu, oracle, tensors, seed):
    from anni_amd.lm_adam import DeviceBuffer, LmAdam
    rng = np.random.default_rng(seed)
    opt = LmAdam(tensors, grad_type=FP8, skip_nonfinite=True)
    n = opt.n
    g32 = (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 2, n)).astype(np.float32)
    for i, (off, cnt) in enumerate(zip(opt.offsets, opt.sizes)):
        g32[off:off + cnt] *= np.float32(1.0 + 3 * (i % 50))
    off2, cnt2 = opt.offsets[2], opt.sizes[2]
    g32[off2:off2 + cnt2] = 0.0                          # amax 0: scale 1e-12, codes 0
    g32[opt.offsets[3] + 1] = np.nan                     # becomes the NaN code
    src = DeviceBuffer(n * 4)
    src.upload(g32)
    return opt, src, g32


def _run(gpu, opt, src, fn):
    n = opt.n
    # junk where the results go, so that a call that wrote nothing cannot pass
    opt.upload("grad", np.full(n, 0x55, np.uint8))
    opt.upload("gscale", np.full(opt.o.n_tensors, 123.0, np.float32))
    assert fn(opt.h, src.ptr) == 0, gpu.gpu_debug_last_error()
    assert gpu.gpu_stream_sync() == 0
    return opt.download("grad"), opt.download("gscale")


def test_static_quantiser_equals_the_allocating_one(gpu, oracle):
    big = [(6000, 3), (64, 0), (4096, 3), (8192 + 3, 3), (1, 0), (4096 * 300 + 17, 3), (3, 0),
           (4096 * 5, 3), (777, 1), (2, 0)]
    small = [(3000, 3), (5, 0), (4096, 3), (4096 * 2 + 9, 3), (1, 0)]
    A = _case(gpu, oracle, big, 1)
    B = _case(gpu, oracle, small, 2)
    assert B[0].n < A[0].n
    ref = [_run(gpu, opt, src, gpu.anni_adam_quantize_grads) for opt, src, _g in (A, B)]
    # the two calls in a row, the second with the smaller input
    got = [_run(gpu, opt, src, gpu.anni_adam_quantize_grads_static) for opt, src, _g in (A, B)]
    for (opt, _src, g32), (q0, s0), (q1, s1) in zip((A, B), ref, got):
        assert (q0 == q1).all()
        assert (s0.view(np.uint32) == s1.view(np.uint32)).all()
        for i, (off, cnt) in enumerate(zip(opt.offsets, opt.sizes)):
            qw, sw = oracle.fp8_quantize(g32[off:off + cnt])
            assert (q1[off:off + cnt] == qw).all(), i
            assert np.float32(s1[i]).view(np.uint32) == np.float32(sw).view(np.uint32), i
    # and once more the other way round: big after small
    q2, s2 = _run(gpu, A[0], A[1], gpu.anni_adam_quantize_grads_static)
    assert (q2 == ref[0][0]).all() and (s2.view(np.uint32) == ref[0][1].view(np.uint32)).all()
    # the same refusals as the allocating entry point
    assert gpu.anni_adam_quantize_grads_static(A[0].h, None) == -1
    assert gpu.anni_adam_quantize_grads_static(A[0].h, A[1].ptr + 4) == -1
    for opt, src, _g in (A, B):
        src.free()
        opt.free()


def test_static_quantiser_refuses_what_its_array_cannot_hold(gpu):
    """More tensors than ANNI_QUANT_STATIC_MAX_TENSORS: -1 and a message; the allocating entry
    point takes the same optimizer."""
    from anni_amd.lm_adam import DeviceBuffer, LmAdam
    opt = LmAdam([(3, 0)] * 4097, grad_type=FP8)
    src = DeviceBuffer(opt.n * 4)
    src.upload(np.ones(opt.n, np.float32))
    gpu.gpu_debug_last_error()                           # clears what earlier tests left
    assert gpu.anni_adam_quantize_grads_static(opt.h, src.ptr) == -1
    assert b"ANNI_QUANT_STATIC_MAX" in gpu.gpu_debug_last_error()
    assert gpu.anni_adam_quantize_grads(opt.h, src.ptr) == 0
    assert gpu.gpu_stream_sync() == 0
    src.free()
    opt.free()


def test_static_quantiser_allocates_no_device_memory(gpu):
    """What the entry point exists for: its first call on a fresh optimizer leaves the device's
    free memory exactly where it was (the allocating entry point's first call takes its scratch
    block then, and the figure drops)."""
    import ctypes as C
    from anni_amd.lm_adam import DeviceBuffer, LmAdam
    # 573 M elements: 2.2 MiB of tile maxima, more than the 2 MiB steps in which the driver's figure moves
    tensors = [(4096 * 100000, 3), (4096 * 40000 + 5, 3), (777, 0)]
    opt = LmAdam(tensors, grad_type=FP8, twins=False)
    src = DeviceBuffer(opt.n * 4)
    assert gpu.gpu_memset(src.ptr, 0, opt.n * 4) == 0
    assert gpu.gpu_stream_sync() == 0

    def free_now():
        hip = C.CDLL("libamdhip64.so")
        fr, tt = C.c_size_t(0), C.c_size_t(0)
        hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
        assert hip.hipMemGetInfo(C.byref(fr), C.byref(tt)) == 0
        return fr.value
    before = free_now()
    assert gpu.anni_adam_quantize_grads_static(opt.h, src.ptr) == 0
    assert gpu.gpu_stream_sync() == 0
    assert free_now() == before
    assert gpu.anni_adam_quantize_grads_static(opt.h, src.ptr) == 0
    assert gpu.gpu_stream_sync() == 0
    assert free_now() == before
    assert gpu.anni_adam_quantize_grads(opt.h, src.ptr) == 0            # the contrast: this one allocates
    assert gpu.gpu_stream_sync() == 0
    seen = free_now() < before
    src.free()
    opt.free()
    if not seen:
        pytest.skip("the driver's free-memory figure did not move for an allocation of this size "
                    "either: the equalities above prove nothing on this box")
