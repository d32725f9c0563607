"""ctypes loader of libanni_gpu_hip.so (the product) and libanni_bench.so (the measuring and
testing utilities of include/anni_bench.h, a library of its own linked against the product).

There is no CPU fallback: if the libraries have not been built, loading raises
``LibraryMissing`` and nothing in this package computes anything.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(HERE, "libanni_gpu_hip.so")
BENCH_SO_PATH = os.path.join(HERE, "libanni_bench.so")

F32, BF16, FP8_E4M3 = 0, 1, 2
T_DECAY, T_TWIN, T_FP8TWIN = 1, 2, 4
LAYOUT_AUTO, LAYOUT_COMPACT, LAYOUT_SPLIT = 0, 1, 2
GPU_PREC_FP32, GPU_PREC_BF16 = 0, 1


class LibraryMissing(RuntimeError):
    pass


class Tensor(C.Structure):
    """anni_tensor (include/anni_adam.h)."""
    _fields_ = [("n", C.c_int64), ("flags", C.c_uint32)]


class Config(C.Structure):
    """anni_adam_config."""
    _fields_ = [("grad_type", C.c_int), ("moment_type", C.c_int), ("twins", C.c_int),
                ("skip_nonfinite", C.c_int), ("grad_slots", C.c_int), ("layout", C.c_int)]


class Adam(C.Structure):
    """anni_adam: the public head of the optimizer handle."""
    _fields_ = [("n", C.c_int64), ("n_tensors", C.c_int), ("t", C.c_int),
                ("beta1", C.c_double), ("beta2", C.c_double), ("eps", C.c_double),
                ("weight_decay", C.c_double), ("grad_clip", C.c_double),
                ("last_sumsq", C.c_double), ("last_grad_norm", C.c_double),
                ("last_grad_scale", C.c_double), ("last_skipped", C.c_int),
                ("last_clipped", C.c_int), ("cfg", Config),
                ("d_param", C.c_void_p), ("d_param_bf16", C.c_void_p),
                ("d_grad", C.c_void_p), ("d_m", C.c_void_p), ("d_v", C.c_void_p),
                ("d_gscale", C.c_void_p), ("d_param_fp8", C.c_void_p), ("d_wscale", C.c_void_p),
                ("d_pack_bf16", C.c_void_p), ("priv", C.c_void_p)]


class Colsum(C.Structure):
    """anni_colsum: one job of anni_colsum_add_batch."""
    _fields_ = [("d_acc", C.c_void_p), ("d_x", C.c_void_p), ("d_y", C.c_void_p),
                ("rows", C.c_int64), ("cols", C.c_int)]


class Pack(C.Structure):
    """anni_pack: a second home for the bf16 of a matrix inside a packed matrix."""
    _fields_ = [("tensor", C.c_int), ("cols", C.c_int32), ("dst_offset", C.c_int64),
                ("dst_stride", C.c_int32)]


# name -> (restype, argtypes) for every entry point the Python side calls.
_PROTOS = {
    # num/gpu.h subset (include/anni_gpu.h)
    "gpu_available": (C.c_int, []),
    "gpu_backend_name": (C.c_char_p, []),
    "gpu_mem_info": (C.c_int, [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "gpu_device_sync": (None, []),
    "gpu_stream_sync": (C.c_int, []),
    "gpu_set_compute_prec": (None, [C.c_int]),
    "gpu_debug_last_error": (C.c_char_p, []),
    "gpu_op_prof_dump": (None, []),
    "gpu_malloc": (C.c_void_p, [C.c_size_t]),
    "gpu_free": (None, [C.c_void_p]),
    "gpu_memcpy_h2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gpu_memcpy_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gpu_host_pin": (C.c_int, [C.c_void_p, C.c_size_t]),
    "gpu_memcpy_d2h_async": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gpu_memcpy_d2d": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gpu_memset": (C.c_int, [C.c_void_p, C.c_int, C.c_size_t]),
    "gpu_host_forget": (None, [C.c_void_p]),
    "gpu_host_alloc": (C.c_void_p, [C.c_size_t]),
    "gpu_host_free": (None, [C.c_void_p]),
    "gpu_adam_set_bf16_flat": (None, [C.c_void_p, C.c_void_p, C.c_int]),
    "gpu_adam_seed_bf16_flat": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "gpu_half_wt_invalidate": (None, [C.c_void_p]),
    "gpu_param_epoch": (C.c_uint, []),
    "anni_gpu_bf16_twin_of": (C.c_void_p, [C.c_void_p, C.c_size_t]),
    "gpu_adam_set_weight_decay": (None, [C.c_double]),
    "gpu_grad_sumsq": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_double)]),
    "gpu_adam_step_dev_bf16": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_void_p, C.c_int, C.c_double, C.c_double,
                                         C.c_double, C.c_double, C.c_int, C.c_double]),
    # include/anni_adam.h
    "anni_adam_create": (C.POINTER(Adam), [C.POINTER(Tensor), C.c_int, C.POINTER(Config)]),
    "anni_adam_free": (None, [C.POINTER(C.POINTER(Adam))]),
    "anni_adam_tensor_offset": (C.c_int64, [C.POINTER(Adam), C.c_int]),
    "anni_adam_grad_slot": (C.c_void_p, [C.POINTER(Adam), C.c_int]),
    "anni_adam_is_split": (C.c_int, [C.POINTER(Adam)]),
    "anni_adam_apart_ratio": (C.c_double, [C.POINTER(Adam)]),
    "anni_adam_probe_gbps": (C.c_double, [C.POINTER(Adam)]),
    "anni_adam_placement_cost": (C.c_int, [C.POINTER(Adam), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "anni_adam_arena_bytes": (C.c_size_t, [C.POINTER(Adam)]),
    "anni_adam_resident_bytes": (C.c_size_t, [C.POINTER(Adam)]),
    "anni_adam_bind_grad": (C.c_int, [C.POINTER(Adam), C.c_void_p]),
    "anni_adam_seed_twins": (C.c_int, [C.POINTER(Adam)]),
    "anni_adam_zero_grad": (C.c_int, [C.POINTER(Adam)]),
    "anni_adam_set_offload": (C.c_int, [C.POINTER(Adam), C.c_int]),
    "anni_adam_mv_on_device": (C.c_int, [C.POINTER(Adam)]),
    "anni_adam_quantize_grads": (C.c_int, [C.POINTER(Adam), C.c_void_p]),
    "anni_adam_quantize_grads_static": (C.c_int, [C.POINTER(Adam), C.c_void_p]),
    "anni_adam_step_scaled": (C.c_int, [C.POINTER(Adam), C.c_double, C.c_double]),
    "anni_adam_step": (C.c_int, [C.POINTER(Adam), C.c_double]),
    "anni_adam_sync_stats": (C.c_int, [C.POINTER(Adam)]),
    "anni_adam_export_mv": (C.c_int, [C.POINTER(Adam), C.c_int64, C.c_int64, C.c_void_p]),
    "anni_adam_import_mv": (C.c_int, [C.POINTER(Adam), C.c_int64, C.c_int64, C.c_void_p]),
    "anni_adam_write_state": (C.c_int, [C.POINTER(Adam), C.c_int, C.c_int, C.c_int]),
    "anni_adam_read_state": (C.c_int, [C.POINTER(Adam), C.c_int, C.POINTER(C.c_int),
                                       C.POINTER(C.c_int)]),
    "anni_adam_enable_derived": (C.c_int, [C.POINTER(Adam), C.POINTER(Pack), C.c_int, C.c_int64]),
    "anni_gpu_device_info": (C.c_int, [C.c_char_p, C.c_size_t, C.POINTER(C.c_int)]),
    "anni_lr_set_schedule": (None, [C.c_int, C.c_int, C.c_char_p]),
    "anni_lr_set_sched_from": (None, [C.c_int]),
    "anni_lr_set_override": (None, [C.c_double]),
    "anni_lr_step": (C.c_double, [C.c_double, C.c_int]),
    "anni_gpu_stream": (C.c_void_p, []),
    "anni_gpu_set_stream": (None, [C.c_void_p]),
    "anni_gpu_flush": (None, []),
    "anni_f32_to_bf16": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64]),
    "anni_fp8_quantize": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64]),
    "anni_colsum_add": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int]),
    "anni_colsum_add_batch": (C.c_int, [C.POINTER(Colsum), C.c_int]),
}

# include/anni_bench.h (libanni_bench.so)
_BENCH_PROTOS = {
    "anni_adam_time_steps": (C.c_int, [C.POINTER(Adam), C.c_int, C.POINTER(C.c_void_p),
                                       C.c_int, C.POINTER(C.c_double),
                                       C.POINTER(C.c_double), C.POINTER(C.c_float),
                                       C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "anni_adam_timed_derived_ms": (C.c_float, [C.POINTER(Adam)]),
    "anni_gpu_reload_switches": (None, []),
    "anni_fill_normal_f32": (C.c_int, [C.c_void_p, C.c_int64, C.c_uint64, C.c_uint64,
                                       C.c_float, C.c_float]),
    "anni_copy_bytes": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "anni_copy_bytes_tiled": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]),
    "anni_fold_guard_stats": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "anni_early_sum_stats": (C.c_int, [C.POINTER(C.c_long), C.POINTER(C.c_long)]),
    "anni_vectors_first_stats": (C.c_int, [C.POINTER(C.c_long), C.POINTER(C.c_long)]),
    "anni_second_stream_state": (C.c_int, []),
}

_lib = None


class _Both:
    """The product library with the bench library's entry points beside it: one object to call."""

    def __init__(self, product, bench):
        self._product, self._bench = product, bench

    def __getattr__(self, name):
        if name in _BENCH_PROTOS:
            return getattr(self._bench, name)
        return getattr(self._product, name)


def load():
    """Returns the loaded library with typed entry points; raises if it was not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise LibraryMissing(
                "%s is missing: build it with `make -C anni_amd/csrc` "
                "(or __graft_entry__.build()); there is no CPU fallback" % SO_PATH)
        if not os.path.exists(BENCH_SO_PATH):
            raise LibraryMissing("%s is missing: build it with `make -C anni_amd/csrc`" % BENCH_SO_PATH)
        L = C.CDLL(SO_PATH)
        B = C.CDLL(BENCH_SO_PATH)
        for lib_, protos in ((L, _PROTOS), (B, _BENCH_PROTOS)):
            for name, (res, args) in protos.items():
                fn = getattr(lib_, name)
                fn.restype = res
                fn.argtypes = args
        _lib = _Both(L, B)
    return _lib


def require_gpu():
    """The library plus a usable device, or an error that says which is missing."""
    L = load()
    if not L.gpu_available():
        raise RuntimeError("libanni_gpu_hip.so loaded but gpu_available() == 0: no HIP device")
    return L
