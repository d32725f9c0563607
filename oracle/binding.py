"""ctypes binding of the CPU oracle (liboracle.so) and, where it was built, of the
reference's own compiled optimizer (oracle/_ref/libanni_ref.so).

Test infrastructure only: imported by tests, by the smoke check and by the
bench's cpu_baseline leg; never by the package that ships.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "liboracle.so")
REF_SO = os.path.join(HERE, "_ref", "libanni_ref.so")

F32, BF16, FP8 = 0, 1, 2
KIND = {"none": 0, "linear": 1, "cosine": 2}


class Seg(C.Structure):
    _fields_ = [("off", C.c_int64), ("n", C.c_int64), ("wd_on", C.c_int),
                ("gscale", C.c_float)]


class OracleAdam(C.Structure):
    _fields_ = [("n", C.c_int64), ("t", C.c_int), ("beta1", C.c_double),
                ("beta2", C.c_double), ("eps", C.c_double),
                ("weight_decay", C.c_double), ("grad_clip", C.c_double),
                ("skip_nonfinite", C.c_int), ("grad_type", C.c_int),
                ("moment_type", C.c_int), ("norm_threads", C.c_int),
                ("last_sumsq", C.c_double), ("last_grad_norm", C.c_double),
                ("last_grad_scale", C.c_double), ("last_clipped", C.c_int),
                ("last_skipped", C.c_int)]


def build(force=False):
    """Compile liboracle.so (and _ref when the reference tree is present)."""
    if force or not all(os.path.exists(os.path.join(HERE, f)) for f in
                        ("liboracle.so", "liboracle_avx2.so", "liboracle_avx512.so")):
        subprocess.check_call(["make", "-C", HERE, "-s"] + (["-B"] if force else []))


_libs = {}


def cpu_simd():
    """Widest of avx512 / avx2 / none that this CPU runs."""
    try:
        flags = open("/proc/cpuinfo").read()
    except OSError:
        return "none"
    if " avx512f" in flags and " avx512dq" in flags:
        return "avx512"
    if " avx2" in flags:
        return "avx2"
    return "none"


def lib(simd="none"):
    """The oracle library; simd = "avx2" / "avx512" selects the auto-vectorised build of the
    same source (bit-identical results, used for the CPU timing leg)."""
    so = ORACLE_SO if simd == "none" else os.path.join(HERE, "liboracle_%s.so" % simd)
    if so not in _libs:
        if not os.path.exists(so):
            build()
        L = C.CDLL(so)
        L.oracle_adam_defaults.argtypes = [C.POINTER(OracleAdam), C.c_int64]
        L.oracle_adam_step_scaled.argtypes = [
            C.POINTER(OracleAdam), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
            C.c_void_p, C.POINTER(Seg), C.c_int, C.c_double, C.c_double,
            C.POINTER(C.c_double), C.c_int]
        L.oracle_adam_step_scaled.restype = C.c_int
        L.oracle_sumsq.argtypes = [C.c_void_p, C.c_int, C.c_int64, C.POINTER(Seg),
                                   C.c_int, C.c_double, C.c_int]
        L.oracle_sumsq.restype = C.c_double
        L.oracle_lr.argtypes = [C.c_double, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        L.oracle_lr.restype = C.c_double
        L.oracle_bf16_rne.argtypes = [C.c_float]
        L.oracle_bf16_rne.restype = C.c_uint16
        L.oracle_fp8_decode.argtypes = [C.c_uint8]
        L.oracle_fp8_decode.restype = C.c_float
        L.oracle_fp8_encode.argtypes = [C.c_float]
        L.oracle_fp8_encode.restype = C.c_uint8
        L.oracle_fp8_scale_from_amax.argtypes = [C.c_float]
        L.oracle_fp8_scale_from_amax.restype = C.c_float
        L.oracle_fp8_quantize.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.oracle_fp8_quantize.restype = C.c_float
        L.oracle_f32_to_bf16.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        L.oracle_adam_step_slots.argtypes = [
            C.c_void_p, C.c_int64, C.c_int, C.c_double, C.c_double, C.c_double,
            C.c_double, C.c_double, C.c_double, C.c_double]
        L.oracle_max_threads.restype = C.c_int
        _libs[so] = L
    return _libs[so]


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def make_segs(tensors):
    """tensors: iterable of (off, n, wd_on, gscale) -> ctypes array."""
    arr = (Seg * len(tensors))()
    for i, (off, n, wd_on, gscale) in enumerate(tensors):
        arr[i] = Seg(off, n, int(wd_on), float(gscale))
    return arr


class Oracle:
    """Host optimizer state over flat numpy arrays, stepped by the C oracle."""

    def __init__(self, n, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0,
                 grad_clip=0.0, skip_nonfinite=False, grad_type=F32, moment_type=F32,
                 tensors=None, threads=1, norm_threads=1, simd="none"):
        self.o = OracleAdam()
        self.L = lib(simd)
        lib().oracle_adam_defaults(C.byref(self.o), n)
        self.o.beta1, self.o.beta2, self.o.eps = beta1, beta2, eps
        self.o.weight_decay, self.o.grad_clip = weight_decay, grad_clip
        self.o.skip_nonfinite = int(skip_nonfinite)
        self.o.grad_type, self.o.moment_type = grad_type, moment_type
        self.o.norm_threads = norm_threads
        self.threads = threads
        self.segs = make_segs(tensors) if tensors is not None else None
        self.nsegs = len(tensors) if tensors is not None else 0

    def set_gscales(self, scales):
        for i, s in enumerate(scales):
            self.segs[i].gscale = float(s)

    def step(self, p, g, m, v, lr, grad_scale=1.0, twin=None, sumsq_override=None):
        ov = None
        if sumsq_override is not None:
            ov = C.byref(C.c_double(float(sumsq_override)))
        return self.L.oracle_adam_step_scaled(
            C.byref(self.o), _ptr(p), _ptr(g), _ptr(m), _ptr(v), _ptr(twin),
            self.segs, self.nsegs, lr, grad_scale, ov, self.threads)

    @property
    def t(self):
        return self.o.t


def sumsq(g, grad_type=F32, tensors=None, grad_scale=1.0, threads=1):
    segs = make_segs(tensors) if tensors is not None else None
    return lib().oracle_sumsq(_ptr(g), grad_type, g.size, segs,
                              len(tensors) if tensors is not None else 0, grad_scale,
                              threads)


def lr(base_lr, step, warmup=0, decay_steps=0, kind="none", sched_from=0):
    return lib().oracle_lr(base_lr, step, warmup, decay_steps, KIND[kind], sched_from)


def bf16_rne(x):
    """float32 array -> uint16 array (round to nearest even)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_f32_to_bf16(_ptr(out), _ptr(x), x.size)
    return out


def same_bytes(a, b):
    """True when two arrays of the same size hold the same bytes (threaded memcmp)."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    if a.nbytes != b.nbytes:
        return False
    L = lib()
    L.oracle_same_bytes.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
    L.oracle_same_bytes.restype = C.c_int
    return bool(L.oracle_same_bytes(_ptr(a), _ptr(b), a.nbytes))


def compare(a, b, tol):
    """a against b, float32 arrays or bf16 bit patterns (uint16): (max |a-b| / max(|b|, rms(b)),
    number of elements with |a-b| > tol*|b|, the largest |b| among those)."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    assert a.dtype == b.dtype and a.size == b.size and a.dtype in (np.float32, np.uint16)
    L = lib()
    L.oracle_compare.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int64, C.c_double,
                                 C.POINTER(C.c_double)]
    L.oracle_compare.restype = None
    out = (C.c_double * 3)()
    L.oracle_compare(_ptr(a), _ptr(b), BF16 if a.dtype == np.uint16 else F32, a.size, tol, out)
    return out[0], int(out[1]), out[2]


def bf16_widen(h):
    return (h.astype(np.uint32) << 16).view(np.float32)


def fp8_decode_table():
    return np.array([lib().oracle_fp8_decode(q) for q in range(256)], dtype=np.float32)


def colsum_add(acc, x, y=None):
    """acc[j] += column sums of the 2-D float32 array x (of x * y), in place, host-loop order."""
    assert acc.dtype == np.float32 and x.dtype == np.float32 and x.flags.c_contiguous
    rows, cols = x.shape
    assert acc.size == cols and (y is None or (y.shape == x.shape and y.dtype == np.float32))
    L = lib()
    L.oracle_colsum_add.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
    L.oracle_colsum_add.restype = None
    L.oracle_colsum_add(_ptr(acc), _ptr(x), _ptr(y) if y is not None else None, rows, cols)
    return acc


def ref_ln_backward_grads(dy, x_hat, dgamma, dbeta):
    """The compiled reference's layernorm_backward: accumulates into dgamma / dbeta in place."""
    R = ref()
    R.ref_ln_backward_grads.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
    R.ref_ln_backward_grads.restype = C.c_int
    assert dy.dtype == np.float32 and dy.shape == x_hat.shape and dy.flags.c_contiguous
    d = R.ref_ln_backward_grads(_ptr(dy), _ptr(x_hat), dy.shape[0], _ptr(dgamma), _ptr(dbeta))
    if d != dy.shape[1]:
        raise RuntimeError("ref_ln_backward_grads: %d" % d)


def fp8_quantize(x):
    """float32 tensor -> (uint8 codes, float scale) by the per-tensor amax convention."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    q = np.empty(x.shape, dtype=np.uint8)
    scale = lib().oracle_fp8_quantize(_ptr(q), _ptr(x), x.size)
    return q, np.float32(scale)


# ---- the reference's own compiled optimizer (present only where it was built) ----

_ref = None


def ref_available():
    return os.path.exists(REF_SO)


def ref():
    global _ref
    if _ref is None:
        R = C.CDLL(REF_SO)
        R.ref_adam_create.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_long, C.c_int, C.c_double, C.c_double,
                                      C.c_double, C.c_double, C.c_double]
        R.ref_adam_create.restype = C.c_void_p
        R.ref_adam_step.argtypes = [C.c_void_p, C.c_double, C.c_double]
        R.ref_adam_step.restype = C.c_int
        R.ref_adam_set.argtypes = [C.c_void_p, C.c_double, C.c_double]
        R.ref_adam_export.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        R.ref_adam_free.argtypes = [C.c_void_p]
        R.ref_step_lr.argtypes = [C.c_double, C.c_int, C.c_int, C.c_int, C.c_char_p,
                                  C.c_int]
        R.ref_step_lr.restype = C.c_double
        _ref = R
    return _ref


class RefAdam:
    """The reference's lm_adam_step_scaled (host path) over flat numpy arrays."""

    def __init__(self, p, g, m=None, v=None, t=0, beta1=0.9, beta2=0.999, eps=1e-8,
                 weight_decay=0.0, grad_clip=0.0):
        self.p, self.g = p, g
        self.h = ref().ref_adam_create(_ptr(p), _ptr(g), _ptr(m), _ptr(v), p.size, t,
                                       beta1, beta2, eps, weight_decay, grad_clip)
        if not self.h:
            raise MemoryError("ref_adam_create")

    def step(self, lr, grad_scale=1.0):
        return ref().ref_adam_step(self.h, lr, grad_scale)

    def moments(self):
        m = np.empty(self.p.size, dtype=np.float32)
        v = np.empty(self.p.size, dtype=np.float32)
        ref().ref_adam_export(self.h, _ptr(m), _ptr(v))
        return m, v

    def close(self):
        if self.h:
            ref().ref_adam_free(self.h)
            self.h = None

    def __del__(self):
        self.close()


def ref_lr(base_lr, step, warmup=0, decay_steps=0, kind="none", sched_from=0):
    return ref().ref_step_lr(base_lr, step, warmup, decay_steps, kind.encode(), sched_from)


# ---- the reference's compiled optimizer linked against THIS repository's HIP backend ----

REF_HIP_SO = os.path.join(HERE, "_ref", "libanni_ref_hip.so")
_ref_hip = None


def ref_hip_available():
    return os.path.exists(REF_HIP_SO)


def ref_hip():
    global _ref_hip
    if _ref_hip is None:
        R = C.CDLL(REF_HIP_SO)
        R.ref_adam_create_device.argtypes = [C.c_void_p, C.c_void_p, C.c_long, C.c_double,
                                             C.c_double, C.c_double, C.c_double, C.c_double]
        R.ref_adam_create_device.restype = C.c_void_p
        R.ref_adam_step.argtypes = [C.c_void_p, C.c_double, C.c_double]
        R.ref_adam_step.restype = C.c_int
        R.ref_adam_sync_host.argtypes = [C.c_void_p]
        R.ref_adam_last_norm.argtypes = [C.c_void_p]
        R.ref_adam_last_norm.restype = C.c_double
        R.ref_adam_on_device.argtypes = [C.c_void_p]
        R.ref_adam_on_device.restype = C.c_int
        R.ref_adam_release_device.argtypes = [C.c_void_p]
        R.ref_adam_export.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        R.ref_adam_free.argtypes = [C.c_void_p]
        _declare_model(R)
        _ref_hip = R
    return _ref_hip


def _declare_model(R):
    R.ref_model_create.argtypes = [C.c_int, C.c_double, C.c_double, C.c_double]
    R.ref_model_create.restype = C.c_void_p
    R.ref_model_create_tied.argtypes = [C.c_int, C.c_double, C.c_double, C.c_double]
    R.ref_model_create_tied.restype = C.c_void_p
    R.ref_model_dims.argtypes = [C.POINTER(C.c_int)] * 4
    R.ref_model_n.argtypes = [C.c_void_p]
    R.ref_model_n.restype = C.c_long
    for f in ("ref_model_n_segs", "ref_model_t", "ref_model_on_device"):
        getattr(R, f).argtypes = [C.c_void_p]
        getattr(R, f).restype = C.c_int
    R.ref_model_last_norm.argtypes = [C.c_void_p]
    R.ref_model_last_norm.restype = C.c_double
    R.ref_model_seg.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_long), C.POINTER(C.c_long),
                                C.POINTER(C.c_int)]
    R.ref_model_get_params.argtypes = [C.c_void_p, C.c_void_p]
    R.ref_model_get_moments.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
    R.ref_model_set_grads.argtypes = [C.c_void_p, C.c_void_p]
    R.ref_model_set_grads.restype = C.c_int
    R.ref_model_step.argtypes = [C.c_void_p, C.c_double, C.c_double]
    R.ref_model_step.restype = C.c_int
    R.ref_model_save_checkpoint.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_char_p]
    R.ref_model_save_checkpoint.restype = C.c_int
    R.ref_model_load_checkpoint.argtypes = [C.c_char_p, C.POINTER(C.c_int), C.POINTER(C.c_int)]
    R.ref_model_load_checkpoint.restype = C.c_void_p
    R.ref_model_free.argtypes = [C.c_void_p]
    R.ref_set_offload.argtypes = [C.c_int]
    R.ref_model_mv_on_device.argtypes = [C.c_void_p]


# The same library compiled with the model sizes of the reference's 555M run
# (scripts/run555m.sh:39-42: D=1536, 24 heads, FF=6272, 14 blocks).
REF_HIP_555M_SO = os.path.join(HERE, "_ref", "libanni_ref_555m_hip.so")
_ref_hip_555m = None


def ref_hip_555m_available():
    return os.path.exists(REF_HIP_555M_SO)


def ref_hip_555m():
    global _ref_hip_555m
    if _ref_hip_555m is None:
        R = C.CDLL(REF_HIP_555M_SO)
        _declare_model(R)
        _ref_hip_555m = R
    return _ref_hip_555m


# The same two flavours with the call-timing interposer (gputrace.c) linked in front of the backend.
REF_TRACE_SO = {"hip_trace": os.path.join(HERE, "_ref", "libanni_ref_hip_trace.so"),
                "hip555m_trace": os.path.join(HERE, "_ref", "libanni_ref_555m_hip_trace.so")}
GPUTRACE_SO = os.path.join(HERE, "_ref", "libgputrace.so")
_ref_trace = {}
_gputrace = None


def ref_trace_available():
    return os.path.exists(GPUTRACE_SO) and all(os.path.exists(p) for p in REF_TRACE_SO.values())


def ref_trace(flavour):
    """The traced flavour "hip_trace" / "hip555m_trace" of the compiled reference."""
    if flavour not in _ref_trace:
        os.environ.setdefault("ANNI_HIP_SO", os.path.join(os.path.dirname(HERE), "anni_amd",
                                                          "libanni_gpu_hip.so"))
        R = C.CDLL(REF_TRACE_SO[flavour])
        _declare_model(R)
        _ref_trace[flavour] = R
    return _ref_trace[flavour]


def gputrace():
    """The interposer's own entry points: start / stop recording, and the recorded calls."""
    global _gputrace
    if _gputrace is None:
        T = C.CDLL(GPUTRACE_SO)
        T.gputrace_get.argtypes = [C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_double),
                                   C.POINTER(C.c_double), C.POINTER(C.c_size_t)]
        T.gputrace_name.restype = C.c_char_p
        T.gputrace_name.argtypes = [C.c_int]
        _gputrace = T
    return _gputrace


def gputrace_events():
    """[(name, start us, end us, bytes)] of the calls recorded since gputrace_start."""
    T = gputrace()
    out = []
    for i in range(T.gputrace_count()):
        a, b, c, d = C.c_int(), C.c_double(), C.c_double(), C.c_size_t()
        T.gputrace_get(i, C.byref(a), C.byref(b), C.byref(c), C.byref(d))
        out.append((T.gputrace_name(a.value).decode(), b.value, c.value, d.value))
    return out


_ref_cpu_model = None


def ref_cpu_model_lib():
    """The reference compiled with its own CPU stub backend, model entry points declared."""
    global _ref_cpu_model
    if _ref_cpu_model is None:
        if not os.path.exists(REF_SO):
            raise FileNotFoundError(REF_SO)
        R = C.CDLL(REF_SO)
        _declare_model(R)
        _ref_cpu_model = R
    return _ref_cpu_model


class RefModelOnBackend:
    """The reference's real lm + lm_adam_create on libanni_gpu_hip.so, at its compile-time 185M
    sizes (backend="hip") or at those of its 555M run (backend="hip555m"), or on its own CPU stub
    (backend="cpu").  tied=True shares the head matrix with the embedding (lm_create_bpe_tied, what
    `--tied` selects in the reference's training scripts)."""

    def __init__(self, vocab=16384, beta2=0.95, weight_decay=0.1, grad_clip=1.0, backend="hip",
                 _handle=None, tied=False):
        self.R = (ref_hip() if backend == "hip" else ref_hip_555m() if backend == "hip555m"
                  else ref_trace(backend) if backend in REF_TRACE_SO else ref_cpu_model_lib())
        create = self.R.ref_model_create_tied if tied else self.R.ref_model_create
        self.h = _handle or create(vocab, beta2, weight_decay, grad_clip)
        if not self.h:
            raise MemoryError("ref_model_create")
        self.n = self.R.ref_model_n(self.h)
        self.n_segs = self.R.ref_model_n_segs(self.h)

    @classmethod
    def load_checkpoint(cls, path, backend="hip"):
        """lm_load_checkpoint: returns (model, epoch, step), or raises when the loader refuses the file."""
        R = ref_hip() if backend == "hip" else ref_cpu_model_lib()
        ep, st = C.c_int(-1), C.c_int(-1)
        h = R.ref_model_load_checkpoint(os.fsencode(path), C.byref(ep), C.byref(st))
        if not h:
            raise ValueError("lm_load_checkpoint refused " + str(path))
        return cls(backend=backend, _handle=h), ep.value, st.value

    def dims(self):
        """(d_model, heads, d_ff, blocks) the library was compiled with."""
        v = [C.c_int(0) for _ in range(4)]
        self.R.ref_model_dims(*[C.byref(x) for x in v])
        return tuple(x.value for x in v)

    def save_checkpoint(self, path, epoch, step):
        if self.R.ref_model_save_checkpoint(self.h, epoch, step, os.fsencode(path)) != 0:
            raise RuntimeError("lm_save_checkpoint")

    @property
    def t(self):
        return self.R.ref_model_t(self.h)

    def segs(self):
        out = []
        off, n, im = C.c_long(0), C.c_long(0), C.c_int(0)
        for i in range(self.n_segs):
            self.R.ref_model_seg(self.h, i, C.byref(off), C.byref(n), C.byref(im))
            out.append((off.value, n.value, bool(im.value)))
        return out

    def params(self):
        p = np.empty(self.n, np.float32)
        self.R.ref_model_get_params(self.h, _ptr(p))
        return p

    def moments(self):
        m = np.empty(self.n, np.float32)
        v = np.empty(self.n, np.float32)
        self.R.ref_model_get_moments(self.h, _ptr(m), _ptr(v))
        return m, v

    def set_grads(self, g):
        assert g.dtype == np.float32 and g.size == self.n
        if self.R.ref_model_set_grads(self.h, _ptr(g)) != 0:
            raise RuntimeError("ref_model_set_grads")

    def step(self, lr, grad_scale=1.0):
        return self.R.ref_model_step(self.h, lr, grad_scale)

    @property
    def on_device(self):
        return bool(self.R.ref_model_on_device(self.h))

    @property
    def last_grad_norm(self):
        return self.R.ref_model_last_norm(self.h)

    def device_flats(self):
        """(d_param, d_param_bf16) of the caller's optimizer, as integers."""
        for name in ("ref_model_d_param", "ref_model_d_param_bf16"):
            fn = getattr(self.R, name)
            fn.argtypes = [C.c_void_p]
            fn.restype = C.c_void_p
        return self.R.ref_model_d_param(self.h), self.R.ref_model_d_param_bf16(self.h)

    def set_offload(self, on):
        """lm_adam_set_offload: a process-wide switch of the reference."""
        self.R.ref_set_offload(int(on))

    @property
    def mv_on_device(self):
        return bool(self.R.ref_model_mv_on_device(self.h))

    def close(self):
        if self.h:
            self.R.ref_model_free(self.h)
            self.h = None


class RefAdamOnBackend:
    """The unchanged lm_adam_step_scaled taking its device path on libanni_gpu_hip.so."""

    def __init__(self, p, g, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, grad_clip=0.0):
        self.p, self.g = p, g
        self.h = ref_hip().ref_adam_create_device(_ptr(p), _ptr(g), p.size, beta1, beta2, eps,
                                                  weight_decay, grad_clip)
        if not self.h:
            raise MemoryError("ref_adam_create_device")

    def step(self, lr, grad_scale=1.0):
        return ref_hip().ref_adam_step(self.h, lr, grad_scale)

    @property
    def last_grad_norm(self):
        return ref_hip().ref_adam_last_norm(self.h)

    @property
    def on_device(self):
        return bool(ref_hip().ref_adam_on_device(self.h))

    def moments(self):
        ref_hip().ref_adam_sync_host(self.h)
        m = np.empty(self.p.size, dtype=np.float32)
        v = np.empty(self.p.size, dtype=np.float32)
        ref_hip().ref_adam_export(self.h, _ptr(m), _ptr(v))
        return m, v

    def close(self):
        if self.h:
            ref_hip().ref_adam_release_device(self.h)
            ref_hip().ref_adam_free(self.h)
            self.h = None
