"""Host-side mirror of the reference's lm_adam interface over the device arena.

Names and argument meaning follow lang/lm_adam.h:56-78 (create, step,
step_scaled, zero_grad, free) and lang/lm_train.c:98-124 (step_lr); the work is
done by libanni_gpu_hip.so through its C ABI (include/anni_adam.h).  numpy is
used only to move test data; nothing here computes the update.
"""
import ctypes as C

import numpy as np

from . import lib as _l

_NP = {_l.F32: np.float32, _l.BF16: np.uint16, _l.FP8_E4M3: np.uint8}


def step_lr(base_lr, step, warmup=0, decay_steps=0, kind="none", sched_from=0):
    """lm_train_step_lr with its setters applied first (lang/lm_train.c:98-124,398-411)."""
    L = _l.load()
    L.anni_lr_set_schedule(warmup, decay_steps, kind.encode())
    L.anni_lr_set_sched_from(sched_from)
    return L.anni_lr_step(base_lr, step)


class DeviceBuffer:
    """A gpu_malloc'ed range (freed with gpu_free)."""

    def __init__(self, nbytes):
        self.L = _l.require_gpu()
        self.nbytes = int(nbytes)
        self.ptr = self.L.gpu_malloc(self.nbytes)
        if not self.ptr:
            raise MemoryError("gpu_malloc(%d)" % self.nbytes)

    def upload(self, arr, offset=0):
        arr = np.ascontiguousarray(arr)
        assert offset + arr.nbytes <= self.nbytes
        if arr.nbytes and self.L.gpu_memcpy_h2d(self.ptr + offset, arr.ctypes.data,
                                                arr.nbytes) != 0:
            raise RuntimeError("gpu_memcpy_h2d failed")
        if self.L.gpu_stream_sync() != 0:
            raise RuntimeError("gpu_stream_sync failed")

    def download(self, dtype, count, offset=0):
        out = np.empty(count, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        if out.nbytes and self.L.gpu_memcpy_d2h(out.ctypes.data, self.ptr + offset,
                                                out.nbytes) != 0:
            raise RuntimeError("gpu_memcpy_d2h failed")
        return out

    def free(self):
        if self.ptr:
            self.L.gpu_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class PinnedArray:
    """A numpy array in page-locked host memory (gpu_host_alloc / gpu_host_free): device copies to
    and from it run at the host link's rate, several times that of copies through pageable memory."""

    def __init__(self, dtype, count):
        self.L = _l.require_gpu()
        self.nbytes = int(count) * np.dtype(dtype).itemsize
        self.ptr = self.L.gpu_host_alloc(max(self.nbytes, 1))
        if not self.ptr:
            raise MemoryError("gpu_host_alloc(%d)" % self.nbytes)
        buf = (C.c_char * self.nbytes).from_address(self.ptr)
        self.a = np.frombuffer(buf, dtype=dtype, count=int(count))

    def free(self):
        if self.ptr:
            self.a = None
            self.L.gpu_host_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class LmAdam:
    """lm_adam over a list of tensors ((n, flags) pairs or (name, n, flags) triples)."""

    def __init__(self, tensors, grad_type=_l.F32, moment_type=_l.F32, twins=True,
                 skip_nonfinite=False, grad_slots=1, layout=_l.LAYOUT_AUTO, beta1=0.9, beta2=0.999, eps=1e-8,
                 weight_decay=0.0, grad_clip=0.0):
        self.L = _l.require_gpu()
        rows = [(t[-2], t[-1]) for t in tensors]
        self.names = [t[0] if len(t) == 3 else "t%d" % i for i, t in enumerate(tensors)]
        arr = (_l.Tensor * len(rows))(*[_l.Tensor(int(n), int(f)) for n, f in rows])
        cfg = _l.Config(grad_type, moment_type, int(twins), int(skip_nonfinite), int(grad_slots),
                         int(layout))
        self.h = self.L.anni_adam_create(arr, len(rows), C.byref(cfg))
        if not self.h:
            raise RuntimeError("anni_adam_create failed: %s"
                               % self.L.gpu_debug_last_error().decode())
        self.grad_type, self.moment_type = grad_type, moment_type
        o = self.h.contents
        o.beta1, o.beta2, o.eps = beta1, beta2, eps
        o.weight_decay, o.grad_clip = weight_decay, grad_clip
        self.sizes = [n for n, _f in rows]
        self.offsets = [self.L.anni_adam_tensor_offset(self.h, i) for i in range(len(rows))]

    # -- the reference's public fields ------------------------------------------------
    @property
    def o(self):
        return self.h.contents

    @property
    def n(self):
        return self.o.n

    @property
    def t(self):
        return self.o.t

    # -- the reference's functions ------------------------------------------------------
    def step_scaled(self, lr, grad_scale=1.0):
        rc = self.L.anni_adam_step_scaled(self.h, lr, grad_scale)
        if rc < 0:
            raise RuntimeError("anni_adam_step_scaled failed: %s"
                               % self.L.gpu_debug_last_error().decode())
        return rc

    def step(self, lr):
        return self.step_scaled(lr, 1.0)

    def zero_grad(self):
        if self.L.anni_adam_zero_grad(self.h) != 0:
            raise RuntimeError("anni_adam_zero_grad failed")

    def seed_twins(self):
        if self.L.anni_adam_seed_twins(self.h) != 0:
            raise RuntimeError("anni_adam_seed_twins failed")

    def enable_derived(self, packs=(), pack_elems=0):
        """packs: (tensor, cols, dst_offset, dst_stride) tuples; E4M3 twins follow the tensor flags."""
        arr = (_l.Pack * max(len(packs), 1))(*[_l.Pack(*[int(x) for x in pk]) for pk in packs])
        if self.L.anni_adam_enable_derived(self.h, arr if packs else None, len(packs),
                                           int(pack_elems)) != 0:
            raise RuntimeError("anni_adam_enable_derived refused")
        self.pack_elems = int(pack_elems)

    def sync_stats(self):
        if self.L.anni_adam_sync_stats(self.h) != 0:
            raise RuntimeError("anni_adam_sync_stats failed")
        return self.o

    def grad_slot(self, k):
        return self.L.anni_adam_grad_slot(self.h, k)

    @property
    def split(self):
        return bool(self.L.anni_adam_is_split(self.h))

    @property
    def apart_ratio(self):
        return self.L.anni_adam_apart_ratio(self.h)

    @property
    def arena_bytes(self):
        return self.L.anni_adam_arena_bytes(self.h)

    @property
    def resident_bytes(self):
        return self.L.anni_adam_resident_bytes(self.h)

    @property
    def probe_gbps(self):
        return self.L.anni_adam_probe_gbps(self.h)

    @property
    def placement_cost(self):
        """(GiB walked, milliseconds, candidates timed) of the search for the second block."""
        gib, ms = C.c_double(0), C.c_double(0)
        timed = self.L.anni_adam_placement_cost(self.h, C.byref(gib), C.byref(ms))
        return gib.value, ms.value, timed

    def bind_grad(self, ptr):
        if self.L.anni_adam_bind_grad(self.h, ptr) != 0:
            raise RuntimeError("anni_adam_bind_grad failed")

    # -- the optimizer block of a checkpoint (lang/lm_serialize.c:263-331,526-587) -----------
    def export_mv(self, first=0, count=None):
        """(m, v) float pairs of slots [first, first+count) as a (count, 2) array."""
        count = self.n - first if count is None else count
        out = np.empty((count, 2), np.float32)
        if self.L.anni_adam_export_mv(self.h, first, count, out.ctypes.data) != 0:
            raise RuntimeError("anni_adam_export_mv failed")
        return out

    def import_mv(self, pairs, first=0):
        pairs = np.ascontiguousarray(pairs, dtype=np.float32).reshape(-1, 2)
        if self.L.anni_adam_import_mv(self.h, first, pairs.shape[0], pairs.ctypes.data) != 0:
            raise RuntimeError("anni_adam_import_mv failed")

    def write_state(self, fd, epoch, step):
        """has_adam, epoch, step, t, n and the n pairs, as lm_save_checkpoint writes them."""
        if self.L.anni_adam_write_state(self.h, fd, epoch, step) != 0:
            raise RuntimeError("anni_adam_write_state failed")

    def read_state(self, fd):
        """Reads the block lm_load_checkpoint reads; restores t; returns (epoch, step)."""
        ep, st = C.c_int(-1), C.c_int(-1)
        if self.L.anni_adam_read_state(self.h, fd, C.byref(ep), C.byref(st)) != 0:
            raise ValueError("anni_adam_read_state refused the block")
        return ep.value, st.value

    def free(self):
        if getattr(self, "h", None):
            hp = C.POINTER(_l.Adam)(self.h.contents)
            self.L.anni_adam_free(C.byref(hp))
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    # -- test / bench data movement --------------------------------------------------------
    def _flat(self, which):
        o = self.o
        return {"param": (o.d_param, np.float32), "grad": (o.d_grad, _NP[self.grad_type]),
                "m": (o.d_m, _NP[self.moment_type]), "v": (o.d_v, _NP[self.moment_type]),
                "twin": (o.d_param_bf16, np.uint16), "gscale": (o.d_gscale, np.float32),
                "fp8twin": (o.d_param_fp8, np.uint8), "wscale": (o.d_wscale, np.float32),
                "pack": (o.d_pack_bf16, np.uint16)}[which]

    def upload(self, which, arr, offset=0):
        ptr, dt = self._flat(which)
        arr = np.ascontiguousarray(arr, dtype=dt)
        if self.L.gpu_memcpy_h2d(ptr + offset * arr.itemsize, arr.ctypes.data, arr.nbytes) != 0 \
                or self.L.gpu_stream_sync() != 0:
            raise RuntimeError("upload(%s) failed" % which)

    def download_into(self, which, out, offset=0):
        """The flat `which` from element `offset` on into the array `out` (its size and type decide how much)."""
        ptr, dt = self._flat(which)
        assert out.dtype == dt and out.flags.c_contiguous
        if self.L.gpu_memcpy_d2h(out.ctypes.data, ptr + offset * out.itemsize, out.nbytes) != 0:
            raise RuntimeError("download(%s) failed" % which)
        return out

    def download(self, which, count=None, offset=0):
        ptr, dt = self._flat(which)
        if count is None:
            count = (self.o.n_tensors if which in ("gscale", "wscale")
                     else self.pack_elems if which == "pack" else self.n)
        out = np.empty(count, dtype=dt)
        if self.L.gpu_memcpy_d2h(out.ctypes.data, ptr + offset * out.itemsize, out.nbytes) != 0:
            raise RuntimeError("download(%s) failed" % which)
        return out
