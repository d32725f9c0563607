"""The C-ABI library loads, exports every declared symbol, and answers as the headers say when
there is no device.  Host-only logic (the learning-rate schedule, the tensor layout) is checked
here too.  No compute calls: runs without a GPU."""
import ctypes as C
import glob
import os
import re

import numpy as np
import pytest

from helpers import GOLDEN

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_in(*headers):
    names = set()
    for h in headers:
        text = open(h).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b((?:gpu|anni)_[a-z0-9_]+)\s*\(", text))
    return names


def exported_by(so):
    import subprocess
    out = subprocess.check_output(["nm", "-D", "--defined-only", so]).decode()
    return {ln.split()[-1] for ln in out.splitlines() if ln.strip()}


def test_every_declared_symbol_is_exported_and_nothing_else():
    """libanni_gpu_hip.so exports exactly what anni_gpu.h, anni_gpu_unserved.h and anni_adam.h
    declare, plus the three hooks of the private header that libanni_bench.so is built on;
    libanni_bench.so exports exactly what anni_bench.h declares.  No C++ symbol, no measuring or
    testing utility in the product library."""
    from anni_amd import lib
    inc = os.path.join(ROOT, "include")
    product = declared_in(os.path.join(inc, "anni_gpu.h"), os.path.join(inc, "anni_gpu_unserved.h"),
                          os.path.join(inc, "anni_adam.h"))
    hooks = declared_in(os.path.join(ROOT, "anni_amd", "csrc", "anni_hooks.h"))
    bench = declared_in(os.path.join(inc, "anni_bench.h")) - product
    assert len([s for s in product if s.startswith("gpu_")]) == 99          # the whole of num/gpu.h
    assert hooks == {"anni_hook_step_events", "anni_hook_reload_switches", "anni_hook_counter"}
    assert exported_by(lib.SO_PATH) == product | hooks
    assert exported_by(lib.BENCH_SO_PATH) == bench
    assert set(glob.glob(os.path.join(inc, "*.h"))) == {os.path.join(inc, h) for h in
                                                        ("anni_gpu.h", "anni_gpu_unserved.h",
                                                         "anni_adam.h", "anni_bench.h")}
    for s_ in lib._PROTOS:
        assert s_ in product, s_
    for s_ in lib._BENCH_PROTOS:
        assert s_ in bench, s_


def test_missing_library_fails_loudly(monkeypatch):
    from anni_amd import lib
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "SO_PATH", "/nonexistent/libanni_gpu_hip.so")
    with pytest.raises(lib.LibraryMissing):
        lib.load()


def _no_device(L):
    return L.gpu_available() == 0


def test_without_a_device_every_entry_declines():
    from anni_amd import lib
    L = lib.load()
    if not _no_device(L):
        pytest.skip("a device is present")
    assert L.gpu_backend_name() == b"hip-gfx950"
    assert L.gpu_malloc(1024) is None
    assert L.gpu_host_alloc(1024) is None
    buf = np.zeros(16, np.float32)
    out = C.c_double(0)
    assert L.gpu_grad_sumsq(buf.ctypes.data, 16, C.byref(out)) == -1
    assert L.gpu_adam_step_dev_bf16(buf.ctypes.data, None, buf.ctypes.data, buf.ctypes.data,
                                    buf.ctypes.data, 16, 1e-3, 0.9, 0.95, 1e-8, 1, 1.0) == -1
    assert L.gpu_memcpy_h2d(buf.ctypes.data, buf.ctypes.data, 64) == -1
    assert L.gpu_memset(buf.ctypes.data, 0, 64) == -1
    assert L.gpu_stream_sync() == -1
    assert L.gpu_adam_seed_bf16_flat(buf.ctypes.data, buf.ctypes.data, 16) == -1
    L.gpu_device_sync()
    L.gpu_free(None)
    t = (lib.Tensor * 1)(lib.Tensor(16, 3))
    cfg = lib.Config(0, 0, 1, 0, 1)
    assert not L.anni_adam_create(t, 1, C.byref(cfg))
    assert L.anni_adam_step_scaled(None, 1e-3, 1.0) == -1


def test_unserved_symbols_answer_like_the_cpu_stub():
    from anni_amd import lib
    L = C.CDLL(lib.SO_PATH)
    for name in ("gpu_mat_mul", "gpu_mat_mul_bt", "gpu_graph_begin", "gpu_graph_replay"):
        fn = getattr(L, name)
        fn.restype = C.c_int
        assert fn(None, None, None) == -1
    for name, want in (("gpu_fp8", 0), ("gpu_graph_supported", 0), ("gpu_graph_replayable", 0),
                       ("gpu_ce_bias_fused", 0)):
        fn = getattr(L, name)
        fn.restype = C.c_int
        assert fn() == want
    L.gpu_attn_qkv_bwd.restype = C.c_int
    assert L.gpu_attn_qkv_bwd(None, None, None, None, None, None, None, None, None) == 1
    L.gpu_set_sync_mode(1)
    assert L.gpu_sync_mode() == 1
    L.gpu_set_sync_mode(0)
    L.gpu_copy_stream.restype = C.c_void_p
    assert L.gpu_copy_stream() is None


def test_weight_epoch_moves_on_invalidate():
    from anni_amd import lib
    L = lib.load()
    e0 = L.gpu_param_epoch()
    L.gpu_half_wt_invalidate(None)
    assert L.gpu_param_epoch() == e0 + 1


def test_lr_schedule_host_logic(oracle):
    from anni_amd import lm_adam
    # the reference's own known answers (tests/test_ann.c:866-879)
    f = lm_adam.step_lr
    assert abs(f(1.0, 29000, 100, 1000, "cosine", 0) - 0.0) < 1e-12
    assert abs(f(1.0, 29000, 100, 1000, "cosine", 29000) - 0.01) < 1e-12
    assert abs(f(1.0, 29099, 100, 1000, "cosine", 29000) - 1.0) < 1e-12
    assert abs(f(1.0, 29600, 100, 1000, "cosine", 29000) - 0.5) < 1e-12
    assert abs(f(1.0, 31000, 100, 1000, "cosine", 29000) - 0.0) < 1e-12
    assert abs(f(1.0, 10, 100, 1000, "cosine", 29000) - 0.01) < 1e-12
    # the table the compiled reference wrote, and the oracle, bit for bit
    T = np.load(os.path.join(GOLDEN, "lr_table.npz"))
    for row, case in zip(T["lr"], T["cases"]):
        w, d, k, frm = str(case).split(",")
        for s, want in zip(T["steps"], row):
            got = f(3e-4, int(s), int(w), int(d), k, int(frm))
            assert got == want == oracle.lr(3e-4, int(s), int(w), int(d), k, int(frm))
    # setters clamp negatives (lm_train.c:398-411)
    assert f(1.0, 5, -3, -7, "cosine", -2) == 1.0
    # the live control (train_control.lr, lm_train.c:104-105): > 0 wins over any schedule, <= 0 does not
    from anni_amd import lib
    L = lib.load()
    for ctl in (2.5e-5, 0.0, -1.0):
        L.anni_lr_set_override(ctl)
        for s in (0, 50, 600, 5000):
            got = f(3e-4, s, 100, 1000, "cosine", 0)
            want = ctl if ctl > 0 else oracle.lr(3e-4, s, 100, 1000, "cosine", 0)
            assert got == want
            if oracle.ref_available():
                R = oracle.ref()
                R.ref_step_lr_controlled.argtypes = [C.c_double, C.c_int, C.c_int, C.c_int, C.c_char_p, C.c_double]
                R.ref_step_lr_controlled.restype = C.c_double
                assert R.ref_step_lr_controlled(3e-4, s, 100, 1000, b"cosine", ctl) == got
    L.anni_lr_set_override(0.0)


def test_layout_parameter_counts():
    from anni_amd import layout
    assert layout.param_count("185m") == 167948288
    assert layout.param_count("555m") == 555848096
    assert layout.param_count("1p4b") == 1413498528
    assert layout.param_count("185m", "reference") == 167899136
    assert layout.param_count("555m", "reference") == 555762080
    assert layout.param_count("1p4b", "reference") == 1413301920
    assert len(layout.tensors("185m")) == 2 + 12 * 12
    assert len(layout.tensors("555m", "reference")) == 2 + 12 * 14
    mats = [t for t in layout.tensors("555m") if t[2]]
    assert all(n >= 1536 * 1536 for _nm, n, _f in mats)


def test_c99_caller_with_the_reference_flags(tmp_path):
    """include/*.h are plain C99 under the reference's own compiler flags (Makefile:21), and a C
    program links against the library and gets the schedule's known answers
    (tests/test_ann.c:866-879: 0.01 at step 0 of a 100-step warmup, 1.0 at step 99, 0.5 half way
    down the cosine, 0 at its end)."""
    import shutil
    import subprocess
    from anni_amd import lib
    if not shutil.which("gcc"):
        pytest.skip("no gcc")
    exe = str(tmp_path / "abi_probe")
    libdir = os.path.dirname(lib.SO_PATH)
    subprocess.check_call(["gcc", "-W", "-Wall", "-Werror", "-ansi", "-pedantic", "-std=c99", "-O2",
                           "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "c", "abi_probe.c"), "-o", exe,
                           "-L", libdir, "-lanni_gpu_hip", "-Wl,-rpath," + libdir, "-lm"])
    out = subprocess.check_output([exe], timeout=120).decode().splitlines()
    lr = [float(x) for x in out[0].split()[1:]]
    assert lr[0] == 0.01 and lr[1] == 1.0 and abs(lr[2] - 0.5) < 1e-15 and abs(lr[3]) < 1e-15
    assert out[1].startswith("backend hip-gfx950 available ")
    assert out[2].startswith("create declined") or out[2].startswith("create ok n 4160 t 1 norm 0")


def test_pool_chunk_bookkeeping_on_the_host(tmp_path):
    """The first-fit block bookkeeping of gpu_malloc's pools (anni_amd/csrc/pool_chunks.h) has no
    device call in it: a random sequence of 20000 takes and gives against a byte map."""
    import shutil
    import subprocess
    if not shutil.which("g++"):
        pytest.skip("no g++")
    exe = str(tmp_path / "pool_chunks_test")
    subprocess.check_call(["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", "-Werror",
                           "-I", os.path.join(ROOT, "anni_amd", "csrc"),
                           os.path.join(ROOT, "tests", "c", "pool_chunks_test.cpp"), "-o", exe])
    out = subprocess.check_output([exe], timeout=120).decode()
    assert out.startswith("ok takes "), out


def test_busy_flag_on_the_host(tmp_path):
    """The flag that lets one gpu_grad_sumsq at a time at the shared result slot
    (anni_amd/csrc/busy_flag.h) has no device call in it: eight threads, never two inside, a
    caller that finds it taken is refused, the flag is free after every scope."""
    import shutil
    import subprocess
    if not shutil.which("g++"):
        pytest.skip("no g++")
    exe = str(tmp_path / "busy_flag_test")
    subprocess.check_call(["g++", "-std=c++17", "-O2", "-Wall", "-Wextra", "-Werror", "-pthread",
                           "-I", os.path.join(ROOT, "anni_amd", "csrc"),
                           os.path.join(ROOT, "tests", "c", "busy_flag_test.cpp"), "-o", exe])
    out = subprocess.check_output([exe], timeout=120).decode()
    assert out.startswith("ok entered "), out


def test_division_by_a_step_constant_equals_the_ieee_quotient(tmp_path):
    """div_by_const (anni_amd/csrc/adam_math.h: q = a * (1/b), one residual folded back, the sign
    of a zero restored) restated on the host with fma() against a / b: b = 1 - beta^t for beta in
    {0.9, 0.95, 0.999}, t = 1..10000, 3570 float-valued numerators each from every binary exponent
    of a float, both signs, bf16-representable mantissas among them: 1.07e8 quotients, none may
    differ.  (Without the sign fix every -0 numerator differed: -0 / b is -0, the residual form
    gave +0.)"""
    import shutil
    import subprocess
    if not shutil.which("gcc"):
        pytest.skip("no gcc")
    exe = str(tmp_path / "div_by_const_test")
    subprocess.check_call(["gcc", "-O2", "-fopenmp", "-ffp-contract=off", "-Wall",
                           os.path.join(ROOT, "tests", "c", "div_by_const_test.c"), "-o", exe, "-lm"])
    out = subprocess.check_output([exe, "7"], timeout=600).decode().strip().splitlines()[-1]
    words = out.split()
    assert words[0] == "compared" and int(words[1]) >= 100000000, out
    assert words[2] == "mismatches" and int(words[3]) == 0, out
