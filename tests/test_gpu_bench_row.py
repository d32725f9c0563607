"""The bench-log row on the GPU: bench.py --ref-jsonl appends a row in the reference's schema whose
adam phase is the row's p50, and the reference's own bench harness (lm_bench_step, compiled from the
reference tree with the small model of its unit tests and linked against this backend) runs a
whole packed training step on this backend and writes the row the fixture was taken from."""
import json
import os
import subprocess
import sys

import pytest

from anni_amd import bench_row

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_appends_a_row_in_the_references_schema(gpu, tmp_path):
    path = str(tmp_path / "bench" / "results.jsonl")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "185m",
                        "--no-cpu", "--steps", "6", "--warmup", "2", "--ref-jsonl", path],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    rows = [json.loads(ln) for ln in open(path).read().splitlines()]
    assert len(rows) == 1
    row = rows[0]
    assert row["mode"] == "step" and row["cfg"]["phase"] == "adam" and row["cfg"]["workload"] == "185m"
    assert row["cfg"]["steps"] == 6 and row["cfg"]["warmup"] == 2 and row["cfg"]["prec"] == "fp32"
    assert row["phase_ms"]["adam"] == row["ms"]["p50"] > 0
    assert row["phase_ms"]["fwd"] == row["phase_ms"]["loss"] == row["phase_ms"]["bwd"] == -1.0
    assert row["ms"]["p10"] <= row["ms"]["p50"] <= row["ms"]["p90"]
    assert row["loss_ok"] is True and row["backend"] == "hip-gfx950" and "gfx950" in row["gpu"]
    assert row["params"] == line["config"]["params"] == 167948288
    assert row["model"] == {"D": 1024, "L": 12, "H": 16, "FF": 4096}
    assert abs(row["ms"]["p50"] - line["ms_per_step"]) < 0.25 * line["ms_per_step"]
    # the line on disk is in the reference writer's format: printed back it is itself
    assert bench_row.format_row(row) == open(path).read().splitlines()[0]
    assert line["ref_jsonl_row"] == row


def test_the_references_bench_harness_runs_on_this_backend(gpu, oracle, tmp_path):
    """`anni lm bench step --profile --json` (lang/lm_bench.c:619-643) through its library entry
    point: a real packed training step of the reference's model code -- forward, loss, backward on
    its host paths (this backend answers -1 for what it does not serve), the optimizer phase on
    this backend -- with a falling loss, and one appended row that our writer reproduces."""
    import ctypes as C
    so = os.path.join(ROOT, "oracle", "_ref", "libanni_ref_small_hip.so")
    if not os.path.exists(so):
        pytest.skip("oracle/_ref/libanni_ref_small_hip.so not built (reference tree absent at build time)")
    R = C.CDLL(so)
    R.ref_bench_step.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    R.ref_bench_step.restype = C.c_int
    path = str(tmp_path / "row.jsonl")
    assert R.ref_bench_step(os.fsencode(path), 4, 32, 512, 2, 12) == 0      # 0: its loss check passed
    lines = open(path).read().splitlines()
    assert len(lines) == 1
    row = json.loads(lines[0])
    assert bench_row.format_row(row) == lines[0]
    ref = json.loads(open(os.path.join(ROOT, "tests", "golden", "bench_row_ref.jsonl")).read())
    assert list(row) == list(ref) and list(row["cfg"]) == list(ref["cfg"])
    assert row["cfg"] == ref["cfg"] and row["model"] == ref["model"]
    assert row["loss"] == ref["loss"]                       # same seed, same arithmetic: the same losses
    assert row["backend"] == "hip-gfx950" and row["phase_ms"]["adam"] > 0 and row["loss_ok"] is True
    assert bench_row.compare_key(row) == bench_row.compare_key(ref)
    gpu.gpu_set_compute_prec(0)
    gpu.gpu_adam_set_weight_decay(0.0)
