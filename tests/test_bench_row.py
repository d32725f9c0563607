"""The bench-log row of the optimizer phase (anni_amd/bench_row.py) against the reference's schema
(lang/lm_bench.c:224-246 statistics, :378-387 head, :586-608 step body) and against the way
scripts/bench_compare.py matches and scores rows.  No GPU: the environment probe is given."""
import json

from anni_amd import bench_row

ENV = {"git": "abc1234", "dirty": False, "backend": "hip", "gpu": "AMD Instinct MI355X (gfx950)",
       "driver": "70200000", "vram_mb": 294896, "busy": False}

# keys the reference prints, in its own order
HEAD_KEYS = ["mode", "git", "dirty", "backend", "gpu", "driver", "vram_mb", "busy", "time", "model"]
CFG_KEYS = ["V", "B", "B_req", "T", "prec", "attn", "graphs", "ckpt", "offload", "warmup", "steps",
            "lr"]
BODY_KEYS = ["ms", "tok_s", "tf_model", "tf_hw", "ceiling_tf", "mfu", "vram_peak_mb", "loss",
             "loss_ok", "phase_ms"]


def test_nearest_rank_statistics():
    # n = 10: p10 = v[0], p50 = v[4], p90 = v[9] (index rules of stats_of)
    v = [5.0, 1.0, 9.0, 3.0, 7.0, 2.0, 8.0, 4.0, 10.0, 6.0]
    s = bench_row.stats_of(v)
    assert (s["p10"], s["p50"], s["p90"]) == (1.0, 5.0, 10.0)
    assert s["mean"] == 5.5
    assert abs(s["cv"] - (sum((x - 5.5) ** 2 for x in v) / 9) ** 0.5 / 5.5) < 1e-15
    # n = 1: everything is the value, cv 0; n = 0: zeros
    assert bench_row.stats_of([3.5]) == {"p10": 3.5, "p50": 3.5, "p90": 3.5, "mean": 3.5, "cv": 0.0}
    assert bench_row.stats_of([])["p50"] == 0.0
    # n = 21: (n-1)/10 = 2, (n-1)/2 = 10, (9*20+9)/10 = 18
    s = bench_row.stats_of(range(21))
    assert (s["p10"], s["p50"], s["p90"]) == (2.0, 10.0, 18.0)


def test_row_has_every_key_of_the_reference_row():
    row = bench_row.adam_row(ENV, "555m", "555m", 0, 0, 555848096, 3, [3.4, 3.5, 3.3], 3e-4,
                             98000.0, True)
    keys = list(row)
    assert keys[:len(HEAD_KEYS)] == HEAD_KEYS
    assert [k for k in BODY_KEYS if k not in row] == []
    assert list(row["cfg"])[:len(CFG_KEYS)] == CFG_KEYS
    assert row["cfg"]["phase"] == "adam" and row["cfg"]["workload"] == "555m"
    assert row["mode"] == "step" and row["model"] == {"D": 1536, "L": 14, "H": 24, "FF": 6272}
    assert set(row["ms"]) == {"p10", "p50", "p90", "mean", "cv"} and row["ms"]["p50"] == 3.4
    assert row["phase_ms"] == {"fwd": -1.0, "loss": -1.0, "bwd": -1.0, "adam": 3.4}
    assert row["loss"] == [-1.0, -1.0] and row["loss_ok"] is True and row["mfu"] == -1.0
    assert row["cfg"]["prec"] == "fp32"
    assert bench_row.adam_row(ENV, "555m-bf16", "555m", 1, 1, 1, 0, [1.0], 3e-4, 0, True)["cfg"]["prec"] == "bf16"
    assert bench_row.adam_row(ENV, "1p4b-fp8", "1p4b", 2, 0, 1, 0, [1.0], 3e-4, 0, False)["loss_ok"] is False


def compare_key(row):
    """How the reference's comparison script identifies a row: mode, gpu, model, cfg without
    warmup / steps / runs / B_req / lr."""
    cfg = {k: v for k, v in row["cfg"].items() if k not in ("warmup", "steps", "runs", "B_req", "lr")}
    return (row["mode"], row["gpu"], json.dumps(row["model"], sort_keys=True),
            json.dumps(cfg, sort_keys=True))


def test_rows_of_two_runs_match_and_never_match_a_whole_step_row(tmp_path):
    a = bench_row.adam_row(ENV, "555m", "555m", 0, 0, 555848096, 3, [3.4] * 10, 3e-4, 98000.0, True)
    b = bench_row.adam_row(ENV, "555m", "555m", 0, 0, 555848096, 5, [3.3] * 20, 1e-4, 98000.0, True)
    assert compare_key(a) == compare_key(b)             # warmup / steps / lr do not matter
    c = bench_row.adam_row(ENV, "555m-bf16", "555m", 1, 1, 555848096, 3, [2.3] * 8, 3e-4, 1.0, True)
    assert compare_key(c) != compare_key(a)
    whole = json.loads(json.dumps(a))
    del whole["cfg"]["phase"], whole["cfg"]["workload"]  # what a row of the reference's own bench has
    assert compare_key(whole) != compare_key(a)
    # the scored metric is ms.p50, which must be a positive number
    assert isinstance(a["ms"]["p50"], float) and a["ms"]["p50"] > 0
    path = str(tmp_path / "bench" / "run.jsonl")
    bench_row.append(path, a)
    bench_row.append(path, b)
    lines = open(path).read().splitlines()
    assert len(lines) == 2 and json.loads(lines[0]) == a and json.loads(lines[1]) == b


def test_strings_are_made_json_safe():
    assert bench_row._json_safe('a"b\\c\n') == "a_b_c_"


def test_bench_refuses_more_than_one_gpu():
    """One GPU is all this build runs on: a larger --gpus ends with a message that says so,
    before any device or library is touched."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr and "--gpus 1" in r.stderr
    assert r.stdout.strip() == ""
