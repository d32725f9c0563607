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


def _fixtures():
    import os
    from helpers import GOLDEN
    line = open(os.path.join(GOLDEN, "bench_row_ref.jsonl")).read().rstrip("\n")
    keys = json.load(open(os.path.join(GOLDEN, "bench_row_keys.json")))
    return line, keys


def _sample_row():
    import importlib.util
    import os
    from helpers import GOLDEN
    spec = importlib.util.spec_from_file_location("make_bench_row",
                                                  os.path.join(GOLDEN, "make_bench_row.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.sample_row()


def test_writer_reproduces_the_line_the_references_writer_wrote():
    """tests/golden/bench_row_ref.jsonl is the line the reference's own lm_bench_step appended when
    its real training step ran on this backend (make_bench_row.py --row).  Parsed and printed back
    by format_row it must be that line, byte for byte: key order, nesting, %.4f / %.1f / %.5f /
    %.0f / %g conversions."""
    line, _keys = _fixtures()
    ref = json.loads(line)
    assert bench_row.format_row(ref) == line
    # and our own rows carry the reference's keys in the reference's order, extras behind them
    ours = _sample_row()
    printed = json.loads(bench_row.format_row(ours))
    assert [k for k in printed if k in ref] == list(ref)
    assert list(printed)[len(ref):] == ["params"]
    assert list(printed["cfg"])[:len(ref["cfg"])] == list(ref["cfg"])
    assert list(printed["cfg"])[len(ref["cfg"]):] == ["phase", "workload"]
    for k in ("model", "ms", "phase_ms"):
        assert list(printed[k]) == list(ref[k])
    assert printed == json.loads(json.dumps(ours))       # nothing lost on the way
    # number formats of our values as the reference prints such values
    text = bench_row.format_row(ours)
    assert '"ms":{"p10":3.1999,"p50":3.2101,' in text and '"lr":0.0003,' in text
    assert '"mfu":-1.0000,' in text and '"loss":[-1.00000,-1.00000]' in text
    assert '"vram_mb":294896,' in text and '"tok_s":0.0,' in text


def test_compare_key_is_the_references_key_of():
    """bench_row.compare_key against the keys that the reference's scripts/bench_compare.py itself
    derived (make_bench_row.py --keys imported it in the build container) for the reference-written
    row and for a row of ours."""
    line, keys = _fixtures()
    ref = json.loads(line)
    assert list(bench_row.compare_key(ref)) == keys["ref_row_key"]
    ours = _sample_row()
    assert json.loads(json.dumps(ours)) == keys["sample_row"]    # the row the key was recorded for
    assert list(bench_row.compare_key(ours)) == keys["sample_row_key"]
    assert sorted(bench_row.IGNORED_CFG) == keys["ignored_cfg"]
    # a whole-step row of the same gpu and model is another key: the two kinds never match
    whole = dict(ref, gpu=ours["gpu"], model=ours["model"])
    assert list(bench_row.compare_key(whole)) == keys["whole_step_row_same_gpu_model_key"]
    assert bench_row.compare_key(whole) != bench_row.compare_key(ours)
    # the scored metric of a step row is ms.p50, lower is better, and ours is a positive number
    assert keys["step_metric"] == [["ms", "p50"], False]
    assert keys["sample_row_metric"] == ours["ms"]["p50"] > 0


def test_rows_of_two_runs_match(tmp_path):
    a = bench_row.adam_row(ENV, "555m", "555m", 0, 0, 555848096, 3, [3.4] * 10, 3e-4, 98000.0, True)
    b = bench_row.adam_row(ENV, "555m", "555m", 0, 0, 555848096, 5, [3.3] * 20, 1e-4, 98000.0, True)
    assert bench_row.compare_key(a) == bench_row.compare_key(b)   # warmup / steps / lr do not matter
    c = bench_row.adam_row(ENV, "555m-bf16", "555m", 1, 1, 555848096, 3, [2.3] * 8, 3e-4, 1.0, True)
    assert bench_row.compare_key(c) != bench_row.compare_key(a)
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
