#!/usr/bin/env python3
"""Writes the fixtures that pin anni_amd/bench_row.py to the reference's own bench-log writer.

Two stages, because the reference's harness refuses to run on its CPU stub
(lang/lm_bench.c:334-339) and the reference tree exists only in the build container:

  --row   (on a GPU box; loads oracle/_ref/libanni_ref_small_hip.so = the reference's library
          sources with the small model of its unit tests, linked against libanni_gpu_hip.so)
          runs the reference's lm_bench_step once -- a packed training step of its real model
          code, the optimizer phase on this backend -- and stores the line its json writer
          (lang/lm_bench.c:378-387,586-608) appended:  tests/golden/bench_row_ref.jsonl
  --keys  (in the build container, where /root/reference exists) imports the reference's
          scripts/bench_compare.py and records the match key it derives for that row and for a
          row written by anni_amd.bench_row:  tests/golden/bench_row_keys.json
"""
import argparse
import ctypes as C
import importlib.util
import json
import os
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
ROW = os.path.join(HERE, "bench_row_ref.jsonl")
KEYS = os.path.join(HERE, "bench_row_keys.json")

# a fixed row of ours: environment as probe_env returns it, per-step times in ms
SAMPLE_ENV = {"git": "abc1234", "dirty": False, "backend": "hip-gfx950",
              "gpu": "AMD Instinct MI355X (gfx950:sramecc+:xnack-)", "driver": "70253211",
              "vram_mb": 294896, "busy": False, "vram_used_mb": 4600}
SAMPLE_MS = [3.2101, 3.2204, 3.1999, 3.25, 3.2077, 3.2163, 3.3012, 3.2139, 3.2081, 3.2]


def sample_row():
    from anni_amd import bench_row
    row = bench_row.adam_row(SAMPLE_ENV, "555m", "555m", 0, 0, 555848096, 3, SAMPLE_MS, 3e-4,
                             41000.0, True)
    row["time"] = 0
    return row


def write_row():
    so = os.path.join(ROOT, "oracle", "_ref", "libanni_ref_small_hip.so")
    R = C.CDLL(so)
    R.ref_bench_step.argtypes = [C.c_char_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
    R.ref_bench_step.restype = C.c_int
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "row.jsonl")
        rc = R.ref_bench_step(os.fsencode(path), 4, 32, 512, 2, 12)
        if rc not in (0, 1):                     # 1 = its loss check failed: the row is written all the same
            sys.exit("lm_bench_step returned %d" % rc)
        lines = open(path).read().splitlines()
    assert len(lines) == 1 and json.loads(lines[0])["mode"] == "step"
    with open(ROW, "w") as f:
        f.write(lines[0] + "\n")
    print(lines[0])


def write_keys():
    spec = importlib.util.spec_from_file_location(
        "bench_compare", "/root/reference/scripts/bench_compare.py")
    bc = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bc)
    ref_row = json.loads(open(ROW).read())
    ours = sample_row()
    whole_step_like = dict(ref_row, gpu=ours["gpu"], model=ours["model"])
    out = {"ref_row_key": list(bc.key_of(ref_row)),
           "sample_row": ours, "sample_row_key": list(bc.key_of(ours)),
           # a whole-step row of the same gpu and model must not match an optimizer-phase row
           "whole_step_row_same_gpu_model_key": list(bc.key_of(whole_step_like)),
           "ignored_cfg": sorted(bc.IGNORED_CFG),
           "step_metric": [list(bc.METRIC["step"][0]), bc.METRIC["step"][1]],
           "sample_row_metric": bc.metric(ours)}
    with open(KEYS, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps(out["sample_row_key"]))


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--row", action="store_true")
    ap.add_argument("--keys", action="store_true")
    a = ap.parse_args()
    if a.row:
        write_row()
    if a.keys:
        write_keys()
