"""One line of the reference's bench log for the optimizer phase of a step.

The reference's `anni lm bench step --profile --json FILE` appends one JSON object per run
(lang/lm_bench.c:378-387 head, :586-608 body) that scripts/bench_compare.py matches by
mode + gpu + model + cfg and compares on ms.p50.  This module writes the same object for a run
of the optimizer step alone: every key of the reference's row is present with the reference's
meaning; what this library does not run (forward, loss, backward, the GEMM ceiling) carries the
reference's own "not measured" value (-1), and cfg carries two extra keys, "phase": "adam" and
"workload", so a row of this kind only ever matches rows of the same kind, never a whole-step row.
"""
import json
import math
import os
import subprocess
import time

from . import layout

PREC_NAME = {(0, 0): "fp32", (1, 1): "bf16", (2, 0): "fp8"}   # (grad_type, moment_type)


def stats_of(values):
    """Nearest-rank p10 / p50 / p90, mean and cv = sd / mean (lang/lm_bench.c:224-246)."""
    v = sorted(float(x) for x in values)
    n = len(v)
    if n == 0:
        return {"p10": 0.0, "p50": 0.0, "p90": 0.0, "mean": 0.0, "cv": 0.0}
    mean = sum(v) / n
    ss = sum((x - mean) * (x - mean) for x in v)
    cv = math.sqrt(ss / (n - 1)) / mean if n > 1 and mean > 0.0 else 0.0
    return {"p10": v[(n - 1) // 10], "p50": v[(n - 1) // 2], "p90": v[(9 * (n - 1) + 9) // 10],
            "mean": mean, "cv": cv}


def _json_safe(s):
    return "".join("_" if (c in '"\\' or ord(c) < 32) else c for c in s)


def _cmd_line(argv, cwd):
    try:
        out = subprocess.run(argv, cwd=cwd, capture_output=True, text=True, timeout=10)
    except (OSError, subprocess.SubprocessError):
        return None
    if out.returncode != 0:
        return None
    return out.stdout.splitlines()[0].strip() if out.stdout.strip() else ""


def probe_env(L, repo_root):
    """git / gpu / driver / vram of the row's head (lang/lm_bench.c:287-335); busy when more than
    8 GiB of device memory is in use before this process allocates its arena (an idle MI355X
    with this library initialised shows 4-5 GiB in use, against the 300-500 MB the reference
    allows for a CUDA context before its 1 GiB limit)."""
    import ctypes as C
    git = _cmd_line(["git", "rev-parse", "--short", "HEAD"], repo_root)
    porcelain = _cmd_line(["git", "status", "--porcelain", "--untracked-files=no"], repo_root)
    name = C.create_string_buffer(96)
    drv = C.c_int(0)
    if L.anni_gpu_device_info(name, len(name), C.byref(drv)) != 0:
        raise RuntimeError("anni_gpu_device_info failed")
    fr, tot = C.c_size_t(0), C.c_size_t(0)
    vram_total = vram_used = 0.0
    if L.gpu_mem_info(C.byref(fr), C.byref(tot)) == 0 and tot.value > 0:
        vram_total = tot.value / 1048576.0
        vram_used = (tot.value - fr.value) / 1048576.0
    return {"git": _json_safe(git) if git else "unknown", "dirty": bool(porcelain),
            "backend": L.gpu_backend_name().decode(), "gpu": _json_safe(name.value.decode()),
            "driver": str(drv.value), "vram_mb": round(vram_total), "busy": vram_used > 8192.0, "vram_used_mb": round(vram_used)}


def adam_row(env, workload, size, grad_type, moment_type, n_params, warmup, step_ms, lr,
             vram_peak_mb, updates_ok):
    """The reference's "step" row for a run whose steps are the optimizer phase only.

    step_ms: the per-step times in ms (device events).  updates_ok: every timed step updated
    the state under a finite gradient norm -- what this row reports as loss_ok, there being no
    loss on this path (loss is the reference's "not sampled" pair).
    """
    ms = stats_of(step_ms)
    d, heads, ff, blocks, vocab = layout.SIZES[size]
    row = {"mode": "step", "git": env["git"], "dirty": env["dirty"], "backend": env["backend"],
           "gpu": env["gpu"], "driver": env["driver"], "vram_mb": env["vram_mb"],
           "busy": env["busy"], "time": int(time.time()), "model": {"D": d, "L": blocks, "H": heads, "FF": ff},
           "cfg": {"V": vocab, "B": 0, "B_req": 0, "T": 0,
                   "prec": PREC_NAME[(grad_type, moment_type)], "attn": "auto", "graphs": 0,
                   "ckpt": 0, "offload": 0, "warmup": warmup, "steps": len(step_ms), "lr": lr,
                   "phase": "adam", "workload": workload},
           "ms": {k: round(ms[k], 4) for k in ("p10", "p50", "p90", "mean", "cv")},
           "tok_s": 0.0, "tf_model": 0.0, "tf_hw": 0.0, "ceiling_tf": 0.0, "mfu": -1.0,
           "vram_peak_mb": round(vram_peak_mb), "loss": [-1.0, -1.0],
           "loss_ok": bool(updates_ok),
           "phase_ms": {"fwd": -1.0, "loss": -1.0, "bwd": -1.0, "adam": round(ms["p50"], 4)},
           "params": int(n_params)}
    return row


def _b(x):
    return "true" if x else "false"


def format_row(row):
    """The row as the reference's writer prints it (lang/lm_bench.c:378-387 head, :586-608 body):
    the same keys in the same order with the same printf conversions (%.0f, %.4f, %.1f, %.5f, %g,
    %d, %ld); keys the reference does not have (cfg.phase, cfg.workload, params) follow the
    reference's keys of their object.  A row parsed from a line of the reference's log prints
    back as that line."""
    m, c = row["model"], row["cfg"]
    out = ('{"mode":"%s","git":"%s","dirty":%s,"backend":"%s","gpu":"%s","driver":"%s",'
           '"vram_mb":%.0f,"busy":%s,"time":%d,"model":{"D":%d,"L":%d,"H":%d,"FF":%d}'
           % (row["mode"], row["git"], _b(row["dirty"]), row["backend"], row["gpu"],
              row["driver"], row["vram_mb"], _b(row["busy"]), row["time"], m["D"], m["L"], m["H"],
              m["FF"]))
    out += (',"cfg":{"V":%d,"B":%d,"B_req":%d,"T":%d,"prec":"%s","attn":"%s","graphs":%d,'
            '"ckpt":%d,"offload":%d,"warmup":%d,"steps":%d,"lr":%g'
            % (c["V"], c["B"], c["B_req"], c["T"], c["prec"], c["attn"], c["graphs"], c["ckpt"],
               c["offload"], c["warmup"], c["steps"], c["lr"]))
    for k in ("phase", "workload"):
        if k in c:
            out += ',"%s":"%s"' % (k, c[k])
    ms = row["ms"]
    out += ('},"ms":{"p10":%.4f,"p50":%.4f,"p90":%.4f,"mean":%.4f,"cv":%.4f},"tok_s":%.1f,'
            '"tf_model":%.4f,"tf_hw":%.4f,"ceiling_tf":%.4f,"mfu":%.4f,"vram_peak_mb":%.0f,'
            '"loss":[%.5f,%.5f],"loss_ok":%s'
            % (ms["p10"], ms["p50"], ms["p90"], ms["mean"], ms["cv"], row["tok_s"],
               row["tf_model"], row["tf_hw"], row["ceiling_tf"], row["mfu"], row["vram_peak_mb"],
               row["loss"][0], row["loss"][1], _b(row["loss_ok"])))
    if "phase_ms" in row:
        ph = row["phase_ms"]
        out += (',"phase_ms":{"fwd":%.4f,"loss":%.4f,"bwd":%.4f,"adam":%.4f}'
                % (ph["fwd"], ph["loss"], ph["bwd"], ph["adam"]))
    if "params" in row:
        out += ',"params":%d' % row["params"]
    return out + "}"


IGNORED_CFG = ("warmup", "steps", "runs", "B_req", "lr")


def compare_key(row):
    """How the reference's scripts/bench_compare.py identifies a row (its key_of): mode, gpu,
    model and cfg without warmup / steps / runs / B_req / lr, the two objects as sorted JSON."""
    cfg = {k: v for k, v in row.get("cfg", {}).items() if k not in IGNORED_CFG}
    return (row.get("mode"), row.get("gpu"), json.dumps(row.get("model", {}), sort_keys=True),
            json.dumps(cfg, sort_keys=True))


def append(path, row):
    """Appends the row as one line (the reference opens its log with "a", lm_bench.c:362-375)."""
    d = os.path.dirname(path)
    if d:
        os.makedirs(d, exist_ok=True)
    with open(path, "a", encoding="utf-8") as fp:
        fp.write(format_row(row) + "\n")
