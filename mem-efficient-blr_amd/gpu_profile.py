"""Kernel-level profiles of one operator function with rocprofv3 (role of the reference's gpu_profile.py + gpu_profile.sh,
which drive nsys / ncu: reference gpu_profile.py:17-171, gpu_profile.sh:47-140).

Three modes, chosen with ``--mode``:

  run       build the operands of ``--function_name`` (same operand shapes per function family as the reference's
            gpu_profile.py:31-163) and call it ``--num_iters`` times.  This is the program that is profiled.
  trace     start ``rocprofv3 --kernel-trace --stats`` on this script in run mode (as a child process), then print and
            write a per-kernel summary: calls, average / min / max microseconds, grid and workgroup size.
  counters  one rocprofv3 ``--pmc`` run per counter (the profiler does not split counters over passes; FETCH_SIZE and
            WRITE_SIZE by default), each followed by the same run over a copy of known size, and a per-kernel summary
            of HBM bytes per dispatch scaled by what the counter reads for the copy.

    python gpu_profile.py --mode trace --function_name triton_funcs.blast_kernels.triton_blast_full_fp16 \
        --num_batches 1 --num_seq 1 --in_f 4096 --out_f 22016 --b 16 --rank 1024 --output_dir out/llama7b/gate_up

The child always is ``python3 gpu_profile.py --mode run ...`` directly behind ``--``: no shell, no env wrapper.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import importlib
import json
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)

CALIB_BYTES = 256 << 20
COPY_KERNEL_HINTS = ("copyBuffer", "elementwise_kernel")        # the device-to-device copy of the calibration run


def _function(name):
    mod, _, fn = name.rpartition(".")
    return getattr(importlib.import_module(mod), fn), fn


def build_call(args):
    """(callable, description) for --function_name on cuda:0; operand shapes as in the reference's gpu_profile.py."""
    import torch
    fn, short = _function(args.function_name)
    dev = torch.device("cuda:0")
    dt = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}[args.dtype]
    if short.endswith("fp32"):
        dt = torch.float32
    b, r, i_f, o_f = args.b, args.rank, args.in_f, args.out_f
    x = torch.randn((args.num_batches, args.num_seq, i_f), device=dev, dtype=dt)
    rn = lambda *s: torch.randn(s, device=dev, dtype=dt) * (1.0 / max(r, 1)) ** 0.5
    if "blast" in short:
        if "torch" in short:
            ops = (rn(b, o_f // b, r), rn(b, r, i_f // b), torch.randn((b, b, r), device=dev, dtype=dt))
        elif "bmm" in short:
            U, V, S = rn(b, o_f // b, r), rn(b, i_f // b, r), torch.randn((r, b, b), device=dev, dtype=dt)
            if "int8" in short or "int4" in short:
                from triton_funcs import blast_sym_quant_kernels as Q
                if args.weight_quant:
                    U, V = Q.quantize_blast_factors(U.float(), V.float(), 4 if "int4" in short else 8)
            ops = (U, V, S)
        else:
            ops = (rn(b, r, o_f // b), rn(b, i_f // b, r), torch.randn((b, b, r), device=dev, dtype=dt))
    elif "monarch" in short:
        if "torch" in short:
            ops = (rn(b, r, i_f // b), rn(b, o_f // b, r))
        else:
            ops = (rn(b, i_f // b, r), rn(b, r, o_f // b) if "left" in short else rn(b, o_f // b, r))
    elif "low_rank" in short:
        ops = (rn(r, i_f), rn(o_f, r)) if "torch" in short else (rn(i_f, r), rn(r, o_f))
    elif "dense" in short:
        ops = (rn(o_f, i_f),) if "torch" in short else (rn(i_f, o_f),)
    else:
        raise SystemExit(f"don't know the operands of {short}")
    return (lambda: fn(x, *ops)), f"{short} x{tuple(x.shape)}"


def run(args):
    import torch
    call, what = build_call(args)
    for _ in range(args.num_warmup_iters):
        call()
    torch.cuda.synchronize()
    for _ in range(args.num_iters):
        call()
    torch.cuda.synchronize()
    print(json.dumps({"ran": what, "iters": args.num_iters, "warmup": args.num_warmup_iters}))


def calib(_args):
    """A device-to-device copy of CALIB_BYTES, four times: the known size the counters are scaled by."""
    import torch
    src = torch.empty(CALIB_BYTES, dtype=torch.uint8, device="cuda:0").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(4):
        dst.copy_(src)
    torch.cuda.synchronize()
    print(json.dumps({"calib_bytes": CALIB_BYTES}))


# ---- summaries of rocprofv3's csv files (no GPU needed) -----------------------------------------------------------------
def summarize_kernel_trace(path, skip_first=0):
    """{(kernel, grid, workgroup): {"calls", "avg_us", "min_us", "max_us"}} from a *_kernel_trace.csv."""
    rows = collections.defaultdict(list)
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            key = (r["Kernel_Name"], int(r["Grid_Size_X"]) * int(r.get("Grid_Size_Y", 1) or 1) * int(r.get("Grid_Size_Z", 1) or 1),
                   int(r["Workgroup_Size_X"]))
            rows[key].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    out = {}
    for key, v in rows.items():
        v = v[skip_first:] or v
        out[key] = {"calls": len(v), "avg_us": sum(v) / len(v), "min_us": min(v), "max_us": max(v)}
    return out


def summarize_counters(path):
    """{(kernel, counter): {"dispatches", "mean", "min", "max"}} from a *_counter_collection.csv."""
    rows = collections.defaultdict(list)
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            rows[(r["Kernel_Name"], r["Counter_Name"])].append(float(r["Counter_Value"]))
    return {k: {"dispatches": len(v), "mean": sum(v) / len(v), "min": min(v), "max": max(v)} for k, v in rows.items()}


def counter_unit_bytes(calib_summary, counter):
    """Bytes that one unit of `counter` stands for, from the calibration copy (CALIB_BYTES read and written per dispatch)."""
    best = None
    for (kernel, name), s in calib_summary.items():
        if name == counter and any(h in kernel for h in COPY_KERNEL_HINTS) and s["mean"] > 1000:
            if best is None or s["mean"] > best["mean"]:
                best = s
    return CALIB_BYTES / best["mean"] if best else None


def _short(kernel, width=72):
    return kernel if len(kernel) <= width else kernel[: width - 3] + "..."


def format_trace(summary, only=None):
    lines = [f"{'kernel':72s} {'grid':>9s} {'wg':>5s} {'calls':>6s} {'avg_us':>9s} {'min_us':>9s} {'max_us':>9s}"]
    for (kernel, grid, wg), s in sorted(summary.items(), key=lambda kv: -kv[1]["avg_us"] * kv[1]["calls"]):
        if only and not any(o in kernel for o in only):
            continue
        lines.append(f"{_short(kernel):72s} {grid:9d} {wg:5d} {s['calls']:6d} {s['avg_us']:9.2f} {s['min_us']:9.2f} {s['max_us']:9.2f}")
    return "\n".join(lines)


# ---- driver modes ---------------------------------------------------------------------------------------------------------
def _child_args(args, mode):
    out = [sys.executable, os.path.abspath(__file__), "--mode", mode, "--function_name", args.function_name,
           "--num_batches", str(args.num_batches), "--num_seq", str(args.num_seq), "--in_f", str(args.in_f), "--out_f", str(args.out_f),
           "--b", str(args.b), "--rank", str(args.rank), "--num_iters", str(args.num_iters), "--num_warmup_iters", str(args.num_warmup_iters),
           "--dtype", args.dtype]
    if args.weight_quant:
        out.append("--weight_quant")
    return out


def _rocprof(extra, out_dir, name, child, timeout):
    cmd = ["rocprofv3"] + extra + ["--output-format", "csv", "-d", out_dir, "-o", name, "--"] + child
    print("running:", " ".join(cmd), flush=True)
    env = dict(os.environ, TMPDIR=os.environ.get("TMPDIR", "/tmp"))
    subprocess.run(cmd, check=True, timeout=timeout, env=env, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    return cmd


def _find(out_dir, suffix):
    hits = glob.glob(os.path.join(out_dir, "**", f"*{suffix}"), recursive=True)
    if not hits:
        raise SystemExit(f"rocprofv3 left no *{suffix} under {out_dir}")
    return hits[0]


def trace(args):
    _, short = _function(args.function_name)
    out_dir = os.path.join(args.output_dir, f"{short}_trace")
    cmd = _rocprof(["--kernel-trace", "--stats"], out_dir, "kt", _child_args(args, "run"), args.timeout)
    summary = summarize_kernel_trace(_find(out_dir, "kernel_trace.csv"), skip_first=0)
    text = "command: " + " ".join(cmd) + "\n" + format_trace(summary, only=args.only)
    print(text)
    with open(os.path.join(args.output_dir, f"{short}_kernels.txt"), "w") as f:
        f.write(text + "\n")


def counters(args):
    _, short = _function(args.function_name)
    lines = []
    for counter in args.counters:
        d_run = os.path.join(args.output_dir, f"{short}_{counter}")
        d_cal = os.path.join(args.output_dir, f"calib_{counter}")
        c1 = _rocprof(["--pmc", counter], d_run, "pmc", _child_args(args, "run"), args.timeout)
        c2 = _rocprof(["--pmc", counter], d_cal, "cal", _child_args(args, "calib"), args.timeout)
        run_s = summarize_counters(_find(d_run, "counter_collection.csv"))
        unit = counter_unit_bytes(summarize_counters(_find(d_cal, "counter_collection.csv")), counter)
        lines += ["command: " + " ".join(c1), "command: " + " ".join(c2),
                  f"{counter}: one unit = {unit:.1f} bytes (from a {CALIB_BYTES >> 20} MiB copy)" if unit else f"{counter}: no calibration kernel found"]
        for (kernel, name), s in sorted(run_s.items(), key=lambda kv: -kv[1]["mean"]):
            if args.only and not any(o in kernel for o in args.only):
                continue
            mb = f"{s['mean'] * unit / 1e6:10.2f} MB" if unit else "         ?"
            lines.append(f"  {_short(kernel):72s} dispatches {s['dispatches']:5d}  {name} mean {s['mean']:12.1f} -> {mb} per dispatch")
    text = "\n".join(lines)
    print(text)
    with open(os.path.join(args.output_dir, f"{short}_counters.txt"), "w") as f:
        f.write(text + "\n")


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--mode", required=True, choices=["run", "calib", "trace", "counters"])
    ap.add_argument("--function_name", required=True, help="module.function, e.g. triton_funcs.blast_kernels.triton_blast_full_fp16")
    ap.add_argument("--num_batches", type=int, default=1)
    ap.add_argument("--num_seq", type=int, required=True)
    ap.add_argument("--in_f", type=int, required=True)
    ap.add_argument("--out_f", type=int, required=True)
    ap.add_argument("--b", type=int, default=1)
    ap.add_argument("--rank", type=int, default=0)
    ap.add_argument("--num_iters", type=int, default=20)
    ap.add_argument("--num_warmup_iters", type=int, default=5)
    ap.add_argument("--dtype", default="fp16", choices=["fp16", "bf16", "fp32"])
    ap.add_argument("--weight_quant", action="store_true", help="int8 / int4 names: quantize the factors once (weight-quantized product)")
    ap.add_argument("--output_dir", default="./output/profile")
    ap.add_argument("--counters", nargs="+", default=["FETCH_SIZE", "WRITE_SIZE"])
    ap.add_argument("--only", nargs="*", default=["blr"], help="substrings of the kernel names to report (default: this library's kernels)")
    ap.add_argument("--timeout", type=int, default=300)
    args = ap.parse_args(argv)
    if args.mode in ("trace", "counters"):
        os.makedirs(args.output_dir, exist_ok=True)
    {"run": run, "calib": calib, "trace": trace, "counters": counters}[args.mode](args)


if __name__ == "__main__":
    main()
