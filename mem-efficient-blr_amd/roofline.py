"""Closed-form bytes / FLOPs per function and the roofline table (role of the reference's roofline.py).

Every `<function stem>_mem_flops` below is looked up by name from the function list of a Layer,
exactly as the reference does (roofline.py:136-142): the stem is the function name without its
trailing `_fp16` / `_fp32`.  The formulas are the reference's, name by name (roofline.py:7-99), so a
table made here is comparable with one made there: a name whose reference kernel writes an
intermediate to memory is charged for it even though this library's kernel for that name may not
(`library_mem_flops` gives the bytes this library's kernels are designed to move: every operand once).
"""
import os

import numpy as np
from tabulate import tabulate


# ---- low rank / dense (reference roofline.py:7-29) -----------------------------------------------------
def torch_low_rank_baseline_mem_flops(n, i, r, o, e):
    return (n * i + i * r + n * r + r * o + n * r + n * o) * e, n * r * (i + o) * 2


def triton_low_rank_mem_flops(n, i, r, o, e):
    return (i * r + r * o + n * o + n * i) * e, n * r * (i + o) * 2


def torch_dense_baseline_mem_flops(n, i, o, e):
    return (n * i + i * o + n * o) * e, n * i * o * 2


def triton_dense_mem_flops(n, i, o, e):
    return torch_dense_baseline_mem_flops(n, i, o, e)


# ---- BLAST (reference roofline.py:31-71) -------------------------------------------------------------------
def torch_blast_baseline_mem_flops(n, i, r, o, b1, b2, e):
    return (n * i + b1 * b2 * r + i * r + 4 * b2 * n * r + 4 * b1 * n * r + r * o + n * o) * e, n * r * (i + o + b1 * b2) * 2


def triton_blast_partial_mem_flops(n, i, r, o, b1, b2, e):
    return (n * i + b1 * b2 * r + i * r + 2 * b2 * n * r + r * o + n * o) * e, n * r * (i + o + b1 * b2) * 2


def triton_blast_bmm_int8_mem_flops(n, i, r, o, b1, b2, e):
    """The reference's int8 name: factors at e bytes, the rank-space intermediates as int8 (roofline.py:46-51)."""
    return (n * i + b1 * b2 * r + i * r + r * o + n * o) * e + 2 * b2 * n * r, n * r * (i + o + b1 * b2) * 2


def triton_blast_partial_grouped_mem_flops(n, i, r, o, b1, b2, e):
    return triton_blast_partial_mem_flops(n, i, r, o, b1, b2, e)


def triton_blast_partial_grouped_persistent_mem_flops(n, i, r, o, b1, b2, e):
    return triton_blast_partial_mem_flops(n, i, r, o, b1, b2, e)


def triton_blast_full_mem_flops(n, i, r, o, b1, b2, e):
    return (n * i + b1 * b2 * r + i * r + r * o + n * o) * e, n * r * (i + o + b1 * b2) * 2


def triton_blast_bmm_mem_flops(n, i, r, o, b1, b2, e):
    return (n * i + b1 * b2 * r + i * r + 2 * b2 * n * r + 2 * b1 * n * r + r * o + n * o) * e, n * r * (i + o + b1 * b2) * 2


def blast_weight_quant_mem_flops(n, i, r, o, b1, b2, e, bits):
    """Weight-quantized BLAST of this library (no reference counterpart): codes at bits / 8 bytes; S, the per-channel
    scales of U (o values) and V (b1 r values) and the activations at e bytes."""
    return r * (i + o) * bits // 8 + e * (b1 * b2 * r + o + b1 * r + n * (i + o)), n * r * (i + o + b1 * b2) * 2


def triton_blast_bmm_int4_mem_flops(n, i, r, o, b1, b2, e):
    """triton_blast_bmm_int4_fp16 exists only with packed 4-bit factors."""
    return blast_weight_quant_mem_flops(n, i, r, o, b1, b2, e, 4)


# ---- Monarch (reference roofline.py:73-99) ------------------------------------------------------------------
def triton_monarch_right_mem_flops(n, i, r, o, b, e):
    return (n * i + i * r + 2 * b * n * r + r * o + n * o + 2 * n * o) * e, n * r * (i + o) * 2


def triton_monarch_right_ideal_mem_flops(n, i, r, o, b, e):
    return (n * i + i * r + 2 * b * n * r + r * o + n * o) * e, n * r * (i + o) * 2


def triton_monarch_right_left_mem_flops(n, i, r, o, b, e):
    return triton_monarch_right_ideal_mem_flops(n, i, r, o, b, e)


def torch_monarch_baseline_mem_flops(n, i, r, o, b, e):
    return (n * i + i * r + 2 * b * n * r + 2 * b * n * r + r * o + n * o + 2 * n * o) * e, n * r * (i + o) * 2


def library_mem_flops(function_name, layer, n, elt=2):
    """(bytes, flops) with every operand moved once - what this library's kernels for `function_name` aim at."""
    i, o = layer.in_f, layer.out_f
    if "dense" in function_name:
        return torch_dense_baseline_mem_flops(n, i, o, elt)
    if "low_rank" in function_name:
        return triton_low_rank_mem_flops(n, i, layer.low_rank["rank"], o, elt)
    if "blast" in function_name:
        r, b = layer.blast["rank"], layer.blast["b"]
        if "int4" in function_name:
            return blast_weight_quant_mem_flops(n, i, r, o, b, b, elt, 4)
        return triton_blast_full_mem_flops(n, i, r, o, b, b, elt)
    r = layer.monarch["rank"]
    return (n * i + i * r + r * o + n * o) * elt, n * r * (i + o) * 2


def mem_flops_for(function_name, layer, n, elt=2):
    """(bytes, flops) of one call of `function_name` on `layer` with n token rows."""
    stem = function_name.rsplit("_", 1)[0] if "triton" in function_name else function_name
    fn = globals()[f"{stem}_mem_flops"]
    i, o = layer.in_f, layer.out_f
    if "dense" in stem:
        return fn(n, i, o, elt)
    if "low_rank" in stem:
        return fn(n, i, layer.low_rank["rank"], o, elt)
    if "blast" in stem:
        return fn(n, i, layer.blast["rank"], o, layer.blast["b"], layer.blast["b"], elt)
    return fn(n, i, layer.monarch["rank"], o, layer.monarch["b"], elt)


def roofline_table(layer, device, measured_ms=None):
    """Rows of (method, intensity, bytes, flops, attainable FLOP/s, ideal runtime s[, measured s, fraction])."""
    n = layer.num_batches * layer.num_seq
    rows = []
    for name in layer.function_names:
        mem, flops = mem_flops_for(name, layer, n)
        ai = flops / mem
        perf = min(device.peak_performance, device.memory_bandwidth * ai)
        row = [name, ai, mem, flops, perf, flops / perf]
        if measured_ms is not None:
            t = measured_ms.get(name)
            row += [t * 1e-3 if t and t > 0 else None, (flops / perf) / (t * 1e-3) if t and t > 0 else None]
        rows.append(row)
    return rows


def plot_roofline(layer, device, measured_ms=None, plot=True):
    rows = roofline_table(layer, device, measured_ms)
    headers = ["Method", "Arithmetic Intensity", "Memory Accesses", "FLOPS", "Performance", "Runtime"]
    if measured_ms is not None:
        headers += ["Measured (s)", "Fraction of roofline"]
    table_str = tabulate(rows, headers=headers, tablefmt="grid")
    print(table_str)
    out_dir = f"output/{layer.network_name}/{layer.layer_name}"
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "roofline_summary.txt"), "w") as f:
        f.write(repr(device) + "\n" + table_str)
    if plot:
        try:
            import matplotlib
            matplotlib.use("Agg")
            import matplotlib.pyplot as plt
        except Exception:
            return rows
        ai = np.linspace(0.01, max(1000.0, 2 * device.break_point), 500)
        fig, ax = plt.subplots(2, 1, figsize=(10, 10), gridspec_kw={"height_ratios": [3, 1]})
        ax[0].plot(ai, np.minimum(device.peak_performance, device.memory_bandwidth * ai), label="roofline")
        ax[0].axvline(device.break_point, linestyle="--", color="green", label=f"break point {device.break_point:.0f} FLOP/B")
        for r in rows:
            ax[0].scatter(r[1], r[4], s=60, label=r[0])
        ax[0].set_xlabel("Arithmetic Intensity (FLOPs/Byte)"); ax[0].set_ylabel("Performance (FLOP/s)")
        ax[0].set_title(f"{device.name} roofline"); ax[0].legend(fontsize=6); ax[0].grid(True)
        ax[1].bar([r[0] for r in rows], [r[5] for r in rows]); ax[1].set_ylabel("Ideal runtime (s)")
        plt.xticks(rotation=45, ha="right"); plt.tight_layout()
        plt.savefig(os.path.join(out_dir, "roofline_plot.png"), dpi=150, bbox_inches="tight")
        plt.close(fig)
    return rows
