"""Per-layer verify / benchmark / summary harness (counterpart of the reference's layer.py:10-507).

Reads the same YAML schema: `configs/config.yaml` shallow-merged with the layer file (layer keys win,
reference layer.py:15-17), function lists given as dotted paths, resolved with importlib, and
dispatched on substrings of the function *names* (reference layer.py:207, 232-240, 304, 365):
BLAST names starting with "triton_blast_bmm" get the bmm layouts, Monarch names starting with
"triton_monarch_right_left" get w2 as (b, r, s), "triton_monarch_right_ideal" is verified on the
permuted intermediate.  Output files are the reference's: output/<net>/<layer>/{summary.txt,
*_best_config.pkl}.  Inputs are drawn with std 1/sqrt(rank) factors (the reference uses std 1).
"""
import importlib
import math
import os
import pickle

import torch
from tabulate import tabulate

from utils import VerificationStatus, do_bench, do_verify, load_yaml

HERE = os.path.dirname(os.path.abspath(__file__))
FAMILIES = ("blast", "blast_sym_quant", "monarch", "low_rank", "dense")


def _resolve(path):
    mod, name = path.rsplit(".", 1)
    return getattr(importlib.import_module(mod), name)


def _get_config_fn(func):
    """get_<name>_config of the module that defines func (or None)."""
    mod = importlib.import_module(func.__module__)
    return getattr(mod, f"get_{func.__name__}_config", None)


class Layer:
    def __init__(self, config_path, default_config_path=None):
        if not config_path:
            raise ValueError("A YAML configuration file path must be provided")
        layer_config = load_yaml(config_path)
        default_config = load_yaml(default_config_path or os.path.join(HERE, "configs", "config.yaml"))
        config = default_config | layer_config
        self.config = config
        self.network_name, self.layer_name = config["network_name"], config["layer_name"]
        self.num_seq, self.num_batches = config["num_seq"], config["num_batches"]
        self.in_f, self.out_f = config["in_f"], config["out_f"]
        self.blast, self.monarch, self.low_rank = config["blast"], config.get("monarch"), config["low_rank"]

        self.verify_funcs, self.bench_funcs, self.status, self.times = {}, {}, {}, {}
        for fam in FAMILIES:
            vkey, bkey = f"triton_{fam}_verify", f"triton_{fam}_benchmark"
            bench = [_resolve(p) for p in sorted(config[bkey]["funcs"])] if bkey in config else []
            ver = [_resolve(p) for p in sorted(config[vkey]["funcs"])] if vkey in config else []
            if fam == "monarch" and self.monarch is None:
                bench, ver = [], []
            if fam != "blast_sym_quant" and bench and ver and len(bench) != len(ver):
                raise ValueError(f"Mismatch: {vkey}.funcs and {bkey}.funcs must have the same length")
            self.bench_funcs[fam], self.verify_funcs[fam] = bench, ver
            self.times[fam] = [-1] * len(bench)
            initial = VerificationStatus.NA if fam == "blast_sym_quant" or not ver else VerificationStatus.UNKNOWN
            self.status[fam] = [initial] * len(bench)

        self.torch_funcs, self.torch_compiled, self.torch_times = {}, {}, {}
        for fam in ("blast", "monarch", "low_rank", "dense"):
            if fam == "monarch" and self.monarch is None:
                continue
            entry = config[f"torch_{fam}"]
            f = _resolve(entry["funcs"])
            self.torch_compiled[fam] = bool(entry.get("compile", False))
            self.torch_funcs[fam] = torch.compile(f) if self.torch_compiled[fam] else f
            self.torch_funcs[fam].__dict__.setdefault("_blr_name", f.__name__)
            self.torch_times[fam] = -1
        names = [f.__name__ for fam in FAMILIES for f in self.bench_funcs[fam]]
        names += [self._torch_name(fam) for fam in self.torch_funcs]
        self.function_names = names

    def _torch_name(self, fam):
        return getattr(self.torch_funcs[fam], "_blr_name", getattr(self.torch_funcs[fam], "__name__", fam))

    # ---- inputs ---------------------------------------------------------------------------------
    def _randn(self, shape, std, dtype, device):
        return (torch.randn(shape, device=device, dtype=torch.float32) * std).to(dtype)

    def _blast_inputs(self, dtype, device):
        b, r = self.blast["b"], self.blast["rank"]
        U = self._randn((b, self.out_f // b, r), 1 / math.sqrt(r), dtype, device)
        Vt = self._randn((b, r, self.in_f // b), 1 / math.sqrt(r), dtype, device)
        S = self._randn((b, b, r), 1.0, dtype, device)
        kern = dict(U=U.transpose(1, 2).contiguous(), V=Vt.transpose(1, 2).contiguous(), S=S.transpose(0, 1).contiguous())
        bmm = dict(U=U, V=kern["V"], S=S.permute(2, 0, 1).contiguous())       # reference layer.py:199-201
        return (U, Vt, S), kern, bmm

    def _monarch_inputs(self, dtype, device):
        b, r = self.monarch["b"], self.monarch["rank"]
        p, s = self.in_f // b, self.out_f // b
        w1_t = self._randn((b, r, p), 1 / math.sqrt(p), dtype, device)
        w2_t = self._randn((b, s, r), 1 / math.sqrt(r), dtype, device)
        w1 = w1_t.transpose(1, 2).contiguous().view(b, p, r // b, b).permute(0, 1, 3, 2).reshape(b, p, r).contiguous()
        return (w1_t, w2_t), w1, w2_t.transpose(1, 2).contiguous()

    def _call(self, fam, f, x, data):
        name = f.__name__
        if fam in ("blast", "blast_sym_quant"):
            _, kern, bmm = data
            d = bmm if name.startswith("triton_blast_bmm") else kern
            if fam == "blast_sym_quant":
                if "q" not in data[2]:
                    from triton_funcs.blast_sym_quant_kernels import quantize_blast_factors
                    data[2]["q"] = quantize_blast_factors(bmm["U"].float(), bmm["V"].float(), self.config.get("quant_bits", 8))
                uq, vq = data[2]["q"]
                return f(x, uq, vq, bmm["S"])
            return f(x, d["U"], d["V"], d["S"])
        if fam == "monarch":
            (w1_t, w2_t), w1, w2 = data
            return f(x, w1, w2 if name.startswith("triton_monarch_right_left") else w2_t)
        if fam == "low_rank":
            return f(x, data["V"], data["U"])
        return f(x, data["W"])

    def _inputs(self, fam, dtype, device):
        if fam in ("blast", "blast_sym_quant"):
            return self._blast_inputs(dtype, device)
        if fam == "monarch":
            return self._monarch_inputs(dtype, device)
        if fam == "low_rank":
            r = self.low_rank["rank"]
            Vt = self._randn((r, self.in_f), 1 / math.sqrt(r), dtype, device)
            Ut = self._randn((self.out_f, r), 1 / math.sqrt(r), dtype, device)
            return dict(Vt=Vt, Ut=Ut, V=Vt.t().contiguous(), U=Ut.t().contiguous())
        Wt = self._randn((self.out_f, self.in_f), 1 / math.sqrt(self.in_f), dtype, device)
        return dict(Wt=Wt, W=Wt.t().contiguous())

    def _torch_call(self, fam, x, data):
        f = self.torch_funcs[fam]
        if fam == "blast":
            return f(x, *data[0])
        if fam == "monarch":
            return f(x, *data[0])
        if fam == "low_rank":
            return f(x, data["Vt"], data["Ut"])
        return f(x, data["Wt"])

    # ---- verify -----------------------------------------------------------------------------------
    def verify(self, method="all", device="cuda:0"):
        dtype = torch.float32
        x = torch.randn((self.num_batches, self.num_seq, self.in_f), device=device, dtype=dtype)
        for fam in ("blast", "monarch", "low_rank", "dense"):
            if method not in (fam, "all") or not self.verify_funcs[fam] or fam not in self.torch_funcs:
                continue
            data = self._inputs(fam, dtype, device)
            ref = self._torch_call(fam, x, data)
            for i, f in enumerate(self.verify_funcs[fam]):
                print(f"Verifying {f.__name__} ...")
                try:
                    got = self._call(fam, f, x, data)
                    if fam == "monarch" and f.__name__.startswith("triton_monarch_right_ideal"):
                        a, b_ = got[1], ref[2]                      # permuted intermediate (reference layer.py:237)
                    elif fam == "dense":
                        a, b_ = got, ref
                    elif fam == "low_rank":
                        a, b_ = got[0], ref
                    else:
                        a, b_ = got[0], ref[0]
                    status = do_verify(a.reshape(b_.shape), b_)
                except Exception as e:                             # keep going, record the failure
                    print(f"An error occured while executing {f.__name__}: {e}")
                    status = VerificationStatus.FAIL
                if i < len(self.status[fam]):
                    self.status[fam][i] = status

    # ---- benchmark ----------------------------------------------------------------------------------
    def _save_config(self, f):
        out_dir = f"output/{self.network_name}/{self.layer_name}"
        os.makedirs(out_dir, exist_ok=True)
        name = f.__name__
        if name.startswith("triton_blast_bmm"):
            mod = importlib.import_module(f.__module__)
            quant = "int8_" if "int8" in name or "int4" in name else ""
            for suffix in ("xv", "sxv", "usxv"):
                getter = getattr(mod, f"get_triton_blast_bmm_{suffix}_{quant}fp16_config", None)
                if getter:
                    with open(os.path.join(out_dir, f"triton_blast_bmm_{suffix}_{quant}fp16_best_config.pkl"), "wb") as fh:
                        pickle.dump(getter(), fh)
            return
        getter = _get_config_fn(f)
        if getter:
            with open(os.path.join(out_dir, f"{name}_best_config.pkl"), "wb") as fh:
                pickle.dump(getter(), fh)

    def benchmark(self, method="all", device="cuda:0", dtype=torch.float16):
        x = torch.randn((self.num_batches, self.num_seq, self.in_f), device=device, dtype=dtype)
        for fam in FAMILIES:
            base = "blast" if fam == "blast_sym_quant" else fam
            if method not in (base, fam, "all") or (fam == "monarch" and self.monarch is None):
                continue
            data = self._inputs(fam, dtype, device)
            if fam in self.torch_funcs:
                try:
                    self.torch_times[fam] = do_bench(lambda: self._torch_call(fam, x, data))
                except Exception as e:
                    print(f"An error occured while executing {self._torch_name(fam)}: {e}")
            for i, f in enumerate(self.bench_funcs[fam]):
                print(f"Benchmarking {f.__name__} ...")
                try:
                    self.times[fam][i] = do_bench(lambda: self._call(fam, f, x, data))
                    self._save_config(f)
                except Exception as e:
                    print(f"An error occured while executing {f.__name__}: {e}")

    def measured_ms(self):
        out = {self._torch_name(fam): t for fam, t in self.torch_times.items()}
        for fam in FAMILIES:
            for f, t in zip(self.bench_funcs[fam], self.times[fam]):
                out[f.__name__] = t
        return out

    # ---- reporting -----------------------------------------------------------------------------------
    def summary(self):
        table = []
        for fam in self.torch_funcs:
            n = self._torch_name(fam)
            table.append((f"torch.compile({n})" if self.torch_compiled[fam] else n, self.torch_times[fam], "N/A"))
        for fam in FAMILIES:
            if not self.bench_funcs[fam]:
                continue
            rows = sorted(zip(self.bench_funcs[fam], self.times[fam], self.status[fam]),
                          key=lambda r: r[1] if r[1] != -1 else float("inf"))
            table.append([None, None, None])
            table.extend([[f.__name__, t, s.name] for f, t, s in rows])
        table_str = tabulate(table, headers=["Function", "Benchmark Time (ms)", "Verification Status"], tablefmt="grid", missingval="—")
        print(table_str)
        out_dir = f"output/{self.network_name}/{self.layer_name}"
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, "summary.txt"), "w") as f:
            f.write(table_str)
        return table_str

    def __repr__(self):
        names = lambda fs: [f.__name__ for f in fs]
        mon = f"B={self.monarch['b']}, Rank={self.monarch['rank']}" if self.monarch else "N/A"
        lines = ["", "=" * 50, "Layer Configuration", "-" * 50,
                 f"Network Name    : {self.network_name}", f"Layer Name      : {self.layer_name}",
                 f"Input Features  : {self.in_f}", f"Output Features : {self.out_f}", f"Num Sequence    : {self.num_seq}", "",
                 f"BLAST Config    : B={self.blast['b']}, Rank={self.blast['rank']}", f"Monarch Config  : {mon}",
                 f"Low-Rank Config : Rank={self.low_rank['rank']}", "", "=" * 50, "Microbenchmark Details", "-" * 50]
        for fam in FAMILIES:
            lines.append(f"{fam:16s} verify    : {names(self.verify_funcs[fam])}")
            lines.append(f"{fam:16s} benchmark : {names(self.bench_funcs[fam])}")
        for fam in self.torch_funcs:
            lines.append(f"torch {fam:10s}: Name={self._torch_name(fam)} Compiled={self.torch_compiled[fam]}")
        lines += ["", "=" * 50, ""]
        return "\n".join(lines)
