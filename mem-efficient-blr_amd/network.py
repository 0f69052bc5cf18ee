"""End-to-end model timing harness (counterpart of the reference's network.py:8-79).

Network YAML schema: method -> layer key -> {rank, b, triton: {func}, torch: {func, compile}}.
The model module `models.<name>` must provide benchmark(method, framework, layer_configs, num_seq,
num_iters, device, dtype).  Results go to output/<name>/end2end_summary_<num_seq>.txt.
"""
import importlib
import os

import torch
from tabulate import tabulate

from utils import load_yaml

METHODS = ["blast", "blast_sym_quant", "monarch", "low_rank", "dense"]


class Network:
    def __init__(self, config_path):
        if not config_path:
            raise ValueError("A YAML configuration file path must be provided")
        cfg = load_yaml(config_path)
        self.name = cfg["name"]
        self.benchmark_func = getattr(importlib.import_module(f"models.{self.name}"), "benchmark")
        self.benchmark_results = {}
        self.num_seq = cfg["num_seq"]
        self.batch = cfg.get("batch", 1)
        self.layer_configs = {}
        for method in METHODS:
            if method not in cfg:
                if method in ("monarch", "blast_sym_quant"):
                    continue
                raise KeyError(f"Method '{method}' missing in network configuration")
            per = {"triton": {}, "torch": {}}
            for layer, details in cfg[method].items():
                if not isinstance(details, dict):
                    continue
                for fw in ("triton", "torch"):
                    if fw in details:
                        per[fw][layer] = {"rank": details.get("rank"), "b": details.get("b"),
                                          "func": details[fw].get("func"), "compile": details[fw].get("compile", False)}
                        if "bits" in details:
                            per[fw][layer]["bits"] = details["bits"]
            self.layer_configs[method] = per

    def benchmark(self, method_filter=METHODS, device="cuda", dtype=torch.float16, num_iters=100):
        for method in method_filter:
            if method not in self.layer_configs:
                continue
            for framework, layer_configs in self.layer_configs[method].items():
                if not layer_configs:
                    continue
                try:
                    t = self.benchmark_func(method, framework, layer_configs, self.num_seq, num_iters, torch.device(device), dtype)
                except Exception as e:
                    print(f"An error occured while benchmarking {method}/{framework}: {e}")
                    continue
                self.benchmark_results.setdefault(method, {}).setdefault(framework, {})["time"] = t

    def summary(self):
        rows = [[m, fw, res["time"]] for m, fws in self.benchmark_results.items() for fw, res in fws.items()]
        table_str = tabulate(rows, headers=["Method", "Framework", "Benchmark Time (ms)"], tablefmt="grid")
        print(table_str)
        out_dir = f"output/{self.name}"
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, f"end2end_summary_{self.num_seq}.txt"), "w") as f:
            f.write(table_str)
        return table_str
