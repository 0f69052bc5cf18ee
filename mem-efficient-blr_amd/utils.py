"""Harness helpers: verification status, YAML loading, do_verify, do_bench, linear-layer replacement.

Counterparts of the reference's utils.py:8-116 (and of triton.testing.do_bench, which the reference's
layer.py uses for timing and which is not available without Triton).
"""
import os
from enum import Enum

import torch
import yaml

from models.wrappers import BlastLinear, DenseLinear, LowRankLinear, MonarchLinear, QuantBlastLinear

try:                                   # GPT-2 style linears, only if transformers is importable
    from transformers import Conv1D
except Exception:                      # pragma: no cover
    Conv1D = None


class VerificationStatus(Enum):
    MATCH = 1
    DIFFER = 0
    FAIL = -1
    UNKNOWN = -2
    NA = -3


def next_power_of_2(x):
    return 1 if x < 1 else 1 << (x - 1).bit_length()


def load_yaml(file_path):
    with open(file_path, "r") as f:
        return yaml.safe_load(f)


def merge_dicts(dst, src):
    """Recursive merge: nested dicts are merged, lists are united, everything else is overwritten."""
    for key, value in src.items():
        if isinstance(value, dict) and key in dst:
            dst[key] = merge_dicts(dst.get(key, {}), value)
        elif isinstance(value, list) and key in dst:
            dst[key] = list(set(dst[key] + value))
        else:
            dst[key] = value
    return dst


def do_verify(triton_out, torch_out, rtol=0, atol=1e-1):
    """allclose(atol=1e-1, rtol=0) like the reference (utils.py:35-44)."""
    if torch.allclose(triton_out, torch_out, atol=atol, rtol=rtol):
        print("✅ kernel and torch baseline match")
        return VerificationStatus.MATCH
    print("❌ kernel and torch baseline differ")
    print(f"Max abs difference = {(triton_out - torch_out).abs().max()}")
    return VerificationStatus.DIFFER


_flush = {}


def do_bench(fn, warmup=25, rep=100, flush_bytes=256 << 20):
    """Mean milliseconds per call, timed with events, a 256 MB buffer zeroed before every timed call.

    Same protocol as triton.testing.do_bench (estimate from 5 calls, ~25 ms warm-up, ~100 ms of
    timed calls, cache flush before each)."""
    dev = torch.cuda.current_device()
    if dev not in _flush:
        _flush[dev] = torch.empty(flush_bytes, dtype=torch.int8, device="cuda")
    cache = _flush[dev]
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        cache.zero_()
        fn()
    e1.record()
    torch.cuda.synchronize()
    est = max(e0.elapsed_time(e1) / 5, 1e-3)
    n_warm, n_rep = max(1, int(warmup / est)), max(1, int(rep / est))
    for _ in range(n_warm):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_rep)]
    for i in range(n_rep):
        cache.zero_()
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    return sum(s.elapsed_time(e) for s, e in zip(starts, ends)) / n_rep


def _is_linear(module):
    return isinstance(module, torch.nn.Linear) or (Conv1D is not None and isinstance(module, Conv1D))


def replace_linear_with_custom(model, layer_configs, method, skip_keys=None):
    """Swap every nn.Linear / Conv1D whose qualified name contains a key of layer_configs.

    Same matching rule as the reference (substring of the module name, utils.py:46-116)."""
    skip_keys = skip_keys or []
    targets = []
    for name, module in model.named_modules():
        if not _is_linear(module) or any(s in name for s in skip_keys):
            continue
        for key, cfg in layer_configs.items():
            if key in name:
                targets.append((name, module, cfg))
                break
    for name, module, cfg in targets:
        parent = model
        *path, attr = name.split(".")
        for part in path:
            parent = getattr(parent, part)
        if isinstance(module, torch.nn.Linear):
            in_f, out_f = module.in_features, module.out_features
        else:
            in_f, out_f = module.nx, module.nf
        common = dict(func_path=cfg["func"], device=module.weight.device, dtype=module.weight.dtype,
                      bias=module.bias is not None, is_compiled=cfg.get("compile", False))
        if method == "blast":
            new = BlastLinear(in_f, out_f, b=cfg["b"], rank=cfg["rank"], **common)
        elif method == "blast_sym_quant":
            if "torch" in cfg["func"]:
                new = BlastLinear(in_f, out_f, b=cfg["b"], rank=cfg["rank"], **common)
            else:
                new = QuantBlastLinear(in_f, out_f, b=cfg["b"], rank=cfg["rank"], bits=cfg.get("bits", 8), **common)
        elif method == "monarch":
            new = MonarchLinear(in_f, out_f, b=cfg["b"], rank=cfg["rank"], **common)
        elif method == "low_rank":
            new = LowRankLinear(in_f, out_f, rank=cfg["rank"], **common)
        elif method == "dense":
            new = DenseLinear(in_f, out_f, **common)
        else:
            raise ValueError(f"unknown method {method}")
        setattr(parent, attr, new)
    print(f"Replaced {len(targets)} linear layers with {method} layers")
    return len(targets)
