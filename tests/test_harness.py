"""Host-side harness: wrappers' parameter layouts per function name, config schema, dispatch strings,
roofline formulas, DiT module naming.  No GPU work (the torch baselines run on CPU tensors)."""
import glob
import importlib
import os
import pickle

import numpy as np
import pytest
import torch
import yaml

from oracle import blr_oracle as O

PKG = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "mem-efficient-blr_amd")


def test_every_func_path_in_configs_resolves():
    paths = set()
    def walk(node):
        if isinstance(node, dict):
            for k, v in node.items():
                if k in ("func", "funcs"):
                    paths.update(v if isinstance(v, list) else [v])
                else:
                    walk(v)
        elif isinstance(node, list):
            for v in node:
                walk(v)
    files = glob.glob(os.path.join(PKG, "configs", "**", "*.yaml"), recursive=True)
    assert len(files) >= 10
    for f in files:
        walk(yaml.safe_load(open(f)))
    assert len(paths) >= 20
    for p in paths:
        mod, name = p.rsplit(".", 1)
        assert callable(getattr(importlib.import_module(mod), name)), p


def test_wrapper_layouts_follow_function_names():
    from models.wrappers import BlastLinear, DenseLinear, LowRankLinear, MonarchLinear
    kw = dict(device="cpu", dtype=torch.float32)
    m = BlastLinear(32, 48, b=4, rank=6, func_path="triton_funcs.blast_kernels.triton_blast_full_fp16", **kw)
    assert m.U.shape == (4, 6, 12) and m.V.shape == (4, 8, 6) and m.S.shape == (4, 4, 6) and m.bias.shape == (48,)
    m = BlastLinear(32, 48, b=4, rank=6, func_path="triton_funcs.blast_kernels.triton_blast_bmm_fp16", bias=False, **kw)
    assert m.U.shape == (4, 12, 6) and m.V.shape == (4, 8, 6) and m.S.shape == (6, 4, 4) and m.bias is None
    m = BlastLinear(32, 48, b=4, rank=6, func_path="torch_funcs.blast_funcs.torch_blast_baseline", **kw)
    assert m.U.shape == (4, 12, 6) and m.V.shape == (4, 6, 8) and m.S.shape == (4, 4, 6)
    m = MonarchLinear(32, 48, b=4, rank=8, func_path="triton_funcs.monarch_kernels.triton_monarch_right_left_fp16", **kw)
    assert m.w1_bfly.shape == (4, 8, 8) and m.w2_bfly.shape == (4, 8, 12)
    m = MonarchLinear(32, 48, b=4, rank=8, func_path="triton_funcs.monarch_kernels.triton_monarch_right_fp16", **kw)
    assert m.w2_bfly.shape == (4, 12, 8)
    m = MonarchLinear(32, 48, b=4, rank=8, func_path="torch_funcs.monarch_funcs.torch_monarch_baseline", **kw)
    assert m.w1_bfly.shape == (4, 8, 8) and m.w2_bfly.shape == (4, 12, 8)
    with pytest.raises(AssertionError):
        MonarchLinear(32, 48, b=4, rank=6, func_path="torch_funcs.monarch_funcs.torch_monarch_baseline", **kw)
    with pytest.raises(AssertionError):
        BlastLinear(30, 48, b=4, rank=6, func_path="torch_funcs.blast_funcs.torch_blast_baseline", **kw)
    m = LowRankLinear(32, 48, rank=6, func_path="triton_funcs.low_rank_kernels.triton_low_rank_fp16", **kw)
    assert m.V.shape == (32, 6) and m.U.shape == (6, 48)
    m = LowRankLinear(32, 48, rank=6, func_path="torch_funcs.low_rank_funcs.torch_low_rank_baseline", **kw)
    assert m.V.shape == (6, 32) and m.U.shape == (48, 6)
    assert DenseLinear(32, 48, func_path="triton_funcs.dense_kernels.triton_dense_fp16", **kw).W.shape == (32, 48)
    assert DenseLinear(32, 48, func_path="torch_funcs.dense_funcs.torch_dense_baseline", **kw).W.shape == (48, 32)


def test_torch_wrappers_forward_match_oracle_with_bias():
    from models.wrappers import BlastLinear, MonarchLinear, LowRankLinear, DenseLinear
    torch.manual_seed(0)
    kw = dict(device="cpu", dtype=torch.float64)
    x = torch.randn(2, 3, 32, dtype=torch.float64)
    m = BlastLinear(32, 48, b=4, rank=6, func_path="torch_funcs.blast_funcs.torch_blast_baseline", **kw)
    ref = O.blast_forward(x.numpy(), m.U.detach().numpy(), m.V.detach().numpy(), m.S.detach().numpy())[0] + m.bias.detach().numpy()
    np.testing.assert_allclose(m(x).detach().numpy(), ref, atol=1e-10)
    m = MonarchLinear(32, 48, b=4, rank=8, func_path="torch_funcs.monarch_funcs.torch_monarch_baseline", **kw)
    ref = O.monarch_forward(x.numpy(), m.w1_bfly.detach().numpy(), m.w2_bfly.detach().numpy())[0] + m.bias.detach().numpy()
    np.testing.assert_allclose(m(x).detach().numpy(), ref, atol=1e-10)
    m = LowRankLinear(32, 48, rank=6, func_path="torch_funcs.low_rank_funcs.torch_low_rank_baseline", bias=False, **kw)
    np.testing.assert_allclose(m(x).detach().numpy(), O.low_rank_forward(x.numpy(), m.V.detach().numpy(), m.U.detach().numpy())[0], atol=1e-10)
    m = DenseLinear(32, 48, func_path="torch_funcs.dense_funcs.torch_dense_baseline", bias=False, **kw)
    np.testing.assert_allclose(m(x).detach().numpy(), O.dense_forward(x.numpy(), m.W.detach().numpy()), atol=1e-10)


def test_torch_funcs_match_oracle_including_bmm_and_intermediates():
    from torch_funcs.blast_funcs import torch_blast_baseline, torch_blast_bmm
    from torch_funcs.monarch_funcs import torch_monarch_baseline
    rng = np.random.default_rng(0)
    b, p, q, r = 3, 4, 5, 6
    x = rng.standard_normal((2, 3, b * p)); U = rng.standard_normal((b, q, r)); Vt = rng.standard_normal((b, r, p)); S = rng.standard_normal((b, b, r))
    t = torch.from_numpy
    for got, ref in zip(torch_blast_baseline(t(x), t(U), t(Vt), t(S)), O.blast_forward(x, U, Vt, S)):
        np.testing.assert_allclose(got.numpy(), ref, atol=1e-10)
    Sb = np.ascontiguousarray(np.transpose(S, (2, 0, 1)))
    for got, ref in zip(torch_blast_bmm(t(x), t(U), t(Vt), t(Sb)), O.blast_bmm_forward(x, U, Vt, Sb)):
        np.testing.assert_allclose(got.numpy(), ref, atol=1e-10)
    w1 = rng.standard_normal((3, 6, 4)); w2 = rng.standard_normal((3, 5, 6))
    for got, ref in zip(torch_monarch_baseline(t(x), t(w1), t(w2)), O.monarch_forward(x, w1, w2)):
        np.testing.assert_allclose(got.numpy(), ref, atol=1e-10)


def test_replace_linear_by_substring_and_dit_module_names():
    from models.dit_xl import DiT
    from utils import replace_linear_with_custom
    from models.wrappers import BlastLinear
    model = DiT(input_size=8, depth=2, hidden=64, heads=4)
    cfg = {k: {"rank": 8, "b": 4, "func": "torch_funcs.blast_funcs.torch_blast_baseline"} for k in ("attn.qkv", "attn.proj", "mlp.fc1", "mlp.fc2")}
    n = replace_linear_with_custom(model.blocks, cfg, "blast")
    assert n == 8
    for blk in model.blocks:
        assert isinstance(blk.attn.qkv, BlastLinear) and isinstance(blk.mlp.fc2, BlastLinear)
        assert isinstance(blk.adaLN_modulation[1], torch.nn.Linear)          # adaLN stays dense
        assert blk.attn.qkv.in_features == 64 and blk.attn.qkv.out_features == 192
    x = torch.randn(2, 4, 8, 8); tt = torch.randint(0, 1000, (2,)); y = torch.randint(0, 1000, (2,))
    out = model(x, tt, y)
    assert out.shape == (2, 8, 8, 8) and torch.isfinite(out).all()


def test_dit_self_consistency_blast_equals_dense_assembly():
    """Replacing a BlastLinear by a dense layer holding its assembled matrix must not change the model."""
    from models.dit_xl import DiT
    from utils import replace_linear_with_custom
    torch.manual_seed(1)
    model = DiT(input_size=8, depth=1, hidden=64, heads=4).double()
    cfg = {"mlp.fc1": {"rank": 8, "b": 4, "func": "torch_funcs.blast_funcs.torch_blast_baseline"}}
    replace_linear_with_custom(model.blocks, cfg, "blast")
    x = torch.randn(2, 4, 8, 8).double(); tt = torch.randint(0, 1000, (2,)); y = torch.randint(0, 1000, (2,))
    out = model(x, tt, y)
    bl = model.blocks[0].mlp.fc1
    W = O.blast_dense_weight(bl.U.detach().numpy(), bl.V.detach().numpy(), bl.S.detach().numpy())
    lin = torch.nn.Linear(64, 256).double()
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(W)); lin.bias.copy_(bl.bias)
    model.blocks[0].mlp.fc1 = lin
    np.testing.assert_allclose(model(x, tt, y).detach().numpy(), out.detach().numpy(), atol=1e-9)


def test_dit_xl_shape_walkthrough():
    from models.dit_xl import DiT_XL_2
    with torch.device("meta"):
        m = DiT_XL_2()
    assert len(m.blocks) == 28 and m.pos_embed.shape == (1, 256, 1152)
    blk = m.blocks[0]
    assert blk.attn.qkv.weight.shape == (3456, 1152) and blk.attn.proj.weight.shape == (1152, 1152)
    assert blk.mlp.fc1.weight.shape == (4608, 1152) and blk.mlp.fc2.weight.shape == (1152, 4608)
    assert blk.adaLN_modulation[1].weight.shape == (6912, 1152) and m.final_layer.linear.weight.shape == (32, 1152)


def test_layer_config_merge_names_and_roofline(tmp_path, monkeypatch):
    from layer import Layer
    from device import Device
    from roofline import mem_flops_for, roofline_table
    l = Layer(os.path.join(PKG, "configs", "layers", "llama7b.gate_up_proj.yaml"))
    assert (l.in_f, l.out_f, l.blast["b"], l.blast["rank"], l.num_seq) == (4096, 22016, 16, 1024, 1024)
    assert "triton_blast_full_fp16" in l.function_names and "torch_dense_baseline" in l.function_names
    assert len(l.verify_funcs["blast"]) == len(l.bench_funcs["blast"]) == 5
    d = Device("MI355X")
    assert abs(d.break_point - 2.5166e15 / 8e12) < 1e-6
    with pytest.raises(ValueError):
        Device("H100")
    by, fl = mem_flops_for("triton_blast_full_fp16", l, 1)
    assert (by, fl) == O.blast_bytes_flops(1, 4096, 1024, 22016, 16)
    by, fl = mem_flops_for("triton_dense_fp16", l, 2048)
    assert (by, fl) == O.dense_bytes_flops(2048, 4096, 22016)
    rows = roofline_table(l, d)
    assert len(rows) == len(l.function_names) and all(r[5] > 0 for r in rows)
    # a layer file that redefines a list replaces it (shallow merge)
    custom = tmp_path / "x.yaml"
    custom.write_text(open(os.path.join(PKG, "configs", "layers", "gpt2s.mlp_c_fc.yaml")).read() +
                      "\ntriton_blast_verify:\n  funcs:\n    - triton_funcs.blast_kernels.triton_blast_bmm_fp32\n"
                      "triton_blast_benchmark:\n  funcs:\n    - triton_funcs.blast_kernels.triton_blast_bmm_fp16\n")
    l2 = Layer(str(custom))
    assert [f.__name__ for f in l2.bench_funcs["blast"]] == ["triton_blast_bmm_fp16"] and l2.num_seq == 128
    monkeypatch.chdir(tmp_path)
    l2.summary()
    assert (tmp_path / "output" / "gpt2s" / "mlp_c_fc" / "summary.txt").exists()


def test_network_config_parse():
    from network import Network
    n = Network(os.path.join(PKG, "configs", "networks", "dit_xl.yaml"))
    assert n.name == "dit_xl" and n.num_seq == 256
    assert n.layer_configs["blast"]["triton"]["mlp.fc1"] == {"rank": 576, "b": 16, "func": "triton_funcs.blast_kernels.triton_blast_bmm_fp16", "compile": False}
    assert set(n.layer_configs["dense"]["torch"]) == {"attn.qkv", "attn.proj", "mlp.fc1", "mlp.fc2"}


def test_get_config_is_picklable_and_none_before_use():
    from triton_funcs import blast_kernels as K
    assert K.get_triton_blast_partial_fp16_config() is None
    pickle.dumps(K.get_triton_blast_partial_fp16_config())


def test_gpu_profile_summaries_from_rocprof_csv(tmp_path):
    """The profile tool's readers of rocprofv3's csv files: per-kernel durations, counter means and the scale taken from a copy
    of known size."""
    import gpu_profile as G
    kt = tmp_path / "kt_kernel_trace.csv"
    kt.write_text('"Kind","Kernel_Name","Start_Timestamp","End_Timestamp","Workgroup_Size_X","Grid_Size_X","Grid_Size_Y","Grid_Size_Z"\n'
                  '"KERNEL_DISPATCH","blr::a",1000,3000,256,1024,1,1\n'
                  '"KERNEL_DISPATCH","blr::a",5000,9000,256,1024,1,1\n'
                  '"KERNEL_DISPATCH","other",100,200,64,64,1,1\n')
    s = G.summarize_kernel_trace(str(kt))
    assert s[("blr::a", 1024, 256)] == {"calls": 2, "avg_us": 3.0, "min_us": 2.0, "max_us": 4.0}
    assert "other" not in G.format_trace(s, only=["blr"]) and "blr::a" in G.format_trace(s, only=["blr"])
    cc = tmp_path / "pmc_counter_collection.csv"
    cc.write_text('"Dispatch_Id","Kernel_Name","Counter_Name","Counter_Value"\n'
                  '1,"__amd_rocclr_copyBuffer","FETCH_SIZE",131072.0\n2,"__amd_rocclr_copyBuffer","FETCH_SIZE",131072.0\n'
                  '3,"blr::a","FETCH_SIZE",1000.0\n4,"blr::a","FETCH_SIZE",3000.0\n')
    c = G.summarize_counters(str(cc))
    assert c[("blr::a", "FETCH_SIZE")] == {"dispatches": 2, "mean": 2000.0, "min": 1000.0, "max": 3000.0}
    assert G.counter_unit_bytes(c, "FETCH_SIZE") == G.CALIB_BYTES / 131072.0
    assert G.counter_unit_bytes(c, "WRITE_SIZE") is None


def test_bench_takes_roofline_traffic_from_the_committed_profile():
    """bench.py's roofline.traffic is read from the counter summary under profiles/, not typed into the script."""
    import importlib.util
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_mod", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec); spec.loader.exec_module(bench)
    assert os.path.exists(os.path.join(root, bench.DOMINANT_PROFILE))
    t = bench.traffic_from_profile(bench.DOMINANT_PROFILE)
    algorithmic = bench.blast_bytes_flops(1, 4096, 1024, 22016)[0]
    assert t is not None and algorithmic <= t <= 1.5 * algorithmic
    assert bench.traffic_from_profile("profiles/no_such_file.txt") is None
    text = open(os.path.join(root, bench.DOMINANT_PROFILE)).read()
    assert bench.DOMINANT_KERNEL.split("<")[0] in text


def test_roofline_formulas_are_the_references_name_by_name():
    """Hand-evaluated values of the reference's formulas (roofline.py:7-99) at n=2, i=8, r=4, o=12, b1=b2=b=2, 2 bytes per element."""
    import roofline as R
    n, i, r, o, b, e = 2, 8, 4, 12, 2, 2
    assert R.torch_low_rank_baseline_mem_flops(n, i, r, o, e) == (272, 320)
    assert R.triton_low_rank_mem_flops(n, i, r, o, e) == (240, 320)
    assert R.torch_dense_baseline_mem_flops(n, i, o, e) == R.triton_dense_mem_flops(n, i, o, e) == (272, 384)
    assert R.torch_blast_baseline_mem_flops(n, i, r, o, b, b, e) == (528, 384)
    assert R.triton_blast_partial_mem_flops(n, i, r, o, b, b, e) == (336, 384)
    assert R.triton_blast_partial_grouped_mem_flops(n, i, r, o, b, b, e) == (336, 384)
    assert R.triton_blast_partial_grouped_persistent_mem_flops(n, i, r, o, b, b, e) == (336, 384)
    assert R.triton_blast_bmm_int8_mem_flops(n, i, r, o, b, b, e) == (304, 384)
    assert R.triton_blast_full_mem_flops(n, i, r, o, b, b, e) == (272, 384)
    assert R.triton_blast_bmm_mem_flops(n, i, r, o, b, b, e) == (400, 384)
    assert R.triton_monarch_right_mem_flops(n, i, r, o, b, e) == (400, 320)
    assert R.triton_monarch_right_ideal_mem_flops(n, i, r, o, b, e) == R.triton_monarch_right_left_mem_flops(n, i, r, o, b, e) == (304, 320)
    assert R.torch_monarch_baseline_mem_flops(n, i, r, o, b, e) == (464, 320)
    # weight-quantized BLAST (this library's own): codes r (i + o) bits / 8, the rest at e bytes
    assert R.triton_blast_bmm_int4_mem_flops(n, i, r, o, b, b, e) == (4 * 20 // 2 + 2 * (16 + 12 + 8 + 2 * 20), 384)


def test_every_exported_operator_name_has_a_roofline_formula():
    import importlib
    import roofline as R
    for mod in ("blast_kernels", "blast_sym_quant_kernels", "monarch_kernels", "low_rank_kernels", "dense_kernels"):
        m = importlib.import_module(f"triton_funcs.{mod}")
        for name in m.__all__:
            if not name.startswith("triton_") or "load_store" in name:
                continue
            stem = name.rsplit("_", 1)[0]
            assert hasattr(R, f"{stem}_mem_flops"), f"{name}: no {stem}_mem_flops in roofline.py"
