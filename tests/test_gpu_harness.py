"""GPU: the harness dispatches every configured function name to the HIP kernels and they verify."""
import os

import numpy as np
import pytest
import torch

from oracle import blr_oracle as O
from gpu_util import assert_close, say

pytestmark = pytest.mark.gpu
PKG = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "mem-efficient-blr_amd")


@pytest.mark.parametrize("cfg", ["gpt2s.mlp_c_fc", "dit_xl.fc1"])
def test_layer_verify_all_match(cfg, tmp_path, monkeypatch):
    from layer import Layer
    from utils import VerificationStatus
    monkeypatch.chdir(tmp_path)
    l = Layer(os.path.join(PKG, "configs", "layers", cfg + ".yaml"))
    l.num_seq = min(l.num_seq, 256)
    say(f"[case] Layer.verify {cfg}")
    l.verify("all")
    for fam in ("blast", "monarch", "low_rank", "dense"):
        assert l.status[fam] and all(s == VerificationStatus.MATCH for s in l.status[fam]), (fam, l.status[fam])
    say(f"[case] Layer.benchmark {cfg}")
    l.benchmark("all")
    ms = l.measured_ms()
    assert all(t > 0 for t in ms.values()), ms
    l.summary()
    assert os.path.exists(f"output/{l.network_name}/{l.layer_name}/triton_blast_full_fp16_best_config.pkl")
    assert os.path.exists(f"output/{l.network_name}/{l.layer_name}/triton_blast_bmm_xv_fp16_best_config.pkl")


REFERENCE_SWEEP_LAYERS = ["dit_xl.adaln", "gpt2s.c_attn", "gpt2s.mlp_c_proj", "llama1b.down_proj", "llama1b.gate_proj", "llama1b.qo_proj",
                          "llama1b.up_proj", "vit_b_patch16_224.attn_qkv", "vit_b_patch16_224.mlp_fc1", "vit_b_patch16_224.mlp_fc2",
                          "vit_b_patch8_224.attn_qkv", "vit_b_patch8_224.mlp_fc1", "vit_b_patch8_224.mlp_fc2"]


@pytest.mark.parametrize("num_seq", [1, 48, 300])
@pytest.mark.parametrize("cfg", REFERENCE_SWEEP_LAYERS)
def test_reference_sweep_layers_verify(cfg, num_seq, tmp_path, monkeypatch):
    """The layer files of the reference's own sweeps (configs/layers/*.yaml: 3, 6, 9 and 16 blocks, Monarch with 16 blocks,
    ranks 128 to 768) through Layer.verify at one row, a few dozen and a few hundred: every function of every family MATCHes."""
    from layer import Layer
    from utils import VerificationStatus
    monkeypatch.chdir(tmp_path)
    l = Layer(os.path.join(PKG, "configs", "layers", cfg + ".yaml"))
    l.num_seq = num_seq
    say(f"[case] Layer.verify {cfg} num_seq={num_seq}")
    l.verify("all")
    for fam in ("blast", "monarch", "low_rank", "dense"):
        if fam == "monarch" and l.monarch is None:
            continue
        assert l.status[fam] and all(s == VerificationStatus.MATCH for s in l.status[fam]), (fam, l.status[fam])


@pytest.mark.parametrize("M", [1, 40])
def test_wrappers_on_gpu_vs_oracle(M):
    from models.wrappers import BlastLinear, MonarchLinear, LowRankLinear, DenseLinear, QuantBlastLinear
    torch.manual_seed(0)
    kw = dict(device="cuda", dtype=torch.float16)
    x = torch.randn(1, M, 256, **kw)
    f64 = lambda t: t.detach().double().cpu().numpy()
    say(f"[case] wrappers M={M}")
    m = BlastLinear(256, 384, b=4, rank=64, func_path="triton_funcs.blast_kernels.triton_blast_full_fp16", **kw)
    Ut, Vt, St = f64(m.U).transpose(0, 2, 1), f64(m.V).transpose(0, 2, 1), f64(m.S).transpose(1, 0, 2)
    assert_close(m(x), O.blast_forward(f64(x), Ut, Vt, St)[0] + f64(m.bias), torch.float16, "BlastLinear")
    m = MonarchLinear(256, 384, b=4, rank=64, func_path="triton_funcs.monarch_kernels.triton_monarch_right_left_fp16", bias=False, **kw)
    out = m(x)
    assert out.shape == (1, M, 384) and torch.isfinite(out).all()
    m = LowRankLinear(256, 384, rank=64, func_path="triton_funcs.low_rank_kernels.triton_low_rank_fp16", **kw)
    assert_close(m(x), O.low_rank_forward(f64(x), f64(m.V).T, f64(m.U).T)[0] + f64(m.bias), torch.float16, "LowRankLinear")
    m = DenseLinear(256, 384, func_path="triton_funcs.dense_kernels.triton_dense_fp16", **kw)
    assert_close(m(x), O.dense_forward(f64(x), f64(m.W).T) + f64(m.bias), torch.float16, "DenseLinear")
    if M <= 16:
        m = QuantBlastLinear(256, 384, b=4, rank=64, func_path="triton_funcs.blast_sym_quant_kernels.triton_blast_bmm_int8_fp16", **kw)
        out = m(x)
        assert out.shape == (1, M, 384) and torch.isfinite(out).all()


def test_dit_small_blast_matches_its_dense_assembly():
    """2-block DiT with BLAST kernels vs the same model with each BlastLinear replaced by its dense matrix."""
    from models.dit_xl import CustomDiT
    torch.manual_seed(0)
    cfg = {k: {"rank": r, "b": 16, "func": "triton_funcs.blast_kernels.triton_blast_bmm_fp16"}
           for k, r in (("attn.qkv", 288), ("attn.proj", 288), ("mlp.fc1", 576), ("mlp.fc2", 576))}
    say("[case] DiT depth 2, BLAST")
    net = CustomDiT(layer_configs=cfg, method="blast", depth=2)
    assert net.replaced == 8
    x = torch.randn(4, 4, 32, 32, device="cuda", dtype=torch.float16)
    t = torch.randint(0, 1000, (4,), device="cuda"); y = torch.randint(0, 1000, (4,), device="cuda")
    with torch.no_grad():
        out = net(x, t, y).float()
        say("  replays equal the eager forward; assembling the dense matrices")

        def assemble(bl):                                   # W[(i,q),(j,p)] = sum_r U[i,q,r] S[r,i,j] V[j,p,r], fp32 on the GPU
            W = torch.einsum("iqr,rij,jpr->iqjp", bl.U.float(), bl.S.float(), bl.V.float())
            return W.reshape(bl.out_features, bl.in_features)

        first = net.model.blocks[0].attn.proj                # the einsum against the oracle's assembly, once
        S0 = first.S.detach().double().cpu().numpy().transpose(1, 2, 0)            # (r,i,j) -> (i,j,r)
        W0 = O.blast_dense_weight(first.U.detach().double().cpu().numpy(), first.V.detach().double().cpu().numpy().transpose(0, 2, 1), S0)
        assert np.abs(assemble(first).double().cpu().numpy() - W0).max() <= 1e-4 * np.abs(W0).max()
        for blk in net.model.blocks:
            for parent, name in ((blk.attn, "qkv"), (blk.attn, "proj"), (blk.mlp, "fc1"), (blk.mlp, "fc2")):
                bl = getattr(parent, name)
                lin = torch.nn.Linear(bl.in_features, bl.out_features).cuda().half()
                lin.weight.copy_(assemble(bl)); lin.bias.copy_(bl.bias)
                setattr(parent, name, lin)
        say("  dense forward")
        ref = net(x, t, y).float()
    assert out.shape == (4, 8, 32, 32)
    assert (out - ref).abs().max() <= 2e-2 * ref.abs().max()


def test_dit_full_depth_graph_replay_is_finite_and_matches_dense_assembly():
    """BASELINE config 5 at full size - 28 blocks, 16 latents of 256 tokens, every block linear a BLAST layer - run the way the
    benchmark runs it (a captured forward, replayed): every replay equals the eager forward bit for bit, the output is finite,
    and it agrees with the same network after each BLAST layer has been replaced by its assembled dense matrix."""
    from models.dit_xl import CustomDiT, capture_forward
    torch.manual_seed(0)
    cfg = {k: {"rank": r, "b": 16, "func": "triton_funcs.blast_kernels.triton_blast_bmm_fp16"}
           for k, r in (("attn.qkv", 288), ("attn.proj", 288), ("mlp.fc1", 576), ("mlp.fc2", 576))}
    say("[case] DiT-XL/2 depth 28 batch 16, BLAST, graph replay")
    net = CustomDiT(layer_configs=cfg, method="blast", depth=28)
    assert net.replaced == 112
    x = torch.randn(16, 4, 32, 32, device="cuda", dtype=torch.float16)
    t = torch.randint(0, 1000, (16,), device="cuda"); y = torch.randint(0, 1000, (16,), device="cuda")
    with torch.no_grad():
        eager = net(x, t, y).clone()
        g, out = capture_forward(net, x, t, y, warmup=1)
        for rep in range(3):
            out.zero_()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager), f"replay {rep} differs from the eager forward"
        assert eager.shape == (16, 8, 32, 32) and torch.isfinite(eager).all()
        say("  replays equal the eager forward; assembling the dense matrices")

        def assemble(bl):                                   # W[(i,q),(j,p)] = sum_r U[i,q,r] S[r,i,j] V[j,p,r], fp32 on the GPU
            W = torch.einsum("iqr,rij,jpr->iqjp", bl.U.float(), bl.S.float(), bl.V.float())
            return W.reshape(bl.out_features, bl.in_features)

        first = net.model.blocks[0].attn.proj                # the einsum against the oracle's assembly, once
        S0 = first.S.detach().double().cpu().numpy().transpose(1, 2, 0)            # (r,i,j) -> (i,j,r)
        W0 = O.blast_dense_weight(first.U.detach().double().cpu().numpy(), first.V.detach().double().cpu().numpy().transpose(0, 2, 1), S0)
        assert np.abs(assemble(first).double().cpu().numpy() - W0).max() <= 1e-4 * np.abs(W0).max()
        for blk in net.model.blocks:
            for parent, name in ((blk.attn, "qkv"), (blk.attn, "proj"), (blk.mlp, "fc1"), (blk.mlp, "fc2")):
                bl = getattr(parent, name)
                lin = torch.nn.Linear(bl.in_features, bl.out_features).cuda().half()
                lin.weight.copy_(assemble(bl)); lin.bias.copy_(bl.bias)
                setattr(parent, name, lin)
        say("  dense forward")
        ref = net(x, t, y).float()
    err = (eager.float() - ref).abs().max().item()
    say(f"  max |blast - dense assembly| = {err:.4g} of max |ref| = {ref.abs().max().item():.4g}")
    assert err <= 5e-2 * ref.abs().max().item()          # 28 blocks of fp16 rounding on both sides


def test_gpu_profile_traces_a_function_under_rocprofv3(tmp_path):
    """The collection tool end to end: rocprofv3 --kernel-trace around the tool's own run mode (a child process), summary on disk."""
    import shutil
    import subprocess
    import sys
    if shutil.which("rocprofv3") is None:
        pytest.skip("rocprofv3 is not on PATH")
    pkg = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "mem-efficient-blr_amd")
    say("[case] gpu_profile trace of triton_blast_full_fp16")
    out = tmp_path / "prof"
    cmd = [sys.executable, os.path.join(pkg, "gpu_profile.py"), "--mode", "trace", "--function_name", "triton_funcs.blast_kernels.triton_blast_full_fp16",
           "--num_seq", "8", "--in_f", "1024", "--out_f", "1024", "--b", "16", "--rank", "128", "--num_iters", "6", "--num_warmup_iters", "2",
           "--output_dir", str(out), "--timeout", "150"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=170, env=dict(os.environ, TMPDIR=str(tmp_path)))
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    text = (out / "triton_blast_full_fp16_kernels.txt").read_text()
    rows = [ln for ln in text.splitlines() if "blr" in ln and "command:" not in ln]
    assert rows, text
    assert any(int(ln.split()[-4]) >= 8 for ln in rows), text          # 2 warm-up + 6 timed calls of at least one kernel


def test_fp32_verification_names_keep_bias_gate_and_residual():
    """The *_fp32 names return their intermediates and never read an armed output stage; a wrapper module built on one must
    apply bias, gate and residual itself (reference DiT/models.py:120-121: x + gate.unsqueeze(1) * f(x))."""
    import torch
    from models import wrappers as W
    from models.dit_xl import _gated
    torch.manual_seed(0)
    lin = W.BlastLinear(128, 160, 4, 32, "triton_funcs.blast_kernels.triton_blast_full_fp32", torch.device("cuda"), torch.float32, bias=True)
    assert lin.fuses is False
    h = torch.randn(2, 24, 128, device="cuda"); gate = torch.randn(2, 160, device="cuda"); resid = torch.randn(2, 24, 160, device="cuda")
    with torch.no_grad():
        plain = lin.func(h, lin.U, lin.V, lin.S)[0] + lin.bias
        got = _gated(lin, h, gate, resid)
    want = resid + gate.unsqueeze(1) * plain
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-5)
