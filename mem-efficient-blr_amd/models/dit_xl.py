"""DiT-XL/2 forward in plain torch, with its linears replaceable by the structured wrappers.

The reference builds Meta's DiT through timm (DiT/models.py:101-249, models/dit_xl.py:10-57); timm is
not a dependency here, so the architecture is restated: 2x2 patch embedding (Conv2d), fixed 2-D
sin-cos position table, timestep and label embedders, 28 adaLN-Zero blocks (hidden 1152, 16 heads,
MLP 4608, GELU-tanh, scaled-dot-product attention) and the adaLN final layer.  Module names
(`blocks.N.attn.qkv`, `attn.proj`, `mlp.fc1`, `mlp.fc2`, `adaLN_modulation.1`) match the keys the
network YAML uses for substring replacement.  Weights are random: the harness measures time only.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from utils import replace_linear_with_custom


def modulate(x, shift, scale):
    """x * (1 + scale) + shift (reference DiT/models.py:19-20) as one pass over x."""
    return torch.addcmul(shift.unsqueeze(1), x, (1 + scale).unsqueeze(1))


def _gated(linear, h, gate, residual):
    """residual + gate.unsqueeze(1) * linear(h) (reference DiT/models.py:120-121).  A structured linear that fuses its output stage
    does the whole update while it writes its result; anything else gets one elementwise pass."""
    if gate is None:
        return linear(h)
    if getattr(linear, "fuses", False):
        from triton_funcs import _lib as L
        with L.gate_residual(gate, h.shape[1], residual):
            return linear(h).reshape(residual.shape)
    return torch.addcmul(residual, gate.unsqueeze(1), linear(h))


class TimestepEmbedder(nn.Module):
    def __init__(self, hidden, freq_dim=256):
        super().__init__()
        self.freq_dim = freq_dim
        self.mlp = nn.Sequential(nn.Linear(freq_dim, hidden), nn.SiLU(), nn.Linear(hidden, hidden))

    def forward(self, t):
        half = self.freq_dim // 2
        freqs = torch.exp(-math.log(10000.0) * torch.arange(half, dtype=torch.float32, device=t.device) / half)
        args = t[:, None].float() * freqs[None]
        emb = torch.cat([torch.cos(args), torch.sin(args)], dim=-1)
        return self.mlp(emb.to(self.mlp[0].weight.dtype))        # model dtype (the reference hard-casts to bf16)


class Attention(nn.Module):
    def __init__(self, dim, heads):
        super().__init__()
        self.heads = heads
        self.qkv = nn.Linear(dim, dim * 3, bias=True)
        self.proj = nn.Linear(dim, dim, bias=True)

    def forward(self, x, gate=None, residual=None):
        """attention(x), or residual + gate * attention(x) with the update done by the last linear's output stage."""
        B, N, C = x.shape
        qkv = self.qkv(x).reshape(B, N, 3, self.heads, C // self.heads).permute(2, 0, 3, 1, 4)
        o = F.scaled_dot_product_attention(qkv[0], qkv[1], qkv[2])
        return _gated(self.proj, o.transpose(1, 2).reshape(B, N, C), gate, residual)


class Mlp(nn.Module):
    def __init__(self, dim, hidden):
        super().__init__()
        self.fc1 = nn.Linear(dim, hidden)
        self.act = nn.GELU(approximate="tanh")
        self.fc2 = nn.Linear(hidden, dim)

    def forward(self, x, gate=None, residual=None):
        h = self.fc1(x)
        if getattr(self.fc1, "fused_act", None) is None:     # a structured fc1 applies the GELU in its kernel's output stage
            h = self.act(h)
        return _gated(self.fc2, h, gate, residual)


class DiTBlock(nn.Module):
    def __init__(self, hidden, heads, mlp_ratio=4.0):
        super().__init__()
        self.norm1 = nn.LayerNorm(hidden, elementwise_affine=False, eps=1e-6)
        self.attn = Attention(hidden, heads)
        self.norm2 = nn.LayerNorm(hidden, elementwise_affine=False, eps=1e-6)
        self.mlp = Mlp(hidden, int(hidden * mlp_ratio))
        self.adaLN_modulation = nn.Sequential(nn.SiLU(), nn.Linear(hidden, 6 * hidden))

    def forward(self, x, c):
        s1, c1, g1, s2, c2, g2 = self.adaLN_modulation(c).chunk(6, dim=1)
        # gate and residual (reference DiT/models.py:120-121) in one elementwise pass each
        x = self.attn(modulate(self.norm1(x), s1, c1), gate=g1, residual=x)
        x = self.mlp(modulate(self.norm2(x), s2, c2), gate=g2, residual=x)
        return x


class FinalLayer(nn.Module):
    def __init__(self, hidden, patch, out_ch):
        super().__init__()
        self.norm_final = nn.LayerNorm(hidden, elementwise_affine=False, eps=1e-6)
        self.linear = nn.Linear(hidden, patch * patch * out_ch)
        self.adaLN_modulation = nn.Sequential(nn.SiLU(), nn.Linear(hidden, 2 * hidden))

    def forward(self, x, c):
        shift, scale = self.adaLN_modulation(c).chunk(2, dim=1)
        return self.linear(modulate(self.norm_final(x), shift, scale))


def sincos_2d(dim, grid):
    def one(d, pos):
        omega = 1.0 / 10000 ** (torch.arange(d // 2, dtype=torch.float64) / (d / 2))
        out = pos.reshape(-1)[:, None] * omega[None]
        return torch.cat([torch.sin(out), torch.cos(out)], dim=1)
    ys, xs = torch.meshgrid(torch.arange(grid, dtype=torch.float64), torch.arange(grid, dtype=torch.float64), indexing="ij")
    return torch.cat([one(dim // 2, xs), one(dim // 2, ys)], dim=1).float()        # (grid*grid, dim)


class DiT(nn.Module):
    def __init__(self, input_size=32, patch=2, in_ch=4, hidden=1152, depth=28, heads=16, mlp_ratio=4.0, classes=1000, learn_sigma=True):
        super().__init__()
        self.patch, self.in_ch, self.out_ch = patch, in_ch, in_ch * 2 if learn_sigma else in_ch
        self.x_embedder = nn.Conv2d(in_ch, hidden, kernel_size=patch, stride=patch)
        self.t_embedder = TimestepEmbedder(hidden)
        self.y_embedder = nn.Embedding(classes + 1, hidden)
        self.register_buffer("pos_embed", sincos_2d(hidden, input_size // patch)[None], persistent=False)
        self.blocks = nn.ModuleList([DiTBlock(hidden, heads, mlp_ratio) for _ in range(depth)])
        self.final_layer = FinalLayer(hidden, patch, self.out_ch)

    def forward(self, x, t, y):
        B, _, H, W = x.shape
        h = self.x_embedder(x).flatten(2).transpose(1, 2) + self.pos_embed.to(x.dtype)
        c = self.t_embedder(t) + self.y_embedder(y)
        for blk in self.blocks:
            h = blk(h, c)
        h = self.final_layer(h, c)                                                   # (B, T, p*p*out_ch)
        g, p = H // self.patch, self.patch
        h = h.reshape(B, g, g, p, p, self.out_ch)
        return torch.einsum("nhwpqc->nchpwq", h).reshape(B, self.out_ch, g * p, g * p)


def DiT_XL_2(**kw):
    return DiT(depth=28, hidden=1152, patch=2, heads=16, **kw)


class CustomDiT(nn.Module):
    """DiT-XL/2 with the linears of its blocks swapped per `layer_configs` (cf. reference models/dit_xl.py:10-30)."""

    def __init__(self, layer_configs=None, method=None, dtype=torch.float16, device="cuda", input_size=32, depth=28):
        super().__init__()
        self.model = DiT(input_size=input_size, depth=depth).eval().to(device).to(dtype)
        self.device, self.dtype = device, dtype
        self.replaced = 0
        if layer_configs is not None and method is not None:
            self.replaced = replace_linear_with_custom(self.model.blocks, layer_configs, method)
            for blk in self.model.blocks:                    # hand the MLP's activation to a structured fc1
                if hasattr(blk.mlp.fc1, "fused_act"):
                    blk.mlp.fc1.fused_act = "gelu_tanh"

    def forward(self, x, t, y):
        return self.model(x, t, y)


def capture_forward(model, x, t, y, warmup=3):
    """One forward of `model` captured into a HIP graph on a side stream.  Returns (graph, output tensor the replays write).

    The eager warm-up runs on the capture stream, so that every workspace the operators keep per stream exists, at its final
    size, before the capture begins; the replays then launch the ~1500 kernels of a forward without a Python or ctypes hop."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        for _ in range(warmup):
            model(x, t, y)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            out = model(x, t, y)
    torch.cuda.synchronize()
    return g, out


def benchmark(method, framework, layer_configs, num_seq, num_iters, device, dtype, batch=16, graph=True, return_output=False):
    """Milliseconds per forward of `batch` latents [batch, 4, 32, 32] (256 tokens per image); graph: replay a captured forward."""
    torch.manual_seed(0)
    side = int(round(math.sqrt(num_seq))) * 2
    model = CustomDiT(layer_configs=layer_configs, method=method, dtype=dtype, device=device, input_size=side)
    x = torch.randn(batch, 4, side, side, device=device, dtype=dtype)
    t = torch.randint(0, 1000, (batch,), device=device)
    y = torch.randint(0, 1000, (batch,), device=device)
    with torch.no_grad():
        if graph:
            g, out = capture_forward(model, x, t, y)
            step = g.replay
        else:
            for _ in range(3):
                out = model(x, t, y)
            step = lambda: model(x, t, y)
        step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(num_iters):
            step()
        e1.record()
        torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / num_iters
    return (ms, out) if return_output else ms
