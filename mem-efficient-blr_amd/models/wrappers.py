"""nn.Module wrappers that own structured factors in the layout their forward function expects.

Counterparts of the reference's models/wrappers.py:5-181.  The forward function is resolved from
a dotted path string; the *name* of that function decides parameter layout and call convention,
exactly as in the reference:
  "triton" in name -> kernel layouts, function returns the output tensor;
  "torch"  in name -> baseline layouts, function returns a tuple whose first item is the output;
  BLAST   "bmm" in name  -> U (b, q, r), S (r, b, b), else U (b, r, q), S (b, b, r); V (b, p, r)
  Monarch "left" in name -> w2 (b, r, s), else (b, s, r); w1 (b, p, r)
The bias is added as `out += bias.to(x.dtype)` (reference wrappers.py:176-177); with a library kernel
("triton" names other than the quantized one) the bias - and an activation the owner of the module asks
for by setting `fused_act` ("gelu_tanh", "silu", or "silu_mul": silu(gate) * up over a fused gate|up projection, whose result
has out_features / 2 columns) - is handed to the kernel's output stage instead.
Factors are drawn with std 1/sqrt(fan-in of the factor) instead of the reference's std 1, so that
fp16 activations stay in range at the ranks the networks use.
"""
import importlib
import math

import torch
import torch.nn as nn


def resolve(func_path):
    module_name, func_name = func_path.rsplit(".", 1)
    return func_name, getattr(importlib.import_module(module_name), func_name)


class _StructuredLinear(nn.Module):
    def __init__(self, in_features, out_features, func_path, device, dtype, bias, is_compiled):
        super().__init__()
        self.device, self.dtype = device, dtype
        self.in_features, self.out_features = in_features, out_features
        self.func_name, self.func = resolve(func_path)
        self.is_compiled = is_compiled
        if is_compiled:
            self.func = torch.compile(self.func)
        self.kind = "triton" if "triton" in self.func_name else "torch"
        if bias:
            self.bias = nn.Parameter(torch.randn(out_features, device=device, dtype=dtype))
        else:
            self.register_parameter("bias", None)
        self.fused_act = None          # set by the owner (e.g. an MLP) to have its activation applied by the kernel
        # (the *_fp32 verification names return their intermediates and never read an armed output stage: bias and activation
        # are applied here for them, as for the torch baselines)
        self.fuses = (self.kind == "triton" and not is_compiled and "int8" not in self.func_name and "int4" not in self.func_name
                      and "fp32" not in self.func_name)

    def _param(self, shape, fan_in):
        return nn.Parameter(torch.randn(shape, device=self.device, dtype=torch.float32).mul_(1.0 / math.sqrt(fan_in)).to(self.dtype))

    def _call(self, *args):
        """The forward function; library kernels take bias and activation into their output stage."""
        if not self.fuses:
            return self.func(*args), False
        from triton_funcs import _lib as L
        if self.bias is None and self.fused_act is None and getattr(L._ep_state, "outer", None) is None:
            return self.func(*args), False
        with L.fused_epilogue(self.bias, self.fused_act):          # (also picks up a gate / residual armed by the caller)
            return self.func(*args), True

    def _finish(self, out, fused=False):
        if isinstance(out, tuple):                     # torch baselines and the *_fp32 names: (out, intermediates...)
            out = out[0]
        if fused:
            return out
        if self.bias is not None:
            out += self.bias.to(out.dtype)
        if self.fused_act == "gelu_tanh":
            out = torch.nn.functional.gelu(out, approximate="tanh")
        elif self.fused_act == "silu":
            out = torch.nn.functional.silu(out)
        elif self.fused_act == "silu_mul":
            gate, up = out.chunk(2, dim=-1)
            out = torch.nn.functional.silu(gate) * up
        return out


class BlastLinear(_StructuredLinear):
    def __init__(self, in_features, out_features, b, rank, func_path, device, dtype, bias=True, is_compiled=False):
        super().__init__(in_features, out_features, func_path, device, dtype, bias, is_compiled)
        assert in_features % b == 0 and out_features % b == 0
        self.b, self.rank = b, rank
        p, q = in_features // b, out_features // b
        if self.kind == "triton":
            bmm = "bmm" in self.func_name
            self.U = self._param((b, q, rank) if bmm else (b, rank, q), rank)
            self.V = self._param((b, p, rank), rank)
            self.S = self._param((rank, b, b) if bmm else (b, b, rank), 1)
        else:
            self.U = self._param((b, q, rank), rank)
            self.V = self._param((b, rank, p), rank)
            self.S = self._param((b, b, rank), 1)

    def forward(self, x):
        return self._finish(*self._call(x, self.U, self.V, self.S))

    def extra_repr(self):
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
                f"rank={self.rank}, b={self.b}, func={self.func_name}")


class QuantBlastLinear(BlastLinear):
    """BLAST with int8 / packed-int4 factors (method "blast_sym_quant").

    The factors are quantized once and kept in the order the kernels stream them: buffers ``u_codes`` (b, r, q[/2]),
    ``u_scales`` (b, q), ``v_codes`` (b, p, r[/2]), ``v_scales`` (b, r); int4 packs two codes per byte along the last
    axis, even index in the low nibble.  These buffers are what ``state_dict()`` holds (plus S, the bias and an extra
    state naming bits and layout), so a packed checkpoint loads without touching the floating factors again.
    ``load_state_dict`` also takes a checkpoint of the floating module (keys ``U`` (b, q, r) and ``V`` (b, p, r), the
    bmm layouts) and repacks it on the way in."""
    PACK_FORMAT = "blr-packed-blast/1: U codes (b,r,q[/2]) + scales (b,q); V codes (b,p,r[/2]) + scales (b,r); int4 low nibble = even index"

    def __init__(self, in_features, out_features, b, rank, func_path, device, dtype, bias=True, is_compiled=False, bits=8):
        super().__init__(in_features, out_features, b, rank, func_path, device, dtype, bias, is_compiled)
        assert "bmm" in self.func_name, "the quantized kernel takes the bmm layouts"
        assert bits in (8, 4)
        self.bits = bits
        U, V = self.U.detach().float(), self.V.detach().float()
        del self.U, self.V
        self._pack(U, V)

    def _pack(self, U, V):
        from triton_funcs.blast_sym_quant_kernels import quantize_blast_factors
        Uq, Vq = quantize_blast_factors(U, V, self.bits)
        for name, t in (("u_codes", Uq.codes), ("u_scales", Uq.scales), ("v_codes", Vq.codes), ("v_scales", Vq.scales)):
            if name in self._buffers:
                self._buffers[name] = t
            else:
                self.register_buffer(name, t)
        self._u_shape, self._v_shape = tuple(Uq.shape), tuple(Vq.shape)

    @property
    def Uq(self):
        from triton_funcs.blast_sym_quant_kernels import QuantFactor
        return QuantFactor(self.u_codes, self.u_scales, self.bits, self._u_shape)

    @property
    def Vq(self):
        from triton_funcs.blast_sym_quant_kernels import QuantFactor
        return QuantFactor(self.v_codes, self.v_scales, self.bits, self._v_shape)

    def get_extra_state(self):
        return {"format": self.PACK_FORMAT, "bits": self.bits, "u_shape": list(self._u_shape), "v_shape": list(self._v_shape)}

    def set_extra_state(self, state):
        if state.get("format") != self.PACK_FORMAT:
            raise RuntimeError(f"unknown packed format {state.get('format')!r}")
        if int(state["bits"]) != self.bits:
            raise RuntimeError(f"checkpoint holds {state['bits']}-bit factors, the module {self.bits}-bit")

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        ku, kv = prefix + "U", prefix + "V"
        if ku in state_dict and kv in state_dict:                  # floating checkpoint: repack
            U, V = state_dict.pop(ku), state_dict.pop(kv)
            if tuple(U.shape) != self._u_shape or tuple(V.shape) != self._v_shape:
                error_msgs.append(f"{prefix}: floating factors {tuple(U.shape)}, {tuple(V.shape)} do not fit {self._u_shape}, {self._v_shape}")
            else:
                self._pack(U.to(self.u_codes.device).float(), V.to(self.u_codes.device).float())
                for name in ("u_codes", "u_scales", "v_codes", "v_scales"):
                    state_dict[prefix + name] = self._buffers[name]
                state_dict.setdefault(prefix + "_extra_state", self.get_extra_state())
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs)

    def forward(self, x):
        return self._finish(self.func(x, self.Uq, self.Vq, self.S))


class MonarchLinear(_StructuredLinear):
    def __init__(self, in_features, out_features, b, rank, func_path, device, dtype, bias=True, is_compiled=False):
        super().__init__(in_features, out_features, func_path, device, dtype, bias, is_compiled)
        assert in_features % b == 0 and out_features % b == 0
        assert rank % b == 0
        self.b, self.rank = b, rank
        p, s = in_features // b, out_features // b
        if self.kind == "triton":
            self.w1_bfly = self._param((b, p, rank), p)
            self.w2_bfly = self._param((b, rank, s) if "left" in self.func_name else (b, s, rank), rank)
        else:
            self.w1_bfly = self._param((b, rank, p), p)
            self.w2_bfly = self._param((b, s, rank), rank)

    def forward(self, x):
        return self._finish(*self._call(x, self.w1_bfly, self.w2_bfly))

    def extra_repr(self):
        return (f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, "
                f"rank={self.rank}, b={self.b}, func={self.func_name}")


class LowRankLinear(_StructuredLinear):
    def __init__(self, in_features, out_features, rank, func_path, device, dtype, bias=True, is_compiled=False):
        super().__init__(in_features, out_features, func_path, device, dtype, bias, is_compiled)
        self.rank = rank
        if self.kind == "triton":
            self.V = self._param((in_features, rank), rank)
            self.U = self._param((rank, out_features), rank)
        else:
            self.V = self._param((rank, in_features), rank)
            self.U = self._param((out_features, rank), rank)

    def forward(self, x):
        out, fused = self._call(x, self.V, self.U)
        if self.kind == "triton" and not isinstance(out, tuple):   # the kernel returns (N, out_f): restore the leading dims
            out = out.reshape(*x.shape[:-1], out.shape[-1])
        return self._finish(out, fused)

    def extra_repr(self):
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, rank={self.rank}, func={self.func_name}"


class DenseLinear(_StructuredLinear):
    def __init__(self, in_features, out_features, func_path, device, dtype, bias=True, is_compiled=False):
        super().__init__(in_features, out_features, func_path, device, dtype, bias, is_compiled)
        shape = (in_features, out_features) if self.kind == "triton" else (out_features, in_features)
        self.W = self._param(shape, in_features)

    def forward(self, x):
        out, fused = self._call(x, self.W)
        if self.kind == "triton" and not isinstance(out, tuple):
            out = out.reshape(*x.shape[:-1], out.shape[-1])
        return self._finish(out, fused)

    def extra_repr(self):
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, func={self.func_name}"
