"""Grouped-query softmax attention over the paged cache with a short causal convolution behind each of
the q, k and v projections, a norm a head on q and k, and a rotation of part of each head.

One kernel does everything between the projection and the attention kernels (convolution with the
request's carried history, norm, rotation, queries out, keys and values into the pages), all in 32-bit,
one rounding at the store.  The attention kernels are the ones every attention layer of the package
uses.  They know one head size; here query/key heads and value heads may differ, so every head is
stored in a row of ``padded`` values with zeros behind its own (zeros change no score and add nothing
to a weighted sum of values), and the output projection's columns are padded alike once, at load.
The last taps - 1 projected rows of a request are its state, beside its pages.
"""

from __future__ import annotations

import math

import torch

from .. import kernels
from ..cache.layout import KVCacheSpec, StateSpec
from ..errors import UnsupportedError
from ..weights.loader import ParamDecl
from .linear import Linear
from .registry import register_mixer


class ConvAttention:
    graph_safe = True
    short_portion = kernels.SHORT_PORTION

    @staticmethod
    def declare(spec, hidden: int) -> list:
        H, G, D, V, t = spec.num_heads, spec.num_kv_heads, spec.head_dim, spec.value_dim, spec.conv_taps
        decls = [ParamDecl("q", (H * D, hidden)), ParamDecl("k", (G * D, hidden)), ParamDecl("v", (G * V, hidden)),
                 ParamDecl("q.conv", (H * D, t)), ParamDecl("k.conv", (G * D, t)), ParamDecl("v.conv", (G * V, t)),
                 ParamDecl("o", (hidden, H * V))]
        if spec.qk_norm_eps is not None:
            decls += [ParamDecl("q.norm", (D,), "gain"), ParamDecl("k.norm", (D,), "gain")]
        return decls

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        H, G, D, V = spec.num_heads, spec.num_kv_heads, spec.head_dim, spec.value_dim
        if H < 1 or G < 1 or H % G:
            raise UnsupportedError(f"{H} query heads over {G} key heads, which do not group evenly")
        unit = 1 if dtype == torch.float32 else 16       # the bfloat16 attention kernels take head sizes in 16s
        self.padded = (max(D, V) + unit - 1) // unit * unit
        if not 1 <= self.padded <= 256:
            raise UnsupportedError(f"heads of {D} and {V}: the attention kernels take head sizes up to 256")
        if not 1 <= spec.conv_taps <= 16:
            raise UnsupportedError(f"a convolution of {spec.conv_taps} taps (1 to 16)")
        if spec.rotary_dim % 2 or not 0 <= spec.rotary_dim <= D:
            raise UnsupportedError(f"a rotation over {spec.rotary_dim} values of a head of {D}")
        self.spec, self.dtype = spec, dtype
        self.H, self.G, self.D, self.V = H, G, D, V
        self.scale = float(spec.scale) if spec.scale is not None else 1.0 / math.sqrt(D)
        self.window = int(spec.window or 0)
        self.proj = Linear.fused([params["q"], params["k"], params["v"]])
        self.channels = H * D + G * D + G * V
        f32 = lambda t: t.to(torch.float32).contiguous()
        self.conv_w = torch.cat([f32(params["q.conv"]), f32(params["k.conv"]), f32(params["v.conv"])], 0).t().contiguous()   # [taps, channels]
        if spec.qk_norm_eps is not None:
            self.q_gain, self.k_gain, self.eps = f32(params["q.norm"]), f32(params["k.norm"]), float(spec.qk_norm_eps)
        else:
            # (no norm: a gain of sqrt(mean square) cannot be written as constants; refuse rather than guess)
            raise UnsupportedError("attention with convolutions and without a norm a head on q and k is not built")
        half = spec.rotary_dim // 2
        self.freq = (torch.tensor([spec.rotary_base ** (-2.0 * i / spec.rotary_dim) for i in range(half)],
                                  dtype=torch.float64).to(torch.float32).to(device) if half else None)
        w_o = params["o"]
        if self.padded != V:
            wide = torch.zeros((hidden, H, self.padded), dtype=w_o.dtype, device=w_o.device)
            wide[:, :, :V] = w_o.view(hidden, H, V)
            w_o = wide.view(hidden, H * self.padded)
        self.o_proj = Linear(w_o)

    def cache_spec(self):
        return KVCacheSpec(self.G, self.padded, self.window or None)

    def state_spec(self):
        taps = self.spec.conv_taps
        return StateSpec(((taps - 1) * self.channels,), torch.float32) if taps > 1 else None

    def forward(self, x, ctx):
        batch, kv = ctx.batch, ctx.kv()
        rows = self.proj.forward(x, out_dtype=torch.float32)
        n = rows.shape[0]
        if self.spec.conv_taps > 1:
            history = ctx.state()
        else:
            history = torch.empty((1, 0), dtype=torch.float32, device=rows.device)
        q = torch.empty((n, self.H * self.padded), dtype=self.dtype, device=rows.device)
        kernels.conv_qk_prepare(rows, 0, self.conv_w, history, self.q_gain, self.k_gain, self.eps, self.freq,
                                self.spec.rotary_dim, batch, kv, self.H, self.G, self.D, self.V, self.padded, q)
        if self.spec.conv_taps > 1:
            kernels.conv_history(rows, 0, self.conv_w, history, batch)
        out = torch.empty((n, self.H * self.padded), dtype=self.dtype, device=rows.device)
        kernels.paged_attention(q, out, batch, kv, self.H, self.G, self.padded, self.scale, self.window)
        return self.o_proj.forward(out, out_dtype=torch.float32)


register_mixer("conv_attention", ConvAttention)
