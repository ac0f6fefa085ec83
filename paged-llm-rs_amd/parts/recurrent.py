"""Mixers that keep a matrix of state a head instead of keys and values in pages: linear attention with
a fixed decay, the matrix memory with exponential gates (mLSTM), and the gated delta rule.

All three are one product for every projection of the layer's input (32-bit sums out), the scan over
the step's tokens request by request (``kernels.recurrent_scan``: state, gates, decays and read-out in
32-bit, from and into the request's state slot), a norm over groups of the read-out times a gate, and
the output projection.  A request's state is one run of 32-bit floats in its slot; what a step's result
is does not depend on how the tokens were cut into steps, since the scan walks tokens one by one.
"""

from __future__ import annotations

import torch

from .. import kernels
from ..cache.layout import StateSpec
from ..errors import ConfigError, UnsupportedError
from ..weights.loader import ParamDecl
from .linear import Linear
from .registry import register_mixer


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).contiguous()


class _ScanMixer:
    """What the three have in common: the fused projection and where its pieces lie in a row."""

    graph_safe = True

    def _fuse(self, params: dict, names: list) -> None:
        self.columns, at = {}, 0
        for name in names:
            self.columns[name] = at
            at += params[name].shape[0]
        self.proj = Linear.fused([params[name] for name in names])

    @staticmethod
    def _sizes(spec, what: str) -> None:
        if spec.num_heads < 1 or not 1 <= spec.head_dim <= kernels.SCAN_MAX_DIM or spec.value_dim < 1:
            raise UnsupportedError(f"{what} of {spec.num_heads} heads of {spec.head_dim} by {spec.value_dim}: the scan "
                                   f"takes q and k up to {kernels.SCAN_MAX_DIM} a head")

    def cache_spec(self):
        return None


class LightningAttention(_ScanMixer):
    @staticmethod
    def declare(spec, hidden: int) -> list:
        qk, v = spec.num_heads * spec.head_dim, spec.num_heads * spec.value_dim
        return [ParamDecl("q", (qk, hidden)), ParamDecl("k", (qk, hidden)), ParamDecl("v", (v, hidden)),
                ParamDecl("g", (v, hidden)), ParamDecl("o", (hidden, v)), ParamDecl("norm", (v,), "gain")]

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        self._sizes(spec, "linear attention")
        if len(spec.decay) != spec.num_heads:
            raise ConfigError(f"{len(spec.decay)} decays for {spec.num_heads} heads")
        self.spec = spec
        self.H, self.D, self.V = spec.num_heads, spec.head_dim, spec.value_dim
        self._fuse(params, ["q", "k", "v", "g"])
        self.o_proj = Linear(params["o"])
        self.gain = _f32(params["norm"])
        self.decay = torch.tensor([float(d) for d in spec.decay], dtype=torch.float32, device=device)
        # (in chunks a decay enters through its logarithm)
        self.chunked = min(float(d) for d in spec.decay) > 0.0
        self.dtype = dtype

    def state_spec(self):
        return StateSpec((self.H * self.D * self.V,), torch.float32)

    def forward(self, x, ctx):
        c = self.columns
        rows = self.proj.forward(x, out_dtype=torch.float32)
        read = kernels.recurrent_scan("lightning", rows, c["q"], c["k"], c["v"], ctx.state(), ctx.batch,
                                      self.H, self.H, self.D, self.V, p1=self.decay, chunked=self.chunked)
        normed = kernels.gated_group_norm(read, self.H * self.V, self.gain, self.spec.eps, self.dtype,
                                          gate=rows, gate_off=c["g"], gate_act="sigmoid")
        return self.o_proj.forward(normed, out_dtype=torch.float32)


class Mlstm(_ScanMixer):
    @staticmethod
    def declare(spec, hidden: int) -> list:
        H = spec.num_heads
        qk, v = H * spec.head_dim, H * spec.value_dim
        return [ParamDecl("q", (qk, hidden)), ParamDecl("k", (qk, hidden)), ParamDecl("v", (v, hidden)),
                ParamDecl("g", (v, hidden)), ParamDecl("o", (hidden, v)), ParamDecl("norm", (v,), "gain"),
                ParamDecl("i", (H, hidden)), ParamDecl("i.b", (H,), "bias"),
                ParamDecl("f", (H, hidden)), ParamDecl("f.b", (H,), "bias")]

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        self._sizes(spec, "a matrix memory")
        if not spec.gate_cap > 0:
            raise ConfigError(f"a gate cap of {spec.gate_cap}")
        self.spec = spec
        self.H, self.D, self.V = spec.num_heads, spec.head_dim, spec.value_dim
        self._fuse(params, ["q", "k", "v", "g", "i", "f"])
        self.o_proj = Linear(params["o"])
        self.gain = _f32(params["norm"])
        self.bias_i, self.bias_f = _f32(params["i.b"]), _f32(params["f.b"])
        self.dtype = dtype

    def state_spec(self):
        # S, the normaliser n and the running maximum m (``kernels.scan_state_floats``)
        return StateSpec((kernels.scan_state_floats("mlstm", self.H, self.D, self.V),), torch.float32)

    def forward(self, x, ctx):
        c = self.columns
        rows = self.proj.forward(x, out_dtype=torch.float32)
        read = kernels.recurrent_scan("mlstm", rows, c["q"], c["k"], c["v"], ctx.state(), ctx.batch,
                                      self.H, self.H, self.D, self.V, gates=rows, g1_off=c["i"], g2_off=c["f"],
                                      p1=self.bias_i, p2=self.bias_f, cap=self.spec.gate_cap, chunked=True)
        normed = kernels.gated_group_norm(read, self.V, self.gain, self.spec.eps, self.dtype,
                                          gate=rows, gate_off=c["g"], gate_act="sigmoid")
        return self.o_proj.forward(normed, out_dtype=torch.float32)


class GatedDelta(_ScanMixer):
    @staticmethod
    def declare(spec, hidden: int) -> list:
        H, G, t = spec.num_heads, spec.num_qk_heads, spec.conv_taps
        qk, v = G * spec.head_dim, H * spec.value_dim
        return [ParamDecl("q", (qk, hidden)), ParamDecl("q.conv", (qk, t)),
                ParamDecl("k", (qk, hidden)), ParamDecl("k.conv", (qk, t)),
                ParamDecl("v", (v, hidden)), ParamDecl("v.conv", (v, t)),
                ParamDecl("b", (H, hidden)), ParamDecl("a", (H, hidden)),
                ParamDecl("A_log", (H,), "bias"), ParamDecl("dt_bias", (H,), "bias"),
                ParamDecl("norm", (spec.value_dim,), "gain"), ParamDecl("g", (v, hidden)), ParamDecl("o", (hidden, v))]

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        self._sizes(spec, "a delta rule")
        if spec.num_qk_heads < 1 or spec.num_heads % spec.num_qk_heads:
            raise UnsupportedError(f"{spec.num_heads} heads over {spec.num_qk_heads} heads of q and k, "
                                   "which do not group evenly")
        if not 1 <= spec.conv_taps <= 16:
            raise UnsupportedError(f"a convolution of {spec.conv_taps} taps (1 to 16)")
        self.spec = spec
        self.H, self.G, self.D, self.V = spec.num_heads, spec.num_qk_heads, spec.head_dim, spec.value_dim
        self._fuse(params, ["q", "k", "v", "g", "b", "a"])       # q | k | v first: the convolution's channels
        self.channels = 2 * self.G * self.D + self.H * self.V
        self.conv_w = torch.cat([_f32(params["q.conv"]), _f32(params["k.conv"]), _f32(params["v.conv"])], 0).t().contiguous()   # [taps, channels]
        self.o_proj = Linear(params["o"])
        self.gain = _f32(params["norm"])
        self.a_log, self.dt_bias = _f32(params["A_log"]), _f32(params["dt_bias"])
        self.dtype = dtype
        self.matrix = self.H * self.D * self.V

    def state_spec(self):
        # S [H, D, V], then the convolution's last taps - 1 inputs [taps - 1, channels]
        return StateSpec((self.matrix + (self.spec.conv_taps - 1) * self.channels,), torch.float32)

    def forward(self, x, ctx):
        c, G, D = self.columns, self.G, self.D
        state = ctx.state()
        history = state[:, self.matrix:]
        rows = self.proj.forward(x, out_dtype=torch.float32)
        mixed = kernels.short_conv(rows, c["q"], self.conv_w, history, ctx.batch, silu=True)
        kernels.conv_history(rows, c["q"], self.conv_w, history, ctx.batch)
        read = kernels.recurrent_scan("delta", mixed, 0, G * D, 2 * G * D, state[:, :self.matrix], ctx.batch,
                                      self.H, G, D, self.V, gates=rows, g1_off=c["b"], g2_off=c["a"],
                                      p1=self.a_log, p2=self.dt_bias, chunked=True)
        normed = kernels.gated_group_norm(read, self.V, self.gain, self.spec.eps, self.dtype,
                                          gate=rows, gate_off=c["g"], gate_act="silu")
        return self.o_proj.forward(normed, out_dtype=torch.float32)


register_mixer("lightning_attention", LightningAttention)
register_mixer("mlstm", Mlstm)
register_mixer("gated_delta", GatedDelta)
