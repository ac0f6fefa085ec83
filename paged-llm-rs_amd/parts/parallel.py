"""Several mixers side by side: all read the same rows, and the layer's result is the weighted sum of
theirs.  At most one of them keeps keys and values in pages (a layer has one set of pools); their
states lie one behind the other in the layer's state slot.
"""

from __future__ import annotations

import torch

from .. import kernels
from ..cache.layout import StateSpec
from ..errors import ConfigError, UnsupportedError
from .registry import MIXERS, lookup, prefixed, register_mixer, scoped


class _BranchContext:
    """The layer's context as one branch sees it: its own run of the state's columns."""

    def __init__(self, ctx, begin: int, end: int):
        self._ctx, self._begin, self._end = ctx, begin, end

    def __getattr__(self, name):
        return getattr(self._ctx, name)

    def state(self):
        return self._ctx.state()[:, self._begin:self._end]


class ParallelMixers:
    @staticmethod
    def declare(spec, hidden: int) -> list:
        decls = []
        for name, branch, _ in spec.branches:
            decls += prefixed(lookup(MIXERS, branch.kind, "mixer").declare(branch, hidden), name)
        return decls

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        if not spec.branches:
            raise ConfigError("mixers side by side, and none of them")
        self.branches = []
        at = 0
        paged = 0
        for name, branch, weight in spec.branches:
            mixer = lookup(MIXERS, branch.kind, "mixer")(branch, hidden, scoped(params, name), dtype, device, shared)
            state = mixer.state_spec()
            size = 0
            if state is not None:
                if state.dtype != torch.float32 or len(state.shape) != 1:
                    raise UnsupportedError(f"mixers side by side keep their states as runs of 32-bit floats; "
                                           f"{branch.kind!r} asks for {state.shape} of {state.dtype}")
                size = int(state.shape[0])
            paged += mixer.cache_spec() is not None
            self.branches.append((mixer, float(weight), at, at + size))
            at += size
        if paged > 1:
            raise UnsupportedError("more than one of the mixers side by side keeps keys and values in pages")
        self.state_floats = at
        self.graph_safe = all(getattr(m, "graph_safe", True) for m, *_ in self.branches)
        limits = [getattr(m, "short_portion", None) for m, *_ in self.branches]
        limits = [x for x in limits if x]
        if limits:
            self.short_portion = limits[0]

    def cache_spec(self):
        for mixer, *_ in self.branches:
            spec = mixer.cache_spec()
            if spec is not None:
                return spec
        return None

    def state_spec(self):
        return StateSpec((self.state_floats,), torch.float32) if self.state_floats else None

    def forward(self, x, ctx):
        total = None
        for mixer, weight, begin, end in self.branches:
            out = mixer.forward(x, _BranchContext(ctx, begin, end))
            if out.dtype != torch.float32:
                raise UnsupportedError("mixers side by side hand back 32-bit rows")
            if total is None:
                total, first = out, weight
            else:
                kernels.weighted_sum_(total, first, out, weight)
                first = 1.0
        if first != 1.0:
            kernels.scale_(total, first)
        return total


register_mixer("parallel_mixers", ParallelMixers)
