"""Transforms of the stream behind the embedding and of the logits that ship with the package."""

from __future__ import annotations

from .. import kernels
from .registry import register_embed_transform


class EmbeddingScale:
    """x <- x * extra["embedding_scale"], on the 32-bit stream."""

    graph_safe = True

    def __init__(self, spec, params: dict, dtype, device):
        self.scale = float(spec.extra["embedding_scale"])

    def __call__(self, x, batch):
        return kernels.scale_(x, self.scale) if self.scale != 1.0 else x


register_embed_transform("scale", EmbeddingScale)
