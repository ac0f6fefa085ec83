"""The typed configuration of the Lefavik design, read from the keys of its own config.json.

A Lefavik model is a list of layers.  A layer norms the stream once and adds what its mixer and its
feed-forward make of those normed rows, x <- x + mixer(n) + ff(n).  Two kinds of mixer:
``latent_attention`` keeps one small vector and one rotated key part a token and rebuilds every
head's keys and values from them (a layer may read the vectors another layer keeps, ``kv_from``);
``attention`` is grouped-query attention with unit q and k, a query temperature, a distance penalty
a head, a window and a sink of score 0.  The embedding is scaled, a learned position vector is added
and the sum is normed; the logits are scaled.  Inside a mixer or a feed-forward a key this reader
does not know is refused: a model that ignores a constant runs and is wrong.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..errors import ConfigError, UnsupportedError
from .papivik import _count, _number, _object
from .specs import (GatedMlpSpec, LatentAttentionSpec, LayerSpec, ModelSpec, NormSpec, ScheduleEntry,
                    SinkAttentionSpec)


def _latent(m, what: str, eps: float, max_positions: int):
    _object(m, what, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "rot", "scale"), ("kv_from",))
    _object(m["rot"], what + ".rot", ("dims", "base"))
    rot_dim = _count(m, "rot_dim", what)
    turned, base = _count(m["rot"], "dims", what + ".rot"), _number(m["rot"], "base", what + ".rot")
    if turned % 2 or turned > rot_dim or not base > 0:
        raise ConfigError(f"{what}: a rotation over {turned} of {rot_dim} values with base {base}")
    source = m.get("kv_from")
    if source is not None and (isinstance(source, bool) or not isinstance(source, int) or source < 0):
        raise ConfigError(f"{what}: kv_from {source!r}, which has to name a layer")
    spec = LatentAttentionSpec(num_heads=_count(m, "heads", what), head_dim=_count(m, "dim", what), rotary_dim=rot_dim,
                               value_dim=_count(m, "vdim", what), kv_rank=_count(m, "kv_rank", what),
                               rotary_turned=turned, rotary_base=base, max_positions=max_positions,
                               scale=_number(m, "scale", what), norm_eps=eps,
                               sink="learned", gated=True, borrows=source is not None)
    return spec, source


def _attention(m, what: str, eps: float, max_positions: int):
    _object(m, what, ("heads", "kv_heads", "dim", "vdim", "scale"), ("mask", "q_temp"))
    heads, kv_heads = _count(m, "heads", what), _count(m, "kv_heads", what)
    if heads % kv_heads:
        raise ConfigError(f"{what}: {heads} heads over {kv_heads} kv_heads")
    window = None
    if m.get("mask") is not None:
        _object(m["mask"], what + ".mask", ("size",))
        window = _count(m["mask"], "size", what + ".mask")
    coef, every = None, 1
    if m.get("q_temp") is not None:
        _object(m["q_temp"], what + ".q_temp", ("coef", "every"))
        coef, every = _number(m["q_temp"], "coef", what + ".q_temp"), _count(m["q_temp"], "every", what + ".q_temp")
    spec = SinkAttentionSpec(num_heads=heads, num_kv_heads=kv_heads, head_dim=_count(m, "dim", what),
                             value_dim=_count(m, "vdim", what), scale=_number(m, "scale", what), qk_unit_eps=eps,
                             temperature_coef=coef, temperature_every=every, distance_slopes="geometric",
                             slope_span=8.0, window=window, sink="zero")
    return spec, None


_MIXERS = {"latent_attention": _latent, "attention": _attention}


@dataclass(frozen=True)
class LefavikConfig:
    raw: dict
    width: int
    vocab: int
    eps: float
    embedding_scale: float
    logit_scale: float
    max_positions: int
    layers: tuple             # (mixer spec, feed-forward spec or None, the layer whose pages are read or None) a layer

    architecture = "Lefavik"

    @classmethod
    def from_dict(cls, d: dict) -> "LefavikConfig":
        _object(d, "config.json", ("architecture", "embedding", "layers", "norm", "vocab", "width", "max_positions"),
                ("logit_scale",), others=True)
        _object(d["embedding"], "embedding", ("scale",))
        _object(d["norm"], "norm", ("eps",))
        eps = _number(d["norm"], "eps", "norm")
        if not eps >= 0:
            raise ConfigError(f"norm: an eps of {eps}")
        max_positions = _count(d, "max_positions", "config.json")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("layers has to be a list of at least one layer")
        layers = []
        for i, layer in enumerate(d["layers"]):
            what = f"layers[{i}]"
            _object(layer, what, ("type", "mixer"), ("mlp",), others=True)
            if layer["type"] not in _MIXERS:
                raise UnsupportedError(f"{what}: a mixer of type {layer['type']!r}, this design has {', '.join(_MIXERS)}")
            mixer, source = _MIXERS[layer["type"]](layer["mixer"], what + ".mixer", eps, max_positions)
            mlp = layer.get("mlp")
            if mlp is not None:
                _object(mlp, what + ".mlp", ("kind", "ff"))
                if mlp["kind"] != "dense":
                    raise UnsupportedError(f"{what}.mlp: kind {mlp['kind']!r}, this design has dense")
                mlp = GatedMlpSpec(intermediate_size=_count(mlp, "ff", what + ".mlp"), activation="gelu_tanh",
                                   names=("gate", "up", "down"))
            layers.append((mixer, mlp, source))
        for i, (mixer, _, source) in enumerate(layers):
            if source is None:
                continue
            if source >= i:
                raise ConfigError(f"layers[{i}].mixer: kv_from {source}, which is no earlier layer")
            other, _, others_source = layers[source]
            if not isinstance(other, LatentAttentionSpec) or others_source is not None:
                raise ConfigError(f"layers[{i}].mixer: kv_from {source}, a layer that keeps no vectors of its own")
            same = ("kv_rank", "rotary_dim", "rotary_turned", "rotary_base")
            if any(getattr(other, k) != getattr(mixer, k) for k in same):
                raise ConfigError(f"layers[{i}].mixer: kv_from {source}, whose kv_rank, rot_dim or rotation differ")
        return cls(raw=d, width=_count(d, "width", "config.json"), vocab=_count(d, "vocab", "config.json"), eps=eps,
                   embedding_scale=_number(d["embedding"], "scale", "embedding"),
                   logit_scale=_number(d, "logit_scale", "config.json") if "logit_scale" in d else 1.0,
                   max_positions=max_positions, layers=tuple(layers))

    def to_dict(self) -> dict:
        return self.raw

    def model_spec(self) -> ModelSpec:
        norm = NormSpec("rms_norm", self.eps)
        layers = tuple(LayerSpec(block="shared_norm", mixer=mixer, feed_forward=mlp, norm=norm, weight_prefix=f"l{i}")
                       for i, (mixer, mlp, _) in enumerate(self.layers))
        return ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab, layers=layers,
            schedule=tuple(ScheduleEntry(i, cache_from=source) for i, (_, _, source) in enumerate(self.layers)),
            final_norm=norm, tie_word_embeddings=False, max_positions=self.max_positions, embed_name="embed",
            final_norm_name="final.norm", head_name="head",
            extra={"embed_transform": ("scale", "learned_position", "stream_norm"),
                   "embedding_scale": self.embedding_scale, "position_table_name": "pos",
                   "stream_norm_name": "embed.norm", "stream_norm": norm,
                   "logit_transform": "scale", "logit_scale": self.logit_scale, "bare_norm_names": True})
