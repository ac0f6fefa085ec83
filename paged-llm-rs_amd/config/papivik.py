"""The typed configuration of the Papivik design, read from the keys of its own config.json.

A Papivik model is a list of layers; each names its mixer (``lightning``: linear attention with a fixed
decay a head; ``mlstm``: a matrix memory with exponential gates; ``parallel``: softmax attention with
short convolutions beside a gated delta rule, their outputs added with a weight each) and, optionally, a
dense feed-forward.  Every sublayer's output is normalised before it joins the stream.  The embedding
is scaled; nothing bounds the positions.  Inside a mixer or a feed-forward a key this reader does not
know is refused: a model that ignores a constant runs and is wrong.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..errors import ConfigError, UnsupportedError
from .specs import (ConvAttentionSpec, DenseMlpSpec, GatedDeltaSpec, LayerSpec, LinearAttentionSpec, MlstmSpec, ModelSpec,
                    NormSpec, ParallelMixersSpec, ScheduleEntry)


def _object(d, what: str, required: tuple, optional: tuple = (), others: bool = False) -> dict:
    """``others``: keys beside the known ones are let through (notes about a model, at the levels that hold no
    constant of a mechanism)."""
    if not isinstance(d, dict):
        raise ConfigError(f"{what} is not an object")
    missing = [k for k in required if k not in d]
    unknown = [] if others else sorted(set(d) - set(required) - set(optional))
    if missing:
        raise ConfigError(f"{what} lacks {', '.join(missing)}")
    if unknown:
        raise UnsupportedError(f"{what} has keys this reader does not know: {', '.join(unknown)}")
    return d


def _count(d: dict, key: str, what: str) -> int:
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"{what}: {key} {v!r}, which has to be a positive integer")
    return v


def _number(d: dict, key: str, what: str) -> float:
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{what}: {key} {v!r}, which has to be a number")
    return float(v)


def _lightning(m, what: str, eps: float):
    _object(m, what, ("heads", "dim", "vdim", "decay"))
    heads = _count(m, "heads", what)
    decay = m["decay"]
    if not isinstance(decay, list) or len(decay) != heads:
        raise ConfigError(f"{what}: decay has to list one number a head ({heads})")
    return LinearAttentionSpec(num_heads=heads, head_dim=_count(m, "dim", what), value_dim=_count(m, "vdim", what),
                               decay=tuple(_number({"decay": x}, "decay", what) for x in decay), eps=eps)


def _mlstm(m, what: str, eps: float):
    _object(m, what, ("heads", "dim", "vdim", "gate_cap"))
    cap = _number(m, "gate_cap", what)
    if not cap > 0:
        raise ConfigError(f"{what}: a gate_cap of {cap}")
    return MlstmSpec(num_heads=_count(m, "heads", what), head_dim=_count(m, "dim", what),
                     value_dim=_count(m, "vdim", what), gate_cap=cap, eps=eps)


def _conv_attention(m, what: str, eps: float):
    _object(m, what, ("heads", "kv_heads", "dim", "vdim", "conv", "scale"), ("rot",))
    rot = m.get("rot")
    dims, base = 0, 10000.0
    if rot is not None:
        _object(rot, what + ".rot", ("dims", "base"))
        dims, base = _count(rot, "dims", what + ".rot"), _number(rot, "base", what + ".rot")
        if dims % 2 or dims > m["dim"] or not base > 0:
            raise ConfigError(f"{what}: a rotation over {dims} of {m['dim']} values with base {base}")
    heads, kv_heads = _count(m, "heads", what), _count(m, "kv_heads", what)
    if heads % kv_heads:
        raise ConfigError(f"{what}: {heads} heads over {kv_heads} kv_heads")
    return ConvAttentionSpec(num_heads=heads, num_kv_heads=kv_heads, head_dim=_count(m, "dim", what),
                             value_dim=_count(m, "vdim", what), conv_taps=_count(m, "conv", what), qk_norm_eps=eps,
                             rotary_dim=dims, rotary_base=base, scale=_number(m, "scale", what))


def _delta(m, what: str, eps: float):
    _object(m, what, ("heads", "kv_heads", "dim", "vdim", "conv"))
    heads, kv_heads = _count(m, "heads", what), _count(m, "kv_heads", what)
    if heads % kv_heads:
        raise ConfigError(f"{what}: {heads} heads over {kv_heads} kv_heads")
    return GatedDeltaSpec(num_heads=heads, num_qk_heads=kv_heads, head_dim=_count(m, "dim", what),
                          value_dim=_count(m, "vdim", what), conv_taps=_count(m, "conv", what), eps=eps)


def _parallel(m, what: str, eps: float):
    _object(m, what, ("left", "right", "left_scale", "right_scale"))
    return ParallelMixersSpec(branches=(
        ("left", _conv_attention(m["left"], what + ".left", eps), _number(m, "left_scale", what)),
        ("right", _delta(m["right"], what + ".right", eps), _number(m, "right_scale", what))))


_MIXERS = {"lightning": _lightning, "mlstm": _mlstm, "parallel": _parallel}


@dataclass(frozen=True)
class PapivikConfig:
    raw: dict
    width: int
    vocab: int
    eps: float
    embedding_scale: float
    layers: tuple             # (mixer spec, feed-forward spec or None) a layer

    architecture = "Papivik"

    @classmethod
    def from_dict(cls, d: dict) -> "PapivikConfig":
        _object(d, "config.json", ("architecture", "embedding", "layers", "norm", "vocab", "width"), others=True)
        _object(d["embedding"], "embedding", ("scale",))
        _object(d["norm"], "norm", ("eps",))
        eps = _number(d["norm"], "eps", "norm")
        if not eps >= 0:
            raise ConfigError(f"norm: an eps of {eps}")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("layers has to be a list of at least one layer")
        layers = []
        for i, layer in enumerate(d["layers"]):
            what = f"layers[{i}]"
            _object(layer, what, ("type", "mixer"), ("mlp",), others=True)
            if layer["type"] not in _MIXERS:
                raise UnsupportedError(f"{what}: a mixer of type {layer['type']!r}, this design has {', '.join(_MIXERS)}")
            mixer = _MIXERS[layer["type"]](layer["mixer"], what + ".mixer", eps)
            mlp = layer.get("mlp")
            if mlp is not None:
                _object(mlp, what + ".mlp", ("kind", "ff"))
                if mlp["kind"] != "dense":
                    raise UnsupportedError(f"{what}.mlp: kind {mlp['kind']!r}, this design has dense")
                mlp = DenseMlpSpec(intermediate_size=_count(mlp, "ff", what + ".mlp"), activation="gelu_tanh")
            layers.append((mixer, mlp))
        return cls(raw=d, width=_count(d, "width", "config.json"), vocab=_count(d, "vocab", "config.json"), eps=eps,
                   embedding_scale=_number(d["embedding"], "scale", "embedding"), layers=tuple(layers))

    def to_dict(self) -> dict:
        return self.raw

    def model_spec(self) -> ModelSpec:
        norm = NormSpec("rms_norm", self.eps)
        layers = tuple(LayerSpec(block="sublayer_norm", mixer=mixer, feed_forward=mlp, norm=norm, weight_prefix=f"l{i}")
                       for i, (mixer, mlp) in enumerate(self.layers))
        return ModelSpec(
            hidden_size=self.width, vocab_size=self.vocab, layers=layers,
            schedule=tuple(ScheduleEntry(i) for i in range(len(layers))), final_norm=norm,
            tie_word_embeddings=False, max_positions=0, embed_name="embed", final_norm_name="final.norm",
            head_name="head",
            extra={"embed_transform": "scale", "embedding_scale": self.embedding_scale, "bare_norm_names": True})
