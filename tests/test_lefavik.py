"""The Lefavik design without a GPU: its configuration reader and what it refuses, the tensors it declares, the
random-weights mode, the cache layout of layers that keep one small vector a token, and properties of the plain
implementation's mechanisms."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import lefavik_util as lu
import plain_lefavik as plain
from paged_llm_rs_amd.config import load_config
from paged_llm_rs_amd.config.specs import LatentAttentionSpec, SinkAttentionSpec
from paged_llm_rs_amd.errors import ConfigError, UnsupportedError
from paged_llm_rs_amd.parts.model import declare_parameters


def test_the_reader_takes_every_size_and_constant_from_the_config():
    spec = load_config(copy.deepcopy(lu.ODD)).model_spec()
    assert spec.hidden_size == 72 and spec.vocab_size == 211 and spec.max_positions == 512
    first, second, third, fourth = (layer.mixer for layer in spec.layers)
    assert isinstance(first, LatentAttentionSpec) and isinstance(second, SinkAttentionSpec)
    assert (first.num_heads, first.head_dim, first.rotary_dim, first.value_dim, first.kv_rank) == (3, 24, 8, 40, 40)
    assert first.scale == 0.21 and first.rotary_base == 500.0 and first.rotary_turned == 8 and first.norm_eps == 1e-5
    assert first.sink == "learned" and first.gated and not first.borrows
    assert (second.num_heads, second.num_kv_heads, second.head_dim, second.value_dim) == (6, 2, 24, 40)
    assert second.window == 5 and (second.temperature_coef, second.temperature_every) == (0.7, 3)
    assert second.scale == 0.9 and second.qk_unit_eps == 1e-5 and second.sink == "zero"
    assert third.window == 37 and spec.layers[1].feed_forward is None and spec.layers[2].feed_forward.intermediate_size == 64
    assert fourth.borrows and [e.cache_from for e in spec.schedule] == [None, None, None, 0]
    assert spec.extra["embedding_scale"] == 1.7 and spec.extra["logit_scale"] == 0.5
    ones = load_config(copy.deepcopy(lu.ONES)).model_spec()
    assert ones.layers[0].mixer.window is None and ones.layers[0].mixer.temperature_coef is None
    assert ones.layers[3].mixer.rotary_turned == 8 and ones.layers[3].mixer.rotary_dim == 16


@pytest.mark.parametrize("damage, error", [
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), ConfigError),
    (lambda c: c["layers"][0]["mixer"].update(extra=1), UnsupportedError),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), ConfigError),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), ConfigError),
    (lambda c: c["layers"][1]["mixer"]["q_temp"].update(every=0), ConfigError),
    (lambda c: c["layers"][0].update(type="other"), UnsupportedError),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), UnsupportedError),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), ConfigError),          # not an earlier layer
    (lambda c: c["layers"][3]["mixer"].update(kv_from=1), ConfigError),          # a layer that keeps no vectors
    (lambda c: c["layers"][3]["mixer"].update(kv_rank=48), ConfigError),         # another size than the layer it reads
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), ConfigError),     # more than the rotated part
    (lambda c: c.pop("max_positions"), ConfigError),
    (lambda c: c["norm"].update(eps=-1.0), ConfigError),
])
def test_what_the_reader_refuses(damage, error):
    config = copy.deepcopy(lu.ODD)
    damage(config)
    with pytest.raises(error):
        load_config(config)


def test_declared_tensors():
    decls = {d.name: tuple(d.shape) for d in declare_parameters(load_config(copy.deepcopy(lu.ODD)).model_spec())}
    assert decls["embed"] == (211, 72) and decls["pos"] == (512, 72) and decls["embed.norm"] == (72,)
    assert decls["l0.mix.q"] == (3 * 32, 72) and decls["l0.mix.dkv"] == (48, 72) and decls["l0.mix.dkv.norm"] == (40,)
    assert decls["l0.mix.uk"] == (72, 40) and decls["l0.mix.uv"] == (120, 40) and decls["l0.mix.sink"] == (3,)
    assert decls["l0.mix.g"] == (3, 72) and decls["l0.mix.o"] == (72, 120) and decls["l0.norm1"] == (72,)
    assert decls["l1.mix.q"] == (144, 72) and decls["l1.mix.k"] == (48, 72) and decls["l1.mix.v"] == (80, 72)
    assert decls["l1.mix.o"] == (72, 240) and "l1.mlp.up" not in decls and "l1.mix.sink" not in decls
    assert decls["l2.mlp.gate"] == (64, 72) and decls["l2.mlp.up"] == (64, 72) and decls["l2.mlp.down"] == (72, 64)
    assert "l3.mix.dkv" not in decls and "l3.mix.dkv.norm" not in decls and decls["l3.mix.uk"] == (80, 40)
    assert decls["final.norm"] == (72,) and decls["head"] == (211, 72)
    assert not any("norm2" in name for name in decls)


def test_the_random_weights_mode_and_the_plain_implementation(tmp_path):
    folder = lu.write_model(tmp_path / "m", lu.ODD, seed=3)
    config, weights = lu.load_plain(folder)
    tokens = [5, 17, 3, 200, 0, 44, 9, 9, 120]
    streams = []
    logits = plain.forward(config, weights, tokens, streams)
    assert logits.shape == (9, 211) and len(streams) == 4 and torch.isfinite(logits).all()
    # causal: a prefix gives the same logits
    assert torch.allclose(plain.forward(config, weights, tokens[:5]), logits[:5], atol=1e-12)
    # the logit scale multiplies the logits and nothing else
    other = copy.deepcopy(config)
    other["logit_scale"] = 1.0
    assert torch.allclose(plain.forward(other, weights, tokens) * 0.5, logits, atol=1e-12)


def test_the_cache_layout_of_layers_that_keep_one_vector_a_token():
    from paged_llm_rs_amd.cache.layout import CacheLayout, KVCacheSpec

    class Mixer:
        def __init__(self, spec):
            self.spec = spec

        def cache_spec(self):
            return self.spec

        def state_spec(self):
            return None

    class Block:
        def __init__(self, spec):
            self.mixer = Mixer(spec)

    from paged_llm_rs_amd.config.specs import ScheduleEntry

    small, heads = KVCacheSpec(1, 48, None, values_in_keys=True), KVCacheSpec(2, 32, 5)
    blocks = [Block(small), Block(heads), Block(small), Block(small)]
    layout = CacheLayout.from_blocks(blocks, (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(3, cache_from=0)))
    assert [g.layers for g in layout.groups] == [[0, 2], [1]] and 3 not in layout.layer_group
    # one row a token for a layer that keeps vectors, keys and values for the other
    assert layout.bytes_per_token(2) == 2 * 48 * 2 + 2 * 2 * 32 * 2
    with pytest.raises(ConfigError):
        CacheLayout.from_blocks(blocks, (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(3, cache_from=2), ScheduleEntry(2)))


def test_properties_of_the_plain_mechanisms():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 3, 12, generator=g, dtype=torch.float64)
    positions = torch.arange(7)
    turned = plain.rotate_neighbours(x, positions, 8, 100.0)
    assert torch.allclose(turned[..., 8:], x[..., 8:]) and torch.allclose(turned[0], x[0])
    pairs = lambda t: t[..., 0:8:2] ** 2 + t[..., 1:8:2] ** 2
    assert torch.allclose(pairs(turned), pairs(x))
    # a score between rotated vectors depends on the distance alone
    a, b = torch.randn(1, 8, generator=g, dtype=torch.float64), torch.randn(1, 8, generator=g, dtype=torch.float64)
    dot = lambda p, q: float((plain.rotate_neighbours(a, torch.tensor([p]), 8, 100.0) * plain.rotate_neighbours(b, torch.tensor([q]), 8, 100.0)).sum())
    assert abs(dot(9, 4) - dot(25, 20)) < 1e-12 and abs(dot(9, 4) - dot(9, 5)) > 1e-6
    # a sink takes its share and has no value: weights sum to less than one, and to one as the sink falls away
    score = torch.randn(5, 5, generator=g, dtype=torch.float64)
    visible = torch.tril(torch.ones(5, 5, dtype=torch.bool))
    w = plain.softmax_with_sink(score, visible, 0.3)
    assert (w.sum(-1) < 1).all() and (w[~visible] == 0).all()
    assert torch.allclose(w.sum(-1), 1 - math.exp(0.3) / (math.exp(0.3) + torch.exp(score.masked_fill(~visible, -math.inf)).sum(-1)))
    assert torch.allclose(plain.softmax_with_sink(score, visible, -800.0).sum(-1), torch.ones(5, dtype=torch.float64))
    # temperature and slopes
    t = plain.query_temperature(torch.tensor([0, 62, 63, 126, 127]), 0.5, 64)
    assert torch.allclose(t, torch.tensor([1.0, 1.0, 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(3)], dtype=torch.float64))
    assert torch.allclose(plain.distance_slopes(4), torch.tensor([0.25, 0.0625, 0.015625, 0.00390625], dtype=torch.float64))
    assert abs(float(plain.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12


def test_a_window_of_the_plain_attention_sees_itself_and_the_tokens_before(tmp_path):
    """Changing a token changes the logits of the positions whose windows hold it and of no other (one window layer)."""
    config = lu.model(40, 50, [lu.attention(2, 1, 16, 16, 0.7, window=4)], max_positions=64)
    folder = lu.write_model(tmp_path / "m", config, seed=5, std=0.3)
    cfg, weights = lu.load_plain(folder)
    tokens = list(range(10, 30))
    base = plain.forward(cfg, weights, tokens)
    changed = list(tokens)
    changed[6] = 49
    moved = (plain.forward(cfg, weights, changed) - base).abs().max(-1).values > 1e-9
    assert moved.tolist() == [6 <= p < 10 for p in range(20)]
