"""CPU tests of the Papivik design: its configuration reader and registry entry, the tensors it declares, the
random-weights mode, and properties of the plain implementation that the GPU tests lean on."""

from __future__ import annotations

import copy
import json

import pytest
import torch

import papivik_util as pu
import plain_papivik as plain

from paged_llm_rs_amd.config import PapivikConfig, load_config
from paged_llm_rs_amd.config.specs import (ConvAttentionSpec, DenseMlpSpec, GatedDeltaSpec, LinearAttentionSpec, MlstmSpec,
                                           ParallelMixersSpec)
from paged_llm_rs_amd.errors import ConfigError, UnsupportedError
from paged_llm_rs_amd.parts.model import declare_parameters


def test_config_json_chooses_the_design_and_every_constant_is_read():
    config = load_config(copy.deepcopy(pu.ODD))
    assert isinstance(config, PapivikConfig)
    spec = config.model_spec()
    assert (spec.hidden_size, spec.vocab_size, spec.max_positions) == (72, 211, 0)
    assert spec.extra["embedding_scale"] == 1.7 and spec.final_norm.eps == 1e-5
    kinds = [type(layer.mixer) for layer in spec.layers]
    assert kinds == [MlstmSpec, ParallelMixersSpec, LinearAttentionSpec, ParallelMixersSpec]
    assert [layer.block for layer in spec.layers] == ["sublayer_norm"] * 4
    assert [type(layer.feed_forward) for layer in spec.layers] == [DenseMlpSpec, type(None), DenseMlpSpec, DenseMlpSpec]
    first = spec.layers[0].mixer
    assert (first.num_heads, first.head_dim, first.value_dim, first.gate_cap, first.eps) == (3, 24, 40, 8.0, 1e-5)
    (ln, left, ls), (rn, right, rs) = spec.layers[1].mixer.branches
    assert (ln, rn, ls, rs) == ("left", "right", 1.3, 0.7)
    assert isinstance(left, ConvAttentionSpec) and isinstance(right, GatedDeltaSpec)
    assert (left.num_heads, left.num_kv_heads, left.head_dim, left.value_dim, left.conv_taps, left.scale,
            left.rotary_dim, left.rotary_base, left.qk_norm_eps) == (6, 2, 24, 40, 2, 0.3, 8, 1000.0, 1e-5)
    assert (right.num_heads, right.num_qk_heads, right.head_dim, right.value_dim, right.conv_taps) == (4, 2, 16, 80, 3)
    assert spec.layers[2].mixer.decay == (0.9, 0.99)
    no_rotation = spec.layers[3].mixer.branches[0][1]
    assert no_rotation.rotary_dim == 0 and no_rotation.conv_taps == 1


def test_the_declared_tensors_carry_the_designs_names_and_shapes():
    decls = {d.name: tuple(d.shape) for d in declare_parameters(load_config(copy.deepcopy(pu.ODD)).model_spec())}
    assert decls["embed"] == (211, 72) and decls["head"] == (211, 72) and decls["final.norm"] == (72,)
    assert decls["l0.norm1"] == (72,) and decls["l0.norm2"] == (72,) and "l1.norm2" not in decls
    assert decls["l0.mix.i"] == (3, 72) and decls["l0.mix.i.b"] == (3,) and decls["l0.mix.norm"] == (120,)
    assert decls["l0.mlp.up"] == (100, 72) and decls["l0.mlp.down"] == (72, 100)
    assert decls["l1.mix.left.q"] == (144, 72) and decls["l1.mix.left.k"] == (48, 72) and decls["l1.mix.left.v"] == (80, 72)
    assert decls["l1.mix.left.q.conv"] == (144, 2) and decls["l1.mix.left.v.conv"] == (80, 2)
    assert decls["l1.mix.left.q.norm"] == (24,) and decls["l1.mix.left.o"] == (72, 240)
    assert decls["l1.mix.right.q"] == (32, 72) and decls["l1.mix.right.v"] == (320, 72) and decls["l1.mix.right.v.conv"] == (320, 3)
    assert decls["l1.mix.right.b"] == (4, 72) and decls["l1.mix.right.A_log"] == (4,) and decls["l1.mix.right.norm"] == (80,)
    assert decls["l2.mix.norm"] == (32,) and decls["l2.mix.o"] == (72, 32)


@pytest.mark.parametrize("change, error", [
    (lambda c: c["layers"][0].update(type="mamba"), UnsupportedError),
    (lambda c: c["layers"][0]["mixer"].update(window=64), UnsupportedError),
    (lambda c: c["layers"][0]["mixer"].pop("gate_cap"), ConfigError),
    (lambda c: c["layers"][1]["mixer"]["left"].update(heads=5), ConfigError),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=26), ConfigError),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.5]), ConfigError),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), UnsupportedError),
    (lambda c: c.pop("norm"), ConfigError),
    (lambda c: c.update(width=0), ConfigError),
])
def test_what_the_reader_refuses(change, error):
    config = copy.deepcopy(pu.ODD)
    change(config)
    with pytest.raises(error):
        load_config(config)


def test_notes_beside_the_known_keys_are_let_through_at_the_top():
    config = copy.deepcopy(pu.ONES)
    config["comment"] = "made from a seed"
    del config["layers"][1]["mlp"]          # a layer without the key has no feed-forward
    assert load_config(config).model_spec().layers[1].feed_forward is None


def test_the_random_weights_mode_writes_a_folder_of_this_design(tmp_path):
    folder = pu.write_model(tmp_path / "m", pu.ONES, seed=3, dtype="bfloat16")
    config, weights = pu.load_plain(folder)
    assert config == pu.ONES
    decls = declare_parameters(load_config(folder).model_spec())
    assert sorted(weights) == sorted(d.name for d in decls)
    assert abs(float(weights["l2.norm1"].mean()) - 1.0) < 0.2, "gains are drawn around one"


# --- the plain implementation ------------------------------------------------------------------------------

def test_plain_short_conv_is_the_librarys_causal_convolution():
    torch.manual_seed(0)
    u, w = torch.randn(19, 7, dtype=torch.float64), torch.randn(7, 4, dtype=torch.float64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(u.T[None], (3, 0)), w[:, None, :], groups=7)[0].T
    assert torch.allclose(plain.short_conv(u, w), want, atol=1e-12)


def test_plain_rotation_keeps_lengths_and_leaves_the_rest_of_a_head():
    torch.manual_seed(1)
    x = torch.randn(5, 3, 12, dtype=torch.float64)
    y = plain.rotate_half(x, torch.arange(5) + 100, 8, 77.0)
    assert torch.equal(y[..., 8:], x[..., 8:])
    assert torch.allclose(y[..., :8].norm(dim=-1), x[..., :8].norm(dim=-1))
    assert torch.allclose(plain.rotate_half(x, torch.zeros(5, dtype=torch.long), 8, 77.0), x)


def test_plain_logits_of_a_prefix_do_not_depend_on_what_follows(tmp_path):
    folder = pu.write_model(tmp_path / "m", pu.ODD, seed=5)
    config, weights = pu.load_plain(folder)
    tokens = [3, 100, 7, 7, 200, 41, 0, 9, 13, 150, 2]
    whole = plain.forward(config, weights, tokens)
    assert torch.allclose(plain.forward(config, weights, tokens[:6]), whole[:6], atol=1e-10)


def test_plain_delta_rule_stores_and_recalls_one_pair():
    """One write with beta 1 into an empty memory and no decay: reading with the written key gives the value back."""
    D, V = 6, 4
    k = torch.nn.functional.normalize(torch.randn(D, dtype=torch.float64), dim=0)
    v = torch.randn(V, dtype=torch.float64)
    S = torch.zeros(D, V, dtype=torch.float64)
    u = 1.0 * (v - S.T @ k)
    S = S + k[:, None] * u[None, :]
    assert torch.allclose(S.T @ k, v)


def test_a_model_without_pages_has_room_without_end_and_still_counts_its_state_slots():
    """A model none of whose layers keeps keys and values: the cache manager has no group of pages, requests are
    bounded by the state slots alone, and the scheduler plans them."""
    from paged_llm_rs_amd.cache.manager import CacheManager
    from paged_llm_rs_amd.engine import scheduler as sched

    manager = CacheManager([], state_slots=2)
    slot = manager.add_sequence(7)
    assert slot in (0, 1) and manager.capacity(7) > 1 << 40 and manager.reserve(7, 5000)
    manager.advance(7, 5000)
    assert manager.tokens(7) == 5000 and manager.available() == 0 and manager.total() == 0
    manager.free_sequence(7)
    assert manager.free_state_slots == 2
    scheduler = sched.Scheduler(manager, max_batch=4, chunk=8, max_positions=0, prefix_cache=False)
    for i, n in enumerate((3, 20, 9)):
        scheduler.submit(i + 1, list(range(n)), 0.0, None, None, 4, [], i)
    seen, steps = set(), 0
    while scheduler.running or scheduler.waiting:
        plan = scheduler.plan()
        assert plan.entries, "the planner has something for every step"
        assert len({e.state_slot for e in plan.entries}) == len(plan.entries) <= 2, "two slots, two residents"
        seen |= {e.seq_id for e in plan.entries}
        scheduler.commit([1] * len(plan.ids))
        steps += 1
        assert steps < 200
    assert seen == {1, 2, 3} and manager.free_state_slots == 2
