"""Configurations, model folders and comparisons for the tests of the Papivik design."""

from __future__ import annotations

import copy
import json
from pathlib import Path

import torch

import plain_papivik as plain


def lightning(heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}, "mlp": mlp}


def mlstm(heads, dim, vdim, cap, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def attention(heads, kv_heads, dim, vdim, conv, scale, rot=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale}
    if rot is not None:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return m


def delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def parallel(left, right, left_scale, right_scale, mlp=None):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale},
            "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def model(width, vocab, layers, eps=1e-6, scale=1.0):
    return {"architecture": "Papivik", "embedding": {"scale": scale}, "layers": layers, "norm": {"eps": eps},
            "vocab": vocab, "width": width}


# Odd sizes: heads of 24 and 40 (no multiple of 16; value heads larger than key heads), a value head of 80 (two
# column tiles of the scan), three query heads a key head, a rotation over a quarter of a head, two and three taps,
# a feed-forward on some layers only, a vocabulary that is a prime.
ODD = model(72, 211, [
    mlstm(3, 24, 40, 8.0, dense(100)),
    parallel(attention(6, 2, 24, 40, 2, 0.3, (8, 1000.0)), delta(4, 2, 16, 80, 3), 1.3, 0.7),
    lightning(2, 80, 16, (0.9, 0.99), dense(64)),
    parallel(attention(2, 2, 32, 16, 1, 0.2), delta(2, 2, 40, 24, 1), 0.5, 1.0, dense(96)),
], eps=1e-5, scale=1.7)

# What a small model tends to make equal or 1 is different here: one head, one key head for four query heads, a rotation
# over the whole head, five taps, a scale of one, a width that is no multiple of eight.
ONES = model(100, 97, [
    parallel(attention(4, 1, 16, 16, 5, 1.0, (16, 50.0)), delta(1, 1, 48, 48, 2), 1.0, 1.0),
    lightning(1, 16, 96, (0.5,)),
    mlstm(1, 64, 16, 30.0),
], eps=1e-6, scale=1.0)

# Larger heads: rows of S beyond 64 and 128 (the scan's deepest shapes), value heads of 128, attention heads of 128.
LARGE = model(256, 300, [
    lightning(2, 128, 128, (0.97, 0.999)),
    mlstm(2, 192, 96, 12.0),
    parallel(attention(4, 2, 128, 128, 3, 0.09, (64, 10000.0)), delta(2, 1, 160, 64, 4), 0.8, 0.6, dense(320)),
], eps=1e-6, scale=0.3)

# Eight and sixteen query heads a key head (single tokens then take the attention kernel that makes a group's heads the
# rows of a tile), heads of 24 in rows of 32, and a model whose first and last layers keep no pages.
GROUPED = model(64, 150, [
    lightning(2, 16, 16, (0.95, 0.8)),
    parallel(attention(8, 1, 32, 32, 3, 0.18, (32, 500.0)), delta(4, 4, 16, 16, 2), 0.7, 0.4, dense(128)),
    parallel(attention(16, 1, 24, 32, 2, 0.2, (12, 10000.0)), delta(2, 1, 32, 16, 4), 1.0, 0.5),
    mlstm(2, 16, 32, 5.0, dense(64)),
], eps=1e-6, scale=2.0)

# Head sizes that are no multiple of 4 (30, 22) or of 8 (20, 36, 44), a rotation over 10 values, a width that is a
# multiple of 4 only, seven taps.
UNEVEN = model(52, 75, [
    parallel(attention(3, 1, 30, 20, 7, 0.21, (10, 123.0)), delta(4, 2, 22, 36, 3), 0.9, 1.1, dense(44)),
    lightning(3, 30, 20, (0.7, 0.93, 0.99)),
    mlstm(2, 22, 44, 9.0),
], eps=3e-6, scale=0.8)

CONFIGS = {"odd": ODD, "ones": ONES, "large": LARGE, "grouped": GROUPED, "uneven": UNEVEN}


def write_model(folder, config, seed=0, dtype="float32", std=0.08, gain_std=0.2, edit=None) -> Path:
    """A model folder with random weights from the package's random-weights mode; ``edit(tensors)`` may change
    them (the folder is then written again)."""
    from paged_llm_rs_amd.weights import write_random_model

    folder = write_random_model(Path(folder), copy.deepcopy(config), seed=seed, std=std, gain_std=gain_std, dtype=dtype)
    if edit is not None:
        from safetensors.torch import load_file, save_file

        tensors = load_file(str(folder / "model.safetensors"))
        edit(tensors)
        save_file({k: v.contiguous() for k, v in tensors.items()}, str(folder / "model.safetensors"))
    return folder


def load_plain(folder):
    from safetensors.torch import load_file

    config = json.loads((Path(folder) / "config.json").read_text())
    weights = {k: v.to(torch.float64) for k, v in load_file(str(Path(folder) / "model.safetensors")).items()}
    return config, weights


def plain_logits(folder, prompts: dict) -> dict:
    config, weights = load_plain(folder)
    return {name: plain.forward(config, weights, tokens) for name, tokens in prompts.items()}


def plain_greedy(folder, prompt, count: int) -> list:
    config, weights = load_plain(folder)
    tokens, out = list(prompt), []
    for _ in range(count):
        nxt = int(plain.forward(config, weights, tokens)[-1].argmax())
        out.append(nxt)
        tokens.append(nxt)
    return out


def sensitivity(folder, prompts: dict) -> dict:
    """name -> a factor a position (>= 1): how much more than the median position this position's logits move when
    every weight matrix is disturbed by 2^-9 of itself (root mean square over the vocabulary).  Random models have single
    positions where rounding is amplified ten- to fiftyfold (a read-out near zero before its norm, a score near a
    tie); a bound on an engine's error there has to grow with it, as the error that rounding alone causes does."""
    config, weights = load_plain(folder)
    g = torch.Generator().manual_seed(1234)
    shaken = {k: v * (1 + (torch.rand(v.shape, generator=g, dtype=v.dtype) - 0.5) * 2.0 ** -8) if v.dim() == 2 and "conv" not in k
              else v for k, v in weights.items()}
    out = {}
    for name, tokens in prompts.items():
        base = plain.forward(config, weights, tokens)
        moved = ((plain.forward(config, shaken, tokens) - base) ** 2).mean(-1).sqrt() / base.std()
        out[name] = torch.clamp(moved / (2 * moved.median()), min=1.0)
    return out
