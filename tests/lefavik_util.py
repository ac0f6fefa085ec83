"""Configurations, model folders and comparisons for the tests of the Lefavik design."""

from __future__ import annotations

import copy
import json
from pathlib import Path

import torch

import plain_lefavik as plain


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, turned=None, kv_from=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"dims": rot_dim if turned is None else turned, "base": base}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def attention(heads, kv_heads, dim, vdim, scale, window=None, q_temp=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def model(width, vocab, layers, eps=1e-6, scale=1.0, logit_scale=1.0, max_positions=512):
    return {"architecture": "Lefavik", "embedding": {"scale": scale}, "layers": layers, "logit_scale": logit_scale,
            "max_positions": max_positions, "norm": {"eps": eps}, "vocab": vocab, "width": width}


# Odd sizes: head parts of 24 and 8 with a vector of 40 (rows of 48 in pages of bfloat16), value heads larger than key
# heads, three query heads a key head, windows of 5 and 37 (inside a page, across two page borders), a temperature every 3
# positions, a layer without a feed-forward, a layer that reads an earlier layer's vectors with another head count.
ODD = model(72, 211, [
    latent(3, 24, 8, 40, 40, 0.21, base=500.0, mlp=dense(100)),
    attention(6, 2, 24, 40, 0.9, window=5, q_temp=(0.7, 3)),
    attention(3, 3, 40, 24, 1.4, window=37, q_temp=(0.2, 16), mlp=dense(64)),
    latent(5, 16, 8, 24, 40, 0.3, base=500.0, kv_from=0, mlp=dense(96)),
], eps=1e-5, scale=1.7, logit_scale=0.5)

# What a small model tends to make equal or 1 is different here: one head, one key head for four query heads, no window,
# no temperature, a rotated part of two values, a scale of one, a width that is no multiple of eight, a logit scale of one.
ONES = model(100, 97, [
    attention(4, 1, 16, 16, 1.0, mlp=dense(48)),
    latent(1, 48, 2, 48, 30, 1.0, base=50.0),
    attention(1, 1, 64, 16, 0.5, window=1),
    latent(2, 16, 16, 16, 30, 0.25, base=50.0, turned=8, mlp=dense(40)),
], eps=1e-6, scale=1.0, logit_scale=1.0)

# Larger sizes: pages' rows of 256 (a vector of 192 with a rotated part of 64), heads of 128, sixteen query heads a key
# head, a window of 64 (page borders on both ends), layers that read vectors kept two and three layers earlier.
LARGE = model(256, 300, [
    latent(4, 64, 64, 64, 192, 0.09, base=10000.0, mlp=dense(320)),
    attention(16, 1, 128, 128, 0.15, window=64, q_temp=(0.5, 32)),
    latent(8, 32, 64, 48, 192, 0.1, base=10000.0, kv_from=0),
    latent(2, 128, 64, 128, 192, 0.07, base=10000.0, kv_from=0, mlp=dense(256)),
], eps=1e-6, scale=0.3, logit_scale=3.0)

# Rows of the pages beyond what the matrix-core kernels take (a vector of 272 with a rotated part of 16), head sizes that
# are no multiple of 4 (30, 22) or of 8 (20, 36), a rotation over 10 of 12 values, a width that is a multiple of 4 only.
UNEVEN = model(52, 75, [
    latent(2, 20, 16, 36, 272, 0.2, base=123.0, mlp=dense(44)),
    attention(3, 1, 30, 22, 0.6, window=9, q_temp=(1.5, 2)),
    latent(3, 22, 12, 30, 50, 0.21, base=123.0, turned=10),
], eps=3e-6, scale=0.8, logit_scale=1.5)

CONFIGS = {"odd": ODD, "ones": ONES, "large": LARGE, "uneven": UNEVEN}


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


def wide_sinks(tensors) -> None:
    """Sinks as drawn are near zero; spread them so that a sink left out, scaled or counted twice shows."""
    for name in tensors:
        if name.endswith(".sink"):
            heads = tensors[name].shape[0]
            tensors[name] = torch.linspace(-1.5, 2.5, heads).to(tensors[name].dtype)


def load_plain(folder):
    from safetensors.torch import load_file

    config = json.loads((Path(folder) / "config.json").read_text())
    weights = {k: v.to(torch.float64) for k, v in load_file(str(Path(folder) / "model.safetensors")).items()}
    return config, weights


def plain_logits(folder, prompts: dict, config=None) -> dict:
    """``config``: another config.json to read the same weights with (a window one larger, say)."""
    own, weights = load_plain(folder)
    return {name: plain.forward(config or own, weights, tokens) for name, tokens in prompts.items()}


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
    positions where rounding is amplified many times (a score near a tie under a sharp softmax); a bound on an engine's
    error there has to grow with it, as the error that rounding alone causes does."""
    config, weights = load_plain(folder)
    g = torch.Generator().manual_seed(1234)
    shaken = {k: v * (1 + (torch.rand(v.shape, generator=g, dtype=v.dtype) - 0.5) * 2.0 ** -8) if v.dim() == 2 else v
              for k, v in weights.items()}
    out = {}
    for name, tokens in prompts.items():
        base = plain.forward(config, weights, tokens)
        moved = ((plain.forward(config, shaken, tokens) - base) ** 2).mean(-1).sqrt() / base.std()
        out[name] = torch.clamp(moved / (2 * moved.median()), min=1.0)
    return out


def drawn_config(seed: int) -> dict:
    """A configuration drawn from the sizes and constants a model of the design may have: any order of layers (the first
    may be a window layer), layers that read an earlier layer's vectors, head counts from 1 to 16, groups of 1 to 8, head
    parts from 8 to 128, vectors from 16 to 224, windows from 3 to beyond the prompts or none, with and without a
    temperature and a feed-forward."""
    import random

    rng = random.Random(seed)
    width = rng.choice([64, 96, 128, 192, 200])
    layers, owners = [], []            # owners: (layer, kv_rank, rot_dim, base, turned) of latent layers that keep vectors
    for i in range(rng.randint(3, 6)):
        mlp = dense(rng.choice([64, 200])) if rng.random() < 0.7 else None
        if rng.random() < 0.55:
            heads, dim, vdim = rng.choice([1, 2, 4, 8, 12, 16]), rng.choice([8, 16, 32, 48, 64]), rng.choice([8, 16, 32, 64])
            if owners and rng.random() < 0.4:
                source, rank, rot, base, turned = rng.choice(owners)
                layers.append(latent(heads, dim, rot, vdim, rank, (dim + rot) ** -0.5, base=base, turned=turned, kv_from=source, mlp=mlp))
            else:
                rank, rot = rng.choice([16, 32, 48, 64, 96, 112, 160, 192, 224]), rng.choice([2, 8, 16, 32, 64])
                base = rng.choice([100.0, 10000.0, 250000.0])
                turned = rot if rng.random() < 0.8 else max(2, rot // 2 // 2 * 2)
                owners.append((i, rank, rot, base, turned))
                layers.append(latent(heads, dim, rot, vdim, rank, (dim + rot) ** -0.5, base=base, turned=turned, mlp=mlp))
        else:
            kv_heads, group = rng.choice([1, 2, 4]), rng.choice([1, 2, 4, 8])
            dim, vdim = rng.choice([16, 32, 48, 64, 128]), rng.choice([16, 32, 48, 64, 128])
            window = rng.choice([None, 3, 20, 64, 100, 500])
            q_temp = (rng.choice([0.1, 0.5, 1.0]), rng.choice([1, 7, 64])) if rng.random() < 0.7 else None
            layers.append(attention(kv_heads * group, kv_heads, dim, vdim, rng.choice([0.5, 1.0, 2.0]) * dim ** -0.5, window=window,
                                    q_temp=q_temp, mlp=mlp))
    return model(width, rng.choice([101, 256, 333]), layers, eps=rng.choice([1e-6, 1e-5]), scale=rng.choice([1.0, width ** 0.5]),
                 logit_scale=rng.choice([1.0, 0.5, 2.0]), max_positions=256)
