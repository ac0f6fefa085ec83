"""A plain, slow implementation of the Lefavik design: whole sequences, no cache, no batches, one
function a mechanism, 64-bit arithmetic.  It shares no code with the package; the tests hold the
engine against it.

``config`` is the dict of a config.json; ``w`` maps tensor names to 64-bit tensors.

A layer is x <- x + mixer(n) + ff(n) with n = norm1(x): one norm, both sublayers read it.  Two mixers:
``latent_attention`` (keys and values of all heads rebuilt from one small vector a token, plus one
rotated key part that all heads share; a learned sink a head; a gate a head on the read-out) and
``attention`` (grouped heads, unit q and k, a query temperature that grows with the position, a
distance penalty a head, a window, a sink of score 0).
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_neighbours(x, positions, dims, base):
    """x [T, ..., n]: of the first ``dims`` values, value 2i turns with value 2i + 1 by position * base^(-2i/dims)."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    angle = positions.to(F)[:, None] * freq[None, :]
    while angle.dim() < x.dim():
        angle = angle.unsqueeze(1)
    cos, sin = angle.cos(), angle.sin()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * cos - v * sin, v * cos + u * sin], -1).flatten(-2)
    return torch.cat([turned, x[..., dims:]], -1)


def softmax_with_sink(score, visible, sink):
    """Weights exp(s_j) / (exp(sink) + sum over the visible j of exp(s_j)); ``score`` [T, T], ``sink`` a number.
    The sink has no value, so the weights of a row sum to less than one."""
    score = score.masked_fill(~visible, -math.inf)
    sink = torch.as_tensor(sink, dtype=F)
    top = torch.clamp(score.max(-1, keepdim=True).values, min=float(sink))
    e = torch.exp(score - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - top))


def latent_of(h, w, p, m, eps, positions):
    """What a latent-attention layer keeps of a token: the normalised small vector c [T, kv_rank] and the
    rotated key part [T, rot_dim] that every head shares."""
    R, rot = m["kv_rank"], m["rot_dim"]
    both = h @ w[p + "dkv"].T
    c = rms(both[:, :R], eps) * w[p + "dkv.norm"]
    k_rot = rotate_neighbours(both[:, R:R + rot], positions, m["rot"]["dims"], m["rot"]["base"])
    return c, k_rot


def latent_attention_mixer(h, w, p, m, eps, kept, positions=None):
    """``kept``: (c, k_rot) of this layer, or of the layer whose kept vectors this one reads."""
    T = h.shape[0]
    H, D, rot, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    positions = torch.arange(T) if positions is None else positions
    c, k_rot = kept
    q = (h @ w[p + "q"].T).view(T, H, D + rot)
    q_plain = q[..., :D]
    q_rot = rotate_neighbours(q[..., D:], positions, m["rot"]["dims"], m["rot"]["base"])
    k_plain = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, V)
    gate = torch.sigmoid(h @ w[p + "g"].T)
    causal = positions[:, None] >= positions[None, :]
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        score = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * m["scale"]
        weights = softmax_with_sink(score, causal, w[p + "sink"][head])
        out[:, head] = (weights @ v[:, head]) * gate[:, head:head + 1]
    return out.reshape(T, H * V) @ w[p + "o"].T


def query_temperature(positions, coef, every):
    """1 + coef * ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * torch.log(torch.floor((positions.to(F) + 1.0) / every) + 1.0)


def distance_slopes(heads):
    """2^(-8 (h + 1) / heads) for head h."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=F)


def window_attention_mixer(h, w, p, m, eps, positions=None):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(T) if positions is None else positions
    q = rms((h @ w[p + "q"].T).view(T, H, D), eps)
    k = rms((h @ w[p + "k"].T).view(T, G, D), eps)
    v = (h @ w[p + "v"].T).view(T, G, V)
    if m.get("q_temp"):
        q = q * query_temperature(positions, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    distance = (positions[:, None] - positions[None, :]).to(F)
    visible = distance >= 0
    if m.get("mask"):
        visible = visible & (distance < m["mask"]["size"])
    slopes = distance_slopes(H)
    each = H // G
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        score = (q[:, head] @ k[:, head // each].T) * m["scale"] - slopes[head] * distance
        out[:, head] = softmax_with_sink(score, visible, torch.tensor(0.0, dtype=F)) @ v[:, head // each]
    return out.reshape(T, H * V) @ w[p + "o"].T


def gated_mlp(h, w, p):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def embed(config, w, tokens, positions):
    x = w["embed"][tokens] * config["embedding"]["scale"] + w["pos"][positions]
    return rms(x, config["norm"]["eps"]) * w["embed.norm"]


def forward(config, w, tokens, streams=None):
    """Logits [T, vocab] of one whole sequence.  ``streams``: a list that receives the stream after every layer."""
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    x = embed(config, w, tokens, positions)
    kept = {}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = rms(x, eps) * w[p + "norm1"]
        if layer["type"] == "latent_attention":
            source = m.get("kv_from")
            if source is None:
                kept[i] = latent_of(h, w, p + "mix.", m, eps, positions)
                source = i
            y = latent_attention_mixer(h, w, p + "mix.", m, eps, kept[source], positions)
        elif layer["type"] == "attention":
            y = window_attention_mixer(h, w, p + "mix.", m, eps, positions)
        else:
            raise ValueError(f"a mixer of type {layer['type']!r}")
        if layer.get("mlp") is not None:
            y = y + gated_mlp(h, w, p + "mlp.")
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    x = rms(x, eps) * w["final.norm"]
    return (x @ w["head"].T) * config["logit_scale"]
