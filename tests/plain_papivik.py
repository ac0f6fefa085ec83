"""A plain, slow implementation of the Papivik design: whole sequences, no cache, no batches, one
function a mechanism, 64-bit arithmetic, token-by-token loops where the design has a recurrence.
It shares no code with the package; the tests hold the engine against it.

``config`` is the dict of a config.json; ``w`` maps tensor names to 64-bit tensors.
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


def silu(z):
    return z * torch.sigmoid(z)


def short_conv(u, taps_w):
    """u [T, C], taps_w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + T] * taps_w[:, j]
    return y


def rotate_half(x, positions, dims, base):
    """x [T, heads, dim]: the first ``dims`` values of a head turn, value i with value i + dims/2."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    angle = positions.to(F)[:, None] * freq[None, :]
    cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., dims:]], -1)


def lightning_mixer(h, w, p, m, eps):
    """Linear attention with one fixed decay a head."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).view(T, H, D)
    k = silu(h @ w[p + "k"].T).view(T, H, D)
    v = silu(h @ w[p + "v"].T).view(T, H, V)
    decay = torch.tensor(m["decay"], dtype=F)
    S = torch.zeros(H, D, V, dtype=F)
    o = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = rms(o.reshape(T, H * V), eps) * w[p + "norm"]
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def mlstm_mixer(h, w, p, m, eps):
    """Matrix memory with exponential gates held stable by a running maximum that starts at 0."""
    T = h.shape[0]
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, V)
    i_gate = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    f_gate = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    S = torch.zeros(H, D, V, dtype=F)
    n = torch.zeros(H, D, dtype=F)
    mx = torch.zeros(H, dtype=F)
    o = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        new = torch.maximum(f_gate[t] + mx, i_gate[t])
        keep, add = torch.exp(f_gate[t] + mx - new), torch.exp(i_gate[t] - new)
        S = keep[:, None, None] * S + add[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + add[:, None] * k[t]
        mx = new
        below = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        o[t] = torch.einsum("hdv,hd->hv", S, q[t]) / below[:, None]
    o = rms(o, eps).reshape(T, H * V) * w[p + "norm"]
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def conv_attention_mixer(h, w, p, m, eps, positions=None):
    """Softmax attention over all earlier tokens, with a short convolution behind every projection,
    a norm a head on q and k, and a rotation of part of each head."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(T) if positions is None else positions
    q = short_conv(h @ w[p + "q"].T, w[p + "q.conv"]).view(T, H, D)
    k = short_conv(h @ w[p + "k"].T, w[p + "k.conv"]).view(T, G, D)
    v = short_conv(h @ w[p + "v"].T, w[p + "v.conv"]).view(T, G, V)
    q = rms(q, eps) * w[p + "q.norm"]
    k = rms(k, eps) * w[p + "k.norm"]
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, positions, rot["dims"], rot["base"])
        k = rotate_half(k, positions, rot["dims"], rot["base"])
    each = H // G
    out = torch.zeros(T, H, V, dtype=F)
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for head in range(H):
        g = head // each
        score = (q[:, head] @ k[:, g].T) * m["scale"]
        score = score.masked_fill(~causal, -math.inf)
        out[:, head] = torch.softmax(score, -1) @ v[:, g]
    return out.reshape(T, H * V) @ w[p + "o"].T


def delta_mixer(h, w, p, m, eps):
    """The gated delta rule: decay the memory, correct what it says for this key, read it out."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * torch.nn.functional.softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    each = H // G
    S = torch.zeros(H, D, V, dtype=F)
    o = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        for head in range(H):
            g = head // each
            S[head] = decay[t, head] * S[head]
            u = beta[t, head] * (v[t, head] - S[head].T @ k[t, g])
            S[head] = S[head] + k[t, g][:, None] * u[None, :]
            o[t, head] = S[head].T @ q[t, g]
    o = rms(o, eps) * w[p + "norm"]
    o = o.reshape(T, H * V) * silu(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps):
    left = conv_attention_mixer(h, w, p + "left.", m["left"], eps)
    right = delta_mixer(h, w, p + "right.", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


MIXERS = {"lightning": lightning_mixer, "mlstm": mlstm_mixer, "parallel": parallel_mixer}


def dense_mlp(h, w, p):
    return gelu_tanh(h @ w[p + "up"].T) @ w[p + "down"].T


def forward(config, w, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence.  ``layers_out``: a list that receives the stream after every layer."""
    eps = config["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        mixed = MIXERS[layer["type"]](x, w, p + "mix.", layer["mixer"], eps)
        x = x + rms(mixed, eps) * w[p + "norm1"]
        if layer.get("mlp") is not None:
            x = x + rms(dense_mlp(x, w, p + "mlp."), eps) * w[p + "norm2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms(x, eps) * w["final.norm"]
    return x @ w["head"].T
