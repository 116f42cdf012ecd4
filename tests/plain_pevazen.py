"""Plain, slow, whole-sequence Pevazen decoder on the CPU: the oracle of the tests of this design.

No cache, no batching, no kernels and no code of the package: every function takes
a whole sequence and writes one mechanism out as loops and small tensor
expressions. ``logits(config, tensors, tokens)`` runs a model folder's contents
(``read_model_folder``); ``dtype`` may be ``torch.float64`` for a sharper oracle.

Notation: T tokens, W the model's width, H query heads, G key/value heads, D the
query/key head size, E the value head size, p a token's index in its sequence.
"""
from __future__ import annotations

import json
import math
import os

import torch


def read_model_folder(folder: str):
    """config.json as a dict and every tensor of model.safetensors (floats as float32)."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            tensors[name] = t.to(torch.float32) if t.is_floating_point() else t
    return config, tensors


# ------------------------------------------------------------------ small pieces
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis, eps under the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def scalar_norm(x, gain, eps):
    """RMS norm whose weight is one number for all coordinates."""
    return unit_rms(x, eps) * gain


def vector_norm(x, weight, eps):
    """RMS norm with a plain weight per coordinate."""
    return unit_rms(x, eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 20, z, torch.log1p(torch.exp(torch.clamp(z, max=20.0))))


def pair_frequencies(dims: int, base: float, dtype) -> torch.Tensor:
    """f_i = base^(-2 i / dims), i < dims / 2."""
    i = torch.arange(dims // 2, dtype=dtype)
    return base ** (-2.0 * i / dims)


def turn_halves(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor, sign: float = 1.0) -> torch.Tensor:
    """x[T, heads, n]: coordinate i is paired with i + r, r = len(freqs), for i < r; the pair (u, v) at position p
    becomes (u cos a - v sin a, v cos a + u sin a), a = sign * p * f_i. Coordinates from 2 r on pass unchanged."""
    r = freqs.shape[0]
    a = sign * positions.to(freqs.dtype)[:, None] * freqs[None, :]            # [T, r]
    cos, sin = a.cos()[:, None, :], a.sin()[:, None, :]
    u, v = x[..., :r], x[..., r:2 * r]
    return torch.cat((u * cos - v * sin, v * cos + u * sin, x[..., 2 * r:]), dim=-1)


def chunk_mask(T: int, size: int) -> torch.Tensor:
    """[T, T] bool: query i sees key j iff j <= i and both lie in the same block of ``size`` positions counted
    from the start of the sequence."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def masked_attention(q, k, v, scale: float, visible: torch.Tensor) -> torch.Tensor:
    """q[T, H, D], k[T, G, D], v[T, G, E] -> [T, H, E]; query head h reads key/value head h // (H / G); ordinary
    softmax over the visible keys."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~visible, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


# ------------------------------------------------------------------ mixers
def rotary_attention(h, w, prefix, m, eps, lent=None, rotate_values=False, biases=False):
    """Softmax attention with rotated queries and keys under a chunk mask. ``m``: the mixer's entry of config.json.
    ``lent``: (keys after rotation, values) of another layer, used in place of this layer's own (which then has no
    key and value projections). ``rotate_values``: the value at position j is turned by j over all its coordinates
    and every head's output at position i is turned back by i. Returns (output [T, W], (keys, values) as cached)."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    rot = m["rot"]
    f = pair_frequencies(rot["dims"], rot["base"], h.dtype)
    if rot.get("scaling"):
        f = f / rot["scaling"]["factor"]

    def project(name, heads, size):
        y = h @ w[prefix + name].T
        if biases:
            y = y + w[prefix + name + ".b"]
        return y.view(T, heads, size)

    q = turn_halves(project("q", H, D), pos, f)
    if lent is None:
        k = turn_halves(project("k", G, D), pos, f)
        v = project("v", G, E)
        if rotate_values:
            v = turn_halves(v, pos, pair_frequencies(E, rot["base"], h.dtype))
    else:
        k, v = lent
    o = masked_attention(q, k, v, m["scale"], chunk_mask(T, m["mask"]["size"]))
    if rotate_values:
        o = turn_halves(o, pos, pair_frequencies(E, rot["base"], h.dtype), sign=-1.0)
    return o.reshape(T, H * E) @ w[prefix + "o"].T, (k, v)


def causal_taps(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x[T, C], taps[C, n]: y[t, c] = sum_j taps[c, j] x[t - (n - 1 - j), c], zeros before the start."""
    T, C = x.shape
    n = taps.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(n):
            s = t - (n - 1 - j)
            if s >= 0:
                y[t] += taps[:, j] * x[s]
    return y


def gated_delta_rule(q, k, v, decay, beta):
    """Per head, token by token: S <- diag(decay_t) S; u = beta_t (v_t - S^T k_t); S <- S + k_t u^T; o_t = S^T q_t.
    q, k, decay: [T, H, D]; v: [T, H, E]; beta: [T, H]; S: [D, E], zero at the start. Returns o [T, H, E]."""
    T, H, D = q.shape
    E = v.shape[-1]
    out = torch.zeros(T, H, E, dtype=q.dtype)
    for h in range(H):
        S = torch.zeros(D, E, dtype=q.dtype)
        for t in range(T):
            S = decay[t, h][:, None] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + torch.outer(k[t, h], u)
            out[t, h] = S.T @ q[t, h]
    return out


def delta_rule_mixer(h, w, prefix, m, eps):
    """The recurrent mixer. ``m``: its entry of config.json (heads, kv_heads, dim, vdim, conv)."""
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]

    def short(name):
        return silu(causal_taps(h @ w[prefix + name].T, w[prefix + name + ".conv"]))

    def unit(x):
        return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)

    rep = H // G
    q = unit(short("q").view(T, G, D)).repeat_interleave(rep, dim=1) * D ** -0.5
    k = unit(short("k").view(T, G, D)).repeat_interleave(rep, dim=1)
    v = short("v").view(T, H, E)
    beta = torch.sigmoid(h @ w[prefix + "b"].T)                                            # [T, H]
    step = softplus((h @ w[prefix + "a1"].T) @ w[prefix + "a2"].T + w[prefix + "dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(w[prefix + "A_log"])[None, :, None] * step)
    o = gated_delta_rule(q, k, v, decay, beta)
    gate = torch.sigmoid((h @ w[prefix + "g1"].T) @ w[prefix + "g2"].T).view(T, H, E)
    o = unit_rms(o, eps) * w[prefix + "norm"] * gate
    return o.reshape(T, H * E) @ w[prefix + "o"].T


def gated_feed_forward(h, w, prefix):
    return (silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


# ------------------------------------------------------------------ the model
def hidden_states(config: dict, tensors: dict, tokens, dtype=torch.float32) -> list[torch.Tensor]:
    """[X after the embedding, X after every layer (after its depth average)], each [T, W]."""
    w = {k: (t.to(dtype) if t.is_floating_point() else t) for k, t in tensors.items()}
    eps = config["norm"]["eps"]
    x = scalar_norm(w["embed"][torch.as_tensor(tokens, dtype=torch.long)], w["embed.norm"], eps)
    outputs = [x]            # X_0, X_1, ...: every layer's own result, before the depth average
    streams = [x]
    cached = {}
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = scalar_norm(x, w[p + "norm1"], eps)
        m = layer["mixer"]
        if layer["type"] == "parallel":
            left, _ = rotary_attention(h, w, p + "mix.left.", m["left"], eps, rotate_values=True)
            right = delta_rule_mixer(h, w, p + "mix.right.", m["right"], eps)
            mixed = 0.5 * (vector_norm(left, w[p + "mix.left.out"], eps) + vector_norm(right, w[p + "mix.right.out"], eps))
        elif layer["type"] == "attention":
            lent = cached[m["kv_from"]] if "kv_from" in m else None
            mixed, cached[i] = rotary_attention(h, w, p + "mix.", m, eps, lent=lent, biases=True)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        update = mixed
        if layer.get("mlp") is not None:
            if layer["mlp"]["kind"] != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind")
            update = update + gated_feed_forward(h, w, p + "mlp.")
        outputs.append(x + update)
        x = sum(w[p + "dwa"][j] * outputs[j] for j in range(i + 2))
        streams.append(x)
    return streams


def logits(config: dict, tensors: dict, tokens, dtype=torch.float32) -> torch.Tensor:
    """[T, vocab]."""
    x = hidden_states(config, tensors, tokens, dtype)[-1]
    g = tensors["final.norm"].to(dtype)
    return scalar_norm(x, g, config["norm"]["eps"]) @ tensors["head"].to(dtype).T


def greedy_generate(config, tensors, prompt, n: int) -> list[int]:
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(logits(config, tensors, ids)[-1].argmax()))
    return ids[len(prompt):]
