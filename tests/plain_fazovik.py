"""The Fazovik decoder, plain and slow: whole sequences, no cache, no batching, one function per mechanism, written
from the design's equations only. It reads a model folder itself (config.json, model.safetensors) and shares no code
with the engine. Everything is evaluated in one element type (float64 by default) from the stored numbers.
"""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


def read_folder(folder: str, dtype=torch.float64):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for key in f.keys():
            t = f.get_tensor(key)
            tensors[key] = t.to(dtype) if t.is_floating_point() else t.long()
    return cfg, tensors


# ---------------------------------------------------------------- small pieces
def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rms_norm(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def layer_norm(x, weight, bias, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight + bias


def bigram_rows(tokens, buckets: int, mul_prev: int, mul_cur: int):
    """Row of the bigram table for every token: the last row for a sequence's first token."""
    rows = []
    for i, t in enumerate(tokens):
        rows.append(buckets if i == 0 else (tokens[i - 1] * mul_prev + t * mul_cur) % buckets)
    return rows


def embed(tokens, W, cfg):
    x = W["embed"][torch.tensor(tokens)]
    b = (cfg.get("embedding") or {}).get("bigram")
    if b:
        x = x + W["bigram"][torch.tensor(bigram_rows(tokens, b["buckets"], b["mul_prev"], b["mul_cur"]))]
    return x


def scaled_frequencies(rot: dict, dtype=torch.float64):
    """(frequencies [dims / 2], factor on cosines and sines) of a rotation with optional YaRN scaling."""
    dims, base = rot["dims"], rot["base"]
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=dtype)
    s = rot.get("scaling")
    if not s:
        return f, 1.0
    factor, original = s["factor"], s["original"]

    def dim_of(turns):
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(s["fast"])), 0)
    hi = min(math.ceil(dim_of(s["slow"])), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)], dtype=dtype)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x, positions, freqs, gain):
    """x [..., T, n]: entries (2i, 2i + 1) of the first 2 len(freqs) turn by position * freqs[i]; the rest pass."""
    n = 2 * freqs.shape[0]
    a = positions.to(freqs.dtype)[:, None] * freqs[None, :]                  # [T, n / 2]
    cos, sin = torch.cos(a) * gain, torch.sin(a) * gain
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out = x.clone()
    out[..., 0:n:2] = u * cos - v * sin
    out[..., 1:n:2] = v * cos + u * sin
    return out


def causal_softmax_attention(q, k, v, scale):
    """q, k [H, T, d], v [H, T, e] -> [H, T, e]; position i reads every j <= i."""
    T = q.shape[1]
    s = torch.einsum("hid,hjd->hij", q, k) * scale
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    s = s.masked_fill(~mask, float("-inf"))
    return torch.einsum("hij,hje->hie", torch.softmax(s, dim=-1), v)


# ---------------------------------------------------------------- mixers
def latent_of(h, W, p, m, eps):
    """The normed latent c [T, kv_rank] of a layer (and what is left of the rows of W_dkv, unnormed)."""
    rank = m["kv_rank"]
    d = h @ W[p + "dkv"].T
    return rms_norm(d[:, :rank], W[p + "dkv.norm"], eps), d[:, rank:]


def latent_attention(h, W, p, m, eps, latents):
    """Rotary latent attention with an output gate. ``latents[i]``: what layer i has cached (c)."""
    T = h.shape[0]
    H, dim, rot, vd = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).view(T, H, dim + rot).transpose(0, 1)            # [H, T, dim + rot]
    c, k_rot = latent_of(h, W, p, m, eps)
    k_flat = (c @ W[p + "uk"].T).view(T, H, dim).transpose(0, 1)
    v = (c @ W[p + "uv"].T).view(T, H, vd).transpose(0, 1)
    freqs, gain = scaled_frequencies(m["rot"], h.dtype)
    pos = torch.arange(T)
    q_rot = rotate_interleaved(q[..., dim:], pos, freqs, gain)
    k_rot = rotate_interleaved(k_rot, pos, freqs, gain)                       # [T, rot], one for all heads
    qq = torch.cat([q[..., :dim], q_rot], dim=-1)
    kk = torch.cat([k_flat, k_rot[None].expand(H, T, rot)], dim=-1)
    o = causal_softmax_attention(qq, kk, v, m["scale"])                       # [H, T, vd]
    gate = torch.sigmoid(h @ W[p + "g"].T)                                    # [T, H]
    o = o * gate.T[:, :, None]
    return o.transpose(0, 1).reshape(T, H * vd) @ W[p + "o"].T, c


def latent_attention_2(h, W, p, m, eps, latents):
    """Latent attention without positions; with ``kv_from`` the latent is another layer's."""
    T = h.shape[0]
    H, dim, vd = m["heads"], m["dim"], m["vdim"]
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).view(T, H, dim).transpose(0, 1)
    if m.get("kv_from") is not None:
        c = latents[m["kv_from"]]
    else:
        c, _ = latent_of(h, W, p, m, eps)
    k = (c @ W[p + "uk"].T).view(T, H, dim).transpose(0, 1)
    v = (c @ W[p + "uv"].T).view(T, H, vd).transpose(0, 1)
    o = causal_softmax_attention(q, k, v, m["scale"])
    return o.transpose(0, 1).reshape(T, H * vd) @ W[p + "o"].T, c


# ---------------------------------------------------------------- feed-forwards
def dense_ff(h, W, p):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def routed_ff(h, W, p, mlp):
    """Every token goes to the ``top`` experts of largest sigmoid score; the score multiplies the expert's input."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = torch.sigmoid(h @ W[p + "router"].T)                                  # [T, E]
    chosen = torch.topk(s, top, dim=-1).indices
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            x = s[t, e] * h[t]
            q = p + f"e{e}."
            out[t] += (silu(W[q + "gate"] @ x) * (W[q + "up"] @ x)) @ W[q + "down"].T
    return out


# ---------------------------------------------------------------- the model
MIXERS = {"latent_attention": latent_attention, "latent_attention_2": latent_attention_2}


def forward(cfg, W, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one sequence (and, if asked, the stream after every layer [layers, T, width])."""
    eps = cfg["norm"]["eps"]
    x = embed(tokens, W, cfg)
    latents, after = {}, []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h1 = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
        mixed, latents[i] = MIXERS[layer["type"]](h1, W, p + "mix.", layer["mixer"], eps, latents)
        mlp = layer.get("mlp")
        if mlp is not None:
            h2 = layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps)
            fed = dense_ff(h2, W, p + "mlp.") if mlp["kind"] == "dense" else routed_ff(h2, W, p + "mlp.", mlp)
            mixed = mixed + fed
        x = x + mixed
        after.append(x)
    y = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    logits = y @ W["embed"].T
    return (logits, torch.stack(after)) if return_layers else logits
