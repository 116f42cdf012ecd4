"""Small Fazovik configurations for the tests, and their random weights under the stored tensor names. The weights
are wide enough that attention is far from uniform and the routers' scores are spread out."""
from __future__ import annotations

import json
import math
import os

import torch
from safetensors.torch import save_file


def _rotary(heads, dim, rot_dim, vdim, q_rank, kv_rank, base, scaling=None, scale=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling is not None:
        rot["scaling"] = scaling
    return {"type": "latent_attention",
            "mixer": {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot": rot, "rot_dim": rot_dim,
                      "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "vdim": vdim}}


def _plain(heads, dim, vdim, q_rank, kv_rank, kv_from=None, scale=None):
    m = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale if scale is not None else dim ** -0.5,
         "vdim": vdim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention_2", "mixer": m}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _model(vocab, width, eps, bigram, layers):
    return {"architecture": "Fazovik", "embedding": {"bigram": bigram}, "layers": [dict(l, mlp=mlp) for l, mlp in layers],
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


# F: every size differs from layer to layer and none is a multiple of 8 where it need not be: two experts a token, a
# layer without feed-forward, a layer that borrows a plain latent and one that borrows the latent of a rotary layer
CONFIG_F = _model(131, 44, 1e-5, {"buckets": 37, "mul_cur": 5, "mul_prev": 11}, [
    (_rotary(3, 6, 4, 10, 9, 13, 10000.0, {"factor": 4.0, "fast": 8.0, "original": 16, "slow": 1.0}), _dense(36)),
    (_plain(2, 12, 7, 14, 18), _moe(5, 2, 20)),
    (_rotary(5, 4, 8, 6, 11, 9, 500.0, None, 0.5), None),
    (_plain(4, 5, 9, 6, 18, kv_from=1), _moe(3, 3, 12)),
    (_plain(2, 8, 8, 8, 13, kv_from=0), _dense(28)),
])
# G: stored rows of 64 and 32 entries (the sizes the matrix-core attention kernels take), 17 heads in one layer (more
# than those kernels' decoding form takes), one expert, one bucket, one head
CONFIG_G = _model(211, 64, 2e-6, {"buckets": 1, "mul_cur": 3, "mul_prev": 2}, [
    (_plain(17, 8, 8, 16, 32), _moe(1, 1, 24)),
    (_rotary(4, 16, 16, 16, 24, 48, 40000.0, {"factor": 3.0, "fast": 16.0, "original": 64, "slow": 0.5}), _dense(96)),
    (_plain(1, 16, 24, 8, 32, kv_from=0), _moe(6, 1, 16)),
    (_rotary(6, 8, 32, 8, 16, 32, 1000.0), _moe(4, 4, 8)),
])
CASES = {"F": (CONFIG_F, 11), "G": (CONFIG_G, 12)}


def random_tensors(config: dict, seed: int, gain: float = 1.6) -> dict[str, torch.Tensor]:
    """Stored tensors by name, bfloat16: matrices N(0, gain^2 / inputs), norm weights about 1, biases about 0.1."""
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    out = {}

    def matrix(name, rows, cols, scale=gain):
        out[name] = (torch.randn(rows, cols, generator=g) * scale / math.sqrt(cols)).to(torch.bfloat16)

    def vector(name, n, mean, std):
        out[name] = (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    out["embed"] = torch.randn(config["vocab"], W, generator=g).to(torch.bfloat16)
    bigram = (config.get("embedding") or {}).get("bigram")
    if bigram:
        out["bigram"] = (0.7 * torch.randn(bigram["buckets"] + 1, W, generator=g)).to(torch.bfloat16)
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        vector(p + "norm1", W, 1.0, 0.2)
        vector(p + "norm1.b", W, 0.0, 0.1)
        H, rot = m["heads"], m.get("rot_dim", 0)
        matrix(p + "mix.dq", m["q_rank"], W)
        vector(p + "mix.dq.norm", m["q_rank"], 1.0, 0.2)
        matrix(p + "mix.uq", H * (m["dim"] + rot), m["q_rank"])
        if m.get("kv_from") is None:
            matrix(p + "mix.dkv", m["kv_rank"] + rot, W)
            vector(p + "mix.dkv.norm", m["kv_rank"], 1.0, 0.2)
        matrix(p + "mix.uk", H * m["dim"], m["kv_rank"])
        matrix(p + "mix.uv", H * m["vdim"], m["kv_rank"], 1.0)
        if layer["type"] == "latent_attention":
            matrix(p + "mix.g", H, W)
        matrix(p + "mix.o", W, H * m["vdim"], 1.0)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        vector(p + "norm2", W, 1.0, 0.2)
        vector(p + "norm2.b", W, 0.0, 0.1)
        if mlp["kind"] == "dense":
            matrix(p + "mlp.gate", mlp["ff"], W)
            matrix(p + "mlp.up", mlp["ff"], W, 1.0)
            matrix(p + "mlp.down", W, mlp["ff"], 1.0)
        else:
            matrix(p + "mlp.router", mlp["router"]["experts"], W, 2.0)
            for e in range(mlp["router"]["experts"]):
                q = p + f"mlp.e{e}."
                matrix(q + "gate", mlp["expert"]["ff"], W)
                matrix(q + "up", mlp["expert"]["ff"], W, 1.0)
                matrix(q + "down", W, mlp["expert"]["ff"], 1.0)
    vector("final.norm", W, 1.0, 0.2)
    vector("final.norm.b", W, 0.0, 0.1)
    return out


def write_model(folder: str, config: dict, seed: int) -> str:
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f, indent=1)
    save_file({k: v.contiguous() for k, v in random_tensors(config, seed).items()}, os.path.join(folder, "model.safetensors"))
    return folder
