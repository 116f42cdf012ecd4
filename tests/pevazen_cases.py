"""Small Pevazen configurations, random weights for them and ways of cutting requests into steps, for the tests.

The configurations differ from each other in every size and option; among them are values that make two sizes
equal or 1 (one head, one tap, a chunk of one position, a chunk longer than any request), a layer without
feed-forward, a partial rotation with and without scaled frequencies, and a layer that reads another layer's keys
and values under a mask of another size. Weights are drawn wide enough that attention is far from uniform and the
recurrent state matters; they are stored in bfloat16, so runs in both element types read the same numbers.
"""
from __future__ import annotations

import json
import os

import torch


def _attention(heads, kv_heads, dim, vdim, chunk, rot_dims, base, scale, factor=None, **more):
    rot = {"base": base, "dims": rot_dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    return dict({"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": chunk}, "rot": rot, "scale": scale,
                 "vdim": vdim}, **more)


def _delta(heads, kv_heads, dim, vdim, conv):
    return {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


CONFIG_P = {
    "architecture": "Pevazen", "norm": {"eps": 1e-5}, "vocab": 97, "width": 40,
    "layers": [
        {"type": "parallel", "mlp": _dense(56),
         "mixer": {"left": _attention(4, 2, 8, 12, 6, 4, 50.0, 0.4, factor=3.0), "right": _delta(4, 2, 8, 6, 4)}},
        {"type": "attention", "mlp": None, "mixer": _attention(3, 1, 12, 4, 9, 12, 200.0, 0.3)},
        {"type": "parallel", "mlp": _dense(24),
         "mixer": {"left": _attention(2, 2, 6, 6, 4, 6, 10.0, 0.5), "right": _delta(3, 3, 5, 7, 2)}},
        {"type": "attention", "mlp": _dense(32), "mixer": _attention(3, 1, 12, 4, 5, 12, 200.0, 0.25, kv_from=1)},
    ],
}
RANKS_P = {0: (5, 3), 2: (8, 8)}

# sizes of one, a chunk of one position and a chunk longer than any request
CONFIG_Q = {
    "architecture": "Pevazen", "norm": {"eps": 1e-6}, "vocab": 61, "width": 24,
    "layers": [
        {"type": "attention", "mlp": _dense(16), "mixer": _attention(1, 1, 10, 10, 1000, 2, 7.0, 0.7, factor=1.5)},
        {"type": "parallel", "mlp": None,
         "mixer": {"left": _attention(1, 1, 4, 2, 1, 0, 30.0, 1.0), "right": _delta(1, 1, 3, 3, 1)}},
        {"type": "attention", "mlp": None, "mixer": _attention(1, 1, 10, 10, 3, 2, 7.0, 0.2, factor=1.5, kv_from=0)},
        {"type": "parallel", "mlp": _dense(40),
         "mixer": {"left": _attention(6, 3, 16, 16, 8, 16, 10000.0, 0.25), "right": _delta(2, 1, 16, 16, 3)}},
    ],
}
RANKS_Q = {1: (1, 2), 3: (16, 8)}

# sizes that the kernels on the matrix cores take (head sizes in steps of 16, equal for keys and values)
CONFIG_R = {
    "architecture": "Pevazen", "norm": {"eps": 1e-6}, "vocab": 128, "width": 128,
    "layers": [
        {"type": "parallel", "mlp": _dense(256),
         "mixer": {"left": _attention(4, 2, 32, 32, 40, 32, 10000.0, 32 ** -0.5, factor=2.0), "right": _delta(2, 2, 64, 64, 4)}},
        {"type": "attention", "mlp": _dense(256), "mixer": _attention(8, 2, 16, 16, 24, 8, 500.0, 0.25)},
    ],
}
RANKS_R = {0: (16, 24)}

# the same kinds of sizes with chunks longer than a page of 64 tokens, one of them no multiple of it
CONFIG_S = {
    "architecture": "Pevazen", "norm": {"eps": 1e-6}, "vocab": 96, "width": 64,
    "layers": [
        {"type": "attention", "mlp": _dense(64), "mixer": _attention(4, 1, 32, 32, 96, 16, 10000.0, 0.2)},
        {"type": "parallel", "mlp": None,
         "mixer": {"left": _attention(2, 2, 48, 48, 160, 48, 1000.0, 0.15, factor=4.0), "right": _delta(2, 1, 32, 16, 4)}},
        {"type": "attention", "mlp": _dense(64), "mixer": _attention(4, 1, 32, 32, 128, 16, 10000.0, 0.2, kv_from=0)},
    ],
}
RANKS_S = {1: (8, 8)}

CASES = {"P": (CONFIG_P, RANKS_P, 11), "Q": (CONFIG_Q, RANKS_Q, 12), "R": (CONFIG_R, RANKS_R, 13), "S": (CONFIG_S, RANKS_S, 14)}


def random_tensors(config: dict, ranks: dict, seed: int) -> dict[str, torch.Tensor]:
    """The stored tensors of a model of this configuration, by their names, in bfloat16."""
    gen = torch.Generator().manual_seed(seed)
    W = config["width"]
    out = {}

    def normal(shape, std, mean=0.0):
        return mean + std * torch.randn(shape, generator=gen)

    def matrix(rows, cols, gain=1.0):
        return normal((rows, cols), gain / cols ** 0.5)

    def attention(p, m, biases, own_kv=True):
        H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for name, rows in (("q", H * D), ("k", G * D), ("v", G * E)) if own_kv else (("q", H * D),):
            out[p + name] = matrix(rows, W, 2.5 if name != "v" else 1.0)
            if biases:
                out[p + name + ".b"] = normal((rows,), 0.5)
        out[p + "o"] = matrix(W, H * E)

    out["embed"] = normal((config["vocab"], W), 1.0)
    out["embed.norm"] = normal((), 0.1, 1.3)
    out["final.norm"] = normal((), 0.1, 0.8)
    out["head"] = matrix(config["vocab"], W, 1.5)
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        out[p + "norm1"] = normal((), 0.1, 1.1)
        out[p + "dwa"] = normal((i + 2,), 0.3 / (i + 2), 1.0 / (i + 2))
        m = layer["mixer"]
        if layer["type"] == "attention":
            attention(p + "mix.", m, True, "kv_from" not in m)
        else:
            attention(p + "mix.left.", m["left"], False)
            r = m["right"]
            H, G, D, E, n = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
            ra, rg = ranks[i]
            for name, rows in (("q", G * D), ("k", G * D), ("v", H * E)):
                out[p + "mix.right." + name] = matrix(rows, W, 1.5)
                out[p + "mix.right." + name + ".conv"] = normal((rows, n), 0.6)
            out[p + "mix.right.b"] = matrix(H, W, 2.0)
            out[p + "mix.right.A_log"] = normal((H,), 0.5, -0.5)
            out[p + "mix.right.norm"] = normal((E,), 0.2, 1.0)
            out[p + "mix.right.a1"] = matrix(ra, W)
            out[p + "mix.right.a2"] = matrix(H * D, ra, 2.0)
            out[p + "mix.right.dt_bias"] = normal((H * D,), 1.0, -0.5)
            out[p + "mix.right.g1"] = matrix(rg, W)
            out[p + "mix.right.g2"] = matrix(H * E, rg, 2.0)
            out[p + "mix.right.o"] = matrix(W, H * E)
            out[p + "mix.left.out"] = normal((W,), 0.2, 1.0)
            out[p + "mix.right.out"] = normal((W,), 0.2, 1.0)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            out[p + "mlp.gate"] = matrix(ff, W, 1.5)
            out[p + "mlp.up"] = matrix(ff, W, 1.5)
            out[p + "mlp.down"] = matrix(W, ff, 1.5)
    return {k: v.to(torch.bfloat16) for k, v in out.items()}


def write_model(folder: str, config: dict, ranks: dict, seed: int) -> str:
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.contiguous() for k, v in random_tensors(config, ranks, seed).items()},
              os.path.join(folder, "model.safetensors"))
    return folder


def tokens(vocab: int, n: int, seed: int) -> list[int]:
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


# ------------------------------------------------------------------ ways of cutting requests into steps
def whole(requests: dict) -> list[dict]:
    return [{"step": i, "entries": [{"id": rid, "tokens": list(toks), "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def in_portions(requests: dict, sizes) -> list[dict]:
    """Each request alone, in portions of the sizes given in turn (the list is walked round and round)."""
    steps, k = [], 0
    for rid, toks in requests.items():
        at = 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
                          "end": [rid] if at + n == len(toks) else []})
            at += n
    return steps


def interleaved(requests: dict, sizes, max_live: int) -> list[dict]:
    """Up to ``max_live`` requests side by side: in every step each live request brings its next portion (sizes
    walked round and round, so portions of several tokens stand beside single ones), a request leaves out every
    fifth step it could take part in, and a finished request's place goes to the next one that waits."""
    waiting = list(requests.items())
    live: dict = {}
    steps, k = [], 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, ended = [], []
        for rid, state in list(live.items()):
            k += 1
            if k % 5 == 0 and len(live) > 1:
                continue
            toks, at = state
            n = min(sizes[k % len(sizes)], len(toks) - at)
            entries.append({"id": rid, "tokens": toks[at:at + n], "want": list(range(n))})
            state[1] = at + n
            if state[1] == len(toks):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": ended})
    return steps


def peak_tokens(steps: list[dict], page_size: int) -> int:
    held, peak = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // page_size) * page_size for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak
