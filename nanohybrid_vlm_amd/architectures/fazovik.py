"""The Fazovik decoder as a recipe of parts.

config.json: {"architecture": "Fazovik", "vocab", "width", "norm": {"eps"}, "embedding": {"bigram": {"buckets",
"mul_prev", "mul_cur"}}, "layers": [...]}. Every entry of ``layers`` has a ``type``, the sizes of its mixer
(``mixer``) and its feed-forward (``mlp``, or null):

* ``latent_attention``: attention over a cached latent with a rotated part: ``heads``, ``dim`` (unrotated entries of
  a query/key head), ``rot_dim`` (rotated entries, one key part for all heads), ``vdim``, ``q_rank``, ``kv_rank``,
  ``scale``, ``rot`` = {"base", "dims", "scaling": {"factor", "original", "fast", "slow"} or absent}; an output
  gate per head.
* ``latent_attention_2``: the same without positions and without the gate; with ``kv_from: j`` the layer has no
  latent of its own and reads what layer j stores.
* ``mlp``: {"kind": "dense", "ff"} (gate passed through the tanh form of GELU) or {"kind": "moe", "expert": {"ff"},
  "router": {"experts", "top"}} (sigmoid scores that multiply the experts' inputs; SiLU inside the experts).

Every layer is x <- x + mixer(norm1(x)) + mlp(norm2(x)) with layer norms (weight and bias); the embedding adds a row
of a second table chosen by a hash of the previous and the current token; the head is the embedding table.

Nothing here computes: ``parse_config`` checks and types the keys, ``build_spec`` turns them into a ``ModelSpec``,
``checkpoint_names`` places the stored tensors in the model's (packed) parameters.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from ..config.model_config import ConfigError, require
from ..config.registry import Architecture, WeightSource, register_architecture
from ..parts.model import LayerSpec, ModelSpec, RunEntry

# positions are int32 in a step; the kernels take angles in double
MAX_POSITION = 1 << 24


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    factor: float | None = None
    original: float | None = None
    fast: float | None = None
    slow: float | None = None


@dataclass(frozen=True)
class LatentSizes:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    gated: bool
    rot: Rotation | None = None
    kv_from: int | None = None


@dataclass(frozen=True)
class FeedForwardSizes:
    kind: str                       # "dense" | "moe"
    ff: int
    experts: int = 0
    top: int = 0


@dataclass(frozen=True)
class LayerSizes:
    type: str
    mixer: LatentSizes
    mlp: FeedForwardSizes | None
    spare_norm: bool = False        # a layer without feed-forward whose checkpoint stores a second norm all the same


@dataclass(frozen=True)
class PairTable:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class FazovikConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple
    pair: PairTable | None
    max_position: int = MAX_POSITION
    raw: dict = field(default_factory=dict, compare=False, repr=False)


def _where(i: int, key: str) -> str:
    return f"config.json: layers[{i}].{key}"


def _rotation(i: int, m: dict, rot_dim: int) -> Rotation:
    rot = m.get("rot")
    if not isinstance(rot, dict):
        raise ConfigError(f"{_where(i, 'mixer.rot')} is missing")
    dims = require(rot, "dims")
    if dims != rot_dim or dims % 2 or dims <= 0:
        raise ConfigError(f"{_where(i, 'mixer.rot.dims')}: {dims} must be even, positive and equal to rot_dim {rot_dim}")
    base = require(rot, "base", float)
    if not base > 1:
        raise ConfigError(f"{_where(i, 'mixer.rot.base')} must be larger than 1")
    s = rot.get("scaling")
    if s is None:
        return Rotation(dims, base)
    r = Rotation(dims, base, require(s, "factor", float), require(s, "original", float), require(s, "fast", float),
                 require(s, "slow", float))
    if not (r.factor > 0 and r.original > 0 and r.fast > 0 and r.slow > 0):
        raise ConfigError(f"{_where(i, 'mixer.rot.scaling')}: factor, original, fast and slow must be positive")
    return r


def _mixer(i: int, kind: str, m: dict, layers: list) -> LatentSizes:
    rotary = kind == "latent_attention"
    rot_dim = require(m, "rot_dim") if rotary else int(m.get("rot_dim") or 0)
    if not rotary and rot_dim:
        raise ConfigError(f"{_where(i, 'mixer.rot_dim')}: a layer of type '{kind}' has no rotated part")
    kv_from = m.get("kv_from")
    if kv_from is not None:
        if rotary:
            raise ConfigError(f"{_where(i, 'mixer.kv_from')}: only layers of type 'latent_attention_2' borrow a latent")
        kv_from = require(m, "kv_from")
    a = LatentSizes(heads=require(m, "heads"), dim=require(m, "dim"), rot_dim=rot_dim, vdim=require(m, "vdim"),
                    q_rank=require(m, "q_rank"), kv_rank=require(m, "kv_rank"), scale=require(m, "scale", float),
                    gated=rotary, rot=_rotation(i, m, rot_dim) if rotary else None, kv_from=kv_from)
    if min(a.heads, a.dim, a.vdim, a.q_rank, a.kv_rank) <= 0:
        raise ConfigError(f"{_where(i, 'mixer')}: sizes must be positive")
    if kv_from is not None:
        if not 0 <= kv_from < i or layers[kv_from].mixer.kv_from is not None:
            raise ConfigError(f"{_where(i, 'mixer.kv_from')}: {kv_from} must name an earlier layer with a latent of its own")
        if layers[kv_from].mixer.kv_rank != a.kv_rank:
            raise ConfigError(f"{_where(i, 'mixer.kv_rank')}: {a.kv_rank} must equal that of layer {kv_from}, whose latent "
                              f"it reads ({layers[kv_from].mixer.kv_rank})")
    return a


def _feed_forward(i: int, mlp) -> FeedForwardSizes | None:
    if mlp is None:
        return None
    if not isinstance(mlp, dict):
        raise ConfigError(f"{_where(i, 'mlp')} must be an object or null")
    kind = mlp.get("kind")
    if kind == "dense":
        f = FeedForwardSizes("dense", require(mlp, "ff"))
    elif kind == "moe":
        expert, router = mlp.get("expert"), mlp.get("router")
        if not isinstance(expert, dict) or not isinstance(router, dict):
            raise ConfigError(f"{_where(i, 'mlp')}: 'expert' and 'router' are needed")
        f = FeedForwardSizes("moe", require(expert, "ff"), require(router, "experts"), require(router, "top"))
        if not 0 < f.top <= f.experts:
            raise ConfigError(f"{_where(i, 'mlp.router')}: top {f.top} of {f.experts} experts")
    else:
        raise ConfigError(f"{_where(i, 'mlp.kind')}: {kind!r} is not known ('dense' and 'moe' are)")
    if f.ff <= 0:
        raise ConfigError(f"{_where(i, 'mlp')}: the inner size must be positive")
    return f


def parse_config(raw: dict, shapes: dict | None = None) -> FazovikConfig:
    """``shapes``: {stored tensor name: shape} of the checkpoint where there is one: a layer without feed-forward may
    or may not store its second norm, and only the stored names tell."""
    eps = require(raw.get("norm") or {}, "eps", float)
    if not eps > 0:
        raise ConfigError("config.json: norm.eps must be positive")
    entries = raw.get("layers")
    if not isinstance(entries, list) or not entries:
        raise ConfigError("config.json: 'layers' must be a list with at least one layer")
    layers: list[LayerSizes] = []
    for i, entry in enumerate(entries):
        kind, m = entry.get("type"), entry.get("mixer")
        if kind not in ("latent_attention", "latent_attention_2"):
            raise ConfigError(f"{_where(i, 'type')}: {kind!r} is not known ('latent_attention' and 'latent_attention_2' are)")
        if not isinstance(m, dict):
            raise ConfigError(f"{_where(i, 'mixer')} is missing")
        mlp = _feed_forward(i, entry.get("mlp"))
        spare = mlp is None and shapes is not None and f"l{i}.norm2" in shapes
        layers.append(LayerSizes(kind, _mixer(i, kind, m, layers), mlp, spare))
    pair = None
    bigram = (raw.get("embedding") or {}).get("bigram")
    if bigram is not None:
        pair = PairTable(require(bigram, "buckets"), require(bigram, "mul_prev"), require(bigram, "mul_cur"))
        if pair.buckets <= 0:
            raise ConfigError("config.json: embedding.bigram.buckets must be positive")
    cfg = FazovikConfig(vocab=require(raw, "vocab"), width=require(raw, "width"), eps=eps, layers=tuple(layers), pair=pair,
                        max_position=min(int(raw.get("max_position") or MAX_POSITION), MAX_POSITION), raw=dict(raw))
    if cfg.vocab <= 0 or cfg.width <= 0:
        raise ConfigError("config.json: 'vocab' and 'width' must be positive")
    return cfg


def build_spec(cfg: FazovikConfig) -> ModelSpec:
    norm = {"kind": "layernorm", "size": cfg.width, "eps": cfg.eps}
    layers, positions, order = [], {}, []
    for i, layer in enumerate(cfg.layers):
        a = layer.mixer
        position = None
        if a.rot is not None:
            position = f"l{i}"
            positions[position] = {"kind": "yarn_frequencies", "rotary_dim": a.rot.dims, "base": a.rot.base,
                                   "factor": a.rot.factor, "original": a.rot.original, "fast": a.rot.fast, "slow": a.rot.slow}
        # a borrower's queries meet zeros where the lender's rows hold its rotated part
        pad = cfg.layers[a.kv_from].mixer.rot_dim if a.kv_from is not None else 0
        mixer = {"kind": "latent_attention", "hidden_size": cfg.width, "num_heads": a.heads, "head_dim": a.dim,
                 "rot_dim": a.rot_dim, "value_dim": a.vdim, "q_rank": a.q_rank, "kv_rank": a.kv_rank, "scale": a.scale,
                 "eps": cfg.eps, "gated": a.gated, "own_kv": a.kv_from is None, "pad_dim": pad}
        f = layer.mlp
        if f is None:
            ff = None
        elif f.kind == "dense":
            ff = {"kind": "swiglu", "hidden_size": cfg.width, "intermediate_size": f.ff, "activation": "gelu_tanh"}
        else:
            ff = {"kind": "routed_experts", "hidden_size": cfg.width, "num_experts": f.experts, "top": f.top,
                  "expert_size": f.ff, "activation": "silu"}
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm=norm, position=position,
                                block={"kind": "parallel_two_norms", "keeps_unused_norm": layer.spare_norm}))
        order.append(RunEntry(i, cache=a.kv_from))
    embedding = None
    if cfg.pair is not None:
        embedding = {"kind": "hashed_pair", "hidden_size": cfg.width, "buckets": cfg.pair.buckets,
                     "mul_prev": cfg.pair.mul_prev, "mul_cur": cfg.pair.mul_cur}
    return ModelSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, layers=layers, final_norm=norm, positions=positions,
                     max_position=cfg.max_position, tie_embeddings=True, run_order=order, embedding=embedding)


def checkpoint_names(cfg: FazovikConfig) -> dict[str, WeightSource]:
    names = {"embed": WeightSource("embed.weight"), "final.norm": WeightSource("final_norm.weight"),
             "final.norm.b": WeightSource("final_norm.bias")}
    if cfg.pair is not None:
        names["bigram"] = WeightSource("embedding.pair.weight")
    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[src + "norm1"] = WeightSource(dst + "mixer_norm.weight")
        names[src + "norm1.b"] = WeightSource(dst + "mixer_norm.bias")
        a = layer.mixer
        ms, md = src + "mix.", dst + "mixer."
        names[ms + "dq"] = WeightSource(md + "down.weight", 0, a.q_rank)
        names[ms + "dq.norm"] = WeightSource(md + "q_norm.weight")
        row = a.q_rank
        if a.kv_from is None:
            names[ms + "dkv"] = WeightSource(md + "down.weight", row, a.kv_rank + a.rot_dim)
            names[ms + "dkv.norm"] = WeightSource(md + "kv_norm.weight")
            row += a.kv_rank + a.rot_dim
        if a.gated:
            names[ms + "g"] = WeightSource(md + "down.weight", row, a.heads)
        for name in ("uq", "uk", "uv", "o"):
            names[ms + name] = WeightSource(md + name + ".weight")
        f = layer.mlp
        if f is not None or layer.spare_norm:
            names[src + "norm2"] = WeightSource(dst + "feed_forward_norm.weight")
            names[src + "norm2.b"] = WeightSource(dst + "feed_forward_norm.bias")
        if f is None:
            continue
        fs, fd = src + "mlp.", dst + "feed_forward."
        if f.kind == "dense":
            names[fs + "gate"] = WeightSource(fd + "gate_up.weight", 0, f.ff)
            names[fs + "up"] = WeightSource(fd + "gate_up.weight", f.ff, f.ff)
            names[fs + "down"] = WeightSource(fd + "down.weight")
        else:
            names[fs + "router"] = WeightSource(fd + "router.weight")
            for e in range(f.experts):
                names[fs + f"e{e}.gate"] = WeightSource(fd + "gate_up.weight", e * 2 * f.ff, f.ff)
                names[fs + f"e{e}.up"] = WeightSource(fd + "gate_up.weight", e * 2 * f.ff + f.ff, f.ff)
                names[fs + f"e{e}.down"] = WeightSource(fd + "down.weight", e * cfg.width, cfg.width)
    return names


def _shape(layers: int, width: int, vocab: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int, kv_rank: int,
           ff: int, experts: int, top: int, expert_ff: int, buckets: int) -> dict:
    """Rotary latent layers with dense and routed feed-forwards in turn; every fourth layer has no positions, and
    the second of those reads the latent of the first."""
    entries, plain = [], []
    for i in range(layers):
        mlp = ({"kind": "dense", "ff": ff} if i % 2 == 0 else
               {"kind": "moe", "expert": {"ff": expert_ff}, "router": {"experts": experts, "top": top}})
        if i % 4 == 3:
            mixer = {"dim": dim + rot_dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank,
                     "scale": (dim + rot_dim) ** -0.5, "vdim": vdim}
            if plain:
                mixer["kv_from"] = plain[0]
            plain.append(i)
            entries.append({"type": "latent_attention_2", "mixer": mixer, "mlp": mlp})
        else:
            rot = {"base": 10000.0, "dims": rot_dim, "scaling": {"factor": 4.0, "fast": 32.0, "original": 4096, "slow": 1.0}}
            entries.append({"type": "latent_attention", "mlp": mlp,
                            "mixer": {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot": rot,
                                      "rot_dim": rot_dim, "scale": (dim + rot_dim) ** -0.5, "vdim": vdim}})
    return {"architecture": "Fazovik", "embedding": {"bigram": {"buckets": buckets, "mul_cur": 5, "mul_prev": 13}},
            "layers": entries, "norm": {"eps": 1e-5}, "vocab": vocab, "width": width}


# config.json contents of sizes that measurements and examples name; the engine takes every size from a config.json
SHAPES = {
    "fazovik-tiny": _shape(8, 64, 197, 3, 16, 8, 16, 24, 24, 96, 4, 2, 32, 61),
    "fazovik-1b": _shape(16, 2048, 32768, 16, 128, 64, 128, 768, 192, 6144, 16, 2, 1536, 65521),
    "fazovik-8b": _shape(36, 4096, 151936, 32, 128, 64, 128, 1536, 192, 12288, 32, 4, 1536, 262139),
    # stored rows of 512 entries: more than the matrix-core attention kernels take (256), so attention is the plain kernel's
    "fazovik-8b-wide": _shape(36, 4096, 151936, 32, 128, 64, 128, 1536, 448, 12288, 32, 4, 1536, 262139),
}


FAZOVIK = Architecture(
    name="Fazovik",
    model_types=("fazovik",),
    parse_config=parse_config,
    build_spec=build_spec,
    checkpoint_names=checkpoint_names,
    named_shapes=SHAPES,
    reads_checkpoint_shapes=True,
)
register_architecture(FAZOVIK, replace=True)
