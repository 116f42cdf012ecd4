"""The Pevazen decoder as a recipe of parts.

config.json: {"architecture": "Pevazen", "vocab", "width", "norm": {"eps"}, "layers": [...]}. Every entry of
``layers`` has a ``type``, the sizes of its mixer (``mixer``) and its feed-forward (``mlp``: {"kind": "dense", "ff"} or
null):

* ``attention``: softmax attention with biases on q, k, v, rotation of the first ``rot.dims`` coordinates of every
  query and key head (``rot.base``, optionally ``rot.scaling.factor``), a chunk mask of ``mask.size`` positions,
  ``scale``, value heads of size ``vdim``; with ``kv_from: j`` the layer has no key and value projections and reads
  the cache of layer j.
* ``parallel``: two mixers side by side (``left``: such an attention without biases whose values are turned by
  their position and whose results are turned back; ``right``: a gated delta rule with short convolutions of
  ``conv`` taps), each result normed, half their sum.

Every layer is one norm (a single number as its weight), mixer and feed-forward side by side on its output, and a
weighted sum over the results of all layers so far (``l<i>.dwa``). The embedding's rows pass a norm of the same kind
before the first layer. Two sizes stand in no key of config.json and are read from the shapes of the stored tensors:
the inner sizes of the recurrent mixer's two low-rank projections (``l<i>.mix.right.a1``, ``.g1``); a config.json
written for random weights names them itself (``decay_rank``, ``gate_rank`` beside the mixer's other sizes).

Nothing here computes: ``parse_config`` checks and types the keys, ``build_spec`` turns them into a ``ModelSpec``,
``checkpoint_names`` places the stored tensors in the model's (packed) parameters.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from ..config.model_config import ConfigError, require
from ..config.registry import Architecture, WeightSource, register_architecture
from ..parts.model import LayerSpec, ModelSpec, RunEntry

# positions are counted in float32 by the kernels that turn queries and keys: every integer up to here is exact
MAX_POSITION = 1 << 24


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int
    rot_dims: int
    rot_base: float
    rot_factor: float | None = None
    kv_from: int | None = None


@dataclass(frozen=True)
class DeltaSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int
    gate_rank: int


@dataclass(frozen=True)
class LayerSizes:
    type: str                               # "attention" | "parallel"
    attention: AttentionSizes               # the attention mixer, or the left one of a pair
    delta: DeltaSizes | None = None         # the right one of a pair
    ff: int | None = None                   # inner size of the feed-forward; None: the layer has none


@dataclass(frozen=True)
class PevazenConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple
    max_position: int = MAX_POSITION
    raw: dict = field(default_factory=dict, compare=False, repr=False)


def _where(i: int, key: str) -> str:
    return f"config.json: layers[{i}].{key}"


def _attention(i: int, m: dict, where: str, borrows: bool) -> AttentionSizes:
    for key in ("mask", "rot"):
        if not isinstance(m.get(key), dict):
            raise ConfigError(f"{_where(i, where)}: '{key}' is missing")
    scaling = m["rot"].get("scaling")
    factor = None
    if scaling is not None:
        factor = require(scaling, "factor", float)
        if not factor > 0:
            raise ConfigError(f"{_where(i, where)}: rot.scaling.factor must be positive")
    a = AttentionSizes(heads=require(m, "heads"), kv_heads=require(m, "kv_heads"), dim=require(m, "dim"),
                       vdim=require(m, "vdim"), scale=require(m, "scale", float), chunk=require(m["mask"], "size"),
                       rot_dims=require(m["rot"], "dims"), rot_base=require(m["rot"], "base", float), rot_factor=factor,
                       kv_from=require(m, "kv_from") if borrows else None)
    if min(a.heads, a.kv_heads, a.dim, a.vdim, a.chunk) <= 0 or a.heads % a.kv_heads:
        raise ConfigError(f"{_where(i, where)}: sizes must be positive and heads a multiple of kv_heads")
    if a.rot_dims < 0 or a.rot_dims % 2 or a.rot_dims > a.dim:
        raise ConfigError(f"{_where(i, where)}: rot.dims {a.rot_dims} must be even and at most dim {a.dim}")
    return a


def parse_config(raw: dict, shapes: dict | None = None) -> PevazenConfig:
    """``shapes``: {stored tensor name: shape} of the checkpoint, for the sizes that config.json does not name."""
    eps = require(raw.get("norm") or {}, "eps", float)
    if not eps > 0:
        raise ConfigError("config.json: norm.eps must be positive")
    entries = raw.get("layers")
    if not isinstance(entries, list) or not entries:
        raise ConfigError("config.json: 'layers' must be a list with at least one layer")
    width = require(raw, "width")
    layers = []
    for i, entry in enumerate(entries):
        kind, m = entry.get("type"), entry.get("mixer")
        if not isinstance(m, dict):
            raise ConfigError(f"{_where(i, 'mixer')} is missing")
        mlp = entry.get("mlp")
        ff = None
        if mlp is not None:
            if mlp.get("kind") != "dense":
                raise ConfigError(f"{_where(i, 'mlp.kind')}: {mlp.get('kind')!r} is not known ('dense' is)")
            ff = require(mlp, "ff")
        if kind == "attention":
            a = _attention(i, m, "mixer", "kv_from" in m)
            if a.kv_from is not None:
                j = a.kv_from
                if not 0 <= j < i or layers[j].type != "attention" or layers[j].attention.kv_from is not None:
                    raise ConfigError(f"{_where(i, 'mixer.kv_from')}: {j} must name an earlier attention layer with keys and "
                                      f"values of its own")
                b = layers[j].attention
                if (a.kv_heads, a.dim, a.vdim, a.rot_dims, a.rot_base, a.rot_factor) != \
                        (b.kv_heads, b.dim, b.vdim, b.rot_dims, b.rot_base, b.rot_factor):
                    raise ConfigError(f"{_where(i, 'mixer')}: head sizes and rotation must equal those of layer {j}, whose "
                                      f"keys and values it reads")
            layers.append(LayerSizes("attention", a, None, ff))
        elif kind == "parallel":
            if not isinstance(m.get("left"), dict) or not isinstance(m.get("right"), dict):
                raise ConfigError(f"{_where(i, 'mixer')}: 'left' and 'right' are needed")
            a = _attention(i, m["left"], "mixer.left", False)
            if a.vdim % 2:
                raise ConfigError(f"{_where(i, 'mixer.left.vdim')}: values that are turned need an even size")
            r = m["right"]
            ranks = {}
            for key, tensor in (("decay_rank", "a1"), ("gate_rank", "g1")):
                name = f"l{i}.mix.right.{tensor}"
                if key in r:
                    ranks[key] = require(r, key)
                elif shapes is not None and name in shapes and len(shapes[name]) == 2:
                    ranks[key] = int(shapes[name][0])
                else:
                    raise ConfigError(f"{_where(i, 'mixer.right')}: the inner size of '{tensor}' stands neither in "
                                      f"'{key}' nor in a stored tensor '{name}'")
            d = DeltaSizes(heads=require(r, "heads"), kv_heads=require(r, "kv_heads"), dim=require(r, "dim"),
                           vdim=require(r, "vdim"), conv=require(r, "conv"), **ranks)
            if min(d.heads, d.kv_heads, d.dim, d.vdim, d.decay_rank, d.gate_rank) <= 0 or d.heads % d.kv_heads:
                raise ConfigError(f"{_where(i, 'mixer.right')}: sizes must be positive and heads a multiple of kv_heads")
            if not 1 <= d.conv <= 16:
                raise ConfigError(f"{_where(i, 'mixer.right.conv')}: 1 to 16 taps are taken, got {d.conv}")
            layers.append(LayerSizes("parallel", a, d, ff))
        else:
            raise ConfigError(f"{_where(i, 'type')}: {kind!r} is not known ('attention' and 'parallel' are)")
    max_position = int(raw.get("max_position") or MAX_POSITION)
    cfg = PevazenConfig(vocab=require(raw, "vocab"), width=width, eps=eps, layers=tuple(layers),
                        max_position=min(max_position, MAX_POSITION), raw=dict(raw))
    if cfg.vocab <= 0 or cfg.width <= 0:
        raise ConfigError("config.json: 'vocab' and 'width' must be positive")
    return cfg


def _attention_part(cfg: PevazenConfig, a: AttentionSizes, bias: bool, rotate_values: bool) -> dict:
    return {"kind": "rotary_attention", "hidden_size": cfg.width, "num_heads": a.heads, "num_kv_heads": a.kv_heads,
            "head_dim": a.dim, "value_dim": a.vdim, "scale": a.scale, "bias": bias, "chunk": a.chunk,
            "rotate_values": rotate_values, "own_kv": a.kv_from is None}


def build_spec(cfg: PevazenConfig) -> ModelSpec:
    norm = {"kind": "scalar_rmsnorm", "eps": cfg.eps, "output": "rows"}
    layers, positions, order = [], {}, []
    for i, layer in enumerate(cfg.layers):
        a = layer.attention
        positions[f"l{i}"] = {"kind": "rotary_frequencies", "rotary_dim": a.rot_dims, "base": a.rot_base,
                              "scaling_factor": a.rot_factor}
        if layer.type == "attention":
            mixer = _attention_part(cfg, a, bias=True, rotate_values=False)
        else:
            d = layer.delta
            mixer = {"kind": "normed_pair", "hidden_size": cfg.width, "eps": cfg.eps,
                     "left": _attention_part(cfg, a, bias=False, rotate_values=True),
                     "right": {"kind": "gated_delta_rule", "hidden_size": cfg.width, "num_heads": d.heads,
                               "num_kv_heads": d.kv_heads, "head_dim": d.dim, "value_dim": d.vdim, "conv_taps": d.conv,
                               "decay_rank": d.decay_rank, "gate_rank": d.gate_rank, "eps": cfg.eps}}
        ff = None if layer.ff is None else {"kind": "swiglu", "hidden_size": cfg.width, "intermediate_size": layer.ff}
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm=norm, position=f"l{i}",
                                block={"kind": "parallel_depth_mix", "depth_index": i, "depth_total": len(cfg.layers)}))
        order.append(RunEntry(i, cache=a.kv_from))
    return ModelSpec(vocab_size=cfg.vocab, hidden_size=cfg.width, layers=layers, final_norm=norm, positions=positions,
                     max_position=cfg.max_position, tie_embeddings=False, run_order=order,
                     embed_norm={"kind": "scalar_rmsnorm", "eps": cfg.eps, "output": "float32"})


def checkpoint_names(cfg: PevazenConfig) -> dict[str, WeightSource]:
    names = {"embed": WeightSource("embed.weight"), "embed.norm": WeightSource("embed_norm.weight"),
             "final.norm": WeightSource("final_norm.weight"), "head": WeightSource("head.weight")}

    def attention(src: str, dst: str, a: AttentionSizes, bias: bool):
        q, k, v = a.heads * a.dim, a.kv_heads * a.dim, a.kv_heads * a.vdim
        bands = (("q", 0, q),) if a.kv_from is not None else (("q", 0, q), ("k", q, k), ("v", q + k, v))
        for name, start, rows in bands:
            names[src + name] = WeightSource(dst + "qkv.weight", start, rows)
            if bias:
                names[src + name + ".b"] = WeightSource(dst + "qkv.bias", start, rows)
        names[src + "o"] = WeightSource(dst + "o.weight")

    for i, layer in enumerate(cfg.layers):
        src, dst = f"l{i}.", f"layers.{i}."
        names[src + "norm1"] = WeightSource(dst + "norm.weight")
        names[src + "dwa"] = WeightSource(dst + "depth.weight")
        if layer.type == "attention":
            attention(src + "mix.", dst + "mixer.", layer.attention, True)
        else:
            attention(src + "mix.left.", dst + "mixer.left.", layer.attention, False)
            names[src + "mix.left.out"] = WeightSource(dst + "mixer.left_out.weight")
            names[src + "mix.right.out"] = WeightSource(dst + "mixer.right_out.weight")
            d = layer.delta
            rs, rd = src + "mix.right.", dst + "mixer.right."
            qk, v = d.kv_heads * d.dim, d.heads * d.vdim
            for name, start, rows in (("q", 0, qk), ("k", qk, qk), ("v", 2 * qk, v)):
                names[rs + name] = WeightSource(rd + "in.weight", start, rows)
                names[rs + name + ".conv"] = WeightSource(rd + "conv.weight", start, rows)
            names[rs + "b"] = WeightSource(rd + "in.weight", 2 * qk + v, d.heads)
            for name in ("a1", "a2", "g1", "g2", "o"):
                names[rs + name] = WeightSource(rd + name + ".weight")
            names[rs + "dt_bias"] = WeightSource(rd + "dt_bias")
            names[rs + "A_log"] = WeightSource(rd + "A_log")
            names[rs + "norm"] = WeightSource(rd + "norm.weight")
        if layer.ff is not None:
            names[src + "mlp.gate"] = WeightSource(dst + "feed_forward.gate_up.weight", 0, layer.ff)
            names[src + "mlp.up"] = WeightSource(dst + "feed_forward.gate_up.weight", layer.ff, layer.ff)
            names[src + "mlp.down"] = WeightSource(dst + "feed_forward.down.weight")
    return names


def _attention_entry(heads, kv_heads, dim, vdim, chunk, rot_dims, base, factor=None, **more):
    rot = {"base": base, "dims": rot_dims}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    return dict({"dim": dim, "heads": heads, "kv_heads": kv_heads, "mask": {"size": chunk}, "rot": rot,
                 "scale": dim ** -0.5, "vdim": vdim}, **more)


def _shape(layers: int, width: int, ff: int, vocab: int, heads: int, kv_heads: int, dim: int, chunk: int,
           delta_heads: int, delta_dim: int, rank: int) -> dict:
    """A model of alternating parallel and attention layers at the sizes of a real model's layers; every fourth layer
    reads the keys and values of the attention layer two before it."""
    entries = []
    for i in range(layers):
        if i % 2 == 0:
            mixer = {"left": _attention_entry(heads, kv_heads, dim, dim, chunk, dim, 10000.0, 2.0),
                     "right": {"conv": 4, "dim": delta_dim, "heads": delta_heads, "kv_heads": delta_heads, "vdim": delta_dim,
                               "decay_rank": rank, "gate_rank": rank}}
            entries.append({"type": "parallel", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff}})
        else:
            more = {"kv_from": i - 2} if i % 4 == 3 and i >= 3 else {}
            entries.append({"type": "attention", "mixer": _attention_entry(heads, kv_heads, dim, dim, chunk, dim // 2, 500000.0, **more),
                            "mlp": {"kind": "dense", "ff": ff}})
    return {"architecture": "Pevazen", "layers": entries, "norm": {"eps": 1e-6}, "vocab": vocab, "width": width}


# config.json contents of sizes that measurements name; the engine itself takes every size from a config.json
SHAPES = {
    "pevazen-tiny": _shape(4, 64, 128, 211, 4, 2, 16, 24, 3, 16, 8),
    "pevazen-1b": _shape(16, 2048, 6144, 32768, 16, 8, 128, 2048, 16, 128, 128),
    "pevazen-8b": _shape(36, 4096, 12288, 151936, 32, 8, 128, 8192, 32, 128, 256),
}


PEVAZEN = Architecture(
    name="Pevazen",
    model_types=("pevazen",),
    parse_config=parse_config,
    build_spec=build_spec,
    checkpoint_names=checkpoint_names,
    named_shapes=SHAPES,
    reads_checkpoint_shapes=True,
)
register_architecture(PEVAZEN, replace=True)
