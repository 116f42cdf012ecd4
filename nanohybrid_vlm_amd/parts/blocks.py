"""How a layer's norm, mixer and feed-forward are arranged."""
from __future__ import annotations

import torch

from ..native import ops
from .base import BLOCKS, ParamSpec, Part


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    """r += mixer(norm(r)); r += feed_forward(norm(r)), with each addition folded into
    the next norm (nanovllm/models/qwen3.py:152-159): the block takes and returns
    (hidden, residual), and ``residual`` is None before the first block."""

    # the norms this arrangement takes, by the names of its constructor's arguments: the model builds one per slot
    # from the layer's description (``LayerSpec.norms[slot]``, else ``LayerSpec.norm``)
    norm_slots = ("mixer_norm", "feed_forward_norm")

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def children(self):
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer,
                "feed_forward_norm": self.feed_forward_norm, "feed_forward": self.feed_forward}

    @property
    def takes_summed(self) -> bool:
        """Whether ``hidden`` may come as an ``ops.Summed`` (the block before has added it to the residual stream
        already): this block's first norm has to know what that is. A block that says so takes ``next_norm=``."""
        return getattr(self.mixer_norm, "takes_summed", False)

    def forward(self, hidden, residual, step, cache, next_norm=None, next_reader=None):
        """``next_norm``: the norm that takes this block's result next (the next block's first norm, or the model's
        last), if it takes an ``ops.Summed`` in place of ``hidden``; ``next_reader``: the part that reads that norm."""
        # A mixer or feed-forward that says ``adds_to_residual`` takes ``add_to=`` (the residual stream and the norm
        # that follows, ``ops.AddTo``) and may let its last product make the addition (it then returns an
        # ``ops.Summed``); one that says ``takes_deferred_norm`` may get an ``ops.Normed`` as its input, whose rows
        # its first product scales. Parts that say neither get tensors and return tensors.
        mixer, ff = self.mixer, self.feed_forward
        if residual is None:
            x, residual = self.mixer_norm.forward_start(hidden)
        else:
            x, residual = self.mixer_norm.forward_add(hidden, residual, **_deferred(self.mixer_norm, mixer))
        x = mixer.forward(x, step, cache, **_add_to(mixer, self.feed_forward_norm, residual, ff))
        x, residual = self.feed_forward_norm.forward_add(x, residual, **_deferred(self.feed_forward_norm, ff))
        x = ff.forward(x, step, **_add_to(ff, next_norm, residual, next_reader))
        return x, residual


def _deferred(norm, reader) -> dict:
    """The argument that lets ``norm`` hand its scaling on to ``reader``, if both are made for that."""
    both = getattr(norm, "defers_to_products", False) and getattr(reader, "takes_deferred_norm", False)
    return {"deferred": True} if both else {}


def _add_to(part, norm, residual, reader) -> dict:
    """The argument that lets ``part`` make the addition that ``norm`` would make, if both are made for that.
    ``reader``: the part that reads ``norm`` (it counts only if it takes the norm with its scaling left to do)."""
    if norm is not None and getattr(part, "adds_to_residual", False) and getattr(norm, "takes_summed", False):
        return {"add_to": norm.add_to(residual, reader if getattr(reader, "takes_deferred_norm", False) else None)}
    return {}


@BLOCKS.register("parallel_depth_mix")
class ParallelDepthMixBlock(Part):
    """One norm, mixer and feed-forward side by side on its output, and a weighted sum over depth:
        h = norm(x);  X_(i+1) = x + (mixer(h) + feed_forward(h));  x <- sum over j <= i + 1 of w[j] X_j,
    where X_0 is the stream that entered the first such block and i = ``depth_index`` counts the blocks before this
    one. The stream is float32 and is what the block takes and returns as ``hidden`` (there is no residual beside
    it); the results X_j of a step live in ``step.scratch`` ([``depth_total`` + 1, tokens, width] float32). The
    feed-forward may be absent."""

    norm_slots = ("norm",)
    # the sum over depth can norm what it hands on in its own kernel: the model names the next block's norm
    # (``next_norm=``), and that block finds its rows normed already in ``step.scratch``
    norms_ahead = True

    def __init__(self, mixer, feed_forward, norm, depth_index: int, depth_total: int):
        if not 0 <= depth_index < depth_total:
            raise ValueError(f"block {depth_index} of {depth_total}")
        self.mixer, self.feed_forward, self.norm = mixer, feed_forward, norm
        self.depth_index, self.depth_total = depth_index, depth_total
        self.row_dtype = None

    def children(self):
        out = {"norm": self.norm, "mixer": self.mixer}
        if self.feed_forward is not None:
            out["feed_forward"] = self.feed_forward
        return out

    def param_specs(self):
        n = self.depth_index + 2
        return {"depth.weight": ParamSpec((n,), always_float32=True, init_mean=1.0 / n, init_std=0.3 / n)}

    def forward(self, hidden, residual, step, cache, next_norm=None):
        if residual is not None:
            raise ValueError("this block carries its stream itself and takes no residual beside it")
        if hidden.dtype != torch.float32:
            hidden = hidden.float()
        T, W = hidden.shape
        results = step.scratch.get("depth_results")
        if results is None or self.depth_index == 0:
            results = step.scratch["depth_results"] = torch.empty((self.depth_total + 1, T, W), dtype=torch.float32,
                                                                   device=hidden.device)
        ahead = step.scratch.pop("normed_ahead", None)
        if ahead is not None and ahead[0] is self.norm and ahead[1] is hidden:
            h = ahead[2]                                   # the block before has normed this very stream for this norm
        else:
            h = self.norm.forward(hidden, out_dtype=self.row_dtype or torch.float32)
        # (a pair of mixers may leave its two norms and their mean to the sum over depth)
        mixed = self.mixer.forward(h, step, cache, **({"deferred": True} if getattr(self.mixer, "defers_pair_norm", False) else {}))
        fed = self.feed_forward.forward(h, step) if self.feed_forward is not None else None
        weight, eps = getattr(next_norm, "weight", None), getattr(next_norm, "eps", None)
        rows = mixed.a if isinstance(mixed, ops.NormedPairMean) else mixed
        if weight is not None and weight.numel() == 1 and eps is not None and rows.dtype == (self.row_dtype or torch.float32):
            out, normed = ops.depth_mix(hidden, mixed, fed, results, self.depth_index, self.depth_weight, gain=weight, eps=eps)
            step.scratch["normed_ahead"] = (next_norm, out, normed)
            return out, None
        return ops.depth_mix(hidden, mixed, fed, results, self.depth_index, self.depth_weight), None


@BLOCKS.register("parallel_two_norms")
class ParallelTwoNormsBlock(Part):
    """x <- x + (mixer(norm_a(x)) + feed_forward(norm_b(x))): both norms read the same x. The stream x is float32 and is
    what the block takes and returns as ``hidden`` (no residual beside it). The two norms share their mean and
    variance, so one kernel makes both; the additions of a block are left to the kernel that norms for the block after
    it (``pending`` in ``step.scratch``), or made by a kernel of their own after the last block. The feed-forward may
    be absent (then there is no second norm)."""

    norm_slots = ("mixer_norm", "feed_forward_norm")
    norms_ahead = True            # the model tells the block whether a block follows (``next_norm`` is that block's ``norm``)

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, keeps_unused_norm: bool = False):
        """``keeps_unused_norm``: a block without feed-forward holds its second norm's tensors all the same (a
        checkpoint that stores them), unused."""
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm
        self.keeps_unused_norm = bool(keeps_unused_norm)
        if feed_forward is not None and feed_forward_norm.eps != mixer_norm.eps:
            raise ValueError("the two norms of this block share their statistics and so their eps")
        self.row_dtype = None

    @property
    def norm(self):
        """What the block before this one is shown as the norm that takes its result: this block adds what is
        pending itself, in its norms' kernel."""
        return self

    def children(self):
        out = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.feed_forward is not None or self.keeps_unused_norm:
            out["feed_forward_norm"] = self.feed_forward_norm
        if self.feed_forward is not None:
            out["feed_forward"] = self.feed_forward
        return out

    def forward(self, hidden, residual, step, cache, next_norm=None):
        if residual is not None:
            raise ValueError("this block carries its stream itself and takes no residual beside it")
        if hidden.dtype != torch.float32:
            hidden = hidden.float()
        pending = step.scratch.pop("pending_additions", None)
        add = pending[1] if pending is not None and pending[0] is hidden else ()
        dtype = self.row_dtype or torch.float32
        a, b = self.mixer_norm, self.feed_forward_norm
        second = (b.weight, b.bias) if self.feed_forward is not None else None
        h1, h2 = ops.layernorm_pair(hidden, (a.weight, a.bias), second, a.eps, dtype, add=add)
        mixed = self.mixer.forward(h1, step, cache)
        fed = self.feed_forward.forward(h2, step) if self.feed_forward is not None else None
        if isinstance(next_norm, ParallelTwoNormsBlock):
            step.scratch["pending_additions"] = (hidden, (mixed, fed))
        else:
            ops.add_streams_(hidden, mixed, fed)
        return hidden, None
