"""Attention over a cached latent: keys and values of all heads are made of one low-rank vector per token, and only
that vector (with an optional rotated key part that all heads share) is stored."""
from __future__ import annotations

import torch

from ..native import ops
from .base import MIXERS, CacheView, PagedKVNeed, ParamSpec, Part


@MIXERS.register("latent_attention")
class LatentAttention(Part):
    """Causal softmax attention whose keys and values come from a latent:

        c_q = rmsnorm(W_dq x),  q_h = W_uq,h c_q = [q_h' (``head_dim``) | q_h'' (``rot_dim``, turned by position)]
        c = rmsnorm(first ``kv_rank`` rows of W_dkv x),  r = the last ``rot_dim`` rows, turned by position
        k_h = [W_uk,h c | r],  v_h = W_uv,h c,  score = (q_h . k_h) * scale,  out = W_o [g_h softmax(score) v_h]_h

    with g_h = sigmoid(W_g x)_h if ``gated``. A token stores the row [c | r] and nothing else. The products with
    W_uk and W_uv are moved to the query side, where they are made once per step's token instead of once per key:
    q_h . k_h = (W_uk,h^T q_h') . c + q_h'' . r, and sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j. So attention runs
    with one key/value head whose key is the stored row and whose value is the same row (``values_in_keys``); of the
    result the first ``kv_rank`` entries go through W_uv,h. Pairs (2i, 2i + 1) of the rotated part turn by position *
    frequency i of ``position`` (an encoding that gives ``frequencies()`` and ``gain()``).
    ``own_kv`` False: the layer has no W_dkv and reads the rows of the run-order entry it borrows from, with W_uk,
    W_uv, queries and output of its own; ``pad_dim``: entries of the lender's rows beyond this layer's ``kv_rank``
    (they meet zeros in the queries)."""

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, q_rank: int,
                 kv_rank: int, scale: float, eps: float, gated: bool = False, own_kv: bool = True, pad_dim: int = 0,
                 position=None):
        if min(hidden_size, num_heads, head_dim, value_dim, q_rank, kv_rank) <= 0 or rot_dim < 0 or rot_dim % 2 or pad_dim < 0:
            raise ValueError("sizes must be positive, the rotated part even and not negative")
        if rot_dim and (position is None or not hasattr(position, "frequencies") or position.rotary_dim != rot_dim):
            raise ValueError(f"a rotated part of {rot_dim} entries needs a position encoding of that many frequencies")
        if not own_kv and rot_dim:
            raise ValueError("a layer that borrows its latent has no rotated key part of its own")
        self.hidden_size, self.num_heads, self.head_dim, self.rot_dim = hidden_size, num_heads, head_dim, rot_dim
        self.value_dim, self.q_rank, self.kv_rank, self.scale, self.eps = value_dim, q_rank, kv_rank, scale, eps
        self.gated, self.own_kv, self.pad_dim, self.position = gated, own_kv, pad_dim, position
        self.row = kv_rank + rot_dim + pad_dim                    # what a token stores
        # rows of the packed down projection: query latent | latent and rotated key part | gates
        self.kv_off = q_rank
        self.gate_off = q_rank + (kv_rank + rot_dim if own_kv else 0)
        self.down_rows = self.gate_off + (num_heads if gated else 0)

    def param_specs(self):
        H = self.num_heads
        specs = {"down.weight": ParamSpec((self.down_rows, self.hidden_size)),
                 "q_norm.weight": ParamSpec((self.q_rank,), init="norm", always_float32=True),
                 "uq.weight": ParamSpec((H * (self.head_dim + self.rot_dim), self.q_rank)),
                 "uk.weight": ParamSpec((H * self.head_dim, self.kv_rank)),
                 "uv.weight": ParamSpec((H * self.value_dim, self.kv_rank)),
                 "o.weight": ParamSpec((self.hidden_size, H * self.value_dim))}
        if self.own_kv:
            specs["kv_norm.weight"] = ParamSpec((self.kv_rank,), init="norm", always_float32=True)
        return specs

    def bind(self, params):
        self.down_weight, self.q_norm_weight = params["down.weight"], params["q_norm.weight"]
        self.uq_weight, self.uk_weight, self.uv_weight = params["uq.weight"], params["uk.weight"], params["uv.weight"]
        self.o_weight, self.kv_norm_weight = params["o.weight"], params.get("kv_norm.weight")

    def cache_need(self):
        return PagedKVNeed(1, self.row, None, values_in_keys=True)

    def forward(self, x, step, cache: CacheView):
        if not self.own_kv and cache.writes:
            raise ValueError("a latent attention layer without a latent of its own must borrow another entry's cache")
        tables = step.groups[cache.group]
        T, H, D, R = x.shape[0], self.num_heads, self.head_dim, self.rot_dim
        writes = self.own_kv and cache.writes
        freqs = self.position.frequencies() if R else None
        gain = self.position.gain() if R else 1.0
        a = ops.linear(x, self.down_weight, out_dtype=torch.float32)
        c_q = ops.latent_prepare(a, 0, self.q_rank, self.kv_off, self.kv_rank, R, self.q_norm_weight, self.kv_norm_weight,
                                 self.eps, freqs, gain, step.token_positions, tables.slot_mapping if writes else None,
                                 cache.k if writes else None, x.dtype)
        q = ops.linear(c_q, self.uq_weight).view(T, H, D + R)
        # the query as the stored rows see it: [W_uk,h^T q_h' | q_h'' turned | zeros]
        make = torch.zeros if self.pad_dim else torch.empty
        q_row = make((T, H, self.row), dtype=x.dtype, device=x.device)
        ops.head_gemm(q, self.uk_weight, True, self.kv_rank, D, out=q_row,
                      turn=(R, D, self.kv_rank, freqs, gain, step.token_positions) if R else None)
        mixed = ops.paged_attention(q_row, cache.k, cache.k, step.attention, tables.block_tables, self.scale)
        o = ops.head_gemm(mixed, self.uv_weight, False, self.value_dim, self.kv_rank,
                          gate=a if self.gated else None, gate_off=self.gate_off)
        return ops.linear(o.view(T, H * self.value_dim), self.o_weight)
