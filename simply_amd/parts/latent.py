"""Attention through latents: what is kept per token is one row for all heads.

The mixer's input goes down to a query latent c_q = norm(W_dq h) and to [c | r] = W_dkv h, where c (normed) is the
key/value latent and r (rotated) one key part that all heads share.  Head h has the query [q_h | s_h] = W_uq c_q (s_h
rotated), the key [W_uk,h c | r] and the value W_uv,h c.  Since q_h . (W_uk,h c) = (W_uk,h^T q_h) . c and
sum_j p_j W_uv,h c_j = W_uv,h sum_j p_j c_j, the products with W_uk and W_uv move to the queries and to the result:
attention runs with one key head whose rows are [c | r], the values are the rows' first entries, and only those
rows are cached: once as key rows and, because the matrix cores want the keys of a value entry side by side, the
latent once more transposed, as value pages.
"""
from __future__ import annotations

import torch

from ..config.spec import PartSpec
from ..kernels import ops
from ..registry import MIXERS, POSITION_ENCODINGS
from .base import Mixer, PagedKVNeed, ParamSpec, as_product_weight


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    """Sizes: per head `key_dim` unrotated and `rot_dim` rotated query/key entries and `value_dim` values; latents of
    `q_rank` and `kv_rank` entries, each normed with a weight.  `scale` is the scores' factor as it is.
    `output_gate`: head h's result is multiplied by sigmoid(W_g h)_h, one number per head, read from the mixer's
    input.  `position_encoding`: 'pair_rope' over the rot_dim part."""

    defers_sum = True

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, rot_dim: int, value_dim: int, q_rank: int,
                 kv_rank: int, scale: float, norm_eps: float, window: int | None = None, output_gate: bool = False,
                 position_encoding: PartSpec | None = None):
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.key_dim, self.rot_dim, self.value_dim = int(key_dim), int(rot_dim), int(value_dim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.scale, self.norm_eps, self.output_gate = float(scale), float(norm_eps), bool(output_gate)
        self.window = int(window) if window else None
        self.position_encoding = (POSITION_ENCODINGS.build(position_encoding.kind, **position_encoding.params)
                                  if position_encoding is not None else None)
        pe = self.position_encoding
        if pe is not None and not hasattr(pe, "mult"):
            raise ValueError("latent_attention: the position encoding must rotate neighbouring pairs (pair_rope)")
        if pe is not None and pe.dims > self.rot_dim:
            raise ValueError(f"latent_attention: {pe.dims} rotated entries in a part of {self.rot_dim}")
        self.in_proj = self.uq_proj = self.o_proj = self.uk_t = self.uv = self.dq_norm = self.dkv_norm = None

    def param_specs(self):
        D, H, dk, dr, dv, Rq, R = (self.hidden_size, self.num_heads, self.key_dim, self.rot_dim, self.value_dim,
                                   self.q_rank, self.kv_rank)
        specs = {"dq_proj": ParamSpec((Rq, D)), "dq_norm": ParamSpec((Rq,), role="vector", init="norm"),
                 "uq_proj": ParamSpec((H * (dk + dr), Rq)), "dkv_proj": ParamSpec((R + dr, D)),
                 "dkv_norm": ParamSpec((R,), role="vector", init="norm"), "uk_proj": ParamSpec((H * dk, R)),
                 "uv_proj": ParamSpec((H * dv, R)), "o_proj": ParamSpec((D, H * dv))}
        if self.output_gate:
            specs["gate_proj"] = ParamSpec((H, D))
        return specs

    def load(self, tensors):
        t = tensors
        H, dk, dv, R = self.num_heads, self.key_dim, self.value_dim, self.kv_rank
        rows = [t["dq_proj"], t["dkv_proj"]] + ([t["gate_proj"]] if self.output_gate else [])
        self.in_proj = as_product_weight(torch.cat(rows, dim=0).contiguous())   # rows [c_q | c | r | gates]
        self.uq_proj = as_product_weight(t["uq_proj"])
        self.o_proj = as_product_weight(t["o_proj"])
        # per head: [kv_rank, key_dim] (W_uk,h transposed: queries go up to the latent) and [value_dim, kv_rank]
        self.uk_t = t["uk_proj"].reshape(H, dk, R).transpose(1, 2).contiguous()
        self.uv = t["uv_proj"].reshape(H, dv, R).contiguous()
        self.dq_norm, self.dkv_norm = t["dq_norm"].contiguous(), t["dkv_norm"].contiguous()
        if self.position_encoding is not None:
            self.position_encoding.to_device(t["o_proj"].device)

    def cache_need(self):
        return PagedKVNeed(1, self.kv_rank + self.rot_dim, self.window, self.kv_rank)

    def forward(self, x, ctx, cache, defer_sum=False):
        H, dk, dr, dv, Rq, R = self.num_heads, self.key_dim, self.rot_dim, self.value_dim, self.q_rank, self.kv_rank
        group = ctx.groups[cache.group_id]
        pe = self.position_encoding
        freq, rot_dims = pe.frequencies() if pe is not None else (None, 0)
        mult = pe.mult if pe is not None else 1.0
        proj = ops.gemm(x, self.in_proj)
        cq = ops.rmsnorm(proj[:, :Rq], self.dq_norm, self.norm_eps, False, ctx.dtype)
        q = ops.gemm(cq, self.uq_proj)                                       # [T, H * (dk + dr)]
        qa = ops.head_product(q, self.uk_t, in_stride=dk + dr, tail=dr)      # [T, H * (R + dr)]: [W_uk^T q | s]
        ops.norm_rope_cache_write(qa, ctx.positions, freq, rot_dims, H, 0, R + dr, 0, rot_mult=mult, q_rot_at=R)
        if cache.write:
            # the token's row [norm(c) | rotated r] into the pages
            ops.norm_rope_cache_write(proj[:, Rq:Rq + R + dr], ctx.positions, freq, rot_dims, 0, 1, R + dr, 0,
                                      rot_mult=mult, eps=self.norm_eps, k_weight=self.dkv_norm, k_norm_dims=R,
                                      k_rot_at=R, slot_mapping=group.slot_mapping, k_pages=cache.k_pages,
                                      v_pages=cache.v_pages, key_values=R)
        if ops.attention_maps_units_takes(qa, cache.k_pages, cache.v_pages, H):
            # bfloat16 at sizes that the matrix cores take: units of 16 rows (heads times tokens), keys cut into ranges
            units, few, many, max_q = ctx.attention_units(16 // ops.attention_maps_heads_per_unit(H, 1))
            o = ops.paged_attention_maps_units(qa, cache.k_pages, cache.v_pages, group.block_table, units, 0, few + many,
                                               H, scale=self.scale, window=self.window, max_kv_len=ctx.max_kv_len,
                                               max_q_len=max_q)
        else:
            o = ops.paged_attention_maps(qa, cache.k_pages, cache.v_pages, group.block_table, ctx.token_seq,
                                         ctx.positions, H, scale=self.scale, window=self.window)     # [T, H * R]
        g_at = Rq + R + dr
        o = ops.head_product(o, self.uv, gate=proj[:, g_at:g_at + H] if self.output_gate else None)   # [T, H * dv]
        return ops.gemm(o, self.o_proj, defer_sum=defer_sum)
