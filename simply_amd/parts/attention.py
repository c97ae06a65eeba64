"""Grouped-query attention over a paged cache.

simply/model_lib.py:1605 (Attention): q/k/v projections, position encoding on q and k,
q / query_scale (:1987-2020), attention over the cache with soft-cap and window
(simply/utils/ragged_paged_attention.py:870-949), output projection (:2362).
"""
from __future__ import annotations

import functools

import torch

from ..config.spec import PartSpec
from ..kernels import ops
from ..registry import MIXERS, POSITION_ENCODINGS
from .base import Mixer, PagedKVNeed, ParamSpec, as_product_weight, pending_fits_product, pending_product, project


@MIXERS.register("paged_attention")
class PagedAttention(Mixer):
    accepts_pending = True
    defers_sum = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, query_scale: float,
                 soft_cap: float | None = None, window: int | None = None,
                 position_encoding: PartSpec | None = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"paged_attention: {num_heads} heads do not split over {num_kv_heads} kv heads")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.query_scale = float(query_scale)
        self.soft_cap = float(soft_cap) if soft_cap else None
        self.window = int(window) if window else None
        self.position_encoding = (POSITION_ENCODINGS.build(position_encoding.kind, **position_encoding.params)
                                  if position_encoding is not None else None)
        self.qkv_proj: torch.Tensor | None = None
        self.o_proj: torch.Tensor | None = None

    def param_specs(self):
        D, H, K, hd = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        return {"q_proj": ParamSpec((H * hd, D)), "k_proj": ParamSpec((K * hd, D)),
                "v_proj": ParamSpec((K * hd, D)), "o_proj": ParamSpec((D, H * hd))}

    def load(self, tensors):
        # one product for q, k and v: rows [q heads | k heads | v heads]
        device = tensors["o_proj"].device
        self.qkv_proj = as_product_weight(torch.cat([tensors["q_proj"], tensors["k_proj"], tensors["v_proj"]], dim=0)
                                          .contiguous())
        self.o_proj = as_product_weight(tensors["o_proj"])
        if self.position_encoding is not None and hasattr(self.position_encoding, "to_device"):
            self.position_encoding.to_device(device)

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.head_dim, self.window)

    def forward(self, x, ctx, cache, defer_sum=False):
        H, K, hd = self.num_heads, self.num_kv_heads, self.head_dim
        group = ctx.groups[cache.group_id]
        pe = self.position_encoding
        rotary = pe.rotary_table() if pe is not None else None
        write = cache.write
        pages = dict(slot_mapping=group.slot_mapping if write else None, k_pages=cache.k_pages if write else None,
                     v_pages=cache.v_pages if write else None)
        if (pe is None or rotary is not None) and hd % 32 == 0 and pending_fits_product(x, self.qkv_proj) \
                and cache.k_pages.dtype == torch.bfloat16:
            # a few tokens: the norms in front of the projection and the rotation, query scale and cache write
            # behind it run in the projection's kernel
            table, sf = rotary if rotary is not None else (None, 1.0)
            qkv = pending_product(x, functools.partial(
                ops.gemm_normed_rotary, w=self.qkv_proj, positions=ctx.positions, timescale=table, scale_factor=sf,
                query_scale=self.query_scale, num_heads=H, num_kv_heads=K, head_dim=hd, **pages))
        else:
            if pe is None or rotary is not None:
                # (the kernel behind the projection adds up its cuts of K, if it has any, on the way)
                table, sf = rotary if rotary is not None else (None, 1.0)
                qkv = ops.rope_cache_write(project(x, self.qkv_proj, defer_sum=True), ctx.positions, table, sf,
                                           self.query_scale, H, K, hd, **pages)
            else:
                qkv = project(x, self.qkv_proj)
                # another position encoding: applied by the part itself, then the plain scale-and-write kernel
                pe.apply(qkv, ctx.positions, H, hd, 1.0)
                pe.apply(qkv[:, H * hd:], ctx.positions, K, hd, 1.0)
                ops.rope_cache_write(qkv, ctx.positions, None, 1.0, self.query_scale, H, K, hd, **pages)
        o = torch.empty((qkv.shape[0], H * hd), dtype=qkv.dtype, device=qkv.device)
        if ops.decode_attention_takes(qkv, cache.k_pages, H, 1):
            # the MFMA kernels take up to 16 query rows (tokens x heads per key head) as a unit: a decoding request
            # is one unit and its keys are cut over workgroups; portions of prompts are cut into units of 16 / G
            # tokens, of which one workgroup takes four
            units, few, many, max_q = ctx.attention_units(16 // (H // K), ops.prefill_units_per_group())
            kw = dict(window=self.window, soft_cap=self.soft_cap, max_kv_len=ctx.max_kv_len, max_q_len=max_q, out=o)
            if few:
                ops.paged_attention_decode(qkv, cache.k_pages, cache.v_pages, group.block_table, units, 0, few, H, **kw)
            if many:
                ops.paged_attention_prefill(qkv, cache.k_pages, cache.v_pages, group.block_table, units, few, many, H,
                                            **kw)
        else:
            ops.paged_attention(qkv, cache.k_pages, cache.v_pages, group.block_table, ctx.token_seq, ctx.positions, H,
                                window=self.window, soft_cap=self.soft_cap, out=o)
        return ops.gemm(o, self.o_proj, defer_sum=defer_sum)


@MIXERS.register("sink_attention")
class SinkAttention(Mixer):
    """Grouped-query attention over a paged cache whose values have a size of their own, with the options

      position_encoding  'partial_rope' (or None): only the first dimensions of a head are rotated;
      qk_norm_eps        queries and keys are divided by their root mean square after the rotation (None: not);
      scale              the scores' factor;
      sinks              one learned logit per query head that joins every softmax sum and has no value;
      value_mix          'source': the values of the step's tokens are left for later layers under `value_mix_key`;
                         'mix': v <- (1 - vmix) v + vmix (those values), before the cache is written;
      output_gate        the heads are multiplied by sigmoid(gate projection of the mixer's input) before the output
                         projection;
      bias               q, k, v and the output projection have biases.

    q, k, v and the gate are one product."""

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, scale: float,
                 sinks: bool = False, qk_norm_eps: float | None = None, output_gate: bool = False,
                 value_mix: str | None = None, value_mix_key: str = "values", window: int | None = None,
                 position_encoding: PartSpec | None = None, bias: bool = False):
        if num_heads % num_kv_heads:
            raise ValueError(f"sink_attention: {num_heads} heads do not split over {num_kv_heads} kv heads")
        if value_mix not in (None, "source", "mix"):
            raise ValueError(f"sink_attention: value_mix is None, 'source' or 'mix', not {value_mix!r}")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim, self.scale = int(key_dim), int(value_dim), float(scale)
        self.sinks, self.output_gate, self.bias = bool(sinks), bool(output_gate), bool(bias)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.value_mix, self.value_mix_key = value_mix, str(value_mix_key)
        self.window = int(window) if window else None
        self.position_encoding = (POSITION_ENCODINGS.build(position_encoding.kind, **position_encoding.params)
                                  if position_encoding is not None else None)
        if self.position_encoding is not None and not hasattr(self.position_encoding, "frequencies"):
            raise ValueError("sink_attention: the position encoding must give frequencies() (partial_rope)")
        self.in_proj = self.o_proj = self.sink = self.vmix = self.in_bias = self.o_bias = None

    def param_specs(self):
        D, H, K, dk, dv = self.hidden_size, self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        specs = {"q_proj": ParamSpec((H * dk, D)), "k_proj": ParamSpec((K * dk, D)), "v_proj": ParamSpec((K * dv, D)),
                 "o_proj": ParamSpec((D, H * dv))}
        if self.output_gate:
            specs["gate_proj"] = ParamSpec((H * dv, D))
        if self.sinks:
            specs["sink"] = ParamSpec((H,), role="vector", init="norm")
        if self.bias:
            specs.update(q_bias=ParamSpec((H * dk,), role="vector", init="norm"),
                         k_bias=ParamSpec((K * dk,), role="vector", init="norm"),
                         v_bias=ParamSpec((K * dv,), role="vector", init="norm"),
                         o_bias=ParamSpec((D,), role="vector", init="norm"))
        if self.value_mix is not None:   # (a source stores the factor too and leaves it unused)
            specs["vmix"] = ParamSpec((), role="vector", init="norm")
        return specs

    def load(self, tensors):
        rows = [tensors["q_proj"], tensors["k_proj"], tensors["v_proj"]]
        if self.output_gate:
            rows.append(tensors["gate_proj"])
        self.in_proj = as_product_weight(torch.cat(rows, dim=0).contiguous())
        self.o_proj = as_product_weight(tensors["o_proj"])
        if self.bias:
            parts = [tensors["q_bias"], tensors["k_bias"], tensors["v_bias"]]
            if self.output_gate:
                parts.append(torch.zeros_like(tensors["q_bias"][:1]).expand(self.num_heads * self.value_dim))
            self.in_bias = torch.cat([p.to(parts[0].dtype) for p in parts]).contiguous()
            self.o_bias = tensors["o_bias"].contiguous()
        self.sink = tensors["sink"].contiguous() if self.sinks else None
        self.sink_f32 = self.sink.to(torch.float32) if self.sinks else None   # what the MFMA kernels read
        self.vmix = tensors["vmix"].reshape(1).contiguous() if self.value_mix is not None else None
        if self.position_encoding is not None:
            self.position_encoding.to_device(tensors["o_proj"].device)

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, self.key_dim, self.window, self.value_dim)

    def forward(self, x, ctx, cache, defer_sum=False):
        H, K, dk, dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        group = ctx.groups[cache.group_id]
        proj = ops.gemm(x, self.in_proj)
        if self.bias:
            ops.bias_add_(proj, self.in_bias)
        inv_freq, rot_dims = self.position_encoding.frequencies() if self.position_encoding is not None else (None, 0)
        v_at = (H + K) * dk
        v_first = None
        if self.value_mix == "mix":
            v_first = ctx.carry.get(self.value_mix_key)
            if v_first is None:
                raise RuntimeError(f"sink_attention: no earlier layer of the step has left {self.value_mix_key!r}")
        write = cache.write
        # the bfloat16 MFMA kernels take values of the keys' size (64, 128 or 256) in pages of a multiple of 16 keys;
        # they have no factor on the scores, so the queries carry it
        mfma = dk == dv and proj.dtype == torch.bfloat16 and ops.decode_attention_takes(proj, cache.k_pages, H, 1)
        ops.qk_norm_rope_cache_write(proj, ctx.positions, inv_freq, rot_dims, self.qk_norm_eps, H, K, dk, dv,
                                     v_first=v_first, v_mix=self.vmix if v_first is not None else None,
                                     slot_mapping=group.slot_mapping if write else None,
                                     k_pages=cache.k_pages if write else None, v_pages=cache.v_pages if write else None,
                                     q_mult=self.scale if mfma else 1.0)
        if self.value_mix == "source":
            ctx.carry[self.value_mix_key] = proj[:, v_at:v_at + K * dv]
        if mfma:
            o = torch.empty((proj.shape[0], H * dv), dtype=proj.dtype, device=proj.device)
            units, few, many, max_q = ctx.attention_units(16 // (H // K), ops.prefill_units_per_group())
            kw = dict(window=self.window, soft_cap=None, max_kv_len=ctx.max_kv_len, max_q_len=max_q, out=o,
                      sinks=self.sink_f32)
            if few:
                ops.paged_attention_decode(proj, cache.k_pages, cache.v_pages, group.block_table, units, 0, few, H, **kw)
            if many:
                ops.paged_attention_prefill(proj, cache.k_pages, cache.v_pages, group.block_table, units, few, many, H,
                                            **kw)
        else:
            o = ops.paged_attention_sink(proj, cache.k_pages, cache.v_pages, group.block_table, ctx.token_seq,
                                         ctx.positions, H, scale=self.scale, sinks=self.sink, window=self.window)
        if self.output_gate:
            g_at = v_at + K * dv
            ops.gated_heads(o, proj[:, g_at:g_at + H * dv], H, dv, kind=ops.GATE_SIGMOID, out=o)
        if self.bias:
            return ops.bias_add_(ops.gemm(o, self.o_proj), self.o_bias)
        return ops.gemm(o, self.o_proj, defer_sum=defer_sum)


@MIXERS.register("differential_attention")
class DifferentialAttention(Mixer):
    """Grouped-query attention with two score maps per head over the same values.  A query row holds, head by head,
    [map 1 | map 2] of `key_dim` entries each, a key row likewise per key head; every map of every head is divided by
    its root mean square and multiplied by a weight of `key_dim` entries that all heads and maps share (`qk_norm`),
    then its first entries are rotated (`position_encoding`: 'pair_rope').  With a_1, a_2 the maps' softmax results
    over the window and lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff (one number for the layer):

        o = a_1 - lambda a_2;   o <- o / sqrt(mean(o^2) + norm_eps) * (1 - diff)   per head, over its values

    q, k and v are one product; the cache holds key rows of 2 * key_dim entries and values of their own size."""

    defers_sum = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, scale: float,
                 diff: float, norm_eps: float, qk_norm: bool = True, window: int | None = None,
                 position_encoding: PartSpec | None = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"differential_attention: {num_heads} heads do not split over {num_kv_heads} kv heads")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim, self.scale = int(key_dim), int(value_dim), float(scale)
        self.diff, self.norm_eps, self.qk_norm = float(diff), float(norm_eps), bool(qk_norm)
        self.window = int(window) if window else None
        self.position_encoding = (POSITION_ENCODINGS.build(position_encoding.kind, **position_encoding.params)
                                  if position_encoding is not None else None)
        if self.position_encoding is not None and not hasattr(self.position_encoding, "mult"):
            raise ValueError("differential_attention: the position encoding must rotate neighbouring pairs (pair_rope)")
        self.in_proj = self.o_proj = self.q_norm = self.k_norm = None
        self.lam = 0.0

    def param_specs(self):
        D, H, K, dk, dv = self.hidden_size, self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        specs = {"q_proj": ParamSpec((H * 2 * dk, D)), "k_proj": ParamSpec((K * 2 * dk, D)),
                 "v_proj": ParamSpec((K * dv, D)), "o_proj": ParamSpec((D, H * dv))}
        if self.qk_norm:
            specs.update(q_norm=ParamSpec((dk,), role="vector", init="norm"),
                         k_norm=ParamSpec((dk,), role="vector", init="norm"))
        for name in ("lq1", "lk1", "lq2", "lk2"):
            specs[name] = ParamSpec((dk,), role="vector", init="norm")
        return specs

    def load(self, tensors):
        t = tensors
        self.in_proj = as_product_weight(torch.cat([t["q_proj"], t["k_proj"], t["v_proj"]], dim=0).contiguous())
        self.o_proj = as_product_weight(t["o_proj"])
        if self.qk_norm:
            self.q_norm, self.k_norm = t["q_norm"].contiguous(), t["k_norm"].to(t["q_norm"].dtype).contiguous()
        f = {n: t[n].to(torch.float32) for n in ("lq1", "lk1", "lq2", "lk2")}
        # one number for the layer, in 32-bit
        self.lam = float(torch.exp((f["lq1"] * f["lk1"]).sum()) - torch.exp((f["lq2"] * f["lk2"]).sum())
                         + torch.tensor(self.diff, dtype=torch.float32))
        if self.position_encoding is not None:
            self.position_encoding.to_device(t["o_proj"].device)

    def cache_need(self):
        return PagedKVNeed(self.num_kv_heads, 2 * self.key_dim, self.window, self.value_dim)

    def forward(self, x, ctx, cache, defer_sum=False):
        H, K, dk, dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        group = ctx.groups[cache.group_id]
        proj = ops.gemm(x, self.in_proj)
        pe = self.position_encoding
        freq, rot_dims = pe.frequencies() if pe is not None else (None, 0)
        write = cache.write
        # every map of every head: norm, rotation; keys and values into their pages
        ops.norm_rope_cache_write(proj, ctx.positions, freq, rot_dims, H, K, 2 * dk, dv,
                                  rot_mult=pe.mult if pe is not None else 1.0, sub=2, eps=self.norm_eps,
                                  q_weight=self.q_norm, q_norm_dims=dk if self.qk_norm else 0,
                                  k_weight=self.k_norm, k_norm_dims=dk if self.qk_norm else 0,
                                  slot_mapping=group.slot_mapping if write else None,
                                  k_pages=cache.k_pages if write else None, v_pages=cache.v_pages if write else None)
        combine = (self.lam, self.norm_eps, 1.0 - self.diff)
        if ops.attention_maps_units_takes(proj, cache.k_pages, cache.v_pages, H, maps=2):
            # bfloat16 at sizes that the matrix cores take: units of 16 rows (heads of a key head times tokens) per map,
            # keys cut into ranges; the maps are combined from the ranges' 32-bit partial results
            units, few, many, max_q = ctx.attention_units(16 // ops.attention_maps_heads_per_unit(H, K))
            o = ops.paged_attention_maps_units(proj, cache.k_pages, cache.v_pages, group.block_table, units, 0,
                                               few + many, H, scale=self.scale, maps=2, window=self.window,
                                               differential=combine, max_kv_len=ctx.max_kv_len, max_q_len=max_q)
        else:
            o = ops.paged_attention_maps(proj, cache.k_pages, cache.v_pages, group.block_table, ctx.token_seq,
                                         ctx.positions, H, scale=self.scale, maps=2, window=self.window,
                                         differential=combine)
        return ops.gemm(o, self.o_proj, defer_sum=defer_sum)
