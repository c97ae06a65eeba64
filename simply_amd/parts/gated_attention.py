"""Windowed grouped-query attention with a gate on its heads, put together from options.

q, k, v and the gate are one product of the mixer's input (`bias`: q and k have biases).  Between that product and
the scores:

  conv_taps       (0: none) every channel of q, k and v passes a causal convolution over time (taps oldest first, zeros before the
                  sequence's start, no activation); a request's last taps - 1 projected rows are its state
  qk_norm         'head': q and k divided by each head's root mean square, times a weight of one head's size that the
                  heads share; 'row': by the root mean square of the whole projection (all heads at once), times a
                  weight per entry; None: no norm
  position_encoding  'partial_rope': the first entries of every head of q and k turn in pairs (i, i + dims / 2),
                  after the norm
  query_temperature  (coef, every): the query at position p times 1 + coef ln(floor((p + 1) / every) + 1)
  values          'projected': a projection of their own; 'keys': the keys as projected (before norm and rotation) are
                  the values, and there is no value projection

and in the scores (32-bit): `scale`; `slope_exponent` c: head h's scores lose 2^(-c (h + 1) / H) times the distance
between query and key; `window`; `zero_sink`: one more term exp(0) in every softmax sum, without a value.  The heads'
results are multiplied by sigmoid(gate projection), entry by entry (`output_gate` 'element') or one number per head
('head'), then projected.

`own_keys_values` False: the layer has queries only and reads the keys and values that another schedule entry keeps
(that entry's `cache_window` then covers this layer's window too).  What is kept per token is a `PagedKVNeed`; with a
convolution the tails are a `StateNeed` beside it (a `CompositeNeed`: pages first, then the state).
"""
from __future__ import annotations

import torch

from ..config.spec import PartSpec
from ..kernels import ops
from ..registry import MIXERS, POSITION_ENCODINGS
from .base import CompositeNeed, Mixer, PagedKVNeed, ParamSpec, StateNeed, as_product_weight


@MIXERS.register("gated_attention")
class GatedAttention(Mixer):
    defers_sum = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, scale: float,
                 norm_eps: float = 0.0, qk_norm: str | None = None, bias: bool = False, conv_taps: int = 0,
                 values: str = "projected", position_encoding: PartSpec | None = None,
                 query_temperature: "tuple[float, int] | None" = None, slope_exponent: float | None = None,
                 zero_sink: bool = False, output_gate: str | None = "element", window: int | None = None,
                 cache_window: "int | None | str" = "window", own_keys_values: bool = True):
        if num_heads % num_kv_heads:
            raise ValueError(f"gated_attention: {num_heads} heads do not split over {num_kv_heads} kv heads")
        if qk_norm not in (None, "head", "row"):
            raise ValueError(f"gated_attention: qk_norm is None, 'head' or 'row', not {qk_norm!r}")
        if values not in ("projected", "keys"):
            raise ValueError(f"gated_attention: values are 'projected' or 'keys', not {values!r}")
        if output_gate not in (None, "element", "head"):
            raise ValueError(f"gated_attention: output_gate is None, 'element' or 'head', not {output_gate!r}")
        if values == "keys" and int(value_dim) != int(key_dim):
            raise ValueError("gated_attention: keys that are the values too have the values' size")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim, self.scale = int(key_dim), int(value_dim), float(scale)
        self.norm_eps, self.qk_norm, self.bias = float(norm_eps), qk_norm, bool(bias)
        self.conv_taps = int(conv_taps or 0)
        self.values_are_keys = values == "keys"
        self.own = bool(own_keys_values)
        self.query_temperature = None if query_temperature is None else (float(query_temperature[0]),
                                                                         int(query_temperature[1]))
        if self.query_temperature is not None and self.query_temperature[1] < 1:
            raise ValueError("gated_attention: the temperature's period is at least one position")
        self.slope_exponent = None if slope_exponent is None else float(slope_exponent)
        self.zero_sink, self.output_gate = bool(zero_sink), output_gate
        self.window = int(window) if window else None
        #: how many tokens back the pages are kept: this layer's window or, where other layers read its pages, the
        #: largest of theirs (None: all)
        self.cache_window = self.window if cache_window == "window" else (int(cache_window) if cache_window else None)
        if self.cache_window is not None and (self.window is None or self.window > self.cache_window):
            raise ValueError("gated_attention: the pages are kept for fewer tokens than the layer's window sees")
        self.position_encoding = (POSITION_ENCODINGS.build(position_encoding.kind, **position_encoding.params)
                                  if position_encoding is not None else None)
        if self.position_encoding is not None and not hasattr(self.position_encoding, "frequencies"):
            raise ValueError("gated_attention: the position encoding must give frequencies() (partial_rope)")
        self.in_proj = self.o_proj = self.in_bias = self.taps = self.taps_by_tap = self.q_norm = self.k_norm = None
        self.sinks = self.slopes = None

    # ------------------------------------------------------------------ sizes
    @property
    def conv_channels(self) -> int:
        """Channels that pass the convolution: queries, and the layer's own keys and values."""
        H, K, dk, dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        if not self.own:
            return H * dk
        return (H + K) * dk + (0 if self.values_are_keys else K * dv)

    @property
    def gate_width(self) -> int:
        return {None: 0, "element": self.num_heads * self.value_dim, "head": self.num_heads}[self.output_gate]

    def param_specs(self):
        D, H, K, dk, dv, n = self.hidden_size, self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim, self.conv_taps
        vec = dict(role="vector", init="norm")
        specs = {"q_proj": ParamSpec((H * dk, D)), "o_proj": ParamSpec((D, H * dv))}
        sections = ["q"]
        if self.own:
            specs["k_proj"] = ParamSpec((K * dk, D))
            sections.append("k")
            if not self.values_are_keys:
                specs["v_proj"] = ParamSpec((K * dv, D))
                sections.append("v")
        if self.bias:
            specs["q_bias"] = ParamSpec((H * dk,), **vec)
            if self.own:
                specs["k_bias"] = ParamSpec((K * dk,), **vec)
        if n >= 1:
            for s in sections:
                specs[s + "_conv"] = ParamSpec((specs[s + "_proj"].shape[0], n), role="vector")
        if self.qk_norm is not None:
            specs["q_norm"] = ParamSpec((dk if self.qk_norm == "head" else H * dk,), **vec)
            if self.own:
                specs["k_norm"] = ParamSpec((dk if self.qk_norm == "head" else K * dk,), **vec)
        if self.output_gate is not None:
            specs["gate_proj"] = ParamSpec((self.gate_width, D))
        return specs

    def load(self, tensors):
        t = tensors
        sections = ["q"] + ((["k"] if self.values_are_keys else ["k", "v"]) if self.own else [])
        rows = [t[s + "_proj"] for s in sections] + ([t["gate_proj"]] if self.output_gate is not None else [])
        self.in_proj = as_product_weight(torch.cat(rows, dim=0).contiguous())
        self.o_proj = as_product_weight(t["o_proj"])
        device = t["o_proj"].device
        if self.bias:
            # one bias row for the whole product: zeros where a section has none
            parts = [t[s + "_bias"] if s + "_bias" in t else torch.zeros(t[s + "_proj"].shape[0], dtype=t["q_bias"].dtype,
                                                                         device=device) for s in sections]
            parts.append(torch.zeros(self.gate_width, dtype=t["q_bias"].dtype, device=device))
            self.in_bias = torch.cat([p.to(t["q_bias"].dtype) for p in parts]).contiguous()
        if self.conv_taps >= 1:
            self.taps = torch.cat([t[s + "_conv"] for s in sections], dim=0).contiguous()
            self.taps_by_tap = self.taps.t().contiguous()   # (what the kernel for aligned rows reads in pieces)
        if self.qk_norm is not None:
            self.q_norm = t["q_norm"].contiguous()
            self.k_norm = t["k_norm"].to(self.q_norm.dtype).contiguous() if self.own else None
        H = self.num_heads
        if self.zero_sink:
            self.sinks = torch.zeros(H, dtype=torch.float32, device=device)
        if self.slope_exponent is not None:
            h = torch.arange(1, H + 1, dtype=torch.float64)
            self.slopes = (2.0 ** (-self.slope_exponent * h / H)).to(torch.float32).to(device)
        if self.position_encoding is not None:
            self.position_encoding.to_device(device)

    def cache_need(self):
        pages = PagedKVNeed(self.num_kv_heads, self.key_dim, self.cache_window, self.value_dim)
        if self.conv_taps > 1:
            return CompositeNeed((pages, StateNeed(((self.conv_taps - 1) * self.conv_channels,), torch.float32)))
        return pages

    # ------------------------------------------------------------------ forward
    def forward(self, x, ctx, cache, defer_sum=False):
        H, K, dk, dv = self.num_heads, self.num_kv_heads, self.key_dim, self.value_dim
        pages, state = (cache.parts[0], cache.parts[1].state) if self.conv_taps > 1 else (cache, None)
        if pages.write != self.own:
            raise RuntimeError("gated_attention: a layer with keys and values of its own writes its pages, one without "
                               "reads another entry's")
        group = ctx.groups[pages.group_id]
        proj = ops.gemm(x, self.in_proj)
        # (without a convolution the biases are added where the rows are read; the gate's columns have none)
        bias_later = self.bias and self.conv_taps == 0
        if self.bias and not bias_later:
            ops.bias_add_(proj, self.in_bias)
        pe = self.position_encoding
        inv_freq, rot_dims = pe.frequencies() if pe is not None else (None, 0)
        coef, every = self.query_temperature if self.query_temperature is not None else (0.0, 0)
        # the bfloat16 MFMA kernels take values of the keys' size (64, 128 or 256) in pages of a multiple of 16 keys;
        # they have no factor on the scores, so the queries carry it
        mfma = dk == dv and proj.dtype == torch.bfloat16 and ops.decode_attention_takes(proj, pages.k_pages, H, 1)
        q = ops.attention_inputs(proj, ctx.seq_meta, ctx.num_seqs, ctx.max_q_len, H, K, dk, dv,
                                 values_are_keys=self.values_are_keys, taps=self.taps, taps_by_tap=self.taps_by_tap,
                                 in_bias=self.in_bias if bias_later else None,
                                 tails=state, norm=self.qk_norm,
                                 q_weight=self.q_norm, k_weight=self.k_norm, eps=self.norm_eps, inv_freq=inv_freq,
                                 rot_dims=rot_dims, temp_coef=coef, temp_every=every, q_mult=self.scale if mfma else 1.0,
                                 slot_mapping=group.slot_mapping if self.own else None,
                                 k_pages=pages.k_pages if self.own else None, v_pages=pages.v_pages if self.own else None)
        if mfma:
            o = torch.empty((q.shape[0], H * dv), dtype=q.dtype, device=q.device)
            units, few, many, max_q = ctx.attention_units(16 // (H // K), ops.prefill_units_per_group())
            kw = dict(window=self.window, soft_cap=None, max_kv_len=ctx.max_kv_len, max_q_len=max_q, out=o,
                      sinks=self.sinks, slopes=self.slopes)
            if few:
                ops.paged_attention_decode(q, pages.k_pages, pages.v_pages, group.block_table, units, 0, few, H, **kw)
            if many:
                ops.paged_attention_prefill(q, pages.k_pages, pages.v_pages, group.block_table, units, few, many, H, **kw)
        else:
            o = ops.paged_attention_sink(q, pages.k_pages, pages.v_pages, group.block_table, ctx.token_seq,
                                         ctx.positions, H, scale=self.scale, sinks=self.sinks, slopes=self.slopes,
                                         window=self.window)
        if self.output_gate is not None:
            g_at = self.conv_channels
            ops.gated_heads(o, proj[:, g_at:g_at + self.gate_width], H, dv, kind=ops.GATE_SIGMOID, out=o,
                            per_head=self.output_gate == "head")
        return ops.gemm(o, self.o_proj, defer_sum=defer_sum)
