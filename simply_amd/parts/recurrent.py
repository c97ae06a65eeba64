"""Recurrent mixers: the gated delta rule, and the real-gated linear recurrent unit (further down).

The gated delta rule:

Per head a matrix state S [key size, value size] in 32-bit, carried from token to token of a request:

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

with q, k, v from projections that pass a short causal convolution per channel and silu, q and k made unit vectors
(q also divided by sqrt(key size)), beta = sigmoid(b x), g = exp(-exp(A_log) softplus(a x + dt_bias)) per head.  Each
head's o is divided by its root mean square, multiplied by a weight (shared by the heads) and by silu(gate x), then
projected.  Value head h reads q/k head h // (heads / qk heads).  Besides S, the last taps - 1 inputs of the
convolution are the request's state; both live in one row of a state slot.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import MIXERS
from .base import Mixer, ParamSpec, StateNeed, as_product_weight


@MIXERS.register("gated_delta")
class GatedDelta(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_qk_heads: int, key_dim: int, value_dim: int,
                 conv_taps: int, norm_eps: float):
        if num_heads % num_qk_heads:
            raise ValueError(f"gated_delta: {num_heads} heads do not split over {num_qk_heads} q/k heads")
        if conv_taps < 1:
            raise ValueError("gated_delta: the convolution has at least one tap")
        self.hidden_size, self.num_heads, self.num_qk_heads = int(hidden_size), int(num_heads), int(num_qk_heads)
        self.key_dim, self.value_dim, self.conv_taps = int(key_dim), int(value_dim), int(conv_taps)
        self.norm_eps = float(norm_eps)
        #: channels that pass the convolution: q heads, k heads, values
        self.channels = 2 * self.num_qk_heads * self.key_dim + self.num_heads * self.value_dim
        self.state_words = self.num_heads * self.key_dim * self.value_dim
        self.in_proj = self.ab_proj = self.o_proj = self.taps = self.a_log = self.dt_bias = self.norm = None

    def param_specs(self):
        D, H, G, dk, dv, n = (self.hidden_size, self.num_heads, self.num_qk_heads, self.key_dim, self.value_dim,
                              self.conv_taps)
        return {"q_proj": ParamSpec((G * dk, D)), "k_proj": ParamSpec((G * dk, D)), "v_proj": ParamSpec((H * dv, D)),
                "q_conv": ParamSpec((G * dk, n), role="vector"), "k_conv": ParamSpec((G * dk, n), role="vector"),
                "v_conv": ParamSpec((H * dv, n), role="vector"),
                "a_proj": ParamSpec((H, D)), "b_proj": ParamSpec((H, D)),
                "a_log": ParamSpec((H,), role="vector", init="norm"), "dt_bias": ParamSpec((H,), role="vector", init="norm"),
                "norm": ParamSpec((dv,), role="vector", init="norm"),
                "gate_proj": ParamSpec((H * dv, D)), "o_proj": ParamSpec((D, H * dv))}

    def load(self, tensors):
        t = tensors
        # one product for q, k, v and the gate; a and b are a product of their own, kept in 32-bit
        self.in_proj = as_product_weight(torch.cat([t["q_proj"], t["k_proj"], t["v_proj"], t["gate_proj"]], dim=0).contiguous())
        self.ab_proj = as_product_weight(torch.cat([t["a_proj"], t["b_proj"]], dim=0).contiguous())
        self.o_proj = as_product_weight(t["o_proj"])
        self.taps = torch.cat([t["q_conv"], t["k_conv"], t["v_conv"]], dim=0).contiguous()
        self.a_log, self.dt_bias = t["a_log"].contiguous(), t["dt_bias"].to(t["a_log"].dtype).contiguous()
        self.norm = t["norm"].contiguous()

    def cache_need(self):
        return StateNeed((self.state_words + (self.conv_taps - 1) * self.channels,), torch.float32)

    def forward(self, x, ctx, cache):
        if not cache.write:
            raise RuntimeError("gated_delta: a recurrent state cannot be read through another entry's cache")
        H, G, dk, dv, C = self.num_heads, self.num_qk_heads, self.key_dim, self.value_dim, self.channels
        proj = ops.gemm(x, self.in_proj)
        ab = ops.gemm(x, self.ab_proj, out_dtype=torch.float32)
        state, tails = cache.state[:, :self.state_words], cache.state[:, self.state_words:]
        qkv, gates = ops.delta_inputs(proj[:, :C], self.taps, tails, ab, self.a_log, self.dt_bias, ctx.seq_meta,
                                      ctx.num_seqs, ctx.max_q_len, H, G, dk)
        o = ops.delta_rule(qkv, gates, state, ctx.seq_meta, ctx.num_seqs, H, G, dk, dv)
        z = ops.gated_heads(o, proj[:, C:C + H * dv], H, dv, kind=ops.GATE_SILU, weight=self.norm, eps=self.norm_eps,
                            out_dtype=ctx.dtype)
        return ops.gemm(z, self.o_proj)


@MIXERS.register("rglru")
class RGLRU(Mixer):
    """A recurrent block with one number of state per channel.  Two branches of `width` channels from the mixer's
    input: y = gelu_tanh(W_y h + b_y), and u = conv(W_x h + b_x), a causal convolution per channel (taps oldest first,
    a bias behind it, no activation).  The channels are cut into `blocks` equal parts; in part b, with square matrices
    R_b and I_b:

        r = sigmoid(R_b u_b + b_r),  i = sigmoid(I_b u_b + b_i),  a = exp(-decay_mult r softplus(lam))
        S <- a S + sqrt(1 - a^2) i u         (32-bit, from 0, no special case for a first token)

    and the result is W_o (S * y).  The request's state is S and the convolution's last taps - 1 inputs, one float32
    row of a state slot.  Gates, decays and the recurrence are 32-bit whatever the activation type is."""

    def __init__(self, hidden_size: int, width: int, blocks: int, conv_taps: int, decay_mult: float = 8.0):
        if blocks < 1 or width % blocks:
            raise ValueError(f"rglru: {width} channels do not split into {blocks} equal parts")
        if conv_taps < 1:
            raise ValueError("rglru: the convolution has at least one tap")
        self.hidden_size, self.width, self.blocks = int(hidden_size), int(width), int(blocks)
        self.conv_taps, self.decay_mult = int(conv_taps), float(decay_mult)
        self.block_size = self.width // self.blocks
        self.in_proj = self.o_proj = self.gate_w = None

    def param_specs(self):
        D, C, B, n, bs = self.hidden_size, self.width, self.blocks, self.conv_taps, self.block_size
        vec = dict(role="vector", init="norm")
        return {"y_proj": ParamSpec((C, D)), "y_bias": ParamSpec((C,), **vec), "x_proj": ParamSpec((C, D)),
                "x_bias": ParamSpec((C,), **vec), "conv": ParamSpec((C, n), role="vector"),
                "conv_bias": ParamSpec((C,), **vec), "r_gate": ParamSpec((B, bs, bs)),
                "r_bias": ParamSpec((B, bs), **vec), "i_gate": ParamSpec((B, bs, bs)), "i_bias": ParamSpec((B, bs), **vec),
                "lam": ParamSpec((C,), **vec), "o_proj": ParamSpec((D, C))}

    def load(self, tensors):
        t = tensors
        self.in_proj = as_product_weight(torch.cat([t["y_proj"], t["x_proj"]], dim=0).contiguous())   # rows [y | x]
        self.o_proj = as_product_weight(t["o_proj"])
        # per part the two gate matrices stacked: one product per part gives [r inputs | i inputs]
        self.gate_w = torch.cat([t["r_gate"], t["i_gate"]], dim=1).contiguous()
        vt = t["lam"].dtype
        self.taps = t["conv"].contiguous()
        for name in ("y_bias", "x_bias", "conv_bias", "r_bias", "i_bias", "lam"):
            setattr(self, name, t[name].to(vt).reshape(-1).contiguous())

    def cache_need(self):
        return StateNeed((self.width * self.conv_taps,), torch.float32)   # S, then the convolution's taps - 1 inputs

    def forward(self, x, ctx, cache):
        if not cache.write:
            raise RuntimeError("rglru: a recurrent state cannot be read through another entry's cache")
        C = self.width
        proj = ops.gemm(x, self.in_proj)
        state, tails = cache.state[:, :C], cache.state[:, C:]
        u = ops.short_conv(proj[:, C:2 * C], self.taps, tails, ctx.seq_meta, ctx.num_seqs, ctx.max_q_len,
                           in_bias=self.x_bias, out_bias=self.conv_bias)
        gates = ops.head_product(u, self.gate_w, out_dtype=torch.float32)
        z = ops.rglru_scan(u, gates, self.block_size, self.r_bias, self.i_bias, self.lam, proj[:, :C], self.y_bias,
                           state, ctx.seq_meta, ctx.num_seqs, c=self.decay_mult, out_dtype=ctx.dtype,
                           max_q_len=ctx.max_q_len)
        return ops.gemm(z, self.o_proj)
