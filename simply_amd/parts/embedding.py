"""Token embedding and the output head.

simply/utils/module.py:450-481: lookup, then times sqrt(dim) * embedding_scale, the factor
rounded to the activation dtype first.  simply/model_lib.py:3184-3189: logits are the product
with the (tied) table, then the final soft-cap if it is > 0.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import EMBEDDINGS, HEADS
from .base import ParamSpec, Part, StateNeed, as_product_weight, project


@EMBEDDINGS.register("scaled_embedding")
class ScaledEmbedding(Part):
    def __init__(self, vocab_size: int, dim: int, scale: float):
        self.vocab_size, self.dim, self.scale = int(vocab_size), int(dim), float(scale)
        self.table: torch.Tensor | None = None

    def param_specs(self):
        return {"table": ParamSpec((self.vocab_size, self.dim), role="matrix", init="weight")}

    def load(self, tensors):
        # tiled like a product weight when it is bfloat16 on the GPU: a tied head reads the same storage
        self.table = as_product_weight(tensors["table"], shared=True)

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        """tokens int32 [T] -> float32 residual stream [T, D]."""
        # the factor is rounded to the table's dtype (module.py:476-480), the product is kept in float32
        scale = float(torch.tensor(self.scale, dtype=self.table.dtype))
        return ops.embed(self.table, tokens, scale)


@EMBEDDINGS.register("normed_embedding")
class NormedEmbedding(Part):
    """The token's row divided by its root mean square (eps inside the root) and multiplied by a weight (`plus_one`:
    by one plus the weight): a norm on the embedding before the first layer."""

    def __init__(self, vocab_size: int, dim: int, eps: float, plus_one: bool = False):
        self.vocab_size, self.dim, self.eps, self.plus_one = int(vocab_size), int(dim), float(eps), bool(plus_one)
        self.table = self.norm = None

    def param_specs(self):
        return {"table": ParamSpec((self.vocab_size, self.dim), role="matrix", init="weight"),
                "norm": ParamSpec((self.dim,), role="vector", init="norm")}

    def load(self, tensors):
        self.table = as_product_weight(tensors["table"], shared=True)
        self.norm = tensors["norm"].contiguous()

    def forward(self, tokens: torch.Tensor) -> torch.Tensor:
        """tokens int32 [T] -> float32 residual stream [T, D]."""
        return ops.rmsnorm(ops.embed(self.table, tokens, 1.0), self.norm, self.eps, self.plus_one, torch.float32)


@EMBEDDINGS.register("summed_embedding")
class SummedEmbedding(Part):
    """The token's row, plus (with `pair_buckets`) a row for the pair of the token and the one before it, chosen by
    (previous * mul_prev + token * mul_cur) mod pair_buckets, a request's first token taking the row behind the
    buckets, plus (with `max_positions`) a learned row for the position, unscaled.  The token before a step's first
    one is the request's state: one int32 per state slot, which this part keeps up to date."""

    #: forward() takes the step's context and this part's cache view
    needs_context = True

    def __init__(self, vocab_size: int, dim: int, pair_buckets: int | None = None, mul_prev: int = 0, mul_cur: int = 0,
                 max_positions: int | None = None):
        self.vocab_size, self.dim = int(vocab_size), int(dim)
        self.pair_buckets = int(pair_buckets) if pair_buckets else None
        self.mul_prev, self.mul_cur = int(mul_prev), int(mul_cur)
        self.max_positions = int(max_positions) if max_positions else None
        self.table = self.pair = self.pos = None

    def param_specs(self):
        specs = {"table": ParamSpec((self.vocab_size, self.dim))}
        if self.pair_buckets:
            specs["pair"] = ParamSpec((self.pair_buckets + 1, self.dim))
        if self.max_positions:
            specs["pos"] = ParamSpec((self.max_positions, self.dim))
        return specs

    def cache_need(self):
        return StateNeed((1,), torch.int32) if self.pair_buckets else None

    def forward(self, tokens, ctx, cache):
        if self.max_positions and ctx.max_kv_len > self.max_positions and not ctx.kv_bound:
            raise ValueError(f"summed_embedding: a position beyond the {self.max_positions} learned ones")
        return ops.embed_sum(tokens, ctx.positions, ctx.seq_meta, ctx.num_seqs, ctx.max_q_len, self.table,
                             pair=self.pair, mul_prev=self.mul_prev, mul_cur=self.mul_cur,
                             last=cache.state if cache is not None else None, pos=self.pos)


@HEADS.register("linear_head")
class LinearHead(Part):
    def __init__(self, vocab_size: int, dim: int, soft_cap: float | None):
        self.vocab_size, self.dim = int(vocab_size), int(dim)
        self.soft_cap = float(soft_cap) if soft_cap else None
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        return {"weight": ParamSpec((self.vocab_size, self.dim), role="matrix", init="weight")}

    def load(self, tensors):
        self.weight = as_product_weight(tensors["weight"], shared=True)

    def forward(self, x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """x [R, D] activations (or a `PendingNorm` of them) -> float32 logits [R, V] (written into `out` if given)."""
        return project(x, self.weight, soft_cap=self.soft_cap, out_dtype=torch.float32, out=out)

