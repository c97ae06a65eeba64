"""Dense gated feed-forward: down(act(gate(x)) * up(x))  (simply/model_lib.py:643-730 with
use_gated_activation_in_ffn=True, ffn_use_bias=False; `act` by its name in the registry, as
simply/model_lib.py:723 looks `ffn_activation` up)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import ACTIVATIONS, FEED_FORWARDS
from .base import FeedForward, ParamSpec, PendingNorm, as_product_weight, project

# activation name -> its code in the gated product's epilogue (simply/model_lib.py:93-104 registers these three)
ACTIVATIONS.register("gelu_tanh", ops.ACT_GELU_TANH)
ACTIVATIONS.register("silu", ops.ACT_SILU)
ACTIVATIONS.register("squared_relu", ops.ACT_SQUARED_RELU)
ACTIVATIONS.register("gelu_erf", ops.ACT_GELU_ERF)   # the exact GELU, x Phi(x)


@FEED_FORWARDS.register("dense")
class Dense(FeedForward):
    """down(act(up(x))): one factor, no gate (simply/model_lib.py:643-730 with use_gated_activation_in_ffn=False)."""

    defers_sum = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "squared_relu"):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation = activation
        self.activation_code = int(ACTIVATIONS.get(activation))
        self.up_proj = self.down_proj = None

    def param_specs(self):
        D, F = self.hidden_size, self.intermediate_size
        return {"up_proj": ParamSpec((F, D)), "down_proj": ParamSpec((D, F))}

    def load(self, tensors):
        self.up_proj = as_product_weight(tensors["up_proj"])
        self.down_proj = as_product_weight(tensors["down_proj"])

    def forward(self, x: torch.Tensor, ctx=None, defer_sum=False) -> torch.Tensor:
        z = ops.gemm(x, self.up_proj, activate=self.activation_code)   # (the activation is the product's epilogue)
        return ops.gemm(z, self.down_proj, defer_sum=defer_sum)


@FEED_FORWARDS.register("gated_dense")
class GatedDense(FeedForward):
    accepts_pending = True
    defers_sum = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "gelu_tanh"):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation = activation
        self.activation_code = int(ACTIVATIONS.get(activation))   # an unknown name is refused with the known ones
        self.gate_proj = self.up_proj = self.down_proj = self.gate_up = None

    def param_specs(self):
        D, F = self.hidden_size, self.intermediate_size
        return {"gate_proj": ParamSpec((F, D)), "up_proj": ParamSpec((F, D)), "down_proj": ParamSpec((D, F))}

    def load(self, tensors):
        gate, up = tensors["gate_proj"], tensors["up_proj"]
        if gate.dtype == torch.bfloat16 and gate.is_cuda:
            # one tiled weight for both factors, their tiles in turn: the fused kernels stream it once
            from ..kernels.packing import pack_gate_up

            self.gate_up, self.gate_proj, self.up_proj = pack_gate_up(gate, up), None, None
        else:
            self.gate_up, self.gate_proj, self.up_proj = None, gate, up
        self.down_proj = as_product_weight(tensors["down_proj"])

    def forward(self, x: torch.Tensor, ctx=None, defer_sum=False) -> torch.Tensor:
        # gelu(x.Wg^T) * (x.Wu^T), one kernel
        if self.gate_up is not None:
            z = project(x, self.gate_up, activation=self.activation_code)
        else:
            if isinstance(x, PendingNorm):
                x = x.materialize()
            z = ops.gemm(x, self.gate_proj, w2=self.up_proj, activation=self.activation_code)
        return ops.gemm(z, self.down_proj, defer_sum=defer_sum)


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    """A mixture of experts: `num_experts` feed-forwards without biases, of which every token uses the `top` ones that
    the router chooses; an expert's result is weighted by its score times `router_scale`, the weights are not
    renormalized.

      gated       True: an expert is down(act(gate x) * (up x)); False: down(act(up x)), and there are no gate tensors
      router      'softmax': scores are the softmax of the router's logits over all experts (32-bit), the largest are
                  chosen; 'sigmoid': scores are sigmoids of the logits, the choice goes by score + a stored correction
                  per expert (`correction`) among the experts of the `keep_groups` best of `num_groups` equal groups of
                  neighbours (a group's score: the sum of its two largest choice scores), and the weights are the
                  scores without the correction
      shared_size one more feed-forward of the experts' form runs for every token and is added, times sigmoid(w . x)
                  (one number per token) if `shared_gate`."""

    def __init__(self, hidden_size: int, num_experts: int, top: int, expert_size: int, router_scale: float = 1.0,
                 activation: str = "silu", shared_size: int | None = None, shared_gate: bool = True, gated: bool = True,
                 router: str = "softmax", correction: bool = False, num_groups: int = 1, keep_groups: int = 1):
        self.hidden_size, self.num_experts, self.top = int(hidden_size), int(num_experts), int(top)
        self.expert_size, self.router_scale = int(expert_size), float(router_scale)
        if not 1 <= self.top <= self.num_experts:
            raise ValueError(f"routed_experts: top {top} of {num_experts} experts")
        if router not in ("softmax", "sigmoid"):
            raise ValueError(f"routed_experts: the router is 'softmax' or 'sigmoid', not {router!r}")
        self.router_kind, self.correction = router, bool(correction)
        self.num_groups, self.keep_groups = int(num_groups), int(keep_groups)
        if router == "softmax" and (self.correction or self.num_groups != 1):
            raise ValueError("routed_experts: a correction and groups go with the sigmoid router")
        if self.num_groups < 1 or self.num_experts % self.num_groups or not 1 <= self.keep_groups <= self.num_groups \
                or self.top > self.keep_groups * (self.num_experts // self.num_groups):
            raise ValueError(f"routed_experts: {num_experts} experts in {num_groups} groups of which {keep_groups} stay "
                             f"do not give {top} choices")
        self.gated = bool(gated)
        self.activation_code = int(ACTIVATIONS.get(activation))
        shared_cls = GatedDense if self.gated else Dense
        self.shared = shared_cls(hidden_size, int(shared_size), activation) if shared_size else None
        self.shared_gate = bool(shared_gate) and self.shared is not None
        self.router = self.gate_w = self.up_w = self.down_w = self.correction_w = None

    def param_specs(self):
        D, F, E = self.hidden_size, self.expert_size, self.num_experts
        specs = {"router": ParamSpec((E, D))}
        if self.correction:
            specs["correction"] = ParamSpec((E,), role="vector", init="norm")
        for e in range(E):
            if self.gated:
                specs[f"e{e}.gate"] = ParamSpec((F, D))
            specs.update({f"e{e}.up": ParamSpec((F, D)), f"e{e}.down": ParamSpec((D, F))})
        if self.shared is not None:
            specs.update({"shared." + n: s for n, s in self.shared.param_specs().items()})
            if self.shared_gate:
                specs["shared.score"] = ParamSpec((1, D))
        return specs

    def load(self, tensors):
        from ..kernels.packing import stack_experts

        E = self.num_experts
        rows = [tensors["router"]] + ([tensors["shared.score"]] if self.shared_gate else [])
        # the router (and the shared expert's score) are one product, its result 32-bit
        self.router = as_product_weight(torch.cat(rows, dim=0).contiguous())
        self.gate_w = stack_experts(tensors[f"e{e}.gate"] for e in range(E)) if self.gated else None
        self.up_w = stack_experts(tensors[f"e{e}.up"] for e in range(E))
        self.down_w = stack_experts(tensors[f"e{e}.down"] for e in range(E))
        self.correction_w = tensors["correction"].contiguous() if self.correction else None
        if self.shared is not None:
            self.shared.load({n: tensors["shared." + n] for n in self.shared.param_specs()})

    def forward(self, x: torch.Tensor, ctx=None) -> torch.Tensor:
        E = self.num_experts
        logits = ops.gemm(x, self.router, out_dtype=torch.float32)
        if self.router_kind == "sigmoid":
            experts, weights = ops.route_choice(logits[:, :E], self.top, self.router_scale, correction=self.correction_w,
                                                groups=self.num_groups, keep=self.keep_groups)
        else:
            experts, weights = ops.route(logits[:, :E], self.top, self.router_scale)
        shared = self.shared.forward(x, ctx) if self.shared is not None else None
        return ops.routed_experts(x, experts, weights, self.gate_w, self.up_w, self.down_w, self.activation_code,
                                  shared=shared, shared_gate=logits[:, E:E + 1] if self.shared_gate else None)
