"""Feed-forward parts. ``SwiGLU`` follows nanovllm/models/qwen3.py:91-117."""
from __future__ import annotations

import torch

from ..native import ops
from .base import FEED_FORWARDS, ParamSpec, Part


@FEED_FORWARDS.register("swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)); gate and up are one packed matrix whose first
    ``intermediate_size`` rows are the gate (nanovllm/layers/linear.py:102-108,
    nanovllm/layers/activation.py:10-11)."""

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        """``activation``: what the gate passes, "silu" (the reference's) or "gelu_tanh"."""
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not known ({sorted(ops.ACTIVATIONS)} are)")
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.activation = activation
        self.gate_up_weight = None
        self.down_weight = None

    def param_specs(self):
        return {
            "gate_up.weight": ParamSpec((2 * self.intermediate_size, self.hidden_size)),
            "down.weight": ParamSpec((self.hidden_size, self.intermediate_size)),
        }

    takes_deferred_norm = True    # x goes straight into a product, which can norm it
    adds_to_residual = True       # the down projection can make the addition to the residual stream

    def first_product(self):
        """(weight, gated) of the product that x goes into."""
        return self.gate_up_weight, True

    def forward(self, x, step, add_to=None):
        if self.activation != "silu":
            return ops.linear(ops.gated_linear(x, self.gate_up_weight, self.activation), self.down_weight, add_to=add_to)
        return ops.linear(ops.gated_linear(x, self.gate_up_weight), self.down_weight, add_to=add_to)


@FEED_FORWARDS.register("plain_mlp")
class PlainMLP(Part):
    """down(act(up(x))) without a gate and without biases; ``activation``: "relu2" (the square of max(z, 0)), "silu"
    or "gelu_tanh". The activation is taken in float: on the up projection's finished sums where a step of few rows
    does both in one kernel, else on its rounded rows."""

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu2"):
        if activation not in ops.PLAIN_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not known ({sorted(ops.PLAIN_ACTIVATIONS)} are)")
        if min(hidden_size, intermediate_size) <= 0:
            raise ValueError(f"a feed-forward of {hidden_size} x {intermediate_size}")
        self.hidden_size, self.intermediate_size, self.activation = hidden_size, intermediate_size, activation
        self.up_weight = self.down_weight = None

    def param_specs(self):
        return {"up.weight": ParamSpec((self.intermediate_size, self.hidden_size)),
                "down.weight": ParamSpec((self.hidden_size, self.intermediate_size))}

    def forward(self, x, step):
        return ops.linear(ops.activated_linear(x, self.up_weight, self.activation), self.down_weight)


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(Part):
    """``num_experts`` gated feed-forwards of inner size ``expert_size`` without biases, of which every token uses the
    ``top`` with the largest router logit z_e = router_e . x (+ b_e with ``router_bias``; summed and kept in float32).
    ``scoring`` "sigmoid": the score s_e = sigmoid(z_e), taken as it is (not renormalised); "softmax_of_chosen": the
    scores are the softmax over the chosen logits alone. ``scores_on`` "input": the score multiplies the expert's input,
    y = sum over chosen e of D_e (act(G_e s_e x) * (U_e s_e x)); "output": it weighs the expert's output,
    y = sum over chosen e of s_e D_e (act(G_e x) * (U_e x)). ``shared``: the description of one more feed-forward that
    every token uses and whose result is added (its tensors lie under ``shared.``).
    All experts' matrices lie in two tensors, [experts * 2 expert_size, width] (per expert its gate rows, then its
    up rows) and [experts * width, expert_size]."""

    def __init__(self, hidden_size: int, num_experts: int, top: int, expert_size: int, activation: str = "silu",
                 scoring: str = "sigmoid", scores_on: str = "input", router_bias: bool = False, shared: dict | None = None,
                 **offered):
        if not 0 < top <= num_experts or min(hidden_size, expert_size) <= 0:
            raise ValueError(f"{top} of {num_experts} experts of size {expert_size}")
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not known ({sorted(ops.ACTIVATIONS)} are)")
        if scoring not in ops.ROUTER_SCORES:
            raise ValueError(f"scoring {scoring!r} is not known ({sorted(ops.ROUTER_SCORES)} are)")
        if scores_on not in ("input", "output"):
            raise ValueError(f"scores on {scores_on!r}: 'input' and 'output' are known")
        self.hidden_size, self.num_experts, self.top, self.expert_size = hidden_size, num_experts, top, expert_size
        self.activation, self.scoring, self.scores_on, self.has_router_bias = activation, scoring, scores_on, bool(router_bias)
        self.shared = FEED_FORWARDS.build(shared, offered=offered) if shared is not None else None
        self.router_bias = None

    def children(self):
        return {"shared": self.shared} if self.shared is not None else {}

    def param_specs(self):
        E, F, W = self.num_experts, self.expert_size, self.hidden_size
        specs = {"router.weight": ParamSpec((E, W)),
                 "gate_up.weight": ParamSpec((E * 2 * F, W)),
                 "down.weight": ParamSpec((E * W, F))}
        if self.has_router_bias:
            specs["router.bias"] = ParamSpec((E,), init="zeros", always_float32=True)
        return specs

    def bind(self, params):
        E, F, W = self.num_experts, self.expert_size, self.hidden_size
        self.router_weight = params["router.weight"]
        self.router_bias = params.get("router.bias")
        self.gate_up_weight = params["gate_up.weight"].view(E, 2 * F, W)
        self.down_weight = params["down.weight"].view(E, W, F)

    def forward(self, x, step):
        ids, scores = ops.route_topk(ops.linear(x, self.router_weight, out_dtype=torch.float32), self.top,
                                     bias=self.router_bias, scoring=self.scoring)
        if self.shared is None and self.scores_on == "input":
            return ops.routed_experts(x, ids, scores, self.gate_up_weight, self.down_weight, self.activation)
        add = self.shared.forward(x, step) if self.shared is not None else None
        return ops.routed_experts(x, ids, scores, self.gate_up_weight, self.down_weight, self.activation,
                                  scores_on=self.scores_on, add=add)
