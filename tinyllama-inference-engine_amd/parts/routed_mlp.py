"""A routed feed-forward: a router scores the experts for every token, the token uses the `top` best, and an
expert that every token uses may run beside them.

    z = W_router x (float sums),  s = sigmoid(z)
    the `top` experts with the largest s are the token's; each is fed with s_e * x:
    out = sum over them of down_e(silu(gate_e(s_e x)) * up_e(s_e x))  +  shared(x)
(the scores are not renormalized, and weigh the expert's input, not its result).

Other designs of the same shape, as options:
    score "softmax_of_chosen"   the `top` largest logits z (+ a bias) are chosen, and their weights are the softmax over
                                the chosen logits only
    weigh "output"              out = sum of w_e * expert_e(x): the weight multiplies what the expert gives
    activation "clamped_swish"  g = min(gate, limit), u = clamp(up, -limit, limit), g * sigmoid(alpha g) * (u + 1), with a
                                limit for the experts and one for the shared expert
    shared_gate                 the shared expert's result is multiplied by sigmoid(w_sg . x), one number a token

All experts' gate and up matrices are one matrix, their rows side by side expert by expert (g0 u0 g1 u1 ...), the
shared expert's last, and all down matrices are one matrix along the inner index: the feed-forward is then two
products around a gate kernel that multiplies an expert's columns by the token's score for it, which is zero for an
expert that the token does not use (silu(0) * 0 adds nothing to the second product, exactly).  Since the products
are linear, s (W x) stands for W (s x); a weight on an expert's result multiplies the columns of the second product's
input in the result's place; and the shared expert's gate is one more row of the router's matrix, which stands outside
the choice.
"""
from __future__ import annotations

from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import register
from ..weights.arena import keep_in
from .base import FeedForward
from .linear import Linear


@register("feed_forward", "routed_mlp")
class RoutedMLP(FeedForward):
    """spec: hidden_size, experts, top, expert_size, shared_size (0: no shared expert), score ("sigmoid" or
    "softmax_of_chosen"), renormalize (False), weigh ("input" or "output"), router_bias (False), activation ("silu" or
    "clamped_swish" with alpha, limit, shared_limit), shared_gate (False), names (router, router_bias, expert: a pattern
    with {} for the expert's number, shared, shared_gate, gate, up, down).
    Tensors: router [experts, hidden] (and its bias [experts]); per expert and for the shared one gate, up [size, hidden],
    down [hidden, size]; the shared expert's gate [1, hidden]."""
    graph_safe = True
    NAMES = {"router": "router.weight", "router_bias": "router.bias", "expert": "experts.{}.", "shared": "shared_expert.",
             "shared_gate": "shared_expert_gate.weight", "gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.experts, self.top = int(spec["experts"]), int(spec["top"])
        self.expert_size, self.shared_size = int(spec["expert_size"]), int(spec.get("shared_size", 0))
        if min(self.experts, self.top, self.expert_size) <= 0 or self.top > self.experts or self.shared_size < 0:
            raise invalid_config("routed_mlp: experts, top (at most experts) and expert_size must be positive")
        self.score, self.weigh = spec.get("score", "sigmoid"), spec.get("weigh", "input")
        self.activation = spec.get("activation", "silu")
        self.alpha, self.limit = float(spec.get("alpha", 1.0)), float(spec.get("limit", 0.0))
        self.shared_limit = float(spec.get("shared_limit", self.limit))
        self.router_bias, self.shared_gate = bool(spec.get("router_bias", False)), bool(spec.get("shared_gate", False))
        if self.score not in ops.ROUTER_SCORES or self.weigh not in ("input", "output") or spec.get("renormalize", False):
            raise invalid_config("routed_mlp: scores are sigmoids or the softmax over the chosen logits, not renormalized, and weigh "
                                 "the expert's input or its output")
        if self.activation not in ops.GATES or (self.weigh == "input" and self.activation != "silu"):
            raise invalid_config("routed_mlp: a score that weighs the expert's input goes with the SiLU gate only")
        if self.activation == "clamped_swish" and not (self.limit > 0.0 and self.shared_limit > 0.0):
            raise invalid_config("routed_mlp: the clamped gate needs positive limits")
        if self.shared_gate and (self.shared_size == 0 or self.weigh != "output"):
            raise invalid_config("routed_mlp: a gate of the shared expert needs a shared expert, and scores that weigh results")
        if self.score == "softmax_of_chosen" and self.top > 64:
            raise invalid_config("routed_mlp: the softmax over the chosen logits takes at most 64 of them")
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.router = self.router_b = self.gate_up = self.down = None

    @classmethod
    def _prefixes(cls, spec, prefix, names):
        places = [prefix + names["expert"].format(e) for e in range(int(spec["experts"]))]
        sizes = [int(spec["expert_size"])] * len(places)
        if int(spec.get("shared_size", 0)) > 0:
            places.append(prefix + names["shared"])
            sizes.append(int(spec["shared_size"]))
        return list(zip(places, sizes))

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden = int(spec["hidden_size"])
        specs = [TensorSpec(prefix + names["router"], (int(spec["experts"]), hidden))]
        if spec.get("router_bias", False):
            specs.append(TensorSpec(prefix + names["router_bias"], (int(spec["experts"]),), init="spread"))
        if spec.get("shared_gate", False):
            specs.append(TensorSpec(prefix + names["shared_gate"], (1, hidden)))
        for place, size in cls._prefixes(spec, prefix, names):
            specs += [TensorSpec(place + names["gate"], (size, hidden)), TensorSpec(place + names["up"], (size, hidden)),
                      TensorSpec(place + names["down"], (hidden, size))]
        return specs

    def load(self, weights, prefix):
        names, keep = self.names, partial(keep_in, weights)
        router = weights[prefix + names["router"]]
        bias = weights[prefix + names["router_bias"]].to(router.dtype) if self.router_bias else None
        if self.shared_gate:
            # the gate's row stands after the experts' rows, outside the choice (its bias: none)
            router = torch.cat([router, weights[prefix + names["shared_gate"]].to(router.dtype).reshape(1, self.hidden)], dim=0)
            if bias is not None:
                bias = torch.cat([bias, torch.zeros(1, dtype=bias.dtype, device=bias.device)])
        self.router = keep(router.contiguous())
        self.router_b = keep(bias.contiguous()) if bias is not None else None
        rows, columns = [], []
        for place, size in self._prefixes(self.spec, prefix, names):
            gate, up = weights[place + names["gate"]], weights[place + names["up"]]
            rows.append(torch.stack([gate, up], dim=1).reshape(2 * size, self.hidden))
            columns.append(weights[place + names["down"]])
        self.gate_up = Linear(torch.cat(rows, dim=0).contiguous(), None, self.dtype, keep=keep)
        self.down = Linear(torch.cat(columns, dim=1).contiguous(), None, self.dtype, keep=keep)

    def forward(self, x, ctx, into=None):
        scale = ops.few_outputs(x, self.router, self.router_b, top=self.top, score=self.score, extra=1 if self.shared_gate else 0)
        hidden = ops.routed_gate(ops.as_product(self.gate_up(x)), scale, self.expert_size, self.dtype, weigh=self.weigh,
                                 shared_scaled=self.shared_gate, gate=self.activation, alpha=self.alpha, limit=self.limit,
                                 shared_limit=self.shared_limit)
        return self.down(hidden)
