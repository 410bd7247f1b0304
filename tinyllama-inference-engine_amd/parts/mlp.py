"""The SiLU-gated feed-forward: down(silu(gate(x)) * up(x)) (src/model.cpp:187-196 of the
reference; SiluMultiply, src/operators.cpp:157-159).  gate and up are one product over the
weight [2 * inter, hidden] whose rows alternate gate and up (g0, u0, g1, u1, ...): the product of
few rows then has a gate and its up in one lane and applies the activation itself."""
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


@register("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    """spec: hidden_size, intermediate_size, activation: "silu" (silu(gate) * up), or "clamped_swish" with
    `alpha` and `limit`: g = min(gate, limit), u = clamp(up, -limit, limit), g * sigmoid(alpha * g) * (u + 1);
    optionally bias (all three products have one) and names (the tensors' names after the prefix, by role:
    gate, up, down, gate_bias, up_bias, down_bias).
    Tensors: `<prefix>{gate,up,down}_proj.weight` unless `names` says otherwise."""
    graph_safe = True
    NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight",
             "gate_bias": "gate_proj.bias", "up_bias": "up_proj.bias", "down_bias": "down_proj.bias"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        self.activation = spec.get("activation", "silu")
        if self.activation not in ops.GATES:
            raise invalid_config(f"gated_mlp: activation '{self.activation}' is not implemented")
        self.alpha, self.limit = float(spec.get("alpha", 1.0)), float(spec.get("limit", 0.0))
        if self.activation == "clamped_swish" and not self.limit > 0.0:
            raise invalid_config("gated_mlp: the clamped gate needs a positive limit")
        self.bias = bool(spec.get("bias", False))
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.gate_up = self.down = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, inter = int(spec["hidden_size"]), int(spec["intermediate_size"])
        shapes = (("gate", (inter, hidden)), ("up", (inter, hidden)), ("down", (hidden, inter)))
        specs = [TensorSpec(prefix + names[role], shape) for role, shape in shapes]
        if spec.get("bias", False):
            specs += [TensorSpec(prefix + names[role + "_bias"], (shape[0],)) for role, shape in shapes]
        return specs

    def load(self, weights, prefix):
        names = self.names
        gate, up = weights[prefix + names["gate"]], weights[prefix + names["up"]]
        keep = partial(keep_in, weights)
        bias = down_bias = None
        if self.bias:
            bias = torch.stack([weights[prefix + names["gate_bias"]], weights[prefix + names["up_bias"]]], dim=1).reshape(2 * self.inter)
            down_bias = weights[prefix + names["down_bias"]]
        self.gate_up = Linear(torch.stack([gate, up], dim=1).reshape(2 * self.inter, self.hidden), bias, self.dtype, keep=keep)
        self.down = Linear(weights[prefix + names["down"]], down_bias, self.dtype, keep=keep)

    @property
    def adds_to_residual(self) -> bool:
        return True

    def takes_normed_rows(self, rows: int) -> bool:
        return self.activation == "silu" and self.gate_up.takes_rows(rows)

    def forward(self, x, ctx, into=None):
        gate = None if self.activation == "silu" else (self.activation, self.alpha, self.limit)
        hidden = self.gate_up(x, gated=True, gate=gate)
        if isinstance(hidden, ops.Product):
            hidden = ops.silu_mul(hidden, self.dtype, interleaved=True, gate=self.activation, alpha=self.alpha, limit=self.limit)
        return self.down(hidden, into=into)


@register("feed_forward", "mlp")
class PlainMLP(FeedForward):
    """down(act(up(x))), no gate.  spec: hidden_size, intermediate_size, activation: "xielu", which has two learned numbers
    (p, q): for z > 0 softplus(p) z^2 + z / 2, otherwise (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2; names (the tensors'
    names after the prefix, by role: up, down, act).
    Tensors: `<prefix>{up,down}_proj.weight`, `<prefix>act` [2] unless `names` says otherwise."""
    graph_safe = True
    NAMES = {"up": "up_proj.weight", "down": "down_proj.weight", "act": "act"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden, self.inter = int(spec["hidden_size"]), int(spec["intermediate_size"])
        self.activation = spec.get("activation", "xielu")
        if self.activation != "xielu":
            raise invalid_config(f"mlp: activation '{self.activation}' is not implemented")
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.up = self.down = self.numbers = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, inter = int(spec["hidden_size"]), int(spec["intermediate_size"])
        return [TensorSpec(prefix + names["up"], (inter, hidden)), TensorSpec(prefix + names["down"], (hidden, inter)),
                TensorSpec(prefix + names["act"], (2,), init="offset")]

    def load(self, weights, prefix):
        keep = partial(keep_in, weights)
        self.up = Linear(weights[prefix + self.names["up"]], None, self.dtype, keep=keep)
        self.down = Linear(weights[prefix + self.names["down"]], None, self.dtype, keep=keep)
        self.numbers = keep(weights[prefix + self.names["act"]].contiguous())

    def forward(self, x, ctx, into=None):
        return self.down(ops.xielu(ops.as_product(self.up(x)), self.numbers, self.dtype))
