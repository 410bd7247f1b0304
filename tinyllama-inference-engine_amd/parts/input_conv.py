"""What may stand between a norm and the sublayer that reads it: h is replaced by h + conv(h), a short causal
convolution over time on each channel, conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the sequence's
start.  The last taps - 1 inputs are a request's state, which the layer's arrangement owns (a row of its block state)."""
from __future__ import annotations

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import register
from ..weights.arena import keep_in
from .base import Part


@register("sublayer_input", "residual_conv")
class ResidualConv(Part):
    """spec: size (channels), taps; optionally tensor (the name after the place; default "weight").
    Tensor: `<place><tensor>` [size, taps], no bias.  Reads float rows (the norm before it leaves floats), sums in
    float, and hands the sublayer rows of the activation type."""
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.size, self.taps = int(spec["size"]), int(spec["taps"])
        if self.size <= 0 or not 1 <= self.taps <= ops.INPUT_CONV_MAX_TAPS:
            raise invalid_config(f"residual_conv: 1 to {ops.INPUT_CONV_MAX_TAPS} taps")
        self.weight = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        return [TensorSpec(prefix + str(spec.get("tensor", "weight")), (int(spec["size"]), int(spec["taps"])))]

    def load(self, weights, prefix):
        self.weight = keep_in(weights, weights[prefix + str(self.spec.get("tensor", "weight"))].contiguous())

    def state_shape(self) -> tuple[int, int]:
        """Of a request's state: the last taps - 1 inputs, oldest first (one row at least)."""
        return (max(self.taps - 1, 1), self.size)

    def forward(self, h: torch.Tensor, ctx, state: torch.Tensor) -> torch.Tensor:
        return ops.input_conv(h, self.weight, state, ctx, self.dtype)
