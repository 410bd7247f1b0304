"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w (src/operators.cpp:22-45 of the reference; its
device form, src/cuda/kernels.cu:67-84).  The residual it reads is float32; the sum of squares,
the scale and the product are float32; the output is in the activation type."""
from __future__ import annotations

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..registry import register
from ..weights.arena import keep_in
from .base import Norm, NormedDelta, ResidualUpdated, as_product


@register("norm", "rms_norm")
class RMSNorm(Norm):
    """spec: size, eps; optionally offset (the stored weight w lies around zero and acts as 1 + w) and
    tensor (the tensor's name after the prefix; default "weight").  Tensor: `<prefix><tensor>` [size]."""
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.offset = bool(spec.get("offset", False))
        self.weight = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        name = prefix + str(spec.get("tensor", "weight"))
        return [TensorSpec(name, (int(spec["size"]),), init="offset" if spec.get("offset", False) else "norm")]

    def load(self, weights, prefix):
        stored = weights[prefix + str(self.spec.get("tensor", "weight"))]
        if self.offset:
            # 1 + w is formed once, in float, and kept so: bfloat16 would round the sum (near 1) to 8 bits
            self.weight = keep_in(weights, (1.0 + stored.float()).contiguous())
        else:
            self.weight = keep_in(weights, stored.contiguous())

    def forward(self, residual):
        return ops.add_rmsnorm(residual, None, self.weight, self.eps, self.dtype)

    def lazy_params(self):
        return self.weight, self.eps

    def add_forward(self, residual, delta, rows=None, lazy=False):
        if isinstance(delta, ResidualUpdated):
            # the residual holds the sum already; if its writer also left this norm's inputs and the
            # reader can fold the norm into its product, nothing is launched here
            if lazy and rows is None and delta.normed is not None:
                return delta.normed
            delta = None
        if isinstance(delta, NormedDelta):
            if delta.weight.dtype == self.weight.dtype:
                return ops.norm_add_rmsnorm(residual, delta.product, delta.weight, delta.eps, self.weight, self.eps,
                                            self.dtype, rows=rows)
            return super().add_forward(residual, delta, rows=rows)      # weights of two types: the add, then this norm
        product = as_product(delta) if delta is not None else None
        return ops.add_rmsnorm(residual, product, self.weight, self.eps, self.dtype, rows=rows)


@register("norm", "layer_norm")
class LayerNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * w + b over a row, the variance the mean of the squared deviations; mean,
    variance and the products float.  spec: size, eps; optionally bias (default True), tensor and bias_tensor (the
    tensors' names after the prefix; defaults "weight" and "bias") and out (the type of the result: "float32" for a
    reader that wants floats; default: the activation type).
    It adds what the residual still lacks in its own kernel: a product, or the two scaled products of a mixer of two
    branches (`ops.ScaledSum`).  It cannot be folded into a product (a row's mean is taken off first)."""
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.has_bias = bool(spec.get("bias", True))
        self.out_dtype = torch.float32 if spec.get("out") == "float32" else dtype
        self.weight = self.bias = None

    @classmethod
    def _names(cls, spec, prefix):
        return prefix + str(spec.get("tensor", "weight")), prefix + str(spec.get("bias_tensor", "bias"))

    @classmethod
    def tensor_specs(cls, spec, prefix):
        weight, bias = cls._names(spec, prefix)
        specs = [TensorSpec(weight, (int(spec["size"]),), init="norm")]
        if spec.get("bias", True):
            specs.append(TensorSpec(bias, (int(spec["size"]),), init="offset"))
        return specs

    def load(self, weights, prefix):
        weight, bias = self._names(self.spec, prefix)
        self.weight = keep_in(weights, weights[weight].contiguous())
        if self.has_bias:
            self.bias = keep_in(weights, weights[bias].to(self.weight.dtype).contiguous())

    def forward(self, residual):
        return ops.layer_norm(residual, None, self.weight, self.bias, self.eps, self.out_dtype)

    def add_forward(self, residual, delta, rows=None, lazy=False, **history):
        """history: `history`, `history_count`, `history_weight`, `mixed` of `ops.layer_norm`: the norm then reads a
        weighted sum over earlier residuals in the residual's place."""
        if isinstance(delta, ResidualUpdated):
            delta = None
        if isinstance(delta, NormedDelta):
            return super().add_forward(residual, delta, rows=rows)
        return ops.layer_norm(residual, delta, self.weight, self.bias, self.eps, self.out_dtype, rows=rows, **history)
