"""The two ends of the model: the token embedding and the output head.

reference: the embedding is a row copy, unscaled (src/model.cpp:94-97); the head is a plain
product of the final norm's output with `lm_head.weight`, no bias, no scaling
(src/model.cpp:224-225).  With tied embeddings the head's matrix is the embedding table.
Logits are float32 whatever the activation type."""
from __future__ import annotations

from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..registry import lookup, register
from ..weights.arena import keep_in
from .base import Part
from .linear import Linear


@register("embedding", "token_embedding")
class TokenEmbedding(Part):
    graph_safe = True
    NAME = "model.embed_tokens.weight"

    def __init__(self, spec: PartSpec, dtype, device):
        """spec: vocab_size, hidden_size; optionally norm (a PartSpec of a norm whose result, as floats, is the
        embedding's output) and norm_prefix (where that norm's tensors lie: a full name's start)."""
        super().__init__(spec, dtype, device)
        self.table = None
        self.norm = None
        if spec.get("norm") is not None:
            norm = spec["norm"]
            norm = PartSpec(norm.kind, {**dict(norm.params), "out": "float32"})
            self.norm = lookup("norm", norm.kind)(norm, dtype, device)
            if getattr(self.norm, "out_dtype", None) != torch.float32:
                raise ops.invalid_argument(f"the embedding's norm '{norm.kind}' cannot leave floats")

    @classmethod
    def tensor_specs(cls, spec, name=""):
        """`name`: the table's full name in the checkpoint (the model's spec gives it; without one,
        the reference's)."""
        specs = [TensorSpec(name or cls.NAME, (int(spec["vocab_size"]), int(spec["hidden_size"])))]
        if spec.get("norm") is not None:
            specs += lookup("norm", spec["norm"].kind).tensor_specs(spec["norm"], str(spec.get("norm_prefix", "")))
        return specs

    def load(self, weights, name=""):
        self.table = keep_in(weights, weights[name or self.NAME].contiguous())
        if self.norm is not None:
            self.norm.load(weights, str(self.spec.get("norm_prefix", "")))

    def forward(self, tokens: torch.Tensor, ctx=None) -> torch.Tensor:
        """The float32 residual [T, H] of the step's tokens.  `ctx` is the step's context: an
        embedding that depends on more than the token (positions learned per place, say) reads it."""
        rows = ops.embed_gather(tokens, self.table)
        return rows if self.norm is None else self.norm.forward(rows)

    def forward_rows(self, tokens: torch.Tensor, next_norm: tuple):
        """For a step of few rows: the residual and the first norm's inputs in one launch."""
        return ops.embed_rows(tokens, self.table, next_norm)


@register("head", "lm_head")
class LMHead(Part):
    graph_safe = True
    NAME = "lm_head.weight"

    def __init__(self, spec: PartSpec, dtype, device):
        """spec: vocab_size, hidden_size, tied (the head's matrix is the embedding's table), and, when
        tied, optionally tied_to: that table's full name (default: the reference's); optionally scale, a factor
        of the logits (applied to the float sums), and softcap c: the logits leave as c * tanh(logits / c)."""
        super().__init__(spec, dtype, device)
        self.tied = bool(spec.get("tied", False))
        self.tied_to = spec.get("tied_to") or TokenEmbedding.NAME
        self.scale = float(spec.get("scale", 1.0))       # what the logits are multiplied by
        self.softcap = float(spec["softcap"]) if spec.get("softcap") is not None else None
        if self.softcap is not None and not self.softcap > 0.0:
            raise ops.invalid_argument("lm_head: a cap of the logits must be positive")
        self.linear = None

    @classmethod
    def tensor_specs(cls, spec, name=""):
        shape = (int(spec["vocab_size"]), int(spec["hidden_size"]))
        # a tied model may still carry the head's matrix; it is then not read
        return [TensorSpec(name or cls.NAME, shape, optional=bool(spec.get("tied", False)))]

    def load(self, weights, name=""):
        matrix = weights[self.tied_to] if self.tied else weights[name or self.NAME]
        self.linear = Linear(matrix, None, self.dtype, keep=partial(keep_in, weights))

    def takes_normed_rows(self, rows: int) -> bool:
        return self.linear.takes_rows(rows)

    def forward(self, normed) -> torch.Tensor:
        logits = self.linear(normed, out_dtype=torch.float32, whole=True).dense(torch.float32)
        if self.scale != 1.0:
            logits = logits.mul_(self.scale)
        return logits if self.softcap is None else ops.softcap(logits.contiguous(), self.softcap)
