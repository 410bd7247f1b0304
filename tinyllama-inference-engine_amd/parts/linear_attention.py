"""Mixers that keep a decaying matrix state per head instead of a cache of keys and values.

Per token and head, with a query q and a key k (dim values each), a value v (vdim values) and a decay w per key channel:
    S_t = diag(w_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t            (S: dim x vdim, zero before the first token)
There is no softmax and no denominator.  What a request carries from token to token is S of every head: a row of
floats in the cache manager's state area, zero when the request is admitted.  The projections are the framework's
products; positions and angles, decays and what they are made of, the state, the scan's sums and the heads' norms are
float whatever the activation type.  The three mixers differ in where the decay comes from and in what stands around
the scan (`ops.decay_scan`, csrc/decay_scan.hip):

    retention                  one fixed decay a head; q and k turned by their positions, k scaled by dim^(-1/2) after
                               that; each head's result divided by its root mean square, times silu(gate), output product
    gated_linear_attention     a decay per token and key channel, sigmoid(z)^(1/tau) with z from a low-rank product with
                               a bias; q scaled by dim^(-1/2); each head's result RMS-normed with a weight the heads
                               share, times silu(gate), output product
    token_shift_mixing         every projection reads its own blend of a token's input and the input of the token before
                               it (part of the state); a decay per token and key channel, exp(-exp(z)) with z from a
                               low-rank product through tanh plus a vector; the result is read before the token joins
                               the state, with a bonus per key channel for the current token; each head's result divided
                               by its root mean square, times a weight, times silu(gate), output product

and `side_by_side` runs two mixers on the same input and hands on their scaled sum.
"""
from __future__ import annotations

from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import lookup, register
from ..weights.arena import keep_in
from .base import Binding, Mixer, StateNeed
from .linear import Linear


def _check_sizes(kind, heads, dim, vdim):
    if min(heads, dim, vdim) <= 0:
        raise invalid_config(f"{kind}: heads, head_dim and value_dim must be positive")
    if dim > ops.SCAN_MAX_DIM:
        raise invalid_config(f"{kind}: head_dim {dim} is beyond what the scan keeps in registers ({ops.SCAN_MAX_DIM})")


@register("mixer", "retention")
class Retention(Mixer):
    """spec: hidden_size, num_heads, head_dim, value_dim, decay (one number a head), norm_eps, position (a PartSpec of a
    position encoding with a rotation table, or none), names (the tensors' names after the prefix, by role).
    Tensors: q and k [heads * head_dim, hidden]; v and gate [heads * value_dim, hidden]; o [hidden, heads * value_dim]."""
    graph_safe = True
    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "gate": "g_proj.weight", "o": "o_proj.weight"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.heads, self.d, self.dv = int(spec["num_heads"]), int(spec["head_dim"]), int(spec["value_dim"])
        _check_sizes("retention", self.heads, self.d, self.dv)
        decay = [float(value) for value in spec["decay"]]
        if len(decay) != self.heads or not all(0.0 <= value <= 1.0 for value in decay):
            raise invalid_config("retention: one decay between 0 and 1 a head")
        self.head_decay = torch.tensor(decay, dtype=torch.float32, device=device)
        self.eps = float(spec["norm_eps"])
        position = spec.get("position") or PartSpec("none")
        self.position = lookup("position_encoding", position.kind)(position, dtype, device)
        table = self.position.rotary_table()
        if table is None and position.kind != "none":
            raise invalid_config("retention: positions are a rotation table or none")
        self.inv_freq, self.rot_dim = table if table is not None else (None, 0)
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.fused = self.o = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, heads, d, dv = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"]), int(spec["value_dim"])
        shapes = (("q", (heads * d, hidden)), ("k", (heads * d, hidden)), ("v", (heads * dv, hidden)),
                  ("gate", (heads * dv, hidden)), ("o", (hidden, heads * dv)))
        return [TensorSpec(prefix + names[role], shape) for role, shape in shapes]

    def load(self, weights, prefix):
        keep = partial(keep_in, weights)
        get = lambda role: weights[prefix + self.names[role]]        # noqa: E731
        self.fused = Linear(torch.cat([get("q"), get("k"), get("v"), get("gate")], dim=0).contiguous(), None, self.dtype, keep=keep)
        self.o = Linear(get("o"), None, self.dtype, keep=keep)

    def state_need(self):
        return StateNeed(ops.decay_scan_state_shape(self.heads, self.d, self.dv), torch.float32)

    def forward(self, x, ctx, binding: Binding, into=None):
        fused = ops.as_product(self.fused(x))
        keys, values = self.heads * self.d, self.heads * self.dv
        # q and k turned, k scaled after that, and v beside them, as floats
        turned = ops.Product(ops.rotate_heads(fused, 0, ctx.positions, self.inv_freq, self.rot_dim, 2 * self.heads, self.heads,
                                              self.d, 1.0, float(self.d) ** -0.5, tail=values))
        scanned = ops.decay_scan((turned, 0), (turned, keys), (turned, 2 * keys), binding.state, ctx.seq_start, ctx.seq_slot,
                                 self.heads, self.d, self.dv, head_decay=self.head_decay, max_new=ctx.max_new)
        normed = ops.head_combine(scanned, self.heads, self.dv, self.eps, self.dtype, gate=fused, gate_col=2 * keys + values,
                                  gate_kind="silu")
        return self.o(normed)


@register("mixer", "gated_linear_attention")
class GatedLinearAttention(Mixer):
    """spec: hidden_size, num_heads, head_dim, value_dim, tau, norm_eps, names; optionally decay_rank (absent: the
    files' tensors give it).
    Tensors: q and k [heads * head_dim, hidden]; v and gate [heads * value_dim, hidden]; decay_down [rank, hidden],
    decay_up [heads * head_dim, rank] with decay_bias [heads * head_dim]; norm [value_dim] (the heads share it);
    o [hidden, heads * value_dim]."""
    graph_safe = True
    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "gate": "g_proj.weight", "o": "o_proj.weight",
             "decay_down": "gk_proj.0.weight", "decay_up": "gk_proj.1.weight", "decay_bias": "gk_proj.1.bias", "norm": "g_norm.weight"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.heads, self.d, self.dv = int(spec["num_heads"]), int(spec["head_dim"]), int(spec["value_dim"])
        _check_sizes("gated_linear_attention", self.heads, self.d, self.dv)
        self.tau, self.eps = float(spec["tau"]), float(spec["norm_eps"])
        if not self.tau > 0.0:
            raise invalid_config("gated_linear_attention: tau must be positive")
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.fused = self.o = self.down = self.up = self.up_bias = self.norm = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, heads, d, dv = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"]), int(spec["value_dim"])
        rank = int(spec.get("decay_rank") or -1)
        shapes = (("q", (heads * d, hidden)), ("k", (heads * d, hidden)), ("v", (heads * dv, hidden)),
                  ("gate", (heads * dv, hidden)), ("o", (hidden, heads * dv)), ("decay_down", (rank, hidden)),
                  ("decay_up", (heads * d, rank)), ("decay_bias", (heads * d,)))
        specs = [TensorSpec(prefix + names[role], shape) for role, shape in shapes]
        specs.append(TensorSpec(prefix + names["norm"], (dv,), init="norm"))
        return specs

    def load(self, weights, prefix):
        keep = partial(keep_in, weights)
        get = lambda role: weights[prefix + self.names[role]]        # noqa: E731
        self.fused = Linear(torch.cat([get("q"), get("k"), get("v"), get("gate")], dim=0).contiguous(), None, self.dtype, keep=keep)
        self.down = Linear(get("decay_down"), None, self.dtype, keep=keep)
        self.up = keep(get("decay_up").contiguous())
        if self.down.out_features != self.up.shape[1]:
            raise invalid_config("gated_linear_attention: the decay's two matrices do not share their inner size")
        self.up_bias = keep(get("decay_bias").to(self.up.dtype).contiguous())
        self.norm = keep(get("norm").repeat(self.heads).contiguous())         # (one entry a head and dim, as the combine kernel reads it)
        self.o = Linear(get("o"), None, self.dtype, keep=keep)

    def state_need(self):
        return StateNeed(ops.decay_scan_state_shape(self.heads, self.d, self.dv), torch.float32)

    def forward(self, x, ctx, binding: Binding, into=None):
        fused = ops.as_product(self.fused(x))
        keys, values = self.heads * self.d, self.heads * self.dv
        # (the inner product's sums stay float: what enters the decay is not rounded on its way)
        decay = ops.low_rank_decay(self.down(x, out_dtype=torch.float32), self.up, self.up_bias, "sigmoid_root", tau=self.tau)
        scanned = ops.decay_scan((fused, 0), (fused, keys), (fused, 2 * keys), binding.state, ctx.seq_start, ctx.seq_slot,
                                 self.heads, self.d, self.dv, decay=decay, q_scale=float(self.d) ** -0.5, max_new=ctx.max_new)
        normed = ops.head_combine(scanned, self.heads, self.dv, self.eps, self.dtype, weight=self.norm, gate=fused,
                                  gate_col=2 * keys + values, gate_kind="silu")
        return self.o(normed)


@register("mixer", "token_shift_mixing")
class TokenShiftMixing(Mixer):
    """spec: hidden_size, num_heads, head_dim (keys and values alike), norm_eps, names; optionally decay_rank (absent:
    the files' tensors give it).
    Tensors: shift_{r,k,v,g,w} [hidden] (the blends); r, k, v and gate [heads * head_dim, hidden]; decay_down
    [rank, hidden], decay_up [heads * head_dim, rank], decay_base [heads * head_dim]; bonus [heads, head_dim];
    norm [heads * head_dim]; o [hidden, heads * head_dim]."""
    graph_safe = True
    NAMES = {"shift_r": "mu.r", "shift_k": "mu.k", "shift_v": "mu.v", "shift_g": "mu.g", "shift_w": "mu.w", "r": "r", "k": "k",
             "v": "v", "gate": "g", "decay_down": "w1", "decay_up": "w2", "decay_base": "w0", "bonus": "u", "norm": "norm", "o": "o"}
    BLENDS = ("r", "k", "v", "g", "w")

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.heads, self.d = int(spec["num_heads"]), int(spec["head_dim"])
        _check_sizes("token_shift_mixing", self.heads, self.d, self.d)
        self.eps = float(spec["norm_eps"])
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.blends = self.products = self.down = self.up = self.base = self.bonus = self.norm = self.o = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, heads, d, rank = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"]), int(spec.get("decay_rank") or -1)
        specs = [TensorSpec(prefix + names["shift_" + blend], (hidden,), init="fraction") for blend in cls.BLENDS]
        shapes = (("r", (heads * d, hidden)), ("k", (heads * d, hidden)), ("v", (heads * d, hidden)), ("gate", (heads * d, hidden)),
                  ("decay_down", (rank, hidden)), ("decay_up", (heads * d, rank)), ("decay_base", (heads * d,)),
                  ("bonus", (heads, d)), ("o", (hidden, heads * d)))
        specs += [TensorSpec(prefix + names[role], shape) for role, shape in shapes]
        specs.append(TensorSpec(prefix + names["norm"], (heads * d,), init="norm"))
        return specs

    def load(self, weights, prefix):
        keep = partial(keep_in, weights)
        get = lambda role: weights[prefix + self.names[role]]        # noqa: E731
        self.blends = keep(torch.stack([get("shift_" + blend) for blend in self.BLENDS], dim=0).contiguous())
        self.products = [Linear(get(role), None, self.dtype, keep=keep) for role in ("r", "k", "v", "gate")]
        self.down = Linear(get("decay_down"), None, self.dtype, keep=keep)
        self.up = keep(get("decay_up").contiguous())
        if self.down.out_features != self.up.shape[1]:
            raise invalid_config("token_shift_mixing: the decay's two matrices do not share their inner size")
        self.base = keep(get("decay_base").to(self.up.dtype).contiguous())
        self.bonus = keep(get("bonus").float().reshape(-1).contiguous())        # (it enters the scan, which is float)
        self.norm = keep(get("norm").contiguous())
        self.o = Linear(get("o"), None, self.dtype, keep=keep)

    def state_need(self):
        """A row of floats: the heads' S, then the input of the token before (hidden values)."""
        heads, tiles, floats = ops.decay_scan_state_shape(self.heads, self.d, self.d)
        return StateNeed((heads * tiles * floats + self.hidden,), torch.float32)

    def forward(self, x, ctx, binding: Binding, into=None):
        shape = ops.decay_scan_state_shape(self.heads, self.d, self.d)
        scan_floats = shape[0] * shape[1] * shape[2]
        before = binding.state[:, scan_floats:]
        blended = ops.token_shift(x, self.blends, before, ctx)
        r, k, v, gate = (ops.as_product(product(blended[index])) for index, product in enumerate(self.products))
        decay = ops.low_rank_decay(self.down(blended[4], out_dtype=torch.float32), self.up, self.base, "exp_neg_exp", inner_tanh=True)
        scanned = ops.decay_scan((r, 0), (k, 0), (v, 0), binding.state, ctx.seq_start, ctx.seq_slot, self.heads, self.d, self.d,
                                 decay=decay, bonus=self.bonus, max_new=ctx.max_new)
        normed = ops.head_combine(scanned, self.heads, self.d, self.eps, self.dtype, weight=self.norm, gate=gate, gate_col=0,
                                  gate_kind="silu")
        return self.o(normed)


@register("mixer", "side_by_side")
class SideBySide(Mixer):
    """Two mixers that read the same input; the result is left_scale * left + right_scale * right.
    spec: left and right (PartSpecs of mixers), left_scale, right_scale, left_place and right_place (what their tensors'
    names continue the prefix with).  The cache manager gives a run one cache and one state row: at most one of the
    two keeps pages and at most one keeps state."""

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.left = lookup("mixer", spec["left"].kind)(spec["left"], dtype, device)
        self.right = lookup("mixer", spec["right"].kind)(spec["right"], dtype, device)
        self.left_scale, self.right_scale = float(spec["left_scale"]), float(spec["right_scale"])
        if self.left.cache_need() is not None and self.right.cache_need() is not None:
            raise invalid_config("side_by_side: only one of the two mixers may keep pages")
        if self.left.state_need() is not None and self.right.state_need() is not None:
            raise invalid_config("side_by_side: only one of the two mixers may keep state")

    @classmethod
    def tensor_specs(cls, spec, prefix):
        specs = []
        for side in ("left", "right"):
            specs += lookup("mixer", spec[side].kind).tensor_specs(spec[side], prefix + str(spec.get(side + "_place", side + ".")))
        return specs

    def load(self, weights, prefix):
        self.left.load(weights, prefix + str(self.spec.get("left_place", "left.")))
        self.right.load(weights, prefix + str(self.spec.get("right_place", "right.")))

    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.left, "graph_safe", False) and getattr(self.right, "graph_safe", False))

    def cache_need(self):
        return self.left.cache_need() or self.right.cache_need()

    def state_need(self):
        return self.left.state_need() or self.right.state_need()

    def forward(self, x, ctx, binding: Binding, into=None):
        left = ops.as_product(self.left.forward(x, ctx, binding))
        right = ops.as_product(self.right.forward(x, ctx, binding))
        return ops.ScaledSum(left, self.left_scale, right, self.right_scale)
