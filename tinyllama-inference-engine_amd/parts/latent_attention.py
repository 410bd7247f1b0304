"""Latent attention: keys and values of all heads are functions of one low-rank vector per position,
and only that vector (and one small rotated key part that all heads share) is cached.

Per token, from the mixer's input h:
    q        = W_q h, per head [plain dims | rot dims]; the rot dims are rotated by the position
    [x | r]  = W_down h;  c = RMSNorm(x) * w (rank dims);  r (rot dims) is rotated by the position
    per head: key = [W_uk c | r], value = W_uv c;  score = (q . key) * scale;  causal softmax with a sink
    out      = W_o concat(heads)
The cache keeps c and the rotated r.  Since q_plain . (W_uk c) = (W_uk^T q_plain) . c, a head's query is
taken to the latent space before the attention (one small product per head), the attention runs over a
single key head of rank + rot dims whose values are the c themselves, and W_uv is applied per head to the
attended latent vector afterwards: the same sums in another order, and no key or value is ever expanded
for a cached position.  A page holds the rows [c | r] and, for the value side, c once more, transposed.
While a key has no more dims than the attention kernels take as a head size, the value side is as wide as
the key side (its last rot rows are never written and stay zero): the cache is then that of one key head
of rank + rot dims, in bfloat16 the kernel on the matrix cores reads it (all heads' columns of a token share
each read of a key), and the attended vector's first rank dims are what goes on.
"""
from __future__ import annotations

import math
from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import lookup, register
from ..weights.arena import keep_in
from .base import Binding, CacheNeed, Mixer
from .linear import Linear


@register("mixer", "latent_attention")
class LatentAttention(Mixer):
    """spec: hidden_size, num_heads, head_dim (a head's unrotated query/key dims), rot_dim (its rotated
    ones), value_dim, rank (of the latent vector), scale, norm_eps (of the latent vector's norm), sink (a
    learned number per head in the softmax's denominator), position (a rotation table over the first dims of the
    rot_dim part: all of them, or fewer, the rest then pass unchanged),
    window (a token sees itself and the window - 1 positions before it; absent: all), output_gate (the heads' results are
    multiplied by sigmoid(W_gate h), h the mixer's input, before the output projection),
    names (the tensors' names after the prefix, by role).
    Tensors: q [H * (head_dim + rot_dim), hidden], down [rank + rot_dim, hidden], down_norm [rank],
    up_keys [H * head_dim, rank], up_values [H * value_dim, rank], o [hidden, H * value_dim], sink [H],
    gate [H * value_dim, hidden]."""
    graph_safe = True
    NAMES = {"q": "q_proj.weight", "down": "kv_a_proj.weight", "down_norm": "kv_a_layernorm.weight",
             "up_keys": "k_b_proj.weight", "up_values": "v_b_proj.weight", "o": "o_proj.weight", "sink": "sinks",
             "gate": "gate_proj.weight"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.heads = int(spec["num_heads"])
        self.plain = int(spec["head_dim"])
        self.rot = int(spec["rot_dim"])
        self.dv = int(spec["value_dim"])
        self.rank = int(spec["rank"])
        self.scale = float(spec.get("scale") or 1.0 / math.sqrt(float(self.plain + self.rot)))
        self.norm_eps = float(spec["norm_eps"])
        self.has_sink = bool(spec.get("sink", False))
        self.window = int(spec["window"]) if spec.get("window") is not None else None
        self.output_gate = bool(spec.get("output_gate", False))
        if self.window is not None and self.window <= 0:
            raise invalid_config("latent_attention: a window must be a positive count of positions")
        if min(self.heads, self.plain, self.dv, self.rank) <= 0 or self.rot < 0:
            raise invalid_config("latent_attention: sizes must be positive")
        # A latent vector wider than the attention kernels' value heads cannot be attended over as it is: the layer then
        # expands every position's keys and values once, when the position is placed, and caches those (per head, as an
        # ordinary attention layer does); without a rotated part only.
        self.expanded = self.rank > ops.ATTENTION_MAX_HEAD_DIM
        if self.expanded and (self.rot > 0 or max(self.plain, self.dv) > ops.ATTENTION_MAX_HEAD_DIM):
            raise invalid_config(f"latent_attention: a latent vector of {self.rank} dims is beyond the attention kernel's "
                                 f"{ops.ATTENTION_MAX_HEAD_DIM} value dims, and the layer's heads cannot be expanded instead")
        # values as wide as keys while that is a head size the attention kernels take
        self.wide_values = self.rank + self.rot <= ops.ATTENTION_MAX_HEAD_DIM
        self.inv_freq, self.turn = None, 0             # turn: how many of the rot dims are rotated (the first ones)
        if self.rot > 0:
            position = spec["position"]
            table = lookup("position_encoding", position.kind)(position, dtype, device).rotary_table()
            if table is None or not 0 < table[1] <= self.rot:
                raise invalid_config("latent_attention: the position encoding must be a rotation table over at most rot_dim dims")
            self.inv_freq, self.turn = table
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.first = self.o = self.down_norm = self.up_keys = self.up_values_t = self.sink = None
        self.up_keys_rows = self.up_values_rows = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, heads, plain, rot = int(spec["hidden_size"]), int(spec["num_heads"]), int(spec["head_dim"]), int(spec["rot_dim"])
        dv, rank = int(spec["value_dim"]), int(spec["rank"])
        specs = [TensorSpec(prefix + names["q"], (heads * (plain + rot), hidden)),
                 TensorSpec(prefix + names["down"], (rank + rot, hidden)),
                 TensorSpec(prefix + names["down_norm"], (rank,), init="norm"),
                 TensorSpec(prefix + names["up_keys"], (heads * plain, rank)),
                 TensorSpec(prefix + names["up_values"], (heads * dv, rank)),
                 TensorSpec(prefix + names["o"], (hidden, heads * dv))]
        if spec.get("sink", False):
            specs.append(TensorSpec(prefix + names["sink"], (heads,)))
        if spec.get("output_gate", False):
            specs.append(TensorSpec(prefix + names["gate"], (heads * dv, hidden)))
        return specs

    def load(self, weights, prefix):
        names, keep = self.names, partial(keep_in, weights)
        # one product for the queries and the down projection (and the gate of the heads' results)
        first = [weights[prefix + names["q"]], weights[prefix + names["down"]]]
        if self.output_gate:
            first.append(weights[prefix + names["gate"]])
        self.first = Linear(torch.cat(first, dim=0), None, self.dtype, keep=keep)
        self.down_norm = keep(weights[prefix + names["down_norm"]].contiguous())
        # per head, as the block-diagonal product wants them, [inner, outer]: a head's query goes to the latent
        # space through W_uk^T (W_uk is [plain, rank] per head: already [inner, outer]); its attended latent
        # vector to its values through W_uv ([value_dim, rank] per head: transposed here)
        self.up_keys = keep(weights[prefix + names["up_keys"]].reshape(self.heads, self.plain, self.rank).contiguous())
        self.up_values_t = keep(weights[prefix + names["up_values"]].reshape(self.heads, self.dv, self.rank).transpose(1, 2).contiguous())
        # and as the product on the matrix cores wants them (steps of many rows, bfloat16), [outer, inner]
        self.up_keys_rows = self.up_values_rows = None
        if self.dtype == torch.bfloat16 and self.up_keys.dtype == torch.bfloat16:
            self.up_keys_rows = keep(self.up_keys.transpose(1, 2).contiguous())
            self.up_values_rows = keep(weights[prefix + names["up_values"]].reshape(self.heads, self.dv, self.rank).contiguous())
        self.o = Linear(weights[prefix + names["o"]], None, self.dtype, keep=keep)
        self.expand = None
        if self.expanded:
            # one product from the normed latent vector to all heads' keys and values
            self.expand = Linear(torch.cat([weights[prefix + names["up_keys"]], weights[prefix + names["up_values"]]], dim=0), None,
                                 self.dtype, keep=keep)
        if self.has_sink:
            self.sink = keep(weights[prefix + names["sink"]].float().contiguous())

    def cache_need(self):
        """One key head of rank + rot dims, [row][dim], then its value dims transposed, [dim][row]: rank of them, or
        with wide values as many as a key has."""
        if self.expanded:       # every head's keys and values, as an attention layer keeps them
            if self.dv == self.plain:
                return CacheNeed((2, self.heads), self.plain, self.window)
            return CacheNeed((self.heads,), self.plain + self.dv, self.window)
        if self.wide_values:
            return CacheNeed((2, 1), self.rank + self.rot, self.window)
        return CacheNeed((1,), 2 * self.rank + self.rot, self.window)

    def _forward_expanded(self, fused, ctx, binding: Binding):
        """The latent vector is normed, every head's keys and values are formed from it by one product and placed in pages
        of their own, and the attention runs over them head by head (window and sink as in the other form)."""
        pages = ctx.groups[binding.group]
        q_width = self.heads * self.plain
        latent = fused.dense(torch.float32)[:, q_width:q_width + self.rank].contiguous()
        c = ops.add_rmsnorm(latent, None, self.down_norm, self.norm_eps, self.dtype)
        expanded = ops.as_product(self.expand(c)).dense(self.dtype)
        qkv = ops.Product(torch.cat([fused.dense(self.dtype)[:, :q_width], expanded], dim=1).contiguous(), 1)
        q = ops.qkv_place(qkv, ctx.positions, pages.slot_map if binding.writes else ctx.no_slots, None, 0, binding.cache, self.heads,
                          self.heads, self.plain, self.dv, self.dtype)
        if self.dv == self.plain and ops.attention_mfma_takes(self.dtype, self.plain, binding.cache.shape[3] // self.plain):
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, 1, self.heads, self.plain)
            attended = ops.attention_mfma(q, binding.cache, pages.block_table, tiles, ctx.positions, self.heads, self.heads, self.plain,
                                          self.window, self.scale, nsplit, split_len, col_tiles, waves, shared, sink=self.sink)
        else:
            attended = ops.attention_generic(q, binding.cache, pages.block_table, ctx.token_seq, ctx.positions, self.heads, self.heads,
                                             self.plain, self.window, self.scale, tiled=ops.attention_generic_plan(ctx, self.plain, self.dv),
                                             seq_start=ctx.seq_start, value_dim=self.dv, sink=self.sink)
        if self.output_gate:
            ops.sigmoid_gate(attended, fused, fused.cols - self.heads * self.dv)
        return self.o(attended)

    def forward(self, x, ctx, binding: Binding, into=None):
        pages = ctx.groups[binding.group]
        key = self.rank + self.rot
        fused = ops.as_product(self.first(x))
        tokens = fused.rows
        if self.expanded:
            return self._forward_expanded(fused, ctx, binding)
        q_plain, q_wide = ops.latent_place(fused, ctx.positions, pages.slot_map if binding.writes else ctx.no_slots, self.inv_freq,
                                           self.down_norm, self.norm_eps, binding.cache, self.heads, self.plain, self.rot,
                                           self.rank, self.dtype, wide_values=self.wide_values, turn=self.turn,
                                           extra_cols=self.heads * self.dv if self.output_gate else 0)
        ops.block_linear(q_plain, 0, self.heads * self.plain, self.plain, self.up_keys, None,
                         q_wide, 0, self.heads * key, key, tokens, weight=self.up_keys_rows)
        value_dim = key if self.wide_values else self.rank
        if self.wide_values and ops.attention_mfma_takes(self.dtype, key, binding.cache.shape[-1] // key):
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, self.heads, 1, key)
            attended = ops.attention_mfma(q_wide, binding.cache, pages.block_table, tiles, ctx.positions, self.heads, 1, key,
                                          self.window, self.scale, nsplit, split_len, col_tiles, waves, shared, sink=self.sink)
        else:
            attended = ops.attention_generic(q_wide, binding.cache, pages.block_table, ctx.token_seq, ctx.positions, self.heads, 1,
                                             key, self.window, self.scale, tiled=ops.attention_generic_plan(ctx, key, value_dim),
                                             seq_start=ctx.seq_start, value_dim=value_dim, sink=self.sink)
        # (of every head's attended vector the first rank dims: with wide values the rest are zeros)
        values = torch.empty((tokens, self.heads * self.dv), dtype=self.dtype, device=attended.device)
        ops.block_linear(attended, 0, self.heads * value_dim, value_dim, self.up_values_t, None,
                         values, 0, self.heads * self.dv, self.dv, tokens, weight=self.up_values_rows)
        if self.output_gate:
            ops.sigmoid_gate(values, fused, fused.cols - self.heads * self.dv)
        return self.o(values)
