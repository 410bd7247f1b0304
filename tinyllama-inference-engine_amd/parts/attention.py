"""Grouped-query causal attention over the paged cache.

reference (one token at a time, src/model.cpp:140-179; src/cuda/model.cu:412-447): q, k, v
projections of the normed input; rotation of q and k; the rotated key and the value go to the
cache at the token's position; each query head h attends over the cached keys 0..pos of kv head
h // (nq / nkv) with scores scaled by 1/sqrt(d) after the dot product; the output projection
follows.  Here the three projections are one product over the concatenated weight, the rotation
and the cache write are one kernel, and all tokens of a step run together.
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
from .base import Binding, CacheNeed, Mixer, PositionEncoding
from .linear import Linear


@register("mixer", "attention")
class Attention(Mixer):
    """spec: hidden_size, num_heads, num_kv_heads, head_dim, bias, window (None or a count of
    positions), position (a PartSpec of a position encoding).  Optionally:
      value_dim          the size of a value head (default head_dim)
      scale              of the scores (default 1 / sqrt(head_dim))
      chunk              a token sees only the keys of its own chunk of so many positions, counted from 0
      sink               a learned number per head whose exponential joins the softmax's denominator
      reads_other_cache  the layer has no key and value projections: it reads the cache its run names
      cache_window       how long the cache keeps a position (default: window, or chunk); the owner of a
                         cache that other layers read names the longest reach among them (None: for good)
      softcap            c: a scaled score s enters the softmax as c * tanh(s / c)
      q_temp             (coef, every): the query at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1)
      values_are_keys    there is no value projection: a key head as projected, before any norm and rotation, is also
                         its value head
      qk_norm            "whole": all of a token's query columns together, and all of its key columns together, are
                         RMS-normed (norm_eps) with a weight of that many entries (q_norm, k_norm), before the rotation
      names              the tensors' names after the prefix, by role (q, k, v, o, q_bias .. o_bias, sink, q_norm, k_norm)
    Tensors: `<prefix>{q,k,v,o}_proj.weight` (and `.bias` when bias) unless `names` says otherwise."""
    NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
             "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias",
             "sink": "sinks", "q_norm": "q_norm.weight", "k_norm": "k_norm.weight"}

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.nq = int(spec["num_heads"])
        self.nkv = int(spec["num_kv_heads"])
        self.d = int(spec["head_dim"])
        self.bias = bool(spec.get("bias", False))
        self.window = spec.get("window")
        if self.nq <= 0 or self.nkv <= 0 or self.nq % self.nkv != 0:
            raise invalid_config("attention: num_heads must be a positive multiple of num_kv_heads")
        if not 0 < self.d <= ops.ATTENTION_MAX_HEAD_DIM:
            # said here, where the model is built, not by the first step's launch
            raise invalid_config(f"attention: head_dim {self.d} is beyond what the attention kernels take "
                                 f"(1 to {ops.ATTENTION_MAX_HEAD_DIM})")
        if self.window is not None and int(self.window) <= 0:
            raise invalid_config("attention: a window must be a positive count of positions")
        position = spec.get("position") or PartSpec("none")
        self.position = lookup("position_encoding", position.kind)(position, dtype, device)
        self.dv = int(spec.get("value_dim") or self.d)
        self.scale = float(spec["scale"]) if spec.get("scale") is not None else 1.0 / math.sqrt(float(self.d))
        self.chunk = spec.get("chunk")
        self.has_sink = bool(spec.get("sink", False))
        self.reads_other_cache = bool(spec.get("reads_other_cache", False))
        if not 0 < self.dv <= ops.ATTENTION_MAX_HEAD_DIM:
            raise invalid_config(f"attention: value_dim {self.dv} is beyond what the attention kernels take")
        if self.chunk is not None and int(self.chunk) <= 0:
            raise invalid_config("attention: a chunk must be a positive count of positions")
        if not (self.scale > 0.0 and math.isfinite(self.scale)):
            raise invalid_config("attention: the scale of the scores must be positive")
        self.softcap = float(spec["softcap"]) if spec.get("softcap") is not None else None
        self.q_temp = tuple(float(number) for number in spec["q_temp"]) if spec.get("q_temp") is not None else None
        self.values_are_keys = bool(spec.get("values_are_keys", False))
        self.qk_norm = spec.get("qk_norm")
        self.norm_eps = float(spec.get("norm_eps", 0.0))
        if self.softcap is not None and not self.softcap > 0.0:
            raise invalid_config("attention: a cap of the scores must be positive")
        if self.q_temp is not None and (len(self.q_temp) != 2 or not self.q_temp[1] > 0.0):
            raise invalid_config("attention: a query temperature is (coef, every) with a positive period")
        if self.values_are_keys and (self.dv != self.d or self.reads_other_cache or self.bias):
            raise invalid_config("attention: values that are the keys have the keys' size, and the layer its own keys and no biases")
        if self.qk_norm not in (None, "whole") or (self.qk_norm is not None and (not self.norm_eps > 0.0 or self.reads_other_cache)):
            raise invalid_config("attention: qk_norm is \"whole\" (with a positive norm_eps, on a layer with keys of its own) or absent")
        # what the kernels that are fused for the plain case (one head size, no sink, no chunks, own keys
        # and values, scores as they are) do not take goes through the kernels for any sizes
        self.placed = self.q_temp is not None or self.values_are_keys or self.qk_norm is not None   # options of the placement kernel alone
        self.general = (self.dv != self.d or self.has_sink or self.chunk is not None or self.reads_other_cache
                        or self.softcap is not None or self.placed)
        self.names = {**self.NAMES, **dict(spec.get("names") or {})}
        self.qkv = self.o = self.sink = self.q_norm = self.k_norm = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        names = {**cls.NAMES, **dict(spec.get("names") or {})}
        hidden, d = int(spec["hidden_size"]), int(spec["head_dim"])
        dv = int(spec.get("value_dim") or d)
        nq, nkv = int(spec["num_heads"]), int(spec["num_kv_heads"])
        shapes = [("q", (nq * d, hidden))]
        if not spec.get("reads_other_cache", False):
            shapes.append(("k", (nkv * d, hidden)))
            if not spec.get("values_are_keys", False):
                shapes.append(("v", (nkv * dv, hidden)))
        shapes.append(("o", (hidden, nq * dv)))
        specs = [TensorSpec(prefix + names[role], shape) for role, shape in shapes]
        if spec.get("qk_norm") is not None:
            specs += [TensorSpec(prefix + names["q_norm"], (nq * d,), init="norm"), TensorSpec(prefix + names["k_norm"], (nkv * d,), init="norm")]
        if spec.get("bias", False):
            specs += [TensorSpec(prefix + names[role + "_bias"], (shape[0],)) for role, shape in shapes]
        if spec.get("sink", False):
            specs.append(TensorSpec(prefix + names["sink"], (nq,)))
        return specs

    def load(self, weights, prefix):
        # The rows of the fused q/k/v weight are stored with the two elements of a rotation pair
        # side by side when the position encoding is a rotation table: the product of few rows then
        # rotates and writes the cache itself; the kernels that read its output know the order.
        # (Not on the route for any sizes, whose kernel takes the columns in their natural order.)
        table = self.position.rotary_table()
        self.paired = table is not None and not self.general
        order = ops.paired_rows(self.nq, self.nkv, self.d, table[1]).to(self.device) if self.paired else None
        names = self.names
        roles = ("q",) if self.reads_other_cache else (("q", "k") if self.values_are_keys else ("q", "k", "v"))

        def cat(suffix):
            joined = torch.cat([weights[prefix + names[role + suffix]] for role in roles], dim=0)
            return joined[order].contiguous() if order is not None else joined
        keep = partial(keep_in, weights)
        self.qkv = Linear(cat(""), cat("_bias") if self.bias else None, self.dtype, keep=keep)
        self.o = Linear(weights[prefix + names["o"]], weights.get(prefix + names["o_bias"]) if self.bias else None,
                        self.dtype, keep=keep)
        if self.has_sink:
            self.sink = keep(weights[prefix + names["sink"]].float().contiguous())     # (it enters the softmax, which is float)
        if self.qk_norm is not None:                       # (norms are float)
            self.q_norm = keep(weights[prefix + names["q_norm"]].float().contiguous())
            self.k_norm = keep(weights[prefix + names["k_norm"]].float().contiguous())

    @property
    def graph_safe(self) -> bool:
        # a rotation table (or none) is fused into this part's own kernels; a position encoding applied
        # as tensors (`apply_qk`) may do anything, so it says itself whether its launches may be recorded
        if self.position.rotary_table() is not None or type(self.position).apply_qk is PositionEncoding.apply_qk:
            return True
        return bool(getattr(self.position, "graph_safe", False))

    @property
    def adds_to_residual(self) -> bool:
        return not self.general

    def takes_normed_rows(self, rows: int) -> bool:
        return not self.general and self.qkv.takes_rows(rows)

    def cache_need(self):
        """A page holds two planes per kv head, [2, nkv, page_size * d]: the rotated keys as
        [position][dim] and the values transposed, [dim][position], which is how the attention
        kernels want them as matrix operands (`ops.rope_cache` writes them so).  With value heads of a
        size dv of their own a page is [nkv, page_size * (d + dv)]: the planes of keys, then those of values."""
        keep = self.window if self.window is not None else self.chunk       # (a chunk's first position is never further back)
        if "cache_window" in self.spec.params:
            keep = self.spec["cache_window"]
        keep = int(keep) if keep is not None else None
        if self.dv != self.d:
            return CacheNeed((self.nkv,), self.d + self.dv, keep)
        return CacheNeed((2, self.nkv), self.d, keep)

    def _forward_general(self, x, ctx, binding: Binding):
        """Any sizes and masks: the product, a kernel that rotates (if there is a rotation) and places q, k
        and v, the plain attention kernel (softmax and scores float), the output product."""
        pages = ctx.groups[binding.group]
        table = self.position.rotary_table()
        if table is None and type(self.position).apply_qk is not PositionEncoding.apply_qk:
            raise invalid_config("attention: a position encoding that is no rotation table goes with the plain options only")
        inv_freq, rot_dim = table if table is not None else (None, 0)
        writes = binding.writes and not self.reads_other_cache
        q = None
        if (table is None and self.dv == self.d and self.d % 2 == 0 and not self.reads_other_cache and not self.placed
                and self.qkv.takes_rows(x.shape[0])):
            # a step of few rows, one head size, own keys and values: the product places q and writes the cache itself
            q = self.qkv(x, rope=ops.RopeTarget(ctx.positions, pages.slot_map if writes else ctx.no_slots, None, 0, binding.cache,
                                                self.nq, self.nkv, self.d))
        if q is None or isinstance(q, ops.Product):
            q = ops.qkv_place(ops.as_product(q if q is not None else self.qkv(x)), ctx.positions, pages.slot_map if writes else ctx.no_slots, inv_freq,
                          rot_dim, binding.cache, self.nq, 0 if self.reads_other_cache else self.nkv, self.d, self.dv, self.dtype,
                          q_norm=self.q_norm, k_norm=self.k_norm, norm_eps=self.norm_eps, values_are_keys=self.values_are_keys,
                          q_temp=self.q_temp)
        if self.dv == self.d and ops.attention_mfma_takes(self.dtype, self.d, binding.cache.shape[3] // self.d):
            # bfloat16, one head size: the kernel on the matrix cores (scores, softmax and sink float)
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, self.nq // self.nkv, self.nkv, self.d)
            attended = ops.attention_mfma(q, binding.cache, pages.block_table, tiles, ctx.positions, self.nq, self.nkv, self.d,
                                          self.window, self.scale, nsplit, split_len, col_tiles, waves, shared,
                                          chunk=self.chunk, sink=self.sink, softcap=self.softcap)
        else:
            attended = ops.attention_generic(q, binding.cache, pages.block_table, ctx.token_seq, ctx.positions, self.nq, self.nkv,
                                             self.d, self.window, self.scale, tiled=ops.attention_generic_plan(ctx, self.d, self.dv),
                                             seq_start=ctx.seq_start, value_dim=self.dv, chunk=self.chunk, sink=self.sink,
                                             softcap=self.softcap)
        return self.o(attended)

    def forward(self, x, ctx, binding: Binding, into=None):
        if self.general:
            return self._forward_general(x, ctx, binding)
        pages = ctx.groups[binding.group]
        slot_map = pages.slot_map if binding.writes else ctx.no_slots
        table = self.position.rotary_table()
        inv_freq, rot_dim = table if table is not None else (None, 0)
        other_positions = table is None and type(self.position).apply_qk is not PositionEncoding.apply_qk
        target = None
        if not other_positions:
            target = ops.RopeTarget(ctx.positions, slot_map, inv_freq, rot_dim, binding.cache, self.nq, self.nkv, self.d)
        q = self.qkv(x, rope=target)
        if isinstance(q, ops.Product):              # the product did not rotate: a kernel of its own does
            if other_positions:
                q = self._apply_other_positions(q, ctx)
            q = ops.rope_cache(q, ctx.positions, slot_map, inv_freq, rot_dim, binding.cache, self.nq, self.nkv, self.d,
                               self.dtype, paired=self.paired)
        page_size = binding.cache.shape[3] // self.d
        if ops.attention_mfma_takes(self.dtype, self.d, page_size):
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, self.nq // self.nkv, self.nkv, self.d)
            attended = ops.attention_mfma(q, binding.cache, pages.block_table, tiles, ctx.positions, self.nq, self.nkv,
                                          self.d, self.window, self.scale, nsplit, split_len, col_tiles, waves, shared)
        else:
            attended = ops.attention_generic(q, binding.cache, pages.block_table, ctx.token_seq, ctx.positions, self.nq,
                                             self.nkv, self.d, self.window, self.scale,
                                             tiled=ops.attention_generic_plan(ctx, self.d), seq_start=ctx.seq_start)
        return self.o(attended, into=into)

    def _apply_other_positions(self, qkv, ctx):
        """A position encoding that is no rotation table: applied to q and k as tensors."""
        dense = qkv.dense(self.dtype)
        qd, kvd = self.nq * self.d, self.nkv * self.d
        q, k = self.position.apply_qk(dense[:, :qd].reshape(-1, self.nq, self.d),
                                      dense[:, qd:qd + kvd].reshape(-1, self.nkv, self.d), ctx.positions)
        joined = torch.cat([q.reshape(-1, qd), k.reshape(-1, kvd), dense[:, qd + kvd:]], dim=1).contiguous()
        return ops.Product(joined, 1)
