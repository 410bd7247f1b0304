"""How a layer's parts are arranged.

"pre_norm" is the reference's block (src/model.cpp:132-203): x += mixer(norm(x)), then
x += feed_forward(norm(x)); the residual itself is never normed in place.  The residual is a
float32 array that lives for the whole step.  A block does not add its last result itself: it
hands it on as `pending`, and whoever norms the residual next (the next block's first norm, or
the model's final norm) adds it in the same kernel.
"""
from __future__ import annotations

import torch

from ..config.spec import LayerSpec
from .. import ops
from ..ops import ResidualUpdated, as_product
from ..registry import lookup, register
from .base import ResidualTarget


@register("block", "pre_norm")
class PreNormBlock:
    """x += mixer(norm(x)), then, if the layer has a feed-forward, x += feed_forward(norm(x)).  With
    `LayerSpec.sublayer_input` a part of the "sublayer_input" table stands between each norm and its sublayer (built
    once for each); what such parts keep per request is this block's state, one row of it each."""

    def __init__(self, layer: LayerSpec, dtype, device):
        from ..config.spec import PartSpec
        from ..errors import invalid_config
        self.layer = layer
        self.dtype = dtype
        between = layer.sublayer_input

        def norm(spec):
            if between is not None:         # what stands behind the norm reads floats
                spec = PartSpec(spec.kind, {**dict(spec.params), "out": "float32"})
            built = lookup("norm", spec.kind)(spec, dtype, device)
            if between is not None and getattr(built, "out_dtype", None) != torch.float32:
                raise invalid_config(f"a norm '{spec.kind}' cannot leave floats for what stands between it and its sublayer")
            return built
        self.mixer_norm = norm(layer.mixer_norm)
        self.mixer = lookup("mixer", layer.mixer.kind)(layer.mixer, dtype, device)
        self.feed_forward_norm = self.feed_forward = self.mixer_input = self.feed_forward_input = None
        if layer.feed_forward is not None:
            self.feed_forward_norm = norm(layer.feed_forward_norm)
            self.feed_forward = lookup("feed_forward", layer.feed_forward.kind)(layer.feed_forward, dtype, device)
        if between is not None:
            self.mixer_input = lookup("sublayer_input", between.kind)(between, dtype, device)
            if self.feed_forward is not None:
                self.feed_forward_input = lookup("sublayer_input", between.kind)(between, dtype, device)
        # the route on which norms are folded into products and products add into the residual is for the plain layer
        self.plain = between is None and self.feed_forward is not None

    @classmethod
    def _parts(cls, layer: LayerSpec):
        """(attribute, registry table, the layer's spec of it) of the parts this layer has."""
        parts = [("mixer_norm", "norm", layer.mixer_norm), ("mixer", "mixer", layer.mixer)]
        if layer.sublayer_input is not None:
            parts.append(("mixer_input", "sublayer_input", layer.sublayer_input))
        if layer.feed_forward is not None:
            parts += [("feed_forward_norm", "norm", layer.feed_forward_norm), ("feed_forward", "feed_forward", layer.feed_forward)]
            if layer.sublayer_input is not None:
                parts.append(("feed_forward_input", "sublayer_input", layer.sublayer_input))
        return parts

    @staticmethod
    def _place(layer: LayerSpec, attribute: str) -> str:
        """Where a part's tensors lie: the layer's prefix and the place the layer's spec names."""
        return layer.prefix + getattr(layer, attribute + "_place")

    @classmethod
    def tensor_specs(cls, layer: LayerSpec):
        specs = []
        for attribute, table, part_spec in cls._parts(layer):
            specs += lookup(table, part_spec.kind).tensor_specs(part_spec, cls._place(layer, attribute))
        return specs

    def load(self, weights):
        for attribute, _, _ in self._parts(self.layer):
            getattr(self, attribute).load(weights, self._place(self.layer, attribute))

    def state_need(self):
        """What the parts between norms and sublayers keep per request: a row each, [parts, rows, channels]."""
        from .base import StateNeed
        inputs = [part for part in (self.mixer_input, self.feed_forward_input) if part is not None]
        if not inputs:
            return None
        return StateNeed((len(inputs), *inputs[0].state_shape()), torch.float32)

    def entry_norm(self):
        """The norm that reads the residual first in this block: whoever writes the residual before
        the block (the embedding, the block before) may leave that norm's inputs with it."""
        return self.mixer_norm

    @property
    def graph_safe(self) -> bool:
        return all(getattr(getattr(self, attribute), "graph_safe", False) for attribute, _, _ in self._parts(self.layer))

    def forward(self, residual, pending, ctx, binding, next_norm=None, first_normed=None):
        """`pending`: what the residual still lacks (a product, a `ResidualUpdated`, or None).
        `next_norm`: the norm that reads the residual after this block, if the caller knows it.
        `first_normed`: the first norm's result, if whoever wrote the residual has formed it already.
        In a step of few rows the parts that offer it fold the norms into their products and add
        their results into the residual themselves; otherwise the norm kernels do both.
        A step that keeps a trace (`ctx.trace`, a dict) leaves there, under `ctx.trace_prefix`, the
        five tensors the reference's ModelTrace keeps per layer
        (src/model.cpp:136-138,176-177,184-185,200-201,204-205), as float32 copies, and takes the route
        on which all five exist; with `ctx.trace_serving_route` a step of few rows takes the route
        it takes without a trace and leaves those that still exist there: "attention_output" and
        "mlp_output" (what the part added into the residual: the residual after it minus the
        residual before) and "output" (the normed inputs are folded away)."""
        trace = getattr(ctx, "trace", None)
        rows = residual.shape[0]
        if not self.plain:
            return self._forward_general(residual, pending, ctx, binding, first_normed)
        few = ops.few_rows_route(rows, self.dtype) and (trace is None or getattr(ctx, "trace_serving_route", False))
        if trace is not None and not few:
            return self._forward_traced(residual, pending, ctx, binding)

        def keep(name, tensor):
            trace[ctx.trace_prefix + name] = tensor.float().clone()
        normed = self.mixer_norm.add_forward(residual, pending, lazy=few and self.mixer.takes_normed_rows(rows))
        before = residual.clone() if trace is not None else None
        if few and self.mixer.adds_to_residual:
            mixed = self.mixer.forward(normed, ctx, binding, into=ResidualTarget(residual, self.feed_forward_norm.lazy_params()))
        else:
            mixed = self.mixer.forward(normed, ctx, binding)
        normed = self.feed_forward_norm.add_forward(residual, mixed, lazy=few and self.feed_forward.takes_normed_rows(rows))
        if trace is not None:
            keep("attention_output", residual - before)        # (whoever added it, the residual holds it now)
            before = residual.clone()
        if few and self.feed_forward.adds_to_residual:
            out = self.feed_forward.forward(normed, ctx, into=ResidualTarget(
                residual, next_norm.lazy_params() if next_norm is not None else None))
        else:
            out = self.feed_forward.forward(normed, ctx)
        if trace is not None:
            added = residual - before if isinstance(out, ResidualUpdated) else as_product(out).dense(torch.float32)
            keep("mlp_output", added)
            keep("output", before + added)
        return out

    def _forward_general(self, residual, pending, ctx, binding, first_normed=None):
        """A layer without a feed-forward, or with parts between its norms and sublayers: norm, that part, sublayer,
        one after the other; the last result is handed on.  With a trace: "input_norm" and "post_attention_norm" are
        what the sublayers read, "attention_output" and "mlp_output" their results, "output" the residual afterwards
        (the block then adds its last result itself and hands on nothing)."""
        trace = getattr(ctx, "trace", None)

        def keep(name, tensor):
            if trace is not None:
                trace[ctx.trace_prefix + name] = tensor.float().clone()
        normed = first_normed if first_normed is not None else self.mixer_norm.add_forward(residual, pending)
        if self.mixer_input is not None:
            normed = self.mixer_input.forward(normed, ctx, binding.block_state[:, 0])
        keep("input_norm", normed)
        out = self.mixer.forward(normed, ctx, binding)
        if trace is not None:
            keep("attention_output", as_product(out).dense(torch.float32))
        if self.feed_forward is not None:
            normed = self.feed_forward_norm.add_forward(residual, out)
            if self.feed_forward_input is not None:
                normed = self.feed_forward_input.forward(normed, ctx, binding.block_state[:, 1])
            keep("post_attention_norm", normed)
            out = self.feed_forward.forward(normed, ctx)
            if trace is not None:
                keep("mlp_output", as_product(out).dense(torch.float32))
        if trace is None:
            return out
        residual += as_product(out).dense(torch.float32)
        keep("output", residual)
        return None

    def _forward_traced(self, residual, pending, ctx, binding):
        def keep(name, tensor):
            ctx.trace[ctx.trace_prefix + name] = tensor.float().clone()

        def dense(result):
            return as_product(result).dense(torch.float32)
        normed = self.mixer_norm.add_forward(residual, pending)
        keep("input_norm", normed)
        mixed = self.mixer.forward(normed, ctx, binding)
        keep("attention_output", dense(mixed))
        normed = self.feed_forward_norm.add_forward(residual, mixed)
        keep("post_attention_norm", normed)
        out = self.feed_forward.forward(normed, ctx)
        keep("mlp_output", dense(out))
        keep("output", residual + dense(out))
        return out


@register("block", "sandwich_norm")
class SandwichNormBlock:
    """x += post1(mixer(pre1(x))), then, if the layer has a feed-forward, x += post2(feed_forward(pre2(x))):
    every sublayer's result is normed before it joins the residual.  The block does neither add itself:
    a result waits, with its norm's weight, as a `NormedDelta`, and whoever norms the residual next
    (this block's second norm, the next block's first, the model's last) norms it, adds it and norms
    the sum in one kernel.  The post norms must be foldable that way (`lazy_params`)."""

    _NORMS = ("mixer_norm", "mixer_post_norm", "feed_forward_norm", "feed_forward_post_norm")

    def __init__(self, layer: LayerSpec, dtype, device):
        from ..errors import invalid_config
        self.layer = layer
        self.dtype = dtype
        if layer.mixer_post_norm is None:
            raise invalid_config("a sandwich_norm layer needs a norm after its mixer")
        if layer.feed_forward is not None and layer.feed_forward_post_norm is None:
            raise invalid_config("a sandwich_norm layer with a feed-forward needs a norm after it")

        def norm(spec):
            return lookup("norm", spec.kind)(spec, dtype, device)
        self.mixer_norm = norm(layer.mixer_norm)
        self.mixer = lookup("mixer", layer.mixer.kind)(layer.mixer, dtype, device)
        self.mixer_post_norm = norm(layer.mixer_post_norm)
        self.feed_forward = self.feed_forward_norm = self.feed_forward_post_norm = None
        if layer.feed_forward is not None:
            self.feed_forward_norm = norm(layer.feed_forward_norm)
            self.feed_forward = lookup("feed_forward", layer.feed_forward.kind)(layer.feed_forward, dtype, device)
            self.feed_forward_post_norm = norm(layer.feed_forward_post_norm)
        for post in (self.mixer_post_norm, self.feed_forward_post_norm):
            if post is not None and post.lazy_params() is None:
                raise invalid_config("a sandwich_norm layer's post norms must be RMS norms that can be folded into the add")

    @classmethod
    def _parts(cls, layer: LayerSpec):
        """(attribute, registry table) of the parts this layer has, in the order they run."""
        parts = [("mixer_norm", "norm"), ("mixer", "mixer"), ("mixer_post_norm", "norm")]
        if layer.feed_forward is not None:
            parts += [("feed_forward_norm", "norm"), ("feed_forward", "feed_forward"), ("feed_forward_post_norm", "norm")]
        return parts

    @classmethod
    def tensor_specs(cls, layer: LayerSpec):
        specs = []
        for attribute, table in cls._parts(layer):
            part_spec = getattr(layer, attribute)
            specs += lookup(table, part_spec.kind).tensor_specs(part_spec, layer.prefix + getattr(layer, attribute + "_place"))
        return specs

    def load(self, weights):
        for attribute, _ in self._parts(self.layer):
            getattr(self, attribute).load(weights, self.layer.prefix + getattr(self.layer, attribute + "_place"))

    def entry_norm(self):
        """None: what is written into the residual before this block is not this block's first norm's
        input yet (a result may still wait to be normed and added)."""
        return None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(getattr(self, attribute), "graph_safe", False) for attribute, _ in self._parts(self.layer))

    def forward(self, residual, pending, ctx, binding, next_norm=None):
        """A step that keeps a trace leaves, under `ctx.trace_prefix`, "input_norm", "attention_output"
        (the mixer's result before its norm), and with a feed-forward "post_attention_norm" and
        "mlp_output" (before its norm), then "output", the residual after the layer; it brings
        the residual up to date itself and hands on nothing."""
        trace = getattr(ctx, "trace", None)

        def keep(name, tensor):
            if trace is not None:
                trace[ctx.trace_prefix + name] = tensor.float().clone()

        def waiting(result, post):
            weight, eps = post.lazy_params()
            return ops.NormedDelta(as_product(result), weight, eps)
        normed = self.mixer_norm.add_forward(residual, pending)
        keep("input_norm", normed)
        out = waiting(self.mixer.forward(normed, ctx, binding), self.mixer_post_norm)
        if trace is not None:
            keep("attention_output", out.product.dense(torch.float32))
        if self.feed_forward is not None:
            normed = self.feed_forward_norm.add_forward(residual, out)
            keep("post_attention_norm", normed)
            out = waiting(self.feed_forward.forward(normed, ctx), self.feed_forward_post_norm)
            if trace is not None:
                keep("mlp_output", out.product.dense(torch.float32))
        if trace is None:
            return out
        ops.norm_add_rmsnorm(residual, out.product, out.weight, out.eps, None, out.eps, self.dtype)
        keep("output", residual)
        return None


@register("block", "parallel")
class ParallelBlock:
    """x += scale * (mixer(norm(x)) + feed_forward(norm(x))): one norm, whose output both sublayers read; the
    feed-forward is optional.  After that, if the layer has one, an input that depends on the step's tokens (a part
    of the "layer_input" table) joins the residual.  The block brings the residual up to date with the two results
    itself, in one kernel; a layer input is normed before it joins and is handed on as a `NormedDelta`, which whoever
    norms the residual next norms, adds and norms in one kernel."""

    def __init__(self, layer: LayerSpec, dtype, device):
        self.layer = layer
        self.dtype = dtype
        self.scale = float(layer.residual_scale)
        self.mixer_norm = lookup("norm", layer.mixer_norm.kind)(layer.mixer_norm, dtype, device)
        self.mixer = lookup("mixer", layer.mixer.kind)(layer.mixer, dtype, device)
        self.feed_forward = self.layer_input = None
        if layer.feed_forward is not None:
            self.feed_forward = lookup("feed_forward", layer.feed_forward.kind)(layer.feed_forward, dtype, device)
        if layer.layer_input is not None:
            self.layer_input = lookup("layer_input", layer.layer_input.kind)(layer.layer_input, dtype, device)

    @classmethod
    def _parts(cls, layer: LayerSpec):
        """(attribute, registry table) of the parts this layer has, in the order they run."""
        parts = [("mixer_norm", "norm"), ("mixer", "mixer")]
        if layer.feed_forward is not None:
            parts.append(("feed_forward", "feed_forward"))
        if layer.layer_input is not None:
            parts.append(("layer_input", "layer_input"))
        return parts

    @classmethod
    def tensor_specs(cls, layer: LayerSpec):
        specs = []
        for attribute, table in cls._parts(layer):
            part_spec = getattr(layer, attribute)
            specs += lookup(table, part_spec.kind).tensor_specs(part_spec, layer.prefix + getattr(layer, attribute + "_place"))
        return specs

    def load(self, weights):
        for attribute, _ in self._parts(self.layer):
            getattr(self, attribute).load(weights, self.layer.prefix + getattr(self.layer, attribute + "_place"))

    def entry_norm(self):
        return None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(getattr(self, attribute), "graph_safe", False) for attribute, _ in self._parts(self.layer))

    def forward(self, residual, pending, ctx, binding, next_norm=None):
        """A step that keeps a trace leaves, under `ctx.trace_prefix`, "input_norm", "attention_output" (the mixer's
        result), "mlp_output" (the feed-forward's, if there is one) and "output", the residual after the layer."""
        trace = getattr(ctx, "trace", None)

        def keep(name, tensor):
            if trace is not None:
                trace[ctx.trace_prefix + name] = tensor.float().clone()
        normed = self.mixer_norm.add_forward(residual, pending)
        keep("input_norm", normed)
        mixed = as_product(self.mixer.forward(normed, ctx, binding))
        if trace is not None:
            keep("attention_output", mixed.dense(torch.float32))
        fed = None
        if self.feed_forward is not None:
            fed = as_product(self.feed_forward.forward(normed, ctx))
            if trace is not None:
                keep("mlp_output", fed.dense(torch.float32))
            if fed.data.dtype != mixed.data.dtype:       # (products of two kernels: as floats, so that one kernel adds both)
                mixed, fed = ops.Product(mixed.dense(torch.float32).contiguous()), ops.Product(fed.dense(torch.float32).contiguous())
        if self.layer_input is None:
            ops.residual_update(residual, mixed, fed, self.scale)
            keep("output", residual)
            return None
        copy = ops.residual_update(residual, mixed, fed, self.scale, copy_dtype=self.layer_input.copy_dtype())
        waiting = self.layer_input.forward(residual, copy, ctx)
        if trace is None:
            return waiting
        ops.norm_add_rmsnorm(residual, waiting.product, waiting.weight, waiting.eps, None, waiting.eps, self.dtype)
        keep("output", residual)
        return None


@register("block", "hyper_connections")
class HyperConnectionBlock:
    """A pre-norm layer on a residual of S streams x_1 .. x_S (`LayerSpec.streams`; float32 [S, tokens, hidden]).  For the
    mixer and then, if the layer has one, the feed-forward, each with three tensors of its own (`in` [S], `mix` [S, S],
    `out` [S]):
        u = sum_s in[s] x_s;   y = sublayer(norm(u));   x_t <- sum_s mix[s, t] x_s + out[t] * y   (all streams at once)
    The block does not bring the streams up to date itself: a result waits as an `ops.StreamUpdate`, and the kernel that
    forms the next sublayer's u (this block's, the next block's, or the model's sum over the streams at the end) applies
    it first.  The norms must be RMS norms that hand out their weight (`lazy_params`)."""

    def __init__(self, layer: LayerSpec, dtype, device):
        from ..errors import invalid_config
        self.layer = layer
        self.dtype = dtype
        self.streams = int(layer.streams)
        if not 0 < self.streams <= ops.MAX_STREAMS:
            raise invalid_config(f"a hyper_connections layer works on 1 to {ops.MAX_STREAMS} streams")
        self.mixer_norm = lookup("norm", layer.mixer_norm.kind)(layer.mixer_norm, dtype, device)
        self.mixer = lookup("mixer", layer.mixer.kind)(layer.mixer, dtype, device)
        self.feed_forward = self.feed_forward_norm = None
        if layer.feed_forward is not None:
            self.feed_forward_norm = lookup("norm", layer.feed_forward_norm.kind)(layer.feed_forward_norm, dtype, device)
            self.feed_forward = lookup("feed_forward", layer.feed_forward.kind)(layer.feed_forward, dtype, device)
        for norm in (self.mixer_norm, self.feed_forward_norm):
            if norm is not None and norm.lazy_params() is None and not hasattr(norm, "weight"):
                raise invalid_config("a hyper_connections layer's norms must be RMS norms")
        self.mixer_streams = self.feed_forward_streams = None      # each (in, mix, out) as float tensors

    @classmethod
    def _parts(cls, layer: LayerSpec):
        parts = [("mixer_norm", "norm"), ("mixer", "mixer")]
        if layer.feed_forward is not None:
            parts += [("feed_forward_norm", "norm"), ("feed_forward", "feed_forward")]
        return parts

    @classmethod
    def _stream_places(cls, layer: LayerSpec):
        places = [("mixer_streams", layer.prefix + layer.mixer_streams_place)]
        if layer.feed_forward is not None:
            places.append(("feed_forward_streams", layer.prefix + layer.feed_forward_streams_place))
        return places

    @classmethod
    def tensor_specs(cls, layer: LayerSpec):
        from ..config.spec import TensorSpec
        specs = []
        for attribute, table in cls._parts(layer):
            part_spec = getattr(layer, attribute)
            specs += lookup(table, part_spec.kind).tensor_specs(part_spec, layer.prefix + getattr(layer, attribute + "_place"))
        count = int(layer.streams)
        for _, place in cls._stream_places(layer):
            specs += [TensorSpec(place + "in", (count,), init="share"), TensorSpec(place + "out", (count,), init="norm"),
                      TensorSpec(place + "mix", (count, count), init="near_identity")]
        return specs

    def load(self, weights):
        from ..weights.arena import keep_in
        for attribute, _ in self._parts(self.layer):
            getattr(self, attribute).load(weights, self.layer.prefix + getattr(self.layer, attribute + "_place"))
        for attribute, place in self._stream_places(self.layer):
            # (the residual's arithmetic is float: so are these few numbers)
            setattr(self, attribute, tuple(keep_in(weights, weights[place + name].float().contiguous()) for name in ("in", "mix", "out")))

    def entry_norm(self):
        return None

    @property
    def graph_safe(self) -> bool:
        return all(getattr(getattr(self, attribute), "graph_safe", False) for attribute, _ in self._parts(self.layer))

    def forward(self, streams, pending, ctx, binding, next_norm=None):
        """`streams`: float32 [S, tokens, hidden]; `pending`: an `ops.StreamUpdate` that the streams still lack, or None.
        A step that keeps a trace leaves, under `ctx.trace_prefix`, "input_norm", "attention_output", with a feed-forward
        "post_attention_norm" and "mlp_output", and "output", the sum of the streams after the layer (the block then
        brings the streams up to date itself and hands on nothing)."""
        trace = getattr(ctx, "trace", None)
        if streams.dim() != 3 or streams.shape[0] != self.streams:
            raise ops.invalid_shape(f"a hyper_connections layer works on [{self.streams}, tokens, hidden] streams, not {list(streams.shape)}")
        if pending is not None and not isinstance(pending, ops.StreamUpdate):
            raise ops.invalid_argument("what a residual of several streams still lacks must say how it joins them")

        def keep(name, tensor):
            if trace is not None:
                trace[ctx.trace_prefix + name] = tensor.float().clone()
        sublayers = [(self.mixer_norm, self.mixer_streams, lambda x: self.mixer.forward(x, ctx, binding), "input_norm", "attention_output")]
        if self.feed_forward is not None:
            sublayers.append((self.feed_forward_norm, self.feed_forward_streams, lambda x: self.feed_forward.forward(x, ctx),
                              "post_attention_norm", "mlp_output"))
        for norm, (read, mix, write), run, normed_name, result_name in sublayers:
            normed, _ = ops.stream_norm(streams, pending, read, norm.weight, norm.eps, self.dtype)
            keep(normed_name, normed)
            result = as_product(run(normed))
            if trace is not None:
                keep(result_name, result.dense(torch.float32))
            pending = ops.StreamUpdate(result, mix, write)
        if trace is None:
            return pending
        _, total = ops.stream_norm(streams, pending, None, None, 0.0, self.dtype, total=True)
        keep("output", total)
        return None
