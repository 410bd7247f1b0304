"""From a `ModelSpec` to a model that runs: the parts are looked up by kind and built with their
own parameters; nothing here names an architecture."""
from __future__ import annotations

import torch

from .. import parts as _parts  # noqa: F401  (fills the part registries)
from ..cache.manager import RunNeed
from ..config.spec import ModelSpec, TensorSpec
from .. import ops
from ..ops import ResidualUpdated
from ..registry import lookup
from ..weights.arena import keep_in


def expected_tensors(spec: ModelSpec) -> list[TensorSpec]:
    """Every tensor the model's parts expect, by full name; the list that weights are checked
    against and that random weights are drawn for (the reference's fixed list of 9 per layer + 3
    is `ExpectedTensors`, src/model_config.cpp:78-97)."""
    specs = list(lookup("embedding", spec.embedding.kind).tensor_specs(spec.embedding, spec.embedding_name))
    for layer in spec.layers:
        specs += lookup("block", layer.block).tensor_specs(layer)
    specs += lookup("norm", spec.final_norm.kind).tensor_specs(spec.final_norm, spec.final_norm_prefix)
    specs += lookup("head", spec.head.kind).tensor_specs(spec.head, spec.head_name)
    specs += list(spec.shared_tensors)
    names = [tensor.name for tensor in specs]
    if len(set(names)) != len(names):
        raise AssertionError("two parts claim the same tensor name")
    return specs


class DecoderModel:
    """Embedding, the layers in the order of `spec.runs`, final norm at the wanted rows, head."""

    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        spec.validate()
        self.spec = spec
        self.dtype = dtype
        self.device = device
        self.embedding = lookup("embedding", spec.embedding.kind)(spec.embedding, dtype, device)
        self.blocks = [lookup("block", layer.block)(layer, dtype, device) for layer in spec.layers]
        self.final_norm = lookup("norm", spec.final_norm.kind)(spec.final_norm, dtype, device)
        self.head = lookup("head", spec.head.kind)(spec.head, dtype, device)
        self.run_vectors: dict[str, torch.Tensor] = {}       # the tensors of which runs add a row to the residual, by name

    def load(self, weights) -> None:
        """weights: tensors on the device by name: a dict, or a `ResidentWeights`, which brings a
        tensor when a part asks for it and is told after each part that what it brought may go."""
        release = getattr(weights, "release", lambda: None)
        self.embedding.load(weights, self.spec.embedding_name)
        release()
        for block in self.blocks:
            block.load(weights)
            release()
        self.final_norm.load(weights, self.spec.final_norm_prefix)
        self.head.load(weights, self.spec.head_name)
        for run in self.spec.runs:
            if run.add_vector is not None and run.add_vector[0] not in self.run_vectors:
                name = run.add_vector[0]
                self.run_vectors[name] = keep_in(weights, weights[name].to(self.embedding.table.dtype).contiguous())
            if run.depth_mix is not None and run.depth_mix not in self.run_vectors:
                self.run_vectors[run.depth_mix] = keep_in(weights, weights[run.depth_mix].to(self.embedding.table.dtype).contiguous())
        release()

    @property
    def graph_safe(self) -> bool:
        """Whether a decode step of this model may be recorded into a HIP graph: every part says so."""
        parts = [self.embedding, self.final_norm, self.head, *self.blocks]
        return all(getattr(part, "graph_safe", False) for part in parts)

    def run_needs(self) -> list[RunNeed]:
        needs = []
        for run in self.spec.runs:
            block = self.blocks[run.layer]
            mixer = block.mixer
            block_state = block.state_need() if hasattr(block, "state_need") else None
            needs.append(RunNeed(cache_of=run.cache_of, cache=mixer.cache_need(), state=mixer.state_need(), block_state=block_state))
        return needs

    def forward(self, ctx, bindings) -> torch.Tensor:
        """Runs the step's tokens; returns float32 logits [wanted rows, vocab].  With `ctx.trace` (a
        dict) the named tensors of the reference's ModelTrace are left there as float32 copies:
        "embedding", per run i "layer{i}.input_norm", ".attention_output", ".post_attention_norm",
        ".mlp_output", ".output", then "final_norm" and "logits" at the wanted rows
        (src/model.cpp:98-231).  A bfloat16 step of at most 16 tokens folds the norms into its
        products when it serves; with a trace it does not, so that every name is left, unless
        `ctx.trace_serving_route` asks for the serving route, which leaves the names that exist
        as tensors there."""
        runs = self.spec.runs
        trace = getattr(ctx, "trace", None)
        if runs[0].depth_mix is not None:
            return self._forward_depth_mixed(ctx, bindings)
        few = ops.few_rows_route(ctx.num_tokens, self.dtype) and (trace is None or getattr(ctx, "trace_serving_route", False))

        def entry_norm(block):
            # a block may say which norm reads the residual first (its writer can then leave that
            # norm's inputs); a block that does not is handed a plain residual
            return block.entry_norm() if hasattr(block, "entry_norm") else None
        first_norm = entry_norm(self.blocks[runs[0].layer])
        lazy = first_norm.lazy_params() if first_norm is not None else None
        if few and hasattr(self.embedding, "forward_rows") and lazy is not None:
            residual, normed = self.embedding.forward_rows(ctx.tokens, lazy)
            pending = ResidualUpdated(normed)
        else:
            residual, pending = self.embedding.forward(ctx.tokens, ctx), None
        if trace is not None:
            trace["embedding"] = residual.float().clone()
        if self.spec.streams:
            # a residual of several streams: all start as the embedding's output; the layers work on all of them
            residual = ops.stream_spread(residual, self.spec.streams)
        for index, run in enumerate(runs):
            next_norm = entry_norm(self.blocks[runs[index + 1].layer]) if index + 1 < len(runs) else self.final_norm
            if trace is not None:
                ctx.trace_prefix = f"layer{index}."
            if run.add_embedding or run.add_vector is not None:
                # what a run takes in before it starts: the residual is brought up to date first
                if pending is not None and not isinstance(pending, ResidualUpdated):
                    self._settle(residual, pending, self.dtype)
                    pending = None
                vector = self.run_vectors[run.add_vector[0]][run.add_vector[1]] if run.add_vector is not None else None
                ops.residual_inject(residual, ctx.tokens, self.embedding.table if run.add_embedding else None, vector)
            pending = self.blocks[run.layer].forward(residual, pending, ctx, bindings[index], next_norm=next_norm)
        if ctx.num_wanted == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        if self.spec.streams:
            # what goes on is the sum of the streams, with what the last sublayer left joined first
            _, residual = ops.stream_norm(residual, pending, None, None, 0.0, self.dtype, total=True)
            pending = None
        if ctx.wants_all_rows:
            lazy = few and self.head.takes_normed_rows(residual.shape[0])
            normed = self.final_norm.add_forward(residual, pending, lazy=lazy)
        else:
            normed = self.final_norm.add_forward(residual, pending, rows=ctx.want_rows)
        logits = self.head.forward(normed)
        if trace is not None:
            if isinstance(normed, torch.Tensor):             # (folded into the head's product on the route of few rows)
                trace["final_norm"] = normed.float().clone()
            trace["logits"] = logits.clone()
        return logits


    def _forward_depth_mixed(self, ctx, bindings) -> torch.Tensor:
        """A model whose runs hand on a weighted sum over the embedding's output and all results so far.  The results
        are kept side by side for the length of the step, [runs + 2, tokens, hidden] floats: entry 0 the embedding's
        output, entry i + 1 the residual that run i works on (it starts as what the run before handed on and ends as
        the run's own result), the last entry what the last run hands on.  The norm that reads the residual next forms
        the sum in its own kernel (it adds what the run's last sublayer left, mixes, writes the next run's residual
        and norms it), so that a run costs no launch more than in a model without the mix."""
        runs = self.spec.runs
        trace = getattr(ctx, "trace", None)
        first = self.embedding.forward(ctx.tokens, ctx)
        tokens, hidden = first.shape
        history = torch.empty((len(runs) + 2, tokens, hidden), dtype=torch.float32, device=first.device)
        history[0].copy_(first)
        history[1].copy_(first)
        if trace is not None:
            trace["embedding"] = first.float().clone()
        normed = None
        logits = None
        for index, run in enumerate(runs):
            if run.add_embedding or run.add_vector is not None:
                raise ops.invalid_argument("runs that take the embedding or a vector again do not go with the mix over results")
            block = self.blocks[run.layer]
            if trace is not None:
                ctx.trace_prefix = f"layer{index}."
            kwargs = {"first_normed": normed} if normed is not None else {}
            pending = block.forward(history[index + 1], None, ctx, bindings[index], **kwargs)
            mix = dict(history=history, history_count=index + 2, history_weight=self.run_vectors[run.depth_mix])
            last = index + 1 == len(runs)
            next_norm = self.final_norm if last else self.blocks[runs[index + 1].layer].entry_norm()
            if not hasattr(next_norm, "out_dtype"):
                raise ops.invalid_argument("the mix over results is formed by the norm that follows it, which this norm cannot")
            if last and trace is None:
                if ctx.num_wanted == 0:
                    # nothing is asked for: the state is up to date, the last sum has no reader
                    return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
                rows = None if ctx.wants_all_rows else ctx.want_rows
                normed = next_norm.add_forward(history[index + 1], pending, rows=rows, mixed=history[index + 2], **mix)
            else:
                normed = next_norm.add_forward(history[index + 1], pending, mixed=history[index + 2], **mix)
                if trace is not None:
                    trace[f"layer{index}.mixed"] = history[index + 2].clone()
                    if last:
                        if ctx.num_wanted == 0:
                            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.device)
                        normed = normed if ctx.wants_all_rows else normed[ctx.want_rows.long()].contiguous()
        logits = self.head.forward(normed)
        if trace is not None:
            trace["final_norm"] = normed.float().clone()
            trace["logits"] = logits.clone()
        return logits

    @staticmethod
    def _settle(residual, pending, dtype) -> None:
        """Adds what a block handed on into the residual now (a block whose result waits for the next norm)."""
        if isinstance(pending, ops.NormedDelta):
            ops.norm_add_rmsnorm(residual, pending.product, pending.weight, pending.eps, None, pending.eps, dtype)
        else:
            residual += ops.as_product(pending).dense(torch.float32)


def build_model(spec: ModelSpec, weights, dtype: torch.dtype, device) -> DecoderModel:
    model = DecoderModel(spec, dtype, device)
    model.load(weights)
    return model
