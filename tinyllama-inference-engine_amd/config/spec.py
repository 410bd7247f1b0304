"""What a configuration turns into: a description of the model as data.

A `ModelSpec` names, layer by layer, which mixer, feed-forward and norm a block is made of and
with which sizes and constants, and in which order the layers run.  Nothing below this point
reads config.json or knows an architecture's name; a part sees only its own `PartSpec`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping


@dataclass(frozen=True)
class PartSpec:
    """One part: the name it is registered under and its parameters (sizes, constants)."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass(frozen=True)
class LayerSpec:
    """One layer's parts, the prefix its tensors are stored under, and under that prefix the place
    of each part's tensors (the defaults are the names of the reference's checkpoints,
    src/model_config.cpp:81-95; an architecture whose files name them otherwise says so here)."""
    prefix: str                 # e.g. "model.layers.3."
    block: str                  # arrangement of the parts, e.g. "pre_norm"
    mixer: PartSpec
    feed_forward: PartSpec | None
    mixer_norm: PartSpec        # the norm in front of the mixer
    feed_forward_norm: PartSpec  # the norm in front of the feed-forward
    mixer_norm_place: str = "input_layernorm."
    mixer_place: str = "self_attn."
    feed_forward_norm_place: str = "post_attention_layernorm."
    feed_forward_place: str = "mlp."
    # for arrangements that also norm a sublayer's result before it joins the residual ("sandwich_norm"):
    # those norms and their places; such a layer may also have no feed-forward at all (feed_forward None)
    mixer_post_norm: PartSpec | None = None
    feed_forward_post_norm: PartSpec | None = None
    mixer_post_norm_place: str = "post_mixer_layernorm."
    feed_forward_post_norm_place: str = "post_feedforward_layernorm."
    # for arrangements that scale what the sublayers add to the residual ("parallel"): the factor
    residual_scale: float = 1.0
    # something that joins the residual after the sublayers and depends on the step's tokens (a part of the
    # "layer_input" table), and its place
    layer_input: PartSpec | None = None
    layer_input_place: str = "side."
    # something that stands between a norm and the sublayer that reads it (a part of the "sublayer_input" table, built
    # once for the mixer and once for the feed-forward), and the places of the two
    sublayer_input: PartSpec | None = None
    mixer_input_place: str = "mixer_input."
    feed_forward_input_place: str = "feed_forward_input."
    # for the arrangement on a residual of several streams ("hyper_connections"): how many streams (the model's
    # `ModelSpec.streams`), and the places of each sublayer's three tensors: `in` [S] (what the sublayer reads: a weighted
    # sum of the streams), `mix` [S, S] ([from, to]: how the streams are mixed among themselves) and `out` [S] (how much of
    # the sublayer's result each stream takes)
    streams: int = 0
    mixer_streams_place: str = "mixer_streams."
    feed_forward_streams_place: str = "feed_forward_streams."


@dataclass(frozen=True)
class Run:
    """One entry of the order in which layers run.

    `layer` indexes `ModelSpec.layers` (a layer may be named by several runs: its weights are
    then shared, each run keeps a cache of its own).  `cache_of` is the index of the run whose
    cache this run's mixer reads; a run that names itself owns a cache and writes to it, a run
    that names an earlier one only reads what that one wrote in the same step and before.
    """
    layer: int
    cache_of: int
    # What joins the residual right before this run: the embedding's output once more, and row `add_vector[1]` of
    # the tensor `add_vector[0]` ([rows, hidden]); for models that run a stretch of layers several times and
    # tell the passes apart.
    add_embedding: bool = False
    add_vector: tuple[str, int] | None = None
    # What goes on after this run in place of its own result: a weighted sum over the embedding's output and the results
    # of all runs so far, this one included (run i: i + 2 summands, in that order), with the weights of the tensor named
    # here ([i + 2]).  A model uses this for all of its runs or for none.
    depth_mix: str | None = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int | None      # None: the architecture sets no bound (the cache pool's size is the only one)
    embedding: PartSpec
    layers: tuple[LayerSpec, ...]
    runs: tuple[Run, ...]
    final_norm: PartSpec
    head: PartSpec
    bos_token_id: int = -1
    eos_token_id: int = -1
    # where the checkpoint keeps what stands outside the layers (the reference's names,
    # src/model_config.cpp:79,96-97): the embedding's table, the final norm's prefix, the head's matrix
    embedding_name: str = "model.embed_tokens.weight"
    final_norm_prefix: str = "model.norm."
    head_name: str = "lm_head.weight"
    # tensors that this architecture's files may carry although no part reads them (buffers that
    # some writers store): regular expressions matched against the whole name.  Anything else that
    # the parts do not expect is an error.
    ignored_tensors: tuple[str, ...] = ()
    # tensors that belong to no single part: tables that several layers read a part of each, the vectors that runs add
    shared_tensors: tuple["TensorSpec", ...] = ()
    # 0: one residual per token.  S > 0: S streams of it, all equal to the embedding's output at the start, which the
    # layers (of an arrangement made for streams) read from and write to; their sum is what the final norm reads.
    streams: int = 0

    def validate(self) -> None:
        from ..errors import invalid_config
        if not self.runs:
            raise invalid_config("a model needs at least one layer to run")
        for layer in self.layers:
            if layer.streams != self.streams:
                raise invalid_config("every layer works on as many streams of the residual as the model has")
        if self.streams and any(run.add_embedding or run.add_vector is not None or run.depth_mix is not None for run in self.runs):
            raise invalid_config("runs that add something to the residual do not go with a residual of several streams")
        for index, run in enumerate(self.runs):
            if not 0 <= run.layer < len(self.layers):
                raise invalid_config(f"run {index} names layer {run.layer}, which does not exist")
            if not 0 <= run.cache_of <= index:
                raise invalid_config(f"run {index} reads the cache of run {run.cache_of}, which does not run before it")
            if self.runs[run.cache_of].cache_of != run.cache_of:
                raise invalid_config(f"run {index} reads the cache of run {run.cache_of}, which owns none")
            if (run.depth_mix is None) != (self.runs[0].depth_mix is None):
                raise invalid_config("either every run mixes the results so far into what goes on, or none does")
            if run.depth_mix is not None:
                shapes = [tensor.shape for tensor in self.shared_tensors if tensor.name == run.depth_mix]
                if shapes != [(index + 2,)]:
                    raise invalid_config(f"run {index} mixes the results so far with '{run.depth_mix}', which is no shared tensor [{index + 2}]")
            if run.add_vector is not None:
                name, row = run.add_vector
                shapes = [tensor.shape for tensor in self.shared_tensors if tensor.name == name]
                if not shapes or len(shapes[0]) != 2 or shapes[0][1] != self.hidden_size or not 0 <= row < shapes[0][0]:
                    raise invalid_config(f"run {index} adds row {row} of '{name}', which is no row of a shared tensor [rows, hidden]")


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part expects in the checkpoint: its full name, shape and kind of values.  An extent of -1 is a size
    that the file gives and no configuration names (random weights draw `free_extent` there)."""
    name: str
    shape: tuple[int, ...]
    init: str = "normal"        # how random weights draw it: "normal", "norm" (around 1), "offset" (a norm's weight stored around 0), "zeros", "forget_bias" (between 3 and 6), "fraction" (between 0 and 1), "mix" (weights of a sum: the last near 1, the others near 0), "near_identity" (a square matrix: 1 on the diagonal, small elsewhere), "share" (numbers around 1 / count), "spread" (of order 1 whatever the scale of the rest)
    free_extent: int = 16
    optional: bool = False       # absent is no error, present it is checked and not read (a tied head's matrix that some files still carry)
