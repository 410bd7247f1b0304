"""The configuration of the Tugalix decoder, read from its own config.json keys.

    architecture    "Tugalix"
    vocab, width    sizes of the vocabulary and of the residual stream
    norm.eps        of every norm
    canon.taps      taps of the causal convolution that stands in front of every sublayer
    logit_scale     what the logits are multiplied by
    layers          one entry a layer: `type` ("retention", "gla", "parallel"), `mixer` (that mixer's sizes and
                    constants) and `mlp` (null: no feed-forward; else kind "dense" with `ff`)

    retention   heads, dim, vdim, decay (one a head), rot (base, dims)
    gla         heads, dim, vdim, tau
    parallel    left (heads, kv_heads, dim, vdim, scale, rot), right (heads, dim), left_scale, right_scale

A layer is pre-norm with layer norms (weight and bias); each sublayer reads h + conv(h) of its norm's result; after a
layer, what goes on is a weighted sum over the embedding's output and all layers' results so far.  Every size and
every constant that can differ between two models of the design is read from here (the rank of the decays' low-rank
products is the stored tensors' own); what the design fixes (the arrangement, rotation of halves, the tensors' names)
is written down in `to_spec`.  The design sets no bound on positions.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Mapping

from ..errors import invalid_config
from .fadutar import _number
from .spec import LayerSpec, ModelSpec, PartSpec, Run, TensorSpec

LAYER_TYPES = ("retention", "gla", "parallel")


@dataclass(frozen=True)
class TugalixConfig:
    raw: Mapping[str, Any]          # config.json as read (validated)
    architecture: str = "Tugalix"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "TugalixConfig":
        config = cls(raw=copy.deepcopy(dict(raw)), architecture=str(raw.get("architecture", "Tugalix")))
        config.validate()
        return config

    def to_dict(self) -> dict:
        return copy.deepcopy(dict(self.raw))

    # ---- checks -----------------------------------------------------------------------------------
    def validate(self) -> None:
        raw = self.raw
        _number("the model", raw, "vocab")
        _number("the model", raw, "width")
        _number("norm", raw.get("norm"), "eps", float)
        _number("canon", raw.get("canon"), "taps")
        _number("the model", raw, "logit_scale", float)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise invalid_config("'layers' must be a list with at least one layer")
        for index, layer in enumerate(layers):
            where = f"layer {index}"
            if not isinstance(layer, Mapping) or layer.get("type") not in LAYER_TYPES:
                kind = layer.get("type") if isinstance(layer, Mapping) else layer
                raise invalid_config(f"{where}: type {kind!r} is not one of {', '.join(LAYER_TYPES)}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, Mapping):
                raise invalid_config(f"{where} lacks 'mixer'")
            getattr(self, "_check_" + layer["type"])(mixer, f"{where}'s mixer")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") != "dense":
                    raise invalid_config(f"{where}: an mlp must be null or of kind 'dense'")
                _number(f"{where}'s mlp", mlp, "ff")

    @staticmethod
    def _check_rot(mixer, where):
        rot = mixer.get("rot")
        _number(f"{where}'s rot", rot, "base", float)
        dims = _number(f"{where}'s rot", rot, "dims")
        if dims > int(mixer["dim"]) or dims % 2 != 0:
            raise invalid_config(f"{where}: rot.dims must be even and at most dim (the dims past it pass unrotated)")

    def _check_retention(self, mixer, where):
        heads = _number(where, mixer, "heads")
        _number(where, mixer, "dim"), _number(where, mixer, "vdim")
        decay = mixer.get("decay")
        if not isinstance(decay, list) or len(decay) != heads or not all(isinstance(value, (int, float)) and 0 <= value <= 1 for value in decay):
            raise invalid_config(f"{where}: 'decay' must list one number between 0 and 1 a head")
        self._check_rot(mixer, where)

    def _check_gla(self, mixer, where):
        for key in ("heads", "dim", "vdim"):
            _number(where, mixer, key)
        _number(where, mixer, "tau", float)

    def _check_parallel(self, mixer, where):
        left, right = mixer.get("left"), mixer.get("right")
        heads, kv_heads = _number(f"{where}'s left", left, "heads"), _number(f"{where}'s left", left, "kv_heads")
        _number(f"{where}'s left", left, "dim"), _number(f"{where}'s left", left, "vdim"), _number(f"{where}'s left", left, "scale", float)
        if heads % kv_heads != 0:
            raise invalid_config(f"{where}: heads {heads} is not a multiple of kv_heads {kv_heads}")
        self._check_rot(left, f"{where}'s left")
        _number(f"{where}'s right", right, "heads"), _number(f"{where}'s right", right, "dim")
        _number(where, mixer, "left_scale", float, positive=False), _number(where, mixer, "right_scale", float, positive=False)

    # ---- the model as data ----------------------------------------------------------------------------
    def to_spec(self) -> ModelSpec:
        raw = self.raw
        width, vocab, eps = int(raw["width"]), int(raw["vocab"]), float(raw["norm"]["eps"])
        taps = int(raw["canon"]["taps"])

        def norm(name):         # weight `<place>`, bias `<place>.b`
            return PartSpec("layer_norm", {"size": width, "eps": eps, "tensor": name, "bias_tensor": name + ".b"})
        layers, runs, shared = [], [], []
        for index, layer in enumerate(raw["layers"]):
            mixer = getattr(self, "_spec_" + layer["type"])(layer["mixer"], width, eps)
            mlp = layer.get("mlp")
            feed_forward = None
            if mlp is not None:
                feed_forward = PartSpec("mlp", {"hidden_size": width, "intermediate_size": int(mlp["ff"]), "activation": "xielu",
                                                "names": {"up": "up", "down": "down", "act": "act"}})
            layers.append(LayerSpec(
                prefix=f"l{index}.", block="pre_norm", mixer=mixer, feed_forward=feed_forward,
                mixer_norm=norm("norm1"), feed_forward_norm=norm("norm2") if mlp is not None else None,
                mixer_norm_place="", mixer_place="mix.", feed_forward_norm_place="", feed_forward_place="mlp.",
                sublayer_input=PartSpec("residual_conv", {"size": width, "taps": taps, "tensor": ""}),
                mixer_input_place="canon1", feed_forward_input_place="canon2"))
            shared.append(TensorSpec(f"l{index}.dwa", (index + 2,), init="mix"))
            runs.append(Run(layer=index, cache_of=index, depth_mix=f"l{index}.dwa"))
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=width, vocab_size=vocab, max_positions=None,
            embedding=PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": width, "norm": norm("embed.norm"),
                                                   "norm_prefix": ""}),
            layers=tuple(layers), runs=tuple(runs), final_norm=norm("final.norm"),
            head=PartSpec("lm_head", {"vocab_size": vocab, "hidden_size": width, "tied": False, "scale": float(raw["logit_scale"])}),
            embedding_name="embed", final_norm_prefix="", head_name="head", shared_tensors=tuple(shared))
        spec.validate()
        return spec

    @staticmethod
    def _rotary(mixer) -> PartSpec:
        rot = mixer["rot"]
        return PartSpec("rotary", {"head_dim": int(mixer["dim"]), "rot_dim": int(rot["dims"]), "theta": float(rot["base"])})

    def _spec_retention(self, mixer, width, eps) -> PartSpec:
        return PartSpec("retention", {
            "hidden_size": width, "num_heads": int(mixer["heads"]), "head_dim": int(mixer["dim"]), "value_dim": int(mixer["vdim"]),
            "decay": tuple(float(value) for value in mixer["decay"]), "norm_eps": eps, "position": self._rotary(mixer),
            "names": {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o"}})

    def _spec_gla(self, mixer, width, eps) -> PartSpec:
        return PartSpec("gated_linear_attention", {
            "hidden_size": width, "num_heads": int(mixer["heads"]), "head_dim": int(mixer["dim"]), "value_dim": int(mixer["vdim"]),
            "tau": float(mixer["tau"]), "norm_eps": eps, "decay_rank": mixer.get("rank"),
            "names": {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o", "decay_down": "a1", "decay_up": "a2",
                      "decay_bias": "a2.b", "norm": "norm"}})

    def _spec_parallel(self, mixer, width, eps) -> PartSpec:
        left, right = mixer["left"], mixer["right"]
        attention = PartSpec("attention", {
            "hidden_size": width, "num_heads": int(left["heads"]), "num_kv_heads": int(left["kv_heads"]),
            "head_dim": int(left["dim"]), "value_dim": int(left["vdim"]), "scale": float(left["scale"]), "bias": False,
            "window": None, "position": self._rotary(left), "names": {"q": "q", "k": "k", "v": "v", "o": "o"}})
        shifted = PartSpec("token_shift_mixing", {
            "hidden_size": width, "num_heads": int(right["heads"]), "head_dim": int(right["dim"]), "norm_eps": eps,
            "decay_rank": right.get("rank")})
        return PartSpec("side_by_side", {"left": attention, "right": shifted, "left_scale": float(mixer["left_scale"]),
                                         "right_scale": float(mixer["right_scale"]), "left_place": "left.", "right_place": "right."})
