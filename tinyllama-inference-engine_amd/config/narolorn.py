"""The configuration of the Narolorn decoder, read from its own config.json keys.

    architecture    "Narolorn"
    vocab, width    sizes of the vocabulary and of the residual stream
    norm.eps        of every RMS norm
    streams         how many copies of the residual a layer's sublayers read from and write to (hyper-connections);
                    absent: one residual that the sublayers' results are added to
    logit_softcap   c: the logits leave as c * tanh(logits / c) (absent: as they are)
    loop            start, stop, times: layers start .. stop - 1 run `times` times in a row, each pass on a cache of its
                    own; nothing is added between passes (absent: every layer runs once)
    layers          one entry a layer: `type` ("attention", "latent_attention", "attention_2"), `mixer` (that mixer's sizes
                    and constants) and `mlp` (null: no feed-forward)

    attention          heads, kv_heads, dim, vdim, scale; optionally softcap (of the scores) and q_temp (coef, every)
    latent_attention   heads, dim, vdim, kv_rank, scale; optionally mask.size (a sliding window)
    attention_2        heads, kv_heads, dim, vdim (= dim: the values are the keys), scale; optionally rot (base, dims) and
                       mask.size (chunks of positions)
    mlp                kind "moe": expert.ff, expert.limit, router.experts, router.top, and optionally shared.ff, shared.limit

Every size and constant that can differ between two models of the design is read from here; what the design fixes is
written down in `to_spec`: the pre-norm arrangement, the head tied to the embedding's table, the gate's factor 1.702,
rotation pairs a half apart, router weights that are the softmax over the chosen logits, a shared expert gated by one
sigmoid a token, the tensors' names.  The design sets no bound on positions.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Mapping

from ..errors import invalid_config
from .fadutar import _number
from .spec import LayerSpec, ModelSpec, PartSpec, Run

LAYER_TYPES = ("attention", "latent_attention", "attention_2")
GATE_ALPHA = 1.702      # g * sigmoid(1.702 g): fixed by the design


@dataclass(frozen=True)
class NarolornConfig:
    raw: Mapping[str, Any]          # config.json as read (validated)
    architecture: str = "Narolorn"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "NarolornConfig":
        config = cls(raw=copy.deepcopy(dict(raw)), architecture=str(raw.get("architecture", "Narolorn")))
        config.validate()
        return config

    def to_dict(self) -> dict:
        return copy.deepcopy(dict(self.raw))

    # ---- checks -----------------------------------------------------------------------------------
    def validate(self) -> None:
        from ..ops import MAX_STREAMS
        raw = self.raw
        _number("the model", raw, "vocab")
        _number("the model", raw, "width")
        _number("norm", raw.get("norm"), "eps", float)
        if raw.get("streams") is not None and _number("the model", raw, "streams") > MAX_STREAMS:
            raise invalid_config(f"'streams' is at most {MAX_STREAMS}")
        if raw.get("logit_softcap") is not None:
            _number("the model", raw, "logit_softcap", float)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise invalid_config("'layers' must be a list with at least one layer")
        loop = raw.get("loop")
        if loop is not None:
            start, stop = _number("loop", loop, "start", positive=False), _number("loop", loop, "stop")
            _number("loop", loop, "times")
            if not 0 <= start < stop <= len(layers):
                raise invalid_config(f"loop: layers {start} .. {stop - 1} are not a stretch of the model's {len(layers)}")
        for index, layer in enumerate(layers):
            where = f"layer {index}"
            if not isinstance(layer, Mapping) or layer.get("type") not in LAYER_TYPES:
                kind = layer.get("type") if isinstance(layer, Mapping) else layer
                raise invalid_config(f"{where}: type {kind!r} is not one of {', '.join(LAYER_TYPES)}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, Mapping):
                raise invalid_config(f"{where} lacks 'mixer'")
            getattr(self, "_check_" + layer["type"])(mixer, f"{where}'s mixer")
            if layer.get("mlp") is not None:
                self._check_mlp(layer["mlp"], f"{where}'s mlp")

    @staticmethod
    def _check_heads(mixer, where, grouped=True):
        heads = _number(where, mixer, "heads")
        for key in ("dim", "vdim"):
            _number(where, mixer, key)
        _number(where, mixer, "scale", float)
        if grouped and heads % _number(where, mixer, "kv_heads") != 0:
            raise invalid_config(f"{where}: heads {heads} is not a multiple of kv_heads {mixer['kv_heads']}")

    @staticmethod
    def _check_mask(mixer, where):
        if mixer.get("mask") is not None:
            _number(f"{where}'s mask", mixer["mask"], "size")

    def _check_attention(self, mixer, where):
        self._check_heads(mixer, where)
        if mixer.get("softcap") is not None:
            _number(where, mixer, "softcap", float)
        if mixer.get("q_temp") is not None:
            _number(f"{where}'s q_temp", mixer["q_temp"], "coef", float, positive=False)
            _number(f"{where}'s q_temp", mixer["q_temp"], "every", float)

    def _check_latent_attention(self, mixer, where):
        self._check_heads(mixer, where, grouped=False)
        _number(where, mixer, "kv_rank")
        self._check_mask(mixer, where)

    def _check_attention_2(self, mixer, where):
        self._check_heads(mixer, where)
        if mixer["vdim"] != mixer["dim"]:
            raise invalid_config(f"{where}: the values are the keys, so vdim must equal dim")
        self._check_mask(mixer, where)
        rot = mixer.get("rot")
        if rot is not None:
            _number(f"{where}'s rot", rot, "base", float)
            dims = _number(f"{where}'s rot", rot, "dims")
            if dims > mixer["dim"] or dims % 2 != 0:
                raise invalid_config(f"{where}: rot.dims must be even and at most dim (the dims past it pass unrotated)")

    def _check_mlp(self, mlp, where):
        if not isinstance(mlp, Mapping) or mlp.get("kind") != "moe":
            raise invalid_config(f"{where}: an mlp must be null or of kind 'moe'")
        _number(f"{where}'s expert", mlp.get("expert"), "ff")
        _number(f"{where}'s expert", mlp.get("expert"), "limit", float)
        experts = _number(f"{where}'s router", mlp.get("router"), "experts")
        top = _number(f"{where}'s router", mlp.get("router"), "top")
        if top > experts:
            raise invalid_config(f"{where}: a token cannot use {top} of {experts} experts")
        if mlp.get("shared") is not None:
            _number(f"{where}'s shared expert", mlp["shared"], "ff")
            _number(f"{where}'s shared expert", mlp["shared"], "limit", float)

    # ---- the model as data ----------------------------------------------------------------------------
    def to_spec(self) -> ModelSpec:
        raw = self.raw
        width, vocab, eps = int(raw["width"]), int(raw["vocab"]), float(raw["norm"]["eps"])
        streams = int(raw["streams"]) if raw.get("streams") is not None else 0
        norm = PartSpec("rms_norm", {"size": width, "eps": eps, "tensor": ""})      # (the tensor is named by the place alone)
        layers = []
        for index, layer in enumerate(raw["layers"]):
            mixer = getattr(self, "_spec_" + layer["type"])(layer["mixer"], width, eps)
            mlp = layer.get("mlp")
            layers.append(LayerSpec(
                prefix=f"l{index}.", block="hyper_connections" if streams else "pre_norm", mixer=mixer,
                feed_forward=self._spec_mlp(mlp, width) if mlp is not None else None,
                mixer_norm=norm, feed_forward_norm=norm if mlp is not None else None,
                mixer_norm_place="norm1", mixer_place="mix.", feed_forward_norm_place="norm2", feed_forward_place="mlp.",
                streams=streams, mixer_streams_place="hc1.", feed_forward_streams_place="hc2."))
        count = len(layers)
        # a layer without a feed-forward reads neither a second norm nor the second sublayer's stream tensors: a file that
        # carries them all the same is taken, and they are left unread
        ignored = tuple(rf"l{index}\.(norm2|hc2\.(in|out|mix))" for index, layer in enumerate(raw["layers"]) if layer.get("mlp") is None)
        order = list(range(count))
        loop = raw.get("loop")
        if loop is not None:
            start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            order = list(range(start)) + list(range(start, stop)) * times + list(range(stop, count))
        runs = [Run(layer=layer, cache_of=index) for index, layer in enumerate(order)]     # (every pass a cache of its own)
        cap = raw.get("logit_softcap")
        head = {"vocab_size": vocab, "hidden_size": width, "tied": True, "tied_to": "embed"}
        if cap is not None:
            head["softcap"] = float(cap)
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=width, vocab_size=vocab, max_positions=None,
            embedding=PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": width}),
            layers=tuple(layers), runs=tuple(runs), final_norm=norm, head=PartSpec("lm_head", head),
            embedding_name="embed", final_norm_prefix="final.norm", head_name="head", streams=streams,
            ignored_tensors=ignored)
        spec.validate()
        return spec

    def _spec_attention(self, mixer, width, eps) -> PartSpec:
        params = {"hidden_size": width, "num_heads": int(mixer["heads"]), "num_kv_heads": int(mixer["kv_heads"]),
                  "head_dim": int(mixer["dim"]), "value_dim": int(mixer["vdim"]), "scale": float(mixer["scale"]),
                  "position": PartSpec("none"), "names": {"q": "q", "k": "k", "v": "v", "o": "o"}}
        if mixer.get("softcap") is not None:
            params["softcap"] = float(mixer["softcap"])
        if mixer.get("q_temp") is not None:
            params["q_temp"] = (float(mixer["q_temp"]["coef"]), float(mixer["q_temp"]["every"]))
        return PartSpec("attention", params)

    def _spec_latent_attention(self, mixer, width, eps) -> PartSpec:
        mask = mixer.get("mask")
        return PartSpec("latent_attention", {
            "hidden_size": width, "num_heads": int(mixer["heads"]), "head_dim": int(mixer["dim"]), "rot_dim": 0,
            "value_dim": int(mixer["vdim"]), "rank": int(mixer["kv_rank"]), "scale": float(mixer["scale"]), "norm_eps": eps,
            "window": int(mask["size"]) if mask is not None else None, "output_gate": True,
            "names": {"q": "q", "down": "dkv", "down_norm": "dkv.norm", "up_keys": "uk", "up_values": "uv", "o": "o", "gate": "g"}})

    def _spec_attention_2(self, mixer, width, eps) -> PartSpec:
        rot, mask = mixer.get("rot"), mixer.get("mask")
        position = PartSpec("none")
        if rot is not None:
            position = PartSpec("rotary", {"head_dim": int(mixer["dim"]), "rot_dim": int(rot["dims"]), "theta": float(rot["base"])})
        return PartSpec("attention", {
            "hidden_size": width, "num_heads": int(mixer["heads"]), "num_kv_heads": int(mixer["kv_heads"]),
            "head_dim": int(mixer["dim"]), "value_dim": int(mixer["vdim"]), "scale": float(mixer["scale"]),
            "chunk": int(mask["size"]) if mask is not None else None, "values_are_keys": True,
            "qk_norm": "whole", "norm_eps": eps, "position": position,
            "names": {"q": "q", "k": "k", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}})

    def _spec_mlp(self, mlp, width) -> PartSpec:
        shared = mlp.get("shared")
        params = {
            "hidden_size": width, "experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
            "expert_size": int(mlp["expert"]["ff"]), "shared_size": int(shared["ff"]) if shared is not None else 0,
            "score": "softmax_of_chosen", "router_bias": True, "weigh": "output", "activation": "clamped_swish",
            "alpha": GATE_ALPHA, "limit": float(mlp["expert"]["limit"]),
            "names": {"router": "router", "router_bias": "router.b", "expert": "e{}.", "shared": "shared.",
                      "shared_gate": "shared.sg", "gate": "gate", "up": "up", "down": "down"}}
        if shared is not None:
            params["shared_limit"] = float(shared["limit"])
            params["shared_gate"] = True
        return PartSpec("routed_mlp", params)
