"""What the Narolorn tests share: configurations of their own, model folders of random weights, and the comparison
with the plain implementation.

The configurations differ from each other in every size and option, and use values that make faults visible: fewer
key/value groups than heads (down to one), value heads of another size than the keys, windows and chunks that are no
multiple of a page (7, 10, 40 positions on pages of 16) so that their edges fall inside pages, rotations over a part of a
head and over all of it, a query temperature whose period is short enough to change within a prompt, one, two and four
streams and a model with a single residual, a loop that starts after the first layer and runs three times, one of a single
layer, and none, routers that choose one, some and all experts, with and without a shared expert, whose limit differs from
the experts', a layer without a feed-forward, a latent vector wider than any head, models with and without capped logits.
"""
import json
import os

import torch
from safetensors.torch import load_file

import plain_narolorn


def _moe(experts, top, ff, limit, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared[0], "limit": shared[1]}
    return mlp


def _attention(heads, groups, dim, vdim, scale, softcap=None, q_temp=None):
    mixer = {"heads": heads, "kv_heads": groups, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap is not None:
        mixer["softcap"] = softcap
    if q_temp is not None:
        mixer["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return mixer


def _latent(heads, dim, vdim, rank, scale, window=None):
    mixer = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if window is not None:
        mixer["mask"] = {"size": window}
    return mixer


def _attention_2(heads, groups, dim, scale, chunk=None, rot=None):
    mixer = {"heads": heads, "kv_heads": groups, "dim": dim, "vdim": dim, "scale": scale}
    if chunk is not None:
        mixer["mask"] = {"size": chunk}
    if rot is not None:
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
    return mixer


CONFIG_P = {
    "architecture": "Narolorn", "vocab": 193, "width": 80, "norm": {"eps": 1e-5}, "streams": 2, "logit_softcap": 12.0,
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "attention", "mixer": _attention(4, 1, 16, 24, 0.2, softcap=6.0, q_temp=(0.3, 5)), "mlp": _moe(5, 2, 24, 1.5, (40, 3.0))},
        {"type": "latent_attention", "mixer": _latent(3, 8, 20, 48, 0.3, window=7), "mlp": _moe(4, 4, 16, 2.5)},
        {"type": "attention_2", "mixer": _attention_2(4, 2, 32, 0.15, chunk=10, rot=(100.0, 8)), "mlp": None},
        {"type": "latent_attention", "mixer": _latent(2, 24, 8, 160, 0.2), "mlp": _moe(3, 1, 12, 1.0, (8, 0.5))},
    ],
}
CONFIG_Q = {        # a single residual, no loop, logits as they are; an attention layer with nothing switched on
    "architecture": "Narolorn", "vocab": 150, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "attention_2", "mixer": _attention_2(2, 2, 16, 0.25), "mlp": _moe(8, 3, 8, 4.0, (16, 4.0))},
        {"type": "attention", "mixer": _attention(3, 3, 32, 32, 0.18), "mlp": _moe(2, 1, 40, 2.0)},
        {"type": "latent_attention", "mixer": _latent(5, 16, 16, 32, 0.25, window=40), "mlp": None},
        {"type": "attention_2", "mixer": _attention_2(6, 1, 8, 0.35, chunk=40, rot=(10.0, 8)), "mlp": _moe(3, 2, 20, 1.0)},
    ],
}
CONFIG_R = {        # one stream (the three small tensors still act), a loop of a single layer; head sizes the matrix cores take
    "architecture": "Narolorn", "vocab": 96, "width": 128, "norm": {"eps": 1e-5}, "streams": 1, "logit_softcap": 25.0,
    "loop": {"start": 0, "stop": 1, "times": 2},
    "layers": [
        {"type": "attention_2", "mixer": _attention_2(4, 2, 64, 0.12, chunk=24, rot=(30000.0, 32)), "mlp": _moe(4, 2, 32, 2.0, (32, 2.0))},
        {"type": "attention", "mixer": _attention(2, 1, 64, 64, 0.13, softcap=20.0, q_temp=(0.7, 16)), "mlp": _moe(4, 1, 32, 2.0)},
        {"type": "latent_attention", "mixer": _latent(4, 32, 32, 64, 0.18, window=24), "mlp": _moe(6, 2, 16, 3.0, (64, 1.0))},
    ],
}
CONFIG_S = {        # four streams, no loop; a width that is no multiple of four
    "architecture": "Narolorn", "vocab": 70, "width": 50, "norm": {"eps": 1e-5}, "streams": 4,
    "layers": [
        {"type": "latent_attention", "mixer": _latent(2, 12, 12, 24, 0.3, window=3), "mlp": _moe(2, 2, 8, 2.0)},
        {"type": "attention", "mixer": _attention(2, 2, 8, 8, 0.4, q_temp=(1.0, 2)), "mlp": None},
    ],
}
CONFIGS = {"P": CONFIG_P, "Q": CONFIG_Q, "R": CONFIG_R, "S": CONFIG_S}
DTYPES = ["float32", "bfloat16"]
# a row's largest error relative to the row's largest value, against float64 on the same stored weights
TOLERANCE = {"float32": 3e-5, "bfloat16": 4e-2}
# two cuts of the same request through the same engine (in bfloat16 a step of few rows takes other product kernels
# than a step of many, whose results are rounded to bfloat16 where the others' stay float partial sums: two results that
# each lie within 4e-2 of the plain one may lie further from each other)
CUT_TOLERANCE = {"float32": 2e-6, "bfloat16": 6e-2}


def make_model(folder, raw_config, seed, std=0.08, norm_std=0.1):
    """Weights are stored in bfloat16, as the design's files are: a float32 run widens the same values."""
    from tlie_amd import write_random_model
    from tlie_amd.registry import config_from_dict
    write_random_model(str(folder), config_from_dict(raw_config), seed, std=std, norm_std=norm_std, dtype=torch.bfloat16)
    return str(folder)


def load_plain(folder):
    with open(os.path.join(folder, "config.json"), "r", encoding="utf-8") as handle:
        raw = json.load(handle)
    weights = {name: tensor.double() for name, tensor in load_file(os.path.join(folder, "model.safetensors")).items()}
    return raw, weights


def plain_generate_greedy(config, weights, prompt, count):
    tokens, out = list(prompt), []
    for _ in range(count):
        token = int(torch.argmax(plain_narolorn.forward(config, weights, tokens)[0][-1]))
        out.append(token)
        tokens.append(token)
    return out


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    got, want = got.double().cpu(), want.double().cpu()
    return (got - want).abs().amax(dim=-1) / want.abs().amax(dim=-1)


def run_cut(engine, request, tokens, cuts):
    """The request's tokens in portions of the sizes `cuts` (repeated as needed); returns logits [T, vocab]."""
    from tlie_amd import StepEntry
    engine.admit(request)
    rows, at, index = [], 0, 0
    while at < len(tokens):
        count = min(cuts[index % len(cuts)], len(tokens) - at)
        rows.append(engine.step([StepEntry(request, tokens[at:at + count], list(range(count)))]).clone())
        at += count
        index += 1
    engine.finish(request)
    return torch.cat(rows, dim=0)
