"""What the Tugalix tests share: configurations of their own, model folders of random weights, and the
comparison with the plain implementation.

The configurations differ from each other in every size and option, and use values that make faults visible:
convolutions of one, two, four and five taps; layers of every kind with and without a feed-forward, in several
orders, a model of a single layer and one without any attention (no pages at all); fewer key/value heads than
query heads and as many; value heads below and above 64 dims and of no multiple of 64; query dims of 8 to 160
(every way the scan splits a head over its waves); rotations over a part of a head and over all of it; scales of
the two sides that are negative, zero-free and unequal; decays' inner sizes of 3 to 16; a factor of the logits
below and above 1; widths and inner sizes that are no multiple of 8.
"""
import json
import os

import torch
from safetensors.torch import load_file

import plain_tugalix


def _retention(heads, dim, vdim, decay, base, dims):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay, "rot": {"base": base, "dims": dims}}


def _parallel(left, right, left_scale, right_scale):
    heads, groups, dim, vdim, scale, base, dims = left
    return {"left": {"heads": heads, "kv_heads": groups, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": base, "dims": dims}},
            "right": dict(zip(("heads", "dim", "rank"), right)), "left_scale": left_scale, "right_scale": right_scale}


CONFIG_U = {
    "architecture": "Tugalix", "vocab": 173, "width": 80, "norm": {"eps": 1e-5}, "canon": {"taps": 4}, "logit_scale": 0.7,
    "layers": [
        {"type": "gla", "mixer": {"heads": 3, "dim": 24, "vdim": 40, "tau": 8.0, "rank": 5}, "mlp": {"kind": "dense", "ff": 56}},
        {"type": "parallel", "mixer": _parallel((4, 2, 16, 24, 0.3, 500.0, 8), (3, 24, 7), 1.3, 0.5), "mlp": None},
        {"type": "retention", "mixer": _retention(3, 16, 20, [0.9, 0.99, 0.5], 100.0, 8), "mlp": {"kind": "dense", "ff": 120}},
        {"type": "parallel", "mixer": _parallel((6, 6, 32, 32, 0.2, 10000.0, 32), (1, 72, 3), -0.4, 1.0), "mlp": {"kind": "dense", "ff": 40}},
    ],
}
CONFIG_V = {        # no attention anywhere: no page is ever asked for; one tap: the convolution keeps nothing
    "architecture": "Tugalix", "vocab": 90, "width": 44, "norm": {"eps": 1e-6}, "canon": {"taps": 1}, "logit_scale": 1.0,
    "layers": [
        {"type": "retention", "mixer": _retention(1, 130, 8, [0.998], 30.0, 2), "mlp": None},
        {"type": "gla", "mixer": {"heads": 2, "dim": 8, "vdim": 130, "tau": 1.0}, "mlp": None},
        {"type": "retention", "mixer": _retention(4, 6, 70, [1.0, 0.25, 0.75, 0.96], 7.0, 6), "mlp": {"kind": "dense", "ff": 44}},
    ],
}
CONFIG_W = {        # a single layer; values wider than keys on the left, heads of 160 dims on the right
    "architecture": "Tugalix", "vocab": 64, "width": 32, "norm": {"eps": 1e-5}, "canon": {"taps": 2}, "logit_scale": 3.5,
    "layers": [
        {"type": "parallel", "mixer": _parallel((2, 1, 8, 70, 0.5, 20.0, 4), (2, 160, 16), 0.6, -1.2), "mlp": {"kind": "dense", "ff": 24}},
    ],
}
CONFIGS = {"U": CONFIG_U, "V": CONFIG_V, "W": CONFIG_W}
DTYPES = ["float32", "bfloat16"]
# a row's largest error relative to the row's largest value, against float64 on the same stored weights.  In
# bfloat16 the engine rounds what stands between its kernels (a sublayer's input, its projections, the heads'
# normed results, the feed-forward's inner values); the sharp comparison is the 32-bit one.
TOLERANCE = {"float32": 3e-5, "bfloat16": 6e-2}
SINGLE_LAYER_TOLERANCE = {"float32": 3e-5, "bfloat16": 3e-2}
# two cuts of the same request through the same engine (in bfloat16 a step of few rows takes other product kernels
# than a step of many; in 32-bit a sequence that brings many tokens takes the scan's sliced walk, whose sums run in
# another order)
CUT_TOLERANCE = {"float32": 1e-5, "bfloat16": 6e-2}


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


def rewrite(folder, changes):
    """Applies `changes(weights)` to the folder's float64 weights and stores them again, in bfloat16."""
    from tlie_amd.weights.safetensors_io import write_safetensors
    config, weights = load_plain(folder)
    changes(weights)
    write_safetensors(os.path.join(folder, "model.safetensors"), {name: tensor.to(torch.bfloat16).contiguous() for name, tensor in weights.items()})
    return load_plain(folder)


def plain_generate_greedy(config, weights, prompt, count):
    tokens, out = list(prompt), []
    for _ in range(count):
        token = int(torch.argmax(plain_tugalix.forward(config, weights, tokens)[0][-1]))
        out.append(token)
        tokens.append(token)
    return out


def row_errors(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
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
