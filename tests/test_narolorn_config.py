"""The Narolorn decoder on the CPU: config.json to the model as data, the tensors it expects, what is refused, and
pieces of the plain implementation against cases worked out by hand."""
import copy
import math

import pytest
import torch

import plain_narolorn as plain
from narolorn_helpers import CONFIGS, CONFIG_P, CONFIG_Q


def spec_of(raw):
    from tlie_amd.registry import config_from_dict
    return config_from_dict(raw).to_spec()


def test_the_configuration_becomes_the_model_as_data():
    spec = spec_of(CONFIG_P)
    assert (spec.architecture, spec.hidden_size, spec.vocab_size, spec.max_positions, spec.streams) == ("Narolorn", 80, 193, None, 2)
    # layers 1 and 2 run three times in a row, every pass on a cache of its own, and nothing joins between passes
    assert [run.layer for run in spec.runs] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert all(run.cache_of == index and not run.add_embedding and run.add_vector is None for index, run in enumerate(spec.runs))
    first, second, third, fourth = spec.layers
    assert all(layer.block == "hyper_connections" and layer.streams == 2 for layer in spec.layers)
    assert (first.mixer.kind, first.mixer["softcap"], first.mixer["q_temp"], first.mixer["value_dim"]) == ("attention", 6.0, (0.3, 5.0), 24)
    assert (second.mixer.kind, second.mixer["window"], second.mixer["rot_dim"], second.mixer["output_gate"]) == ("latent_attention", 7, 0, True)
    assert (third.mixer.kind, third.mixer["chunk"], third.mixer["values_are_keys"], third.mixer["qk_norm"]) == ("attention", 10, True, "whole")
    assert third.mixer["position"].kind == "rotary" and third.mixer["position"]["rot_dim"] == 8 and third.feed_forward is None
    assert fourth.mixer["window"] is None
    mlp = first.feed_forward
    assert (mlp.kind, mlp["score"], mlp["weigh"], mlp["activation"], mlp["limit"], mlp["shared_limit"], mlp["shared_gate"]) == \
        ("routed_mlp", "softmax_of_chosen", "output", "clamped_swish", 1.5, 3.0, True)
    assert spec.head["tied"] and spec.head["tied_to"] == "embed" and spec.head["softcap"] == 12.0


def test_what_config_json_leaves_out_is_absent():
    spec = spec_of(CONFIG_Q)
    assert spec.streams == 0 and all(layer.block == "pre_norm" for layer in spec.layers)
    assert [run.layer for run in spec.runs] == [0, 1, 2, 3]
    assert spec.head.get("softcap") is None
    plain_attention = spec.layers[1].mixer
    assert plain_attention.get("softcap") is None and plain_attention.get("q_temp") is None
    assert spec.layers[0].mixer["position"].kind == "none" and spec.layers[0].mixer["chunk"] is None
    assert spec.layers[1].feed_forward["shared_size"] == 0 and not spec.layers[1].feed_forward.get("shared_gate", False)


def test_the_expected_tensors_carry_the_designs_names_and_shapes():
    from tlie_amd.models.builder import expected_tensors
    shapes = {tensor.name: tensor.shape for tensor in expected_tensors(spec_of(CONFIG_P)) if not tensor.optional}
    assert shapes["embed"] == (193, 80) and shapes["final.norm"] == (80,) and "head" not in shapes
    assert shapes["l0.mix.q"] == (64, 80) and shapes["l0.mix.k"] == (16, 80) and shapes["l0.mix.v"] == (24, 80) and shapes["l0.mix.o"] == (80, 96)
    assert shapes["l0.hc1.in"] == (2,) and shapes["l0.hc2.mix"] == (2, 2) and shapes["l0.hc2.out"] == (2,)
    assert shapes["l0.mlp.router"] == (5, 80) and shapes["l0.mlp.router.b"] == (5,) and shapes["l0.mlp.shared.sg"] == (1, 80)
    assert shapes["l0.mlp.e4.down"] == (80, 24) and shapes["l0.mlp.shared.gate"] == (40, 80)
    assert shapes["l1.mix.dkv"] == (48, 80) and shapes["l1.mix.dkv.norm"] == (48,) and shapes["l1.mix.uk"] == (24, 48)
    assert shapes["l1.mix.uv"] == (60, 48) and shapes["l1.mix.g"] == (60, 80) and "l1.mlp.shared.gate" not in shapes
    assert shapes["l2.mix.q.norm"] == (128,) and shapes["l2.mix.k.norm"] == (64,) and "l2.mix.v" not in shapes
    assert "l2.hc2.in" not in shapes and "l2.norm2" not in shapes          # a layer without a feed-forward
    import re
    assert any(re.fullmatch(pattern, "l2.norm2") for pattern in spec_of(CONFIG_P).ignored_tensors)      # (a file may still carry them)
    assert not any(re.fullmatch(pattern, "l1.norm2") for pattern in spec_of(CONFIG_P).ignored_tensors)
    single = {tensor.name for tensor in expected_tensors(spec_of(CONFIG_Q))}
    assert not any(".hc" in name for name in single)


@pytest.mark.parametrize("change,message", [
    (lambda raw: raw["layers"][0].update(type="mamba"), "not one of"),
    (lambda raw: raw["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda raw: raw["layers"][2]["mixer"].update(vdim=16), "values are the keys"),
    (lambda raw: raw["layers"][2]["mixer"]["rot"].update(dims=7), "even"),
    (lambda raw: raw["layers"][0]["mlp"]["router"].update(top=9), "cannot use"),
    (lambda raw: raw["layers"][0]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda raw: raw.update(loop={"start": 2, "stop": 7, "times": 2}), "stretch"),
    (lambda raw: raw.update(streams=9), "at most"),
    (lambda raw: raw["norm"].pop("eps"), "eps"),
    (lambda raw: raw["layers"][1]["mixer"].update(mask={"size": 0}), "positive"),
])
def test_configurations_that_are_refused(change, message):
    from tlie_amd import EngineError
    raw = copy.deepcopy(CONFIG_P)
    change(raw)
    with pytest.raises(EngineError, match=message):
        spec_of(raw)


def test_every_configuration_of_the_tests_is_read():
    for raw in CONFIGS.values():
        spec_of(raw)


# ---- the plain implementation's pieces, by hand ------------------------------------------------------------
def test_plain_masks():
    window = plain.visible(6, window=3)
    assert window[5].tolist() == [False, False, False, True, True, True] and window[1].tolist() == [True, True] + [False] * 4
    chunk = plain.visible(7, chunk=3)
    assert chunk[4].tolist() == [False, False, False, True, True, False, False]
    assert chunk[6].tolist() == [False] * 6 + [True] and chunk[2].tolist() == [True, True, True] + [False] * 4


def test_plain_query_temperature_and_rotation():
    factor = plain.query_temperature(torch.tensor([0, 3, 4, 9, 14]), 0.5, 5.0)
    want = [1.0, 1.0, 1.0 + 0.5 * math.log(2.0), 1.0 + 0.5 * math.log(3.0), 1.0 + 0.5 * math.log(4.0)]
    assert torch.allclose(factor, torch.tensor(want, dtype=torch.float64))
    x = torch.zeros(1, 1, 6, dtype=torch.float64)
    x[0, 0] = torch.tensor([1.0, 2.0, 3.0, 4.0, 5.0, 6.0])
    turned = plain.rotate_halves(x, torch.tensor([1]), 4, 100.0)[0, 0]
    a0, a1 = 1.0, 100.0 ** -0.5
    want = [math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1), 3 * math.cos(a0) + math.sin(a0),
            4 * math.cos(a1) + 2 * math.sin(a1), 5.0, 6.0]
    assert torch.allclose(turned, torch.tensor(want, dtype=torch.float64))


def test_plain_router_and_expert():
    chosen, weights = plain.router_choice(torch.tensor([[0.0, 2.0, -1.0, 1.0]], dtype=torch.float64), 2)
    assert chosen.tolist() == [[1, 3]]
    assert torch.allclose(weights, torch.tensor([[math.e / (1 + math.e), 1 / (1 + math.e)]], dtype=torch.float64))
    w = {"gate": torch.tensor([[3.0], [-1.0]], dtype=torch.float64), "up": torch.tensor([[5.0], [0.5]], dtype=torch.float64),
         "down": torch.tensor([[1.0, 10.0]], dtype=torch.float64)}
    out = plain.expert(w, "", torch.tensor([[1.0]], dtype=torch.float64), 2.0)
    first = 2.0 / (1 + math.exp(-1.702 * 2.0)) * (2.0 + 1.0)                 # gate 3 -> 2, up 5 -> 2
    second = -1.0 / (1 + math.exp(1.702)) * (0.5 + 1.0)                       # a negative gate is not clamped
    assert abs(float(out) - (first + 10.0 * second)) < 1e-12


def test_plain_streams_with_unit_numbers_are_a_plain_residual():
    streams = torch.randn(3, 4, 5, dtype=torch.float64)
    w = {"in": torch.tensor([1.0, 0.0, 0.0], dtype=torch.float64), "mix": torch.eye(3, dtype=torch.float64),
         "out": torch.tensor([1.0, 0.0, 2.0], dtype=torch.float64)}
    after = plain.hyper_sublayer(streams, w, "", lambda u: 2.0 * u)
    assert torch.allclose(after[0], 3.0 * streams[0]) and torch.allclose(after[1], streams[1])
    assert torch.allclose(after[2], streams[2] + 4.0 * streams[0])
    # mix is indexed [from, to]
    w["mix"] = torch.tensor([[0.0, 1.0, 0.0], [0.0, 0.0, 0.0], [0.0, 0.0, 0.0]], dtype=torch.float64)
    w["out"] = torch.zeros(3, dtype=torch.float64)
    after = plain.hyper_sublayer(streams, w, "", lambda u: u)
    assert torch.allclose(after[1], streams[0]) and float(after[0].abs().max()) == 0.0
