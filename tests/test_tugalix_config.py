"""The Tugalix configuration on the CPU: config.json -> the model as data, the tensors it expects, what it
refuses; and properties of the plain implementation's own pieces."""
import copy
import math

import pytest
import torch

import plain_tugalix as plain
from tugalix_helpers import CONFIG_U, CONFIG_V, CONFIG_W
from tlie_amd.errors import EngineError
from tlie_amd.models.builder import expected_tensors
from tlie_amd.registry import config_from_dict


def test_the_architecture_is_found_by_its_name_and_turned_into_data():
    spec = config_from_dict(CONFIG_U).to_spec()
    assert spec.architecture == "Tugalix" and spec.max_positions is None
    assert (spec.hidden_size, spec.vocab_size) == (80, 173)
    assert [layer.block for layer in spec.layers] == ["pre_norm"] * 4
    assert [layer.mixer.kind for layer in spec.layers] == ["gated_linear_attention", "side_by_side", "retention", "side_by_side"]
    assert [None if layer.feed_forward is None else layer.feed_forward.kind for layer in spec.layers] == ["mlp", None, "mlp", "mlp"]
    assert all(layer.feed_forward["activation"] == "xielu" for layer in spec.layers if layer.feed_forward is not None)
    assert all(layer.sublayer_input.kind == "residual_conv" and layer.sublayer_input["taps"] == 4 for layer in spec.layers)
    assert all(layer.mixer_norm.kind == "layer_norm" and layer.mixer_norm["eps"] == 1e-5 for layer in spec.layers)
    # every layer runs once, owns what it keeps, and hands on a sum over all results so far
    assert [(run.layer, run.cache_of, run.depth_mix) for run in spec.runs] == [(i, i, f"l{i}.dwa") for i in range(4)]
    assert spec.head["scale"] == 0.7 and not spec.head["tied"]
    side = spec.layers[1].mixer
    assert (side["left_scale"], side["right_scale"]) == (1.3, 0.5)
    left, right = side["left"], side["right"]
    assert (left.kind, left["num_heads"], left["num_kv_heads"], left["head_dim"], left["value_dim"], left["scale"]) == ("attention", 4, 2, 16, 24, 0.3)
    assert (left["position"]["rot_dim"], left["position"]["theta"], left["window"]) == (8, 500.0, None)
    assert (right.kind, right["num_heads"], right["head_dim"], right["decay_rank"]) == ("token_shift_mixing", 3, 24, 7)
    retention = spec.layers[2].mixer
    assert retention["decay"] == (0.9, 0.99, 0.5) and retention["position"]["rot_dim"] == 8 and retention["value_dim"] == 20
    assert spec.layers[0].mixer["tau"] == 8.0


def test_layers_in_another_order_and_a_model_of_one_layer():
    spec = config_from_dict(CONFIG_V).to_spec()
    assert [layer.mixer.kind for layer in spec.layers] == ["retention", "gated_linear_attention", "retention"]
    assert [layer.feed_forward is None for layer in spec.layers] == [True, True, False]
    assert spec.layers[1].mixer["decay_rank"] is None               # (the stored tensors give it)
    spec = config_from_dict(CONFIG_W).to_spec()
    assert len(spec.runs) == 1 and spec.runs[0].depth_mix == "l0.dwa" and spec.head["scale"] == 3.5


def test_expected_tensors_follow_the_layers():
    names = {tensor.name: tuple(tensor.shape) for tensor in expected_tensors(config_from_dict(CONFIG_U).to_spec())}
    assert names["embed"] == (173, 80) and names["head"] == (173, 80)
    for norm in ("embed.norm", "final.norm", "l0.norm1", "l0.norm2", "l1.norm1", "l3.norm2"):
        assert names[norm] == (80,) and names[norm + ".b"] == (80,)
    assert "l1.norm2" not in names and "l1.canon2" not in names and "l1.mlp.up" not in names
    assert names["l0.canon1"] == (80, 4) and names["l0.canon2"] == (80, 4) and names["l1.canon1"] == (80, 4)
    assert [names[f"l{i}.dwa"] for i in range(4)] == [(2,), (3,), (4,), (5,)]
    assert names["l0.mix.q"] == (72, 80) and names["l0.mix.k"] == (72, 80) and names["l0.mix.v"] == (120, 80)
    assert names["l0.mix.g"] == (120, 80) and names["l0.mix.o"] == (80, 120) and names["l0.mix.norm"] == (40,)
    assert names["l0.mix.a1"] == (5, 80) and names["l0.mix.a2"] == (72, 5) and names["l0.mix.a2.b"] == (72,)
    assert names["l0.mlp.up"] == (56, 80) and names["l0.mlp.down"] == (80, 56) and names["l0.mlp.act"] == (2,)
    assert names["l1.mix.left.q"] == (64, 80) and names["l1.mix.left.k"] == (32, 80) and names["l1.mix.left.v"] == (48, 80)
    assert names["l1.mix.left.o"] == (80, 96)
    for blend in "rkvgw":
        assert names["l1.mix.right.mu." + blend] == (80,)
    for product in "rkvg":
        assert names["l1.mix.right." + product] == (72, 80)
    assert names["l1.mix.right.w1"] == (7, 80) and names["l1.mix.right.w2"] == (72, 7) and names["l1.mix.right.w0"] == (72,)
    assert names["l1.mix.right.u"] == (3, 24) and names["l1.mix.right.norm"] == (72,) and names["l1.mix.right.o"] == (80, 72)
    assert names["l2.mix.q"] == (48, 80) and names["l2.mix.v"] == (60, 80) and names["l2.mix.g"] == (60, 80) and names["l2.mix.o"] == (80, 60)
    assert "l2.mix.norm" not in names and "l2.mix.a1" not in names
    # without a rank in the configuration the decays' inner size is the file's own
    names = {tensor.name: tuple(tensor.shape) for tensor in expected_tensors(config_from_dict(CONFIG_V).to_spec())}
    assert names["l1.mix.a1"] == (-1, 44) and names["l1.mix.a2"] == (16, -1)


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.5, 0.5]), "decay"),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.5, 0.5, 1.5]), "decay"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "kind"),
    (lambda c: c["layers"][0]["mixer"].pop("tau"), "tau"),
    (lambda c: c.pop("logit_scale"), "logit_scale"),
    (lambda c: c["canon"].pop("taps"), "taps"),
    (lambda c: c["layers"][1]["mixer"].pop("right_scale"), "right_scale"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_what_the_configuration_refuses(change, what):
    raw = copy.deepcopy(CONFIG_U)
    change(raw)
    with pytest.raises(EngineError) as caught:
        config_from_dict(raw).to_spec()
    assert what in str(caught.value)


def test_sizes_the_kernels_do_not_take_are_refused_when_the_model_is_built():
    from tlie_amd.registry import lookup
    raw = copy.deepcopy(CONFIG_U)
    raw["layers"][0]["mixer"]["dim"] = 300
    spec = config_from_dict(raw).to_spec()
    with pytest.raises(EngineError):
        lookup("mixer", spec.layers[0].mixer.kind)(spec.layers[0].mixer, torch.float32, "cpu")
    raw = copy.deepcopy(CONFIG_U)
    raw["canon"]["taps"] = 40
    spec = config_from_dict(raw).to_spec()
    with pytest.raises(EngineError):
        lookup("sublayer_input", "residual_conv")(spec.layers[0].sublayer_input, torch.float32, "cpu")


def test_random_weights_follow_the_expected_tensors(tmp_path):
    from tugalix_helpers import load_plain, make_model
    folder = make_model(tmp_path, CONFIG_W, seed=3)
    raw, weights = load_plain(folder)
    assert {key: value for key, value in raw.items() if key != "torch_dtype"} == CONFIG_W
    assert weights["l0.mix.right.w1"].shape == (16, 32) and weights["l0.dwa"].shape == (2,)
    assert float(weights["l0.mix.right.mu.k"].min()) >= 0.0 and float(weights["l0.mix.right.mu.k"].max()) <= 1.0
    assert abs(float(weights["l0.dwa"][-1]) - 1.0) < 0.8


# ---- the plain implementation's own pieces ------------------------------------------------------------------
def test_plain_layer_norm_and_unit_rms():
    x = torch.randn(5, 12, dtype=torch.float64)
    weight, bias = torch.randn(12, dtype=torch.float64), torch.randn(12, dtype=torch.float64)
    want = torch.nn.functional.layer_norm(x, (12,), weight, bias, 1e-5)
    assert torch.allclose(plain.layer_norm(x, weight, bias, 1e-5), want, atol=1e-12)
    normed = plain.unit_rms(x, 0.0)
    assert torch.allclose((normed * normed).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-12)


def test_plain_input_convolution_is_causal_and_its_last_tap_weighs_the_token_itself():
    h = torch.randn(9, 4, dtype=torch.float64)
    taps = torch.randn(4, 3, dtype=torch.float64)
    out = plain.input_convolution(h, taps)
    assert torch.allclose(out[0], h[0] * (1 + taps[:, 2]))
    assert torch.allclose(out[5], h[5] * (1 + taps[:, 2]) + h[4] * taps[:, 1] + h[3] * taps[:, 0])
    changed = h.clone()
    changed[6] += 1.0
    assert torch.equal(plain.input_convolution(changed, taps)[:6], out[:6])


def test_plain_rotation_keeps_lengths_and_depends_on_distance_only():
    x, y = torch.randn(1, 1, 10, dtype=torch.float64), torch.randn(1, 1, 10, dtype=torch.float64)
    def dot(p, q):
        a = plain.rotate_halves(x, torch.tensor([p]), 6, 50.0)
        b = plain.rotate_halves(y, torch.tensor([q]), 6, 50.0)
        return float((a * b).sum())
    assert abs(dot(3, 1) - dot(40, 38)) < 1e-9
    turned = plain.rotate_halves(x, torch.tensor([17]), 6, 50.0)
    assert abs(float(turned.norm()) - float(x.norm())) < 1e-12 and torch.equal(turned[..., 6:], x[..., 6:])
    assert torch.equal(plain.rotate_halves(x, torch.tensor([0]), 6, 50.0), x)


def test_plain_xielu_is_continuous_with_slope_one_half_at_zero():
    p, q = 0.3, -0.2
    z = torch.tensor([-1e-7, 0.0, 1e-7], dtype=torch.float64)
    out = plain.xielu(z, p, q)
    assert abs(float(out[1])) == 0.0 and abs(float((out[2] - out[0]) / 2e-7) - 0.5) < 1e-6
    assert float(plain.xielu(torch.tensor([2.0], dtype=torch.float64), p, q)) == pytest.approx(math.log1p(math.exp(p)) * 4 + 1)
    want = (0.5 + math.log1p(math.exp(q))) * (math.exp(-3.0) - 1 + 3.0) - 1.5
    assert float(plain.xielu(torch.tensor([-3.0], dtype=torch.float64), p, q)) == pytest.approx(want)


def test_plain_state_walk_equals_the_sum_over_earlier_tokens():
    """o_t = sum_(s <= t) (q_t . (prod_(s < r <= t) decay_r) k_s) v_s.  With a bonus the result reads the state before
    the token's own decay acts on it (the products end at t - 1) and the current token's share is weighed by the bonus."""
    T, dim, vdim = 7, 3, 4
    q, k, decay = (torch.rand(T, dim, dtype=torch.float64) for _ in range(3))
    v = torch.randn(T, vdim, dtype=torch.float64)
    bonus = torch.randn(dim, dtype=torch.float64)
    got, got_bonus = plain.decayed_state_walk(q, k, v, decay), plain.decayed_state_walk(q, k, v, decay, bonus=bonus)

    def summed(t, last, upto):
        total = torch.zeros(vdim, dtype=torch.float64)
        for s in range(upto):
            keep = torch.ones(dim, dtype=torch.float64)
            for r in range(s + 1, last + 1):
                keep = keep * decay[r]
            total += float((q[t] * keep * k[s]).sum()) * v[s]
        return total
    for t in range(T):
        assert torch.allclose(got[t], summed(t, t, t + 1), atol=1e-12)
        assert torch.allclose(got_bonus[t], summed(t, t - 1, t) + float((q[t] * bonus * k[t]).sum()) * v[t], atol=1e-12)


def test_plain_attention_sees_no_later_token_and_groups_share_keys():
    mixer = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 5, "scale": 0.4, "rot": {"base": 10.0, "dims": 4}}
    generator = torch.Generator().manual_seed(1)
    w = {"q": torch.randn(24, 8, generator=generator, dtype=torch.float64), "k": torch.randn(12, 8, generator=generator, dtype=torch.float64),
         "v": torch.randn(10, 8, generator=generator, dtype=torch.float64), "o": torch.eye(20, dtype=torch.float64)}
    h = torch.randn(6, 8, generator=generator, dtype=torch.float64)
    out = plain.softmax_attention(mixer, w, "", h, torch.arange(6))
    changed = h.clone()
    changed[4] += 1.0
    assert torch.equal(plain.softmax_attention(mixer, w, "", changed, torch.arange(6))[:4], out[:4])
    # the first token sees itself only: every head gives its group's value
    v0 = (h[0] @ w["v"].T).reshape(2, 5)
    assert torch.allclose(out[0].reshape(4, 5), v0[[0, 0, 1, 1]], atol=1e-12)


def test_plain_depth_average_of_a_model_whose_last_weight_is_one(tmp_path):
    """With weights (0, .., 0, 1) the sum over the results so far is the layer's own result."""
    from tugalix_helpers import load_plain, make_model, rewrite
    folder = make_model(tmp_path, CONFIG_V, seed=5)

    def last_only(weights):
        for index in range(3):
            weights[f"l{index}.dwa"][:] = 0.0
            weights[f"l{index}.dwa"][-1] = 1.0
    config, weights = rewrite(folder, last_only)
    tokens = [3, 1, 4, 1, 5, 9, 2, 6]
    logits, after = plain.forward(config, weights, tokens)
    assert logits.shape == (8, 90) and len(after) == 3
    # the same model with a weight on the embedding's output differs from the first layer on
    config, weights = rewrite(folder, lambda w: w["l0.dwa"].__setitem__(0, 0.5))
    assert float((plain.forward(config, weights, tokens)[1][0] - after[0]).abs().max()) > 1e-3
