"""The Tugalix decoder on the GPU against the plain implementation (tests/plain_tugalix.py): each mechanism
alone, then whole models through the engine's step function, cache manager, scheduler and entry point,
however the work is cut."""
import math
import random
from types import SimpleNamespace

import pytest
import torch

import plain_tugalix as plain
from tugalix_helpers import (CONFIGS, CUT_TOLERANCE, DTYPES, SINGLE_LAYER_TOLERANCE, TOLERANCE, load_plain, make_model,
                             plain_generate_greedy, rewrite, row_errors, run_cut)

pytestmark = pytest.mark.gpu
CASES = [(name, dtype) for name in CONFIGS for dtype in DTYPES]
DEVICE = "cuda:0"
TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def tokens_of(seed, count, vocab, avoid=()):
    rng = random.Random(seed)
    out = []
    while len(out) < count:
        token = rng.randrange(vocab)
        if token not in avoid:
            out.append(token)
    return out


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            folder = make_model(tmp_path_factory.mktemp(f"tugalix_{name}"), CONFIGS[name], seed=37)
            raw, weights = load_plain(folder)
            made[name] = {"folder": folder, "raw": raw, "weights": weights, "plain": {}}
        return made[name]
    return get


def plain_logits(setup, tokens):
    key = tuple(tokens)
    if key not in setup["plain"]:
        setup["plain"][key] = plain.forward(setup["raw"], setup["weights"], list(tokens))[0]
    return setup["plain"][key]


def new_engine(setup, dtype, max_tokens=640, page_size=16, max_requests=4, **options):
    from tlie_amd import Engine
    return Engine(setup["folder"], dtype=dtype, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests, **options)


def assert_rows(got, want, tolerance, what):
    errors = row_errors(got, want)
    worst = int(errors.argmax())
    assert float(errors.max()) <= tolerance, f"{what}: row {worst} is off by {float(errors[worst]):.3g} of its largest value (allowed {tolerance})"


def split_product(dense, nsplit, generator):
    """A product as `nsplit` float partial sums that add up to `dense`."""
    from tlie_amd import ops
    if nsplit == 1:
        return ops.Product(dense.to(DEVICE).contiguous(), 1)
    parts = torch.randn(nsplit, *dense.shape, generator=generator)
    parts[0] += dense.float() - parts.sum(0)
    return ops.Product(parts.to(DEVICE).contiguous(), nsplit)


def step_arrays(counts, slots):
    """The arrays of a step in which sequence i brings counts[i] tokens and sits in slots[i]; one sequence more without
    a slot and without tokens stands for the padding of a recorded step."""
    starts, token_seq, token_slot = [0], [], []
    for index, (count, slot) in enumerate(zip(counts, slots)):
        starts.append(starts[-1] + count)
        token_seq += [index] * count
        token_slot += [slot] * count
    as_int = lambda values: torch.tensor(values, dtype=torch.int32, device=DEVICE)     # noqa: E731
    return SimpleNamespace(seq_start=as_int(starts + [starts[-1]]), seq_slot=as_int(list(slots) + [-1]), token_seq=as_int(token_seq),
                           token_slot=as_int(token_slot), max_new=max(counts)), starts


def in_steps(lengths, steps, slots, run):
    """Walks sequences of `lengths` through `steps` (per step the tokens each sequence brings; 0: it pauses) and
    returns, per sequence, what run(ctx, pieces) gave for its tokens; pieces[i] = (sequence, from, to) of the step's i-th
    live sequence."""
    got, at = [[] for _ in lengths], [0] * len(lengths)
    for counts in steps:
        live = [s for s in range(len(lengths)) if counts[s] > 0]
        ctx, starts = step_arrays([counts[s] for s in live], [slots[s] for s in live])
        out = run(ctx, [(s, at[s], at[s] + counts[s]) for s in live])
        for i, s in enumerate(live):
            got[s].append(out[..., starts[i]:starts[i + 1], :].cpu())
            at[s] += counts[s]
    assert at == list(lengths)
    return [torch.cat(pieces, dim=-2) for pieces in got]


SHORT_STEPS = ([23, 9], [(1, 4), (5, 0), (2, 1), (1, 1), (14, 3)])
LONG_STEPS = ([260, 41], [(97, 1), (1, 30), (130, 0), (31, 9), (1, 1)])


# ---- each mechanism alone ----------------------------------------------------------------------------------
@pytest.mark.parametrize("tokens,hidden,nsplit,out_dtype", [(6, 80, 1, torch.float32), (3, 203, 2, torch.bfloat16), (20, 32, 1, torch.float32)])
def test_layer_norm_adds_what_the_residual_lacks(tokens, hidden, nsplit, out_dtype):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(hidden)
    x, a, b = (torch.randn(tokens, hidden, generator=generator) for _ in range(3))
    x = x * 3.0 + 5.0                                           # (a mean that is not small beside the deviations)
    weight, bias = (torch.randn(hidden, generator=generator).to(out_dtype) for _ in range(2))       # (stored in the run's type)
    tolerance = 1e-5 if out_dtype == torch.float32 else 2e-2
    residual = x.clone().to(DEVICE)
    got = ops.layer_norm(residual, None, weight.to(DEVICE), bias.to(DEVICE), 1e-5, out_dtype)
    assert got.dtype == out_dtype and torch.equal(residual.cpu(), x)
    assert float((got.cpu().double() - plain.layer_norm(x.double(), weight.double(), bias.double(), 1e-5)).abs().max()) < tolerance * 4
    # a product; then the two scaled products of a mixer of two branches
    residual = x.clone().to(DEVICE)
    got = ops.layer_norm(residual, split_product(a, nsplit, generator), weight.to(DEVICE), bias.to(DEVICE), 1e-5, out_dtype)
    assert float((residual.cpu().double() - (x.double() + a.double())).abs().max()) < 1e-5
    assert float((got.cpu().double() - plain.layer_norm(x.double() + a.double(), weight.double(), bias.double(), 1e-5)).abs().max()) < tolerance * 4
    residual = x.clone().to(DEVICE)
    both = ops.ScaledSum(split_product(a, nsplit, generator), 0.8, split_product(b, 1, generator), -1.7)
    got = ops.layer_norm(residual, both, weight.to(DEVICE), None, 1e-5, out_dtype)
    summed = x.double() + 0.8 * a.double() - 1.7 * b.double()
    assert float((residual.cpu().double() - summed).abs().max()) < 1e-5
    assert float((got.cpu().double() - plain.layer_norm(summed, weight.double(), torch.zeros(hidden, dtype=torch.float64), 1e-5)).abs().max()) < tolerance * 4
    # only some rows: nothing but the result is written
    rows = torch.tensor([tokens - 1, 0], dtype=torch.int32, device=DEVICE)
    residual = x.clone().to(DEVICE)
    got = ops.layer_norm(residual, split_product(a, nsplit, generator), weight.to(DEVICE), bias.to(DEVICE), 1e-5, out_dtype, rows=rows)
    want = plain.layer_norm((x.double() + a.double())[[tokens - 1, 0]], weight.double(), bias.double(), 1e-5)
    assert torch.equal(residual.cpu(), x) and float((got.cpu().double() - want).abs().max()) < tolerance * 4


@pytest.mark.parametrize("entries,count", [(5, 2), (5, 4), (3, 3), (9, 8)])
def test_layer_norm_reads_a_weighted_sum_over_earlier_results(entries, count):
    """The residual is the last of `count` results; what is normed and handed on is their weighted sum.  Weights that
    single out each summand in turn show a summand that is left out or taken twice."""
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(entries * count)
    tokens, hidden = 7, 48
    results = torch.randn(entries, tokens, hidden, generator=generator)
    delta = torch.randn(tokens, hidden, generator=generator)
    weight, bias = torch.randn(hidden, generator=generator), torch.randn(hidden, generator=generator)
    choices = [torch.randn(count, generator=generator)] + [torch.eye(count)[j] for j in range(count)]
    for mix in choices:
        history = results.clone().to(DEVICE)
        mixed = history[count] if count < entries else torch.empty(tokens, hidden, device=DEVICE)
        got = ops.layer_norm(history[count - 1], ops.Product(delta.to(DEVICE), 1), weight.to(DEVICE), bias.to(DEVICE), 1e-5, torch.float32,
                             history=history, history_count=count, history_weight=mix.to(DEVICE), mixed=mixed)
        own = results[count - 1].double() + delta.double()
        want = sum(float(mix[j]) * results[j].double() for j in range(count - 1)) + float(mix[count - 1]) * own
        assert float((history[count - 1].cpu().double() - own).abs().max()) < 1e-5            # the run's own result stays
        assert float((mixed.cpu().double() - want).abs().max()) < 1e-5
        assert float((got.cpu().double() - plain.layer_norm(want, weight.double(), bias.double(), 1e-5)).abs().max()) < 1e-4
        assert torch.equal(history[:count - 1].cpu(), results[:count - 1])
        rows = torch.tensor([3, 6], dtype=torch.int32, device=DEVICE)
        history = results.clone().to(DEVICE)
        some = ops.layer_norm(history[count - 1], ops.Product(delta.to(DEVICE), 1), weight.to(DEVICE), bias.to(DEVICE), 1e-5, torch.float32,
                              rows=rows, history=history, history_count=count, history_weight=mix.to(DEVICE))
        assert float((some - got[[3, 6]]).abs().max()) < 1e-6 and torch.equal(history.cpu(), results)


@pytest.mark.parametrize("taps,channels,plan,out_dtype", [(4, 80, SHORT_STEPS, torch.float32), (1, 44, SHORT_STEPS, torch.float32),
                                                           (2, 32, LONG_STEPS, torch.bfloat16), (5, 203, SHORT_STEPS, torch.float32),
                                                           (8, 16, LONG_STEPS, torch.float32)])
def test_the_input_convolution_carries_its_last_inputs(taps, channels, plan, out_dtype):
    """Two sequences in steps of unequal portions (shorter than the taps reach, down to one token), in slots that are
    not in order; a slot that belongs to nobody stays as it is."""
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(taps * channels)
    (lengths, steps), slots = plan, [2, 0]
    inputs = [torch.randn(length, channels, generator=generator) for length in lengths]
    weight = torch.randn(channels, taps, generator=generator).to(out_dtype)
    area = torch.zeros(3, 2, max(taps - 1, 1), channels, device=DEVICE)       # (two parts' rows side by side: the slots lie apart)
    area[1] = 5.0
    state = area[:, 1]

    def run(ctx, pieces):
        h = torch.cat([inputs[s][a:b] for s, a, b in pieces]).to(DEVICE).contiguous()
        return ops.input_conv(h, weight.to(DEVICE), state, ctx, out_dtype)
    got = in_steps(lengths, steps, slots, run)
    for s in (0, 1):
        want = plain.input_convolution(inputs[s].double(), weight.double())
        assert float((got[s].double() - want).abs().max()) < (1e-5 if out_dtype == torch.float32 else 5e-2), f"sequence {s}"
    assert float((area[1] - 5.0).abs().max()) == 0.0 and float(area[[0, 2], 0].abs().max()) == 0.0
    if taps > 1:                                                 # what is kept: the last inputs, oldest first
        assert torch.equal(state[2].cpu(), inputs[0][-(taps - 1):])


@pytest.mark.parametrize("width,mixes,plan,dtype", [(80, 5, SHORT_STEPS, torch.float32), (44, 1, LONG_STEPS, torch.float32),
                                                    (203, 5, SHORT_STEPS, torch.bfloat16)])
def test_the_token_shift_blends_with_the_token_before(width, mixes, plan, dtype):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(width + mixes)
    (lengths, steps), slots = plan, [1, 0]
    inputs = [torch.randn(length, width, generator=generator).to(dtype) for length in lengths]
    mu = torch.rand(mixes, width, generator=generator).to(dtype)
    area = torch.zeros(3, 11 + width, device=DEVICE)
    area[2] = 5.0
    state = area[:, 11:]                                          # a row's end: the slots lie apart

    def run(ctx, pieces):
        x = torch.cat([inputs[s][a:b] for s, a, b in pieces]).to(DEVICE).contiguous()
        return ops.token_shift(x, mu.to(DEVICE), state, ctx)
    got = in_steps(lengths, steps, slots, run)
    for s in (0, 1):
        x = inputs[s].double()
        before = torch.cat([torch.zeros(1, width, dtype=torch.float64), x[:-1]])
        want = x[None] + (before - x)[None] * mu.double()[:, None, :]
        assert got[s].shape == want.shape
        assert float((got[s].double() - want).abs().max()) < (1e-5 if dtype == torch.float32 else 5e-2), f"sequence {s}"
        assert torch.equal(state[slots[s]].cpu(), inputs[s][-1].float())
    assert float((area[2] - 5.0).abs().max()) == 0.0 and float(area[:2, :11].abs().max()) == 0.0


@pytest.mark.parametrize("nsplit,out_dtype", [(1, torch.float32), (3, torch.float32), (1, torch.bfloat16)])
def test_xielu(nsplit, out_dtype):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(nsplit)
    pre = torch.randn(9, 56, generator=generator) * 3.0
    pre[0, :4] = torch.tensor([0.0, -0.0, 1e-6, -1e-6])
    for p, q in ((0.3, -0.2), (-2.0, 1.5)):
        numbers = torch.tensor([p, q]).to(out_dtype)
        got = ops.xielu(split_product(pre, nsplit, generator), numbers.to(DEVICE), out_dtype)
        want = plain.xielu(pre.double(), float(numbers[0]), float(numbers[1]))
        assert got.dtype == out_dtype
        assert float(((got.cpu().double() - want).abs() / (1.0 + want.abs())).max()) < (1e-5 if out_dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("heads,heads_a,dim,rot_dim,tail,nsplit", [(6, 3, 16, 8, 20, 1), (2, 1, 130, 2, 0, 2), (8, 4, 6, 6, 7, 1), (4, 2, 32, 0, 5, 1)])
def test_heads_are_turned_by_their_positions_and_scaled(heads, heads_a, dim, rot_dim, tail, nsplit):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(heads * dim)
    tokens, col, base = 11, 3, 100.0
    fused = torch.randn(tokens, col + heads * dim + tail + 2, generator=generator)
    positions = torch.tensor([0, 1, 2, 3, 17, 64, 65, 1000, 4095, 70000, 5], dtype=torch.int32)
    inv_freq = torch.tensor([base ** (-2.0 * i / rot_dim) for i in range(rot_dim // 2)], dtype=torch.float32) if rot_dim else None
    got = ops.rotate_heads(split_product(fused, nsplit, generator), col, positions.to(DEVICE), inv_freq.to(DEVICE) if rot_dim else None,
                           rot_dim, heads, heads_a, dim, 1.0, 0.25, tail=tail)
    x = fused[:, col:col + heads * dim].double().reshape(tokens, heads, dim)
    want = plain.rotate_halves(x, positions, rot_dim, base) if rot_dim else x.clone()
    want[:, heads_a:] *= 0.25
    want = torch.cat([want.reshape(tokens, -1), fused[:, col + heads * dim:col + heads * dim + tail].double()], dim=1)
    # (an angle of 70000 radians in 32-bit is known to 4e-3; positions this far show a table that is indexed wrongly, not rounding)
    close = (got.cpu().double() - want).abs()
    assert got.shape == want.shape and float(close[:9].max()) < 2e-3 and float(close.max()) < 5e-2
    assert float(close[:7].max()) < 2e-5


@pytest.mark.parametrize("kind,tokens,channels,rank,dtype", [("sigmoid_root", 9, 72, 5, torch.float32), ("exp_neg_exp", 4, 320, 16, torch.bfloat16),
                                                             ("sigmoid_root", 3, 16, 64, torch.bfloat16), ("exp_neg_exp", 70, 8, 3, torch.float32)])
def test_decays_from_a_low_rank_product(kind, tokens, channels, rank, dtype):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(channels + rank)
    low = torch.randn(tokens, rank, generator=generator) * 2.0
    weight = torch.randn(channels, rank, generator=generator).to(dtype)
    bias = (torch.randn(channels, generator=generator) * 4.0).to(dtype)          # (far into both tails of the sigmoid)
    tau = 7.0
    for inner_tanh in (False, True):
        got = ops.low_rank_decay(low.to(DEVICE), weight.to(DEVICE), bias.to(DEVICE), kind, tau=tau, inner_tanh=inner_tanh)
        inner = torch.tanh(low.double()) if inner_tanh else low.double()
        z = inner @ weight.double().T + bias.double()
        want = torch.sigmoid(z) ** (1.0 / tau) if kind == "sigmoid_root" else torch.exp(-torch.exp(z))
        assert got.dtype == torch.float32 and float((got.cpu().double() - want).abs().max()) < 2e-5
        # the logarithm, which is what a long product of decays feels
        mask = want > 1e-30
        assert float((torch.log(got.cpu().double()[mask]) - torch.log(want[mask])).abs().div(1.0 + torch.log(want[mask]).abs()).max()) < 1e-4


def _scan_case(kind, heads, dim, vdim, plan, nsplit, dtype, generator):
    """q, k, v of two sequences, decays of the kind asked for, and the plain walk's results."""
    lengths, steps = plan
    width = 2 * heads * dim + heads * vdim + 5                     # q | k | v | columns of someone else's
    fused = [(torch.randn(length, width, generator=generator) * 0.5).to(dtype) for length in lengths]
    head_decay = torch.tensor([(0.999, 0.5, 1.0, 0.0, 0.97)[h % 5] for h in range(heads)])
    # the first sequence forgets next to nothing, the second quickly
    decay = [torch.rand(length, heads * dim, generator=generator) * (0.02, 0.9)[s] + (0.98, 0.05)[s] for s, length in enumerate(lengths)]
    bonus = torch.randn(heads * dim, generator=generator)
    want = []
    for s, x in enumerate(fused):
        x = x.double()
        q = x[:, :heads * dim].reshape(-1, heads, dim) * 0.7
        k = x[:, heads * dim:2 * heads * dim].reshape(-1, heads, dim) * 1.3
        v = x[:, 2 * heads * dim:2 * heads * dim + heads * vdim].reshape(-1, heads, vdim)
        outs = []
        for h in range(heads):
            w = decay[s].double().reshape(-1, heads, dim)[:, h] if kind != "head" else torch.full((x.shape[0], dim), float(head_decay[h]), dtype=torch.float64)
            outs.append(plain.decayed_state_walk(q[:, h], k[:, h], v[:, h], w, bonus=bonus.double().reshape(heads, dim)[h] if kind == "bonus" else None))
        want.append(torch.cat(outs, dim=-1))
    return fused, head_decay, decay, bonus, want


@pytest.mark.parametrize("kind", ["head", "channel", "bonus"])
@pytest.mark.parametrize("heads,dim,vdim,plan,nsplit,dtype", [
    (3, 24, 40, SHORT_STEPS, 1, torch.float32), (2, 72, 130, SHORT_STEPS, 2, torch.float32), (1, 160, 16, LONG_STEPS, 1, torch.float32),
    (2, 8, 70, LONG_STEPS, 1, torch.float32), (4, 32, 64, LONG_STEPS, 1, torch.bfloat16), (1, 256, 5, SHORT_STEPS, 1, torch.float32),
    (5, 6, 64, LONG_STEPS, 3, torch.float32)])
def test_the_decaying_state_is_carried_from_step_to_step(kind, heads, dim, vdim, plan, nsplit, dtype):
    """Two sequences of unequal length in steps of unequal portions (one token; just below and above where the walk goes
    in slices, and no multiple of a slice), in slots that are not in order, against the plain walk over each whole
    sequence.  The state rows are wider than the scan's part, as a mixer's that keeps more than S."""
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(dim + vdim)
    (lengths, steps), slots = plan, [2, 0]
    fused, head_decay, decay, bonus, want = _scan_case(kind, heads, dim, vdim, plan, nsplit, dtype, generator)
    shape = ops.decay_scan_state_shape(heads, dim, vdim)
    floats = shape[0] * shape[1] * shape[2]
    state = torch.zeros(3, floats + 9, device=DEVICE)
    state[1] = 5.0
    state[:, floats:] = 7.0

    def run(ctx, pieces):
        rows = torch.cat([fused[s][a:b] for s, a, b in pieces])
        product = split_product(rows, nsplit, generator) if dtype == torch.float32 else ops.Product(rows.to(DEVICE).contiguous(), 1)
        options = {"head_decay": head_decay.to(DEVICE)} if kind == "head" else {"decay": torch.cat([decay[s][a:b] for s, a, b in pieces]).to(DEVICE).contiguous()}
        if kind == "bonus":
            options["bonus"] = bonus.to(DEVICE)
        return ops.decay_scan((product, 0), (product, heads * dim), (product, 2 * heads * dim), state, ctx.seq_start, ctx.seq_slot,
                              heads, dim, vdim, q_scale=0.7, k_scale=1.3, max_new=ctx.max_new, **options)
    got = in_steps(lengths, steps, slots, run)
    for s in (0, 1):
        error = (got[s].double() - want[s]).abs().max() / want[s].abs().max()
        assert float(error) < 2e-5, f"sequence {s}: {float(error):.3g}"
    assert float((state[1, :floats] - 5.0).abs().max()) == 0.0 and float((state[:, floats:] - 7.0).abs().max()) == 0.0


def test_a_sliced_walk_equals_the_walk_in_order():
    """The same step once token by token in order and once in slices side by side, at counts around a slice's and the
    switch's edges: the state left behind and the results agree to rounding."""
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(77)
    heads, dim, vdim = 2, 48, 70
    for count in (ops.SCAN_SLICE - 1, ops.SCAN_SLICE, ops.SCAN_SLICE + 1, ops.SCAN_SLICED_FROM - 1, ops.SCAN_SLICED_FROM, ops.SCAN_SLICED_FROM + 1, 4 * ops.SCAN_SLICE, 201):
        fused = torch.randn(count + 3, 2 * heads * dim + heads * vdim, generator=generator).to(DEVICE)
        decay = (torch.rand(count + 3, heads * dim, generator=generator) * 0.3 + 0.7).to(DEVICE)
        product = ops.Product(fused, 1)
        ctx, _ = step_arrays([count, 3], [1, 0])
        results, states = [], []
        for max_new in (1, max(count, ops.SCAN_SLICED_FROM)):          # (the first never slices, the second always)
            state = torch.randn(2, *ops.decay_scan_state_shape(heads, dim, vdim), generator=torch.Generator().manual_seed(5)).to(DEVICE)
            results.append(ops.decay_scan((product, 0), (product, heads * dim), (product, 2 * heads * dim), state, ctx.seq_start, ctx.seq_slot,
                                          heads, dim, vdim, decay=decay, max_new=max_new))
            states.append(state)
        scale = float(results[0].abs().max())
        assert float((results[0] - results[1]).abs().max()) < 2e-5 * scale, f"{count} tokens"
        assert float((states[0] - states[1]).abs().max()) < 2e-5 * float(states[0].abs().max()), f"{count} tokens"


@pytest.mark.parametrize("heads,dv,nsplit", [(3, 40, 1), (2, 130, 2), (6, 8, 1)])
def test_heads_are_normed_weighed_and_gated(heads, dv, nsplit):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(heads * dv)
    tokens, eps = 7, 1e-5
    a = torch.randn(tokens, heads, dv, generator=generator) * 4.0
    a[0] = 1e-4                                                    # a head whose mean square is of eps' size
    gate = torch.randn(tokens, 11 + heads * dv, generator=generator)
    weight = torch.randn(heads * dv, generator=generator)
    silu = plain.silu(gate[:, 11:].double())
    got = ops.head_combine(a.reshape(tokens, -1).contiguous().to(DEVICE), heads, dv, eps, torch.float32, gate=split_product(gate, nsplit, generator),
                           gate_col=11, gate_kind="silu")
    want = plain.unit_rms(a.double(), eps).reshape(tokens, -1) * silu
    assert float((got.cpu().double() - want).abs().max()) < 2e-5
    got = ops.head_combine(a.reshape(tokens, -1).contiguous().to(DEVICE), heads, dv, eps, torch.float32, weight=weight.to(DEVICE),
                           gate=split_product(gate, nsplit, generator), gate_col=11, gate_kind="silu")
    assert float((got.cpu().double() - want * weight.double()).abs().max()) < 5e-5


# ---- single layers through the engine: a mixer's result from its input, and inputs made so that a fault shows ---------
def _single_layer(tmp_path, layer, seed, vocab=97, width=48, taps=3, changes=None):
    raw = {"architecture": "Tugalix", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "canon": {"taps": taps}, "logit_scale": 1.0,
           "layers": [layer]}
    folder = make_model(tmp_path, raw, seed=seed)
    config, weights = load_plain(folder)
    if changes is not None:
        config, weights = rewrite(folder, changes)
    return folder, config, weights


def _mixer_alone(folder, tokens, dtype, cuts):
    """The mixer's input and result of every token, from the traces of steps of the sizes `cuts`."""
    from tlie_amd import Engine, StepEntry
    engine = Engine(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=2)
    engine.admit("a")
    inputs, results, at, index = [], [], 0, 0
    while at < len(tokens):
        count = min(cuts[index % len(cuts)], len(tokens) - at)
        trace = {}
        engine.step([StepEntry("a", tokens[at:at + count], [count - 1])], trace=trace)
        inputs.append(trace["layer0.input_norm"].cpu())
        results.append(trace["layer0.attention_output"].cpu())
        at += count
        index += 1
    return torch.cat(inputs).double(), torch.cat(results).double()


RETENTIONS = [
    {"heads": 3, "dim": 16, "vdim": 20, "decay": [0.9, 0.99, 0.5], "rot": {"base": 100.0, "dims": 8}},
    {"heads": 1, "dim": 130, "vdim": 8, "decay": [0.998], "rot": {"base": 30.0, "dims": 2}},
    {"heads": 4, "dim": 6, "vdim": 70, "decay": [1.0, 0.0, 0.75, 0.96], "rot": {"base": 7.0, "dims": 6}},
    {"heads": 2, "dim": 64, "vdim": 128, "decay": [0.97, 0.999], "rot": {"base": 500000.0, "dims": 64}},
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mixer", RETENTIONS)
def test_retention_alone(tmp_path, mixer, dtype):
    folder, config, weights = _single_layer(tmp_path, {"type": "retention", "mixer": mixer, "mlp": None}, seed=5)
    tokens = tokens_of(6, 150, 97)
    for cuts in ([150], [33, 1, 2, 20, 97], [1]):
        h, got = _mixer_alone(folder, tokens, dtype, cuts)
        want = plain.retention(mixer, weights, "l0.mix.", h, torch.arange(len(tokens)), 1e-5)
        assert_rows(got, want, 3e-5 if dtype == "float32" else 3e-2, f"cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mixer", [{"heads": 3, "dim": 24, "vdim": 40, "tau": 8.0, "rank": 5}, {"heads": 2, "dim": 8, "vdim": 130, "tau": 1.0},
                                   {"heads": 1, "dim": 160, "vdim": 16, "tau": 64.0, "rank": 40}, {"heads": 4, "dim": 64, "vdim": 64, "tau": 16.0}])
def test_gated_linear_attention_alone(tmp_path, mixer, dtype):
    folder, config, weights = _single_layer(tmp_path, {"type": "gla", "mixer": mixer, "mlp": None}, seed=7)
    assert weights["l0.mix.a1"].shape[0] == mixer.get("rank", 16)
    tokens = tokens_of(8, 150, 97)
    for cuts in ([150], [30, 1, 2, 9, 100], [1]):
        h, got = _mixer_alone(folder, tokens, dtype, cuts)
        want = plain.gated_linear_attention(mixer, weights, "l0.mix.", h, 1e-5)
        assert_rows(got, want, 3e-5 if dtype == "float32" else 3e-2, f"cuts {cuts}")


SIDES = [
    {"left": (4, 2, 16, 24, 0.3, 500.0, 8), "right": (3, 24, 7), "scales": (1.3, 0.5)},
    {"left": (6, 6, 32, 32, 0.2, 10000.0, 32), "right": (1, 72, 3), "scales": (-0.4, 1.0)},
    {"left": (2, 1, 8, 70, 0.5, 20.0, 4), "right": (2, 160, 16), "scales": (0.6, -1.2)},
    {"left": (4, 4, 64, 64, 0.11, 10000.0, 64), "right": (5, 8, 16), "scales": (1.0, 0.0)},         # the left side alone
    {"left": (2, 2, 16, 16, 0.25, 10000.0, 16), "right": (2, 64, 16), "scales": (0.0, 1.0)},        # the right side alone
]


def _side_mixer(side):
    heads, groups, dim, vdim, scale, base, dims = side["left"]
    return {"left": {"heads": heads, "kv_heads": groups, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": base, "dims": dims}},
            "right": dict(zip(("heads", "dim", "rank"), side["right"])), "left_scale": side["scales"][0], "right_scale": side["scales"][1]}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("side", SIDES)
def test_attention_beside_token_shift_mixing_alone(tmp_path, side, dtype):
    mixer = _side_mixer(side)
    folder, config, weights = _single_layer(tmp_path, {"type": "parallel", "mixer": mixer, "mlp": None}, seed=9)
    tokens = tokens_of(10, 300, 97)             # (long enough for the keys to be cut into parts that are merged)
    for cuts in ([300], [33, 1, 2, 20, 150], [280] + [1] * 20):
        h, got = _mixer_alone(folder, tokens, dtype, cuts)
        want = plain.side_by_side(mixer, weights, "l0.mix.", h, torch.arange(len(tokens)), 1e-5)
        assert_rows(got, want, 3e-5 if dtype == "float32" else 3e-2, f"cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps,ff", [(1, 56), (2, 120), (5, 20)])
def test_the_feed_forward_and_both_convolutions(tmp_path, taps, ff, dtype):
    """A layer's second sublayer from its input: the activation's two numbers on both sides of zero, a convolution of its
    own state beside the mixer's."""
    from tlie_amd import Engine, StepEntry
    layer = {"type": "retention", "mixer": RETENTIONS[0], "mlp": {"kind": "dense", "ff": ff}}
    folder, config, weights = _single_layer(tmp_path, layer, seed=15, taps=taps,
                                            changes=lambda w: w["l0.mlp.act"].copy_(torch.tensor([0.7, -0.4], dtype=torch.float64)))
    tokens = tokens_of(16, 70, 97)
    whole = None
    for cuts in ([70], [2], [1], [9, 1, 3]):
        engine = Engine(folder, dtype=dtype, max_tokens=256, page_size=16, max_requests=2)
        engine.admit("a")
        normed, conved, results, at, index = [], [], [], 0, 0
        while at < len(tokens):
            count = min(cuts[index % len(cuts)], len(tokens) - at)
            trace = {}
            engine.step([StepEntry("a", tokens[at:at + count], [count - 1])], trace=trace)
            conved.append(trace["layer0.post_attention_norm"].cpu())
            results.append(trace["layer0.mlp_output"].cpu())
            at += count
            index += 1
        h, got = torch.cat(conved).double(), torch.cat(results).double()
        assert_rows(got, plain.dense_feed_forward(weights, "l0.mlp.", h), 3e-5 if dtype == "float32" else 3e-2, f"cuts {cuts}")
        if whole is None:
            whole = h
        else:                                                    # what the feed-forward reads does not depend on the cut
            assert_rows(h, whole, 1e-5 if dtype == "float32" else 3e-2, f"the convolution's result, cuts {cuts}")


def _boosted(tmp_path, layer, seed, boost, taps=3):
    """A single-layer model whose weights `boost(weights, h_of)` has changed; h_of(token) is what the mixer reads for a
    token that stands alone among tokens it does not resemble (the norm's result with its own tap of the convolution)."""
    def changes(weights):
        def h_of(token):
            x = plain.layer_norm(weights["embed"][token], weights["embed.norm"], weights["embed.norm.b"], 1e-5)
            h = plain.layer_norm(x, weights["l0.norm1"], weights["l0.norm1.b"], 1e-5)
            return h * (1.0 + weights["l0.canon1"][:, -1])
        weights["l0.canon1"][:, :-1] *= 0.05                     # the neighbours' share of a token's input stays small
        boost(weights, h_of)
    return _single_layer(tmp_path, layer, seed, taps=taps, changes=changes)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("far", [0, 1, 15, 16, 17, 31, 32, 250])
def test_one_far_key_among_hundreds_decides_the_result(tmp_path, dtype, far):
    """One head of the attention is made to look at one position only: token B's key and token A's query are large in a
    dim that does not turn, so that B's value decides what A's head gives.  B stands at a page's first or last row, in
    the sequence's first tokens, or hundreds of positions back; A comes last, in a prompt's portion and decoded alone."""
    A, B, length = 95, 96, 300
    mixer = _side_mixer({"left": (2, 1, 12, 20, 0.3, 100.0, 8), "right": (2, 8, 4), "scales": (1.0, 0.3)})

    def boost(weights, h_of):
        a, b = h_of(A), h_of(B)
        weights["l0.mix.left.q"][10] = 14.0 * a / (a @ a)        # head 0, dim 10 (past the rotated 8)
        weights["l0.mix.left.k"][10] = 14.0 * b / (b @ b)
    folder, config, weights = _boosted(tmp_path, {"type": "parallel", "mixer": mixer, "mlp": None}, 11, boost)
    tokens = tokens_of(12, length, 97, avoid=(A, B))
    tokens[far], tokens[-1] = B, A
    other = list(tokens)
    other[far] = tokens[far + 1]
    want = plain.forward(config, weights, tokens)[0]
    lost = plain.forward(config, weights, other)[0]
    assert float(row_errors(lost[-1:], want[-1:])) > 0.15                            # the test shows a key that is lost
    from tlie_amd import Engine
    engine = Engine(folder, dtype=dtype, max_tokens=640, page_size=16, max_requests=2)
    for cuts in ([length], [length - 1, 1], [7, 64, 2]):
        got = run_cut(engine, "a", tokens, cuts)
        assert_rows(got[-1:], want[-1:], SINGLE_LAYER_TOLERANCE[dtype], f"B at {far}, cuts {cuts}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["retention", "gla", "parallel"])
def test_what_the_state_took_in_long_ago_is_still_there(tmp_path, dtype, kind):
    """Decays close to 1, and a key and value written at the third token that stand out: token B alone has a large
    channel 0, which its key's dim 10 and its value read, and token A alone a large channel 1, which the query's dim 10
    reads (past the dims that turn).  A comes last.  A state that is lost or zeroed on the way (between steps, at a
    slice's edge, in a slot that is used again) changes the last tokens' results."""
    A, B, length = 95, 96, 260
    if kind == "retention":
        mixer = {"heads": 2, "dim": 12, "vdim": 12, "decay": [0.9995, 0.9], "rot": {"base": 100.0, "dims": 8}}
        q, k, v, o = ("l0.mix." + name for name in "qkvo")
    elif kind == "gla":
        mixer = {"heads": 2, "dim": 12, "vdim": 12, "tau": 16.0, "rank": 4}
        q, k, v, o = ("l0.mix." + name for name in "qkvo")
    else:
        mixer = _side_mixer({"left": (2, 1, 8, 8, 0.3, 100.0, 8), "right": (2, 12, 4), "scales": (0.2, 1.0)})
        q, k, v, o = ("l0.mix.right." + name for name in "rkvo")

    def boost(weights):
        weights["embed"][:, :2] = 0.0
        weights["embed"][B, 0], weights["embed"][A, 1] = 4.0, 4.0
        weights["l0.canon1"][:, :-1] *= 0.05                     # the neighbours' share of a token's input stays small
        weights[q][10], weights[k][10] = 0.0, 0.0
        weights[q][10, 1], weights[k][10, 0] = 3.0, 3.0          # head 0, dim 10
        weights[v][:12, 0] = torch.linspace(-2.0, 2.0, 12, dtype=torch.float64)
        weights[o] *= 12.0
        if kind == "gla":
            weights["l0.mix.a2.b"][:] = 9.0                      # sigmoid(9)^(1/16) a token: nothing is forgotten
        if kind == "parallel":
            weights["l0.mix.right.w0"][:] = -9.0                 # exp(-exp(-9)) a token
            for blend in "rkv":
                weights["l0.mix.right.mu." + blend][:] = 0.0     # they read the token itself
    folder, config, weights = _single_layer(tmp_path, {"type": kind, "mixer": mixer, "mlp": None}, seed=13, changes=boost)
    tokens = tokens_of(14, length, 97, avoid=(A, B))
    tokens[2], tokens[-1] = B, A
    other = list(tokens)
    other[2] = tokens[3]
    want = plain.forward(config, weights, tokens)[0]
    lost = plain.forward(config, weights, other)[0]
    assert float(row_errors(lost[-2:], want[-2:]).min()) > 0.05                     # the test shows a state that is lost
    from tlie_amd import Engine
    engine = Engine(folder, dtype=dtype, max_tokens=640, page_size=16, max_requests=1)      # one slot: used again by every cut
    for cuts in ([length], [length - 40] + [1] * 40, [5, 64, 2, 1], [3, 96, 33, 97]):
        got = run_cut(engine, "a", tokens, cuts)
        assert_rows(got[-2:], want[-2:], SINGLE_LAYER_TOLERANCE[dtype], f"cuts {cuts[:4]}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_first_tokens_of_a_request_see_nothing_of_the_slots_last_owner(tmp_path, dtype):
    """One slot, two requests after each other: the second's first tokens (whose convolution, token shift and states
    start from zeros) equal the same request in a fresh engine, and differ from what a kept state would give."""
    from tlie_amd import Engine
    mixer = _side_mixer({"left": (2, 1, 8, 8, 0.3, 100.0, 8), "right": (2, 12, 4), "scales": (0.7, 1.0)})
    folder, config, weights = _single_layer(tmp_path, {"type": "parallel", "mixer": mixer, "mlp": {"kind": "dense", "ff": 40}}, seed=21, taps=4)
    first, second = tokens_of(22, 50, 97), tokens_of(23, 9, 97)
    want = plain.forward(config, weights, second)[0]
    joined = plain.forward(config, weights, first + second)[0][len(first):]
    assert float(row_errors(joined[:1], want[:1])) > 0.02
    engine = Engine(folder, dtype=dtype, max_tokens=64, page_size=16, max_requests=1)
    for cuts in ([9], [1], [2, 1]):
        run_cut(engine, "x", first, [50])
        got = run_cut(engine, "y", second, cuts)
        assert_rows(got, want, SINGLE_LAYER_TOLERANCE[dtype], f"cuts {cuts}")


# ---- whole models through the engine -----------------------------------------------------------------------
@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompt_matches_the_plain_implementation(setups, name, dtype):
    setup = setups(name)
    tokens = tokens_of(1, 150, CONFIGS[name]["vocab"])
    engine = new_engine(setup, dtype)
    got = run_cut(engine, "a", tokens, [len(tokens)])
    assert_rows(got, plain_logits(setup, tokens), TOLERANCE[dtype], f"{name} {dtype}")
    engine.cache.check()


@pytest.mark.parametrize("name", list(CONFIGS))
def test_every_layer_matches_the_plain_implementation(setups, name):
    """What every layer hands on, in 32-bit: a fault shows in the first layer it touches."""
    from tlie_amd import StepEntry
    setup = setups(name)
    tokens = tokens_of(2, 61, CONFIGS[name]["vocab"])
    layers = plain.forward(setup["raw"], setup["weights"], tokens)[1]
    engine = new_engine(setup, "float32")
    engine.admit("a")
    trace = {}
    engine.step([StepEntry("a", tokens, [len(tokens) - 1])], trace=trace)
    assert len(layers) == len(engine.spec.runs)
    for index, want in enumerate(layers):
        assert_rows(trace[f"layer{index}.mixed"], want, TOLERANCE["float32"], f"{name}: what layer {index} hands on")


@pytest.mark.parametrize("name,dtype", CASES)
def test_cuts_agree_with_each_other_and_with_the_plain_implementation(setups, name, dtype):
    """Token by token from the first token on; portions of changing sizes down to two tokens and one; most of a
    prompt and then a long run of single tokens over several page borders."""
    setup = setups(name)
    tokens = tokens_of(3, 131, CONFIGS[name]["vocab"])
    want = plain_logits(setup, tokens)
    engine = new_engine(setup, dtype)
    whole = run_cut(engine, "w", tokens, [len(tokens)])
    for cuts in ([1], [2], [7, 2, 33, 1, 16, 3], [40] + [1] * 200, [100, 31]):
        got = run_cut(engine, ("c", tuple(cuts[:3])), tokens, cuts)
        assert_rows(got, want, TOLERANCE[dtype], f"{name} {dtype} cut {cuts[:6]}")
        assert_rows(got, whole, CUT_TOLERANCE[dtype], f"{name} {dtype} cut {cuts[:6]} against the whole prompt")
    engine.cache.check()


@pytest.mark.parametrize("name,dtype", CASES)
def test_batches_of_unequal_requests_with_pages_and_slots_used_again(setups, name, dtype):
    """Up to three live requests of unequal lengths in three slots more than once: portions of some beside single
    tokens of others, requests that pause for a step, a pool that only holds what is live."""
    from tlie_amd import StepEntry
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    lengths = {"a": 70, "b": 9, "c": 41, "d": 1, "e": 120, "f": 30}
    # (a retention head's first result is sign(q . k) v / rms(v): a first token whose q . k of some head is next to zero
    # would turn on bfloat16's rounding; these seeds have none)
    prompts = {key: tokens_of(20 + index, length, vocab) for index, (key, length) in enumerate(lengths.items())}
    engine = new_engine(setup, dtype, max_tokens=256, max_requests=3)
    rng = random.Random(5)
    waiting, live, at, rows = list(prompts), [], {}, {key: [] for key in prompts}
    steps = 0
    while waiting or live:
        while waiting and len(live) < 3 and sum((lengths[key] + 15) // 16 * 16 for key in live + [waiting[0]]) <= 256:
            key = waiting.pop(0)
            engine.admit(key)
            live.append(key)
            at[key] = 0
        entries, counts = [], {}
        for key in live:
            if len(live) > 1 and rng.random() < 0.25:
                continue                                              # left out of this step
            count = min(lengths[key] - at[key], rng.choice([1, 1, 2, 3, 9, 30, 100]))
            entries.append(StepEntry(key, prompts[key][at[key]:at[key] + count], list(range(count))))
            counts[key] = count
        if not entries:
            continue
        logits = engine.step(entries)
        row = 0
        for entry in entries:
            rows[entry.request].append(logits[row:row + counts[entry.request]].clone())
            row += counts[entry.request]
            at[entry.request] += counts[entry.request]
            if at[entry.request] == lengths[entry.request]:
                engine.finish(entry.request)
                live.remove(entry.request)
        engine.cache.check()
        steps += 1
    assert steps > 12
    for key, tokens in prompts.items():
        assert_rows(torch.cat(rows[key]), plain_logits(setup, tokens), TOLERANCE[dtype], f"{name} {dtype} request {key}")


@pytest.mark.parametrize("name", list(CONFIGS))
def test_recorded_steps_equal_launched_steps_bit_for_bit(setups, name):
    """Steps replayed from recordings (padded to the recording's size, with padding tokens and sequences that belong to
    no request) against the same steps launched kernel by kernel: the same bits, also for the layers that carry state."""
    from tlie_amd import StepEntry
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    prompts = [tokens_of(40 + index, length, vocab) for index, length in enumerate((37, 20, 50))]
    results = []
    for capture in (True, False):
        engine = new_engine(setup, "bfloat16", capture_graphs=capture)
        assert engine.runner.use_graphs
        rows = []
        for key in range(3):
            engine.admit(key)
        at = [0, 0, 0]
        for counts in [(5, 3, 0), (1, 1, 1), (1, 1, 1), (6, 2, 9), (1, 1, 1), (5, 3, 0), (1, 1, 1), (6, 0, 9), (1, 1, 1), (1, 0, 1)]:
            entries = [StepEntry(key, prompts[key][at[key]:at[key] + count], [count - 1]) for key, count in enumerate(counts) if count]
            rows.append(engine.step(entries).clone())
            for key, count in enumerate(counts):
                at[key] += count
        results.append(torch.cat(rows))
    assert torch.equal(results[0], results[1])
    assert bool(torch.isfinite(results[0]).all())


@pytest.mark.parametrize("name", list(CONFIGS))
def test_greedy_generation_through_the_scheduler(setups, name):
    """The engine's own entry point: prompts of unequal lengths together under the scheduler, prompts cut into
    portions, greedy tokens equal to the plain implementation's in 32-bit."""
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    prompts = [tokens_of(70 + index, length, vocab) for index, length in enumerate((45, 3, 18))]
    want = [plain_generate_greedy(setup["raw"], setup["weights"], prompt, 10) for prompt in prompts]
    engine = new_engine(setup, "float32", max_tokens=256)
    assert engine.generate(prompts, max_tokens=10, chunk_size=16, max_tokens_per_step=24) == want
    assert engine.generate([prompts[1]], max_tokens=10) == [want[1]]
    engine.cache.check()
    assert len(new_engine(setup, "bfloat16").generate(prompts, max_tokens=5)[2]) == 5


def test_a_preempted_request_is_recomputed_from_a_state_of_zero(setups):
    """A pool too small for all requests at once: the scheduler preempts and recomputes; a recomputed request must not
    see the states its earlier admission left in a slot."""
    setup = setups("U")
    prompts = [tokens_of(90 + index, 40, CONFIGS["U"]["vocab"]) for index in range(4)]
    want = [plain_generate_greedy(setup["raw"], setup["weights"], prompt, 16) for prompt in prompts]
    engine = new_engine(setup, "float32", max_tokens=176, max_requests=4)
    assert engine.generate(prompts, max_tokens=16, admit_partial=True) == want
    engine.cache.check()


def test_long_decoding_keeps_to_the_plain_implementation(setups):
    """A short prompt and then hundreds of single tokens through recorded steps, in bfloat16 and in 32-bit."""
    setup = setups("U")
    tokens = tokens_of(55, 330, CONFIGS["U"]["vocab"])
    want = plain_logits(setup, tokens)
    for dtype in DTYPES:
        engine = new_engine(setup, dtype)
        got = run_cut(engine, "a", tokens, [6] + [1] * 400)
        assert_rows(got, want, TOLERANCE[dtype], f"{dtype}")


def test_the_command_line_and_the_replay_program_run_the_design(setups, tmp_path):
    """`generate` and `logits` of the framework's command line, and a trace of steps through `bin/trace_run` (a portion
    beside a single token, a request that ends and whose slot and pages are used again), on a model of this design."""
    import json
    import os
    import subprocess
    import sys
    import numpy
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    setup = setups("W")
    vocab = CONFIGS["W"]["vocab"]
    tokens, other = tokens_of(61, 40, vocab), tokens_of(62, 21, vocab)
    prompt = "ids:" + ",".join(str(token) for token in tokens[:9])
    cli = [sys.executable, os.path.join(root, "bin", "tinyllama_amd")]
    run = subprocess.run(cli + ["generate", setup["folder"], prompt, "6", "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert json.loads(run.stdout)["generated_tokens"] == plain_generate_greedy(setup["raw"], setup["weights"], tokens[:9], 6)
    run = subprocess.run(cli + ["logits", setup["folder"], prompt, "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert_rows(torch.tensor(json.loads(run.stdout)["logits"])[None], plain_logits(setup, tokens[:9])[-1:], TOLERANCE["float32"], "logits")
    lines = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": tokens[30:31], "want": [0]}, {"id": "b", "tokens": other, "want": [20]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "c", "tokens": other[:7], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": tokens[31:], "want": [8]}, {"id": "c", "tokens": other[7:], "want": [13]}], "end": ["a", "c"]}]
    for dtype in DTYPES:
        out = tmp_path / dtype
        run = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", setup["folder"], "--dtype", dtype,
                              "--out", str(out), "--max-tokens", "128", "--max-requests", "2"],
                             input="".join(json.dumps(line) + "\n" for line in lines), capture_output=True, text=True, timeout=300)
        assert run.returncode == 0 and run.stdout.split() == ["done", "0", "done", "1", "done", "2", "done", "3"], run.stderr
        assert not (out / "2.f32").exists()
        read = lambda step: torch.from_numpy(numpy.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, vocab))      # noqa: E731
        want, want_other = plain_logits(setup, tokens), plain_logits(setup, other)
        assert_rows(read(0), want[[0, 29]], TOLERANCE[dtype], f"{dtype} step 0")
        assert_rows(read(1), torch.stack([want[30], want_other[20]]), TOLERANCE[dtype], f"{dtype} step 1")
        assert_rows(read(3), torch.stack([want[39], want_other[20]]), TOLERANCE[dtype], f"{dtype} step 3")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["two_attentions", "equal_sizes", "odd_sizes"])
def test_models_of_other_orders_and_sizes(tmp_path, which, dtype):
    """Two layers with attention after each other (two page groups' worth of caches) at a width that is no multiple of 8;
    a model whose sizes are all equal (heads' dims, values, width over heads, the inner size), which would hide
    two sizes taken for each other, next to one whose sizes all differ; and one whose width, vocabulary, heads' sizes
    and inner sizes are all odd or twice an odd number (no kernel's wide form fits), with eight taps."""
    if which == "odd_sizes":
        raw = {"architecture": "Tugalix", "vocab": 61, "width": 54, "norm": {"eps": 1e-5}, "canon": {"taps": 8}, "logit_scale": 0.9,
               "layers": [{"type": "parallel", "mixer": _side_mixer({"left": (3, 1, 6, 5, 0.4, 300.0, 2), "right": (3, 9, 5), "scales": (0.9, 1.1)}),
                           "mlp": {"kind": "dense", "ff": 35}},
                          {"type": "gla", "mixer": {"heads": 3, "dim": 7, "vdim": 9, "tau": 2.5, "rank": 3}, "mlp": None},
                          {"type": "retention", "mixer": {"heads": 5, "dim": 10, "vdim": 3, "decay": [0.5, 0.9, 0.99, 0.999, 0.8],
                                                          "rot": {"base": 1000.0, "dims": 6}}, "mlp": {"kind": "dense", "ff": 27}}]}
    elif which == "two_attentions":
        raw = {"architecture": "Tugalix", "vocab": 77, "width": 100, "norm": {"eps": 1e-5}, "canon": {"taps": 3}, "logit_scale": 1.5,
               "layers": [{"type": "parallel", "mixer": _side_mixer(SIDES[0]), "mlp": {"kind": "dense", "ff": 52}},
                          {"type": "parallel", "mixer": _side_mixer(SIDES[1]), "mlp": None},
                          {"type": "gla", "mixer": {"heads": 5, "dim": 4, "vdim": 7, "tau": 3.0, "rank": 2}, "mlp": {"kind": "dense", "ff": 9}}]}
    else:
        raw = {"architecture": "Tugalix", "vocab": 64, "width": 64, "norm": {"eps": 1e-6}, "canon": {"taps": 2}, "logit_scale": 1.0,
               "layers": [{"type": "retention", "mixer": {"heads": 4, "dim": 16, "vdim": 16, "decay": [0.9] * 4, "rot": {"base": 64.0, "dims": 16}},
                           "mlp": {"kind": "dense", "ff": 64}},
                          {"type": "gla", "mixer": {"heads": 4, "dim": 16, "vdim": 16, "tau": 4.0}, "mlp": {"kind": "dense", "ff": 64}},
                          {"type": "parallel", "mixer": _side_mixer({"left": (4, 4, 16, 16, 0.25, 64.0, 16), "right": (4, 16, 16), "scales": (1.0, 1.0)}),
                           "mlp": {"kind": "dense", "ff": 64}}]}
    folder = make_model(tmp_path, raw, seed=17)
    config, weights = load_plain(folder)
    tokens = tokens_of(19, 140, raw["vocab"])
    want = plain.forward(config, weights, tokens)[0]
    from tlie_amd import Engine
    engine = Engine(folder, dtype=dtype, max_tokens=320, page_size=16, max_requests=2)
    for cuts in ([140], [100] + [1] * 40, [3, 64, 2, 1]):
        assert_rows(run_cut(engine, "a", tokens, cuts), want, TOLERANCE[dtype], f"{which} {dtype} cuts {cuts[:4]}")
    engine.cache.check()
    assert engine.generate([tokens[:12], tokens[20:25]], max_tokens=4, chunk_size=8) is not None
