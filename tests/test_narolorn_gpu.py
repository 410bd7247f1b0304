"""The Narolorn decoder on the GPU against the plain implementation (tests/plain_narolorn.py): each mechanism alone,
inputs made so that a fault shows, then whole models through the engine's step function, cache manager, scheduler and
entry point, however the work is cut."""
import math
import random

import pytest
import torch

import plain_narolorn as plain
from narolorn_helpers import (CONFIGS, CUT_TOLERANCE, DTYPES, TOLERANCE, load_plain, make_model, plain_generate_greedy, row_errors,
                              run_cut)

pytestmark = pytest.mark.gpu
CASES = [(name, dtype) for name in CONFIGS for dtype in DTYPES]
DEVICE = "cuda:0"
F64 = torch.float64


def tokens_of(seed, count, vocab):
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(count)]


@pytest.fixture(scope="module")
def setups(tmp_path_factory):
    made = {}

    def get(name):
        if name not in made:
            folder = make_model(tmp_path_factory.mktemp(f"narolorn_{name}"), CONFIGS[name], seed=47)
            raw, weights = load_plain(folder)
            made[name] = {"folder": folder, "raw": raw, "weights": weights, "plain": {}, "margin": {}}
        return made[name]
    return get


def plain_logits(setup, tokens):
    key = tuple(tokens)
    if key not in setup["plain"]:
        margins = []
        logits = plain.forward(setup["raw"], setup["weights"], list(tokens), margins)[0]
        setup["plain"][key] = logits
        setup["margin"][key] = torch.stack(margins).amin(dim=0) if margins else torch.full((len(key),), math.inf, dtype=F64)
    return setup["plain"][key]


# A router's choice is a step function: in bfloat16 a token whose `top`-th and next logits lie closer than rounding moves
# them may take another expert than the plain implementation.  Such a row says nothing about a kernel; bfloat16
# comparisons leave out the tokens whose closest call, over all routers that run, is below this (logits are of order 1),
# (random weights give a router's biases a spread of 2, so that the experts stand well apart) and hold that they are few.
# (What such a token leaves in the caches moves later tokens by less than the tolerance.)
CLOSE_CALL = 0.12


def settled_rows(setup, tokens, dtype, least=0.6):
    """The rows that a comparison in `dtype` holds to its tolerance: all in float32; in bfloat16 those of tokens without a
    close call of a router."""
    plain_logits(setup, tokens)
    count = len(tokens)
    if dtype == "float32":
        return list(range(count))
    rows = (setup["margin"][tuple(tokens)] >= CLOSE_CALL).nonzero().flatten().tolist()
    assert len(rows) >= least * count or count < 8, "too many close calls for a comparison"
    return rows


def assert_settled(got, setup, tokens, dtype, tolerance, what, places=None, other=None, least=0.6):
    """got: logits at `places` of the request (default: all); compared with the plain implementation's (or with `other`,
    another result of the engine at the same places) at the rows without a router's close call."""
    places = list(range(len(tokens))) if places is None else list(places)
    settled = set(settled_rows(setup, tokens, dtype, least))
    keep = [index for index, place in enumerate(places) if place in settled]
    want = plain_logits(setup, tokens)[places] if other is None else other
    if keep:
        assert_rows(got[keep], want[keep], tolerance, what)


def new_engine(setup, dtype, max_tokens=640, page_size=16, max_requests=4, **options):
    from tlie_amd import Engine
    return Engine(setup["folder"], dtype=dtype, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests, **options)


def assert_rows(got, want, tolerance, what):
    errors = row_errors(got, want)
    worst = int(errors.argmax())
    assert float(errors.max()) <= tolerance, f"{what}: row {worst} is off by {float(errors[worst]):.3g} of its largest value (allowed {tolerance})"


# ---- a residual of several streams -----------------------------------------------------------------------------
@pytest.mark.parametrize("count,tokens,hidden,nsplit", [(1, 5, 96, 1), (2, 3, 201, 2), (3, 17, 256, 1), (8, 4, 1000, 3), (4, 1, 64, 1)])
def test_streams_take_a_result_are_read_and_normed(count, tokens, hidden, nsplit):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(count * hidden)
    streams = torch.randn(count, tokens, hidden, generator=generator)
    parts = torch.randn(nsplit, tokens, hidden, generator=generator)
    mix, write, read = (torch.randn(shape, generator=generator) for shape in ((count, count), (count,), (count,)))
    weight = 1.0 + 0.1 * torch.randn(hidden, generator=generator)
    y = parts.double().sum(0)
    fresh = torch.einsum("sr,std->rtd", mix.double(), streams.double()) + write.double()[:, None, None] * y[None]
    u = torch.einsum("s,std->td", read.double(), fresh)
    want = plain.rms_norm(u, weight.double(), 1e-5)
    on = streams.to(DEVICE).clone()
    update = ops.StreamUpdate(ops.Product(parts.to(DEVICE).contiguous() if nsplit > 1 else parts[0].to(DEVICE).contiguous(), nsplit),
                              mix.to(DEVICE), write.to(DEVICE))
    normed, total = ops.stream_norm(on, update, read.to(DEVICE), weight.to(DEVICE), 1e-5, torch.float32, total=True)
    assert float((on.cpu().double() - fresh).abs().max()) < 2e-5              # the streams were brought up to date in place
    assert float((normed.cpu().double() - want).abs().max()) < 2e-5
    assert float((total.cpu().double() - fresh.sum(0)).abs().max()) < 3e-5
    # nothing waits: the streams are read as they are; and the sum alone
    again, none = ops.stream_norm(on, None, read.to(DEVICE), weight.to(DEVICE), 1e-5, torch.float32)
    assert none is None and float((again.cpu().double() - want).abs().max()) < 2e-5
    nothing, total = ops.stream_norm(on, None, None, None, 0.0, torch.float32, total=True)
    assert nothing is None and float((total.cpu().double() - fresh.sum(0)).abs().max()) < 3e-5
    spread = ops.stream_spread(streams[0].to(DEVICE).contiguous(), count)
    assert spread.shape == (count, tokens, hidden) and all(torch.equal(spread[s].cpu(), streams[0]) for s in range(count))


# ---- placement: norms over whole projections, values that are the keys, a query temperature ---------------------
@pytest.mark.parametrize("heads,groups,d,rot,page_size,nsplit", [(4, 2, 16, 8, 16, 1), (3, 1, 10, 10, 4, 2), (2, 2, 64, 0, 16, 1)])
def test_placement_norms_whole_projections_and_keeps_the_projected_keys_as_values(heads, groups, d, rot, page_size, nsplit):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(d + rot)
    tokens = 11
    parts = torch.randn(nsplit, tokens, (heads + groups) * d, generator=generator)
    q_weight, k_weight = 1.0 + 0.2 * torch.randn(heads * d, generator=generator), 1.0 + 0.2 * torch.randn(groups * d, generator=generator)
    positions = torch.tensor([3 + 7 * t for t in range(tokens)])
    full = parts.double().sum(0)
    q = plain.rms_norm(full[:, :heads * d], q_weight.double(), 1e-5).reshape(tokens, heads, d)
    k = plain.rms_norm(full[:, heads * d:], k_weight.double(), 1e-5).reshape(tokens, groups, d)
    if rot:
        q, k = plain.rotate_halves(q, positions, rot, 50.0), plain.rotate_halves(k, positions, rot, 50.0)
    q = q * plain.query_temperature(positions, 0.4, 6.0)[:, None, None]
    inv_freq = torch.tensor([50.0 ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=DEVICE) if rot else None
    pages = 4
    cache = torch.zeros((pages, 2, groups, page_size * d), dtype=torch.float32, device=DEVICE)
    slots = torch.tensor([(t * 5) % (pages * page_size) for t in range(tokens)], dtype=torch.int32, device=DEVICE)
    product = ops.Product(parts.to(DEVICE).contiguous() if nsplit > 1 else parts[0].to(DEVICE).contiguous(), nsplit)
    placed = ops.qkv_place(product, positions.to(torch.int32).to(DEVICE), slots, inv_freq, rot, cache, heads, groups, d, d, torch.float32,
                           q_norm=q_weight.to(DEVICE), k_norm=k_weight.to(DEVICE), norm_eps=1e-5, values_are_keys=True, q_temp=(0.4, 6.0))
    assert float((placed.cpu().double().reshape(tokens, heads, d) - q).abs().max()) < 3e-5
    cache = cache.cpu().double()
    for t in range(tokens):
        page, row = int(slots[t]) // page_size, int(slots[t]) % page_size
        keys = cache[page, 0].reshape(groups, page_size, d)[:, row]
        values = cache[page, 1].reshape(groups, d, page_size)[:, :, row]
        assert float((keys - k[t]).abs().max()) < 3e-5
        assert float((values - full[t, heads * d:].reshape(groups, d)).abs().max()) < 1e-5   # as projected: no norm, no turn


# ---- attention: capped scores, windows and chunks, keys made to stand out --------------------------------------
def _pages(tokens, page_size):
    blocks = (tokens + page_size - 1) // page_size
    order = list(range(blocks + 3))
    random.Random(blocks).shuffle(order)
    return blocks, order


def _attend(q, k, v, scale, page_size, cuts, window=None, chunk=None, softcap=None, dtype=torch.float32, matrix_cores=False):
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence through the placing kernel and an attention kernel, in steps
    of the sizes `cuts`, with the sequence's pages in a scrambled order."""
    from types import SimpleNamespace
    import numpy as np
    from tlie_amd import ops
    tokens, heads, d = q.shape
    groups, dv = k.shape[1], v.shape[2]
    blocks, order = _pages(tokens, page_size)
    shape = (blocks + 3, 2, groups, page_size * d) if d == dv else (blocks + 3, groups, page_size * (d + dv))
    cache = torch.zeros(shape, dtype=dtype, device=DEVICE)
    table = torch.tensor([order[:blocks]], dtype=torch.int32, device=DEVICE)
    outs, at, index = [], 0, 0
    while at < tokens:
        count = min(cuts[index % len(cuts)], tokens - at)
        index += 1
        positions = torch.arange(at, at + count, dtype=torch.int32, device=DEVICE)
        slots = torch.tensor([order[p // page_size] * page_size + p % page_size for p in range(at, at + count)], dtype=torch.int32, device=DEVICE)
        fused = torch.cat([q[at:at + count].reshape(count, -1), k[at:at + count].reshape(count, -1), v[at:at + count].reshape(count, -1)], dim=1)
        placed = ops.qkv_place(ops.Product(fused.to(DEVICE).contiguous(), 1), positions, slots, None, 0, cache, heads, groups, d, dv, dtype)
        if matrix_cores:
            host = {"seq_start": np.asarray([0, count], dtype=np.int32), "seq_len": np.asarray([at + count], dtype=np.int32)}
            ctx = SimpleNamespace(max_new=count, num_seqs=1, num_tokens=count, max_context=at + count, scratch={}, tile_owner=None,
                                  compute_units=256, host=host, tokens=positions)
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, heads // groups, groups, d)
            outs.append(ops.attention_mfma(placed, cache, table, tiles, positions, heads, groups, d, window, scale, nsplit, split_len,
                                           col_tiles, waves, shared, chunk=chunk, softcap=softcap))
        else:
            seq = torch.zeros(count, dtype=torch.int32, device=DEVICE)
            start = torch.tensor([0, count], dtype=torch.int32, device=DEVICE)
            for tiled in ((0, 1) if max(d, dv) <= 64 else (0,)):
                out = ops.attention_generic(placed, cache, table, seq, positions, heads, groups, d, window, scale, tiled=tiled,
                                            seq_start=start, value_dim=dv, chunk=chunk, softcap=softcap)
                if tiled:
                    assert torch.equal(out, outs[-1]), "the two forms of the attention kernel differ in bits"
                else:
                    outs.append(out)
        at += count
    return torch.cat(outs, dim=0).reshape(tokens, heads, dv)


def _plain_attend(q, k, v, scale, window=None, chunk=None, softcap=None):
    tokens, heads, _ = q.shape
    groups = k.shape[1]
    mask = plain.visible(tokens, window=window, chunk=chunk)
    out = [plain.softmax_attention(q[:, h].double(), k[:, h // (heads // groups)].double(), v[:, h // (heads // groups)].double(), scale, mask,
                                   softcap) for h in range(heads)]
    return torch.stack(out, dim=1)


@pytest.mark.parametrize("heads,groups,d,dv,window,chunk,softcap,page_size", [
    (4, 2, 16, 24, None, None, 5.0, 16), (3, 3, 9, 5, 7, None, 2.0, 4), (2, 1, 72, 8, None, 33, 50.0, 16), (4, 1, 64, 64, 21, None, 1.0, 16)])
def test_attention_with_capped_scores(heads, groups, d, dv, window, chunk, softcap, page_size):
    generator = torch.Generator().manual_seed(d * dv)
    tokens = 150
    q, k, v = (torch.randn(tokens, n, size, generator=generator) for n, size in ((heads, d), (groups, d), (groups, dv)))
    want = _plain_attend(q, k, v, 0.6, window, chunk, softcap)
    assert float((want - _plain_attend(q, k, v, 0.6, window, chunk, None)).abs().max()) > 0.05        # the cap is no detail here
    for cuts in ([tokens], [1], [37, 2, 5, 1]):
        got = _attend(q, k, v, 0.6, page_size, cuts, window, chunk, softcap)
        assert float((got.cpu().double() - want).abs().max()) < 2e-5, f"cut {cuts}"


@pytest.mark.parametrize("heads,groups,d,window,chunk,softcap,page_size,tokens", [
    (4, 2, 64, None, None, 6.0, 16, 300), (6, 1, 128, 72, None, None, 16, 400), (2, 2, 32, None, 40, 3.0, 16, 200), (8, 4, 64, None, None, 30.0, 16, 1000)])
def test_attention_on_the_matrix_cores_with_capped_scores_and_windows(heads, groups, d, window, chunk, softcap, page_size, tokens):
    generator = torch.Generator().manual_seed(d + tokens)
    q, k, v = (torch.randn(tokens, n, d, generator=generator).bfloat16().float() for n in (heads, groups, groups))
    want = _plain_attend(q, k, v, 0.25, window, chunk, softcap)
    for cuts in ([tokens], [tokens - 40] + [1] * 40, [37, 2, 5, 1, 130]):
        got = _attend(q, k, v, 0.25, page_size, cuts, window, chunk, softcap, dtype=torch.bfloat16, matrix_cores=True)
        assert float((got.float().cpu().double() - want).abs().max()) < 3e-2, f"cut {cuts[:5]}"
    if softcap is not None and softcap < 10:
        assert float((_plain_attend(q, k, v, 0.25, window, chunk, None) - want).abs().max()) > 0.1


@pytest.mark.parametrize("matrix_cores", [False, True])
def test_keys_at_the_edges_of_windows_chunks_and_pages_and_far_away_show(matrix_cores):
    """Inputs made so that faults show: one query and one key are scaled so that their score towers over all others.  Just
    inside the query's window or chunk that key takes nearly all the weight, just outside it none; a key hundreds of
    positions back among small ones is found; the cap bounds the towering score, so that the others keep a share."""
    heads, groups, d, page_size = 2, 1, 16, 16
    dtype = torch.bfloat16 if matrix_cores else torch.float32
    generator = torch.Generator().manual_seed(3)
    tokens = 700
    q, k, v = (0.1 * torch.randn(tokens, n, d, generator=generator).bfloat16().float() for n in (heads, groups, groups))
    tolerance = 2e-2 if matrix_cores else 1e-5

    def shows(query, target, window=None, chunk=None, softcap=None, cuts=None):
        qq, kk = q[:query + 1].clone(), k[:query + 1].clone()
        qq[query, :, 0], kk[target, :, 0] = 32.0, 32.0
        cuts = cuts or [query, 1]                                         # the asker decoded alone
        got = _attend(qq, kk, v[:query + 1], 1.0, page_size, cuts, window, chunk, softcap, dtype=dtype, matrix_cores=matrix_cores)[query].float().cpu()
        want = _plain_attend(qq, kk, v[:query + 1], 1.0, window, chunk, softcap)[query]
        assert float((got.double() - want).abs().max()) < tolerance, f"query {query}, key {target}"
        return float((got - v[target, 0]).abs().max()) < 2e-2
    # a window of 20: position 99 sees 80 .. 99
    for target, inside in ((80, True), (79, False), (99, True), (64, False)):
        assert shows(99, target, window=20) == inside
        assert shows(99, target, window=20, cuts=[100]) == inside           # in a prompt's portion
        assert shows(99, target, window=20, cuts=[90, 2, 3, 5]) == inside
    # chunks of 24: position 100 is in 96 .. 119
    for target, inside in ((96, True), (95, False), (100, True), (72, False)):
        assert shows(100, target, chunk=24) == inside
        assert shows(100, target, chunk=24, cuts=[97, 4]) == inside
    # far back, at page borders, and the very first keys
    for target in (0, 1, 15, 16, 17, 31, 32, 333, 640):
        assert shows(699, target)
        assert shows(699, target, cuts=[650, 50])
    # capped at 4, the towering score weighs exp(4) against some 700 keys near exp(0): a twelfth, not all
    assert not shows(699, 333, softcap=4.0)


# ---- the router and the experts' gate --------------------------------------------------------------------------
@pytest.mark.parametrize("tokens,inner,experts,top,extra,dtype", [(5, 96, 6, 2, 1, torch.float32), (3, 1000, 16, 16, 0, torch.bfloat16),
                                                                  (9, 80, 3, 1, 1, torch.bfloat16), (4, 64, 70, 64, 0, torch.float32)])
def test_the_router_takes_the_softmax_over_the_chosen_logits(tokens, inner, experts, top, extra, dtype):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(inner + top)
    x = torch.randn(tokens, inner, generator=generator).to(dtype)
    weight = (torch.randn(experts + extra, inner, generator=generator) / math.sqrt(inner)).to(dtype)
    bias = torch.randn(experts + extra, generator=generator).to(dtype)
    if extra:
        bias[experts:] = 0.0
    z = x.double() @ weight.double().T + bias.double()
    chosen, weights = plain.router_choice(z[:, :experts], top)
    want = torch.zeros(tokens, experts + extra, dtype=F64)
    want[:, :experts].scatter_(1, chosen, weights)
    want[:, experts:] = torch.sigmoid(z[:, experts:])
    got = ops.few_outputs(x.to(DEVICE), weight.to(DEVICE), bias.to(DEVICE), top=top, score="softmax_of_chosen", extra=extra).cpu().double()
    assert float((got - want).abs().max()) < 1e-5
    assert torch.allclose(got[:, :experts].sum(1), torch.ones(tokens, dtype=F64), atol=1e-5)


@pytest.mark.parametrize("tokens,experts,block,shared,nsplit,dtype", [(5, 4, 6, 10, 1, torch.float32), (3, 7, 24, 0, 2, torch.float32),
                                                                      (18, 2, 8, 16, 1, torch.bfloat16)])
def test_the_experts_gate_weighs_results_with_a_limit_of_its_own_for_the_shared_expert(tokens, experts, block, shared, nsplit, dtype):
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(block)
    inter = experts * block + shared
    parts = (2.0 * torch.randn(nsplit, tokens, 2 * inter, generator=generator)).to(torch.float32 if nsplit > 1 else dtype)
    scale = torch.rand(tokens, experts + (1 if shared else 0), generator=generator)
    scale[:, 0] = 0.0                                                     # an expert no token uses
    full = parts.double().sum(0)
    g, u = full[:, 0::2], full[:, 1::2]
    limit = torch.cat([torch.full((experts * block,), 1.5), torch.full((shared,), 0.5)]).double()
    act = torch.minimum(g, limit)
    act = act * torch.sigmoid(1.702 * act) * (torch.clamp(u, min=-limit, max=limit) + 1.0)
    per_column = torch.cat([scale[:, :experts].double().repeat_interleave(block, dim=1), scale[:, experts:].double().expand(tokens, shared)], dim=1)
    product = ops.Product(parts.to(DEVICE).contiguous() if nsplit > 1 else parts[0].to(DEVICE).contiguous(), nsplit)
    got = ops.routed_gate(product, scale.to(DEVICE), block, dtype, weigh="output", shared_scaled=bool(shared), gate="clamped_swish",
                          alpha=1.702, limit=1.5, shared_limit=0.5).float().cpu().double()
    tolerance = 1e-5 if dtype == torch.float32 else 2e-2
    assert float((got - per_column * act).abs().max()) < tolerance


def test_a_gate_on_heads_and_capped_logits():
    from tlie_amd import ops
    generator = torch.Generator().manual_seed(8)
    values, pre = torch.randn(7, 30, generator=generator), torch.randn(2, 7, 50, generator=generator)
    got = ops.sigmoid_gate(values.to(DEVICE).clone(), ops.Product(pre.to(DEVICE).contiguous(), 2), 20).cpu().double()
    assert float((got - values.double() * torch.sigmoid(pre.double().sum(0)[:, 20:])).abs().max()) < 1e-6
    logits = 40.0 * torch.randn(5, 33, generator=generator)
    got = ops.softcap(logits.to(DEVICE).clone(), 11.0).cpu().double()
    assert float((got - 11.0 * torch.tanh(logits.double() / 11.0)).abs().max()) < 1e-5 and float(got.abs().max()) <= 11.0


# ---- whole models ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompt_matches_the_plain_implementation(setups, name, dtype):
    setup = setups(name)
    tokens = tokens_of(1, 90, CONFIGS[name]["vocab"])
    engine = new_engine(setup, dtype)
    assert_settled(run_cut(engine, "r", tokens, [len(tokens)]), setup, tokens, dtype, TOLERANCE[dtype], f"{name} {dtype}")
    engine.cache.check()


@pytest.mark.parametrize("name", list(CONFIGS))
def test_every_layer_matches_the_plain_implementation(setups, name):
    from tlie_amd import StepEntry
    setup = setups(name)
    tokens = tokens_of(2, 45, CONFIGS[name]["vocab"])
    _, residuals = plain.forward(setup["raw"], setup["weights"], tokens)
    engine = new_engine(setup, "float32")
    engine.admit("r")
    trace = {}
    engine.step([StepEntry("r", tokens, [len(tokens) - 1])], trace=trace)
    for index in range(residuals.shape[0]):
        got = trace[f"layer{index}.output"].cpu().double()
        scale = float(residuals[index].abs().max())
        assert float((got - residuals[index]).abs().max()) < 3e-5 * scale, f"{name}: the residual after layer run {index}"


@pytest.mark.parametrize("name,dtype", CASES)
def test_cuts_agree_with_each_other_and_with_the_plain_implementation(setups, name, dtype):
    """Whole, token by token from the first token, in portions of two, and in portions of changing sizes that end inside
    pages, windows and chunks."""
    setup = setups(name)
    tokens = tokens_of(3, 75, CONFIGS[name]["vocab"])
    engine = new_engine(setup, dtype, max_tokens=128)
    whole = run_cut(engine, "w", tokens, [len(tokens)])
    for cuts in ([1], [2], [3, 5, 2, 1, 17], [40, 1, 1, 1, 30, 2]):
        got = run_cut(engine, "c", tokens, cuts)
        assert_settled(got, setup, tokens, dtype, TOLERANCE[dtype], f"{name} {dtype} cut {cuts}")
        assert_settled(got, setup, tokens, dtype, CUT_TOLERANCE[dtype], f"{name} {dtype} cut {cuts} against the whole prompt", other=whole)
    engine.cache.check()


@pytest.mark.parametrize("name,dtype", CASES)
def test_batches_of_unequal_requests_with_pages_and_slots_used_again(setups, name, dtype):
    """Up to three live requests of unequal lengths in three slots more than once: portions of some beside single tokens
    of others, requests that pause for a step, a pool that only holds what is live."""
    from tlie_amd import StepEntry
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    lengths = {"a": 70, "b": 9, "c": 41, "d": 1, "e": 55, "f": 30}
    prompts = {key: tokens_of(10 + index, length, vocab) for index, (key, length) in enumerate(lengths.items())}
    engine = new_engine(setup, dtype, max_tokens=192, max_requests=3)
    rng = random.Random(5)
    waiting, live, at, rows = list(prompts), [], {}, {key: [] for key in prompts}
    steps = 0
    while waiting or live:
        while waiting and len(live) < 3 and sum((lengths[key] + 15) // 16 * 16 for key in live + [waiting[0]]) <= 192:
            key = waiting.pop(0)
            engine.admit(key)
            live.append(key)
            at[key] = 0
        entries, counts = [], {}
        for key in live:
            if len(live) > 1 and rng.random() < 0.25:
                continue                                              # left out of this step
            count = min(lengths[key] - at[key], rng.choice([1, 1, 2, 3, 9, 30]))
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
        assert_settled(torch.cat(rows[key]), setup, tokens, dtype, TOLERANCE[dtype], f"{name} {dtype} request {key}")


@pytest.mark.parametrize("name", list(CONFIGS))
def test_recorded_steps_equal_launched_steps_bit_for_bit(setups, name):
    from tlie_amd import StepEntry
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    prompts = [tokens_of(40 + index, length, vocab) for index, length in enumerate((37, 20, 50))]
    results = []
    for capture in (True, False):
        engine = new_engine(setup, "bfloat16", capture_graphs=capture)
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
    setup = setups(name)
    vocab = CONFIGS[name]["vocab"]
    prompts = [tokens_of(70 + index, length, vocab) for index, length in enumerate((45, 3, 18))]
    want = [plain_generate_greedy(setup["raw"], setup["weights"], prompt, 12) for prompt in prompts]
    engine = new_engine(setup, "float32", max_tokens=256)
    assert engine.generate(prompts, max_tokens=12, chunk_size=16, max_tokens_per_step=24) == want
    assert engine.generate([prompts[1]], max_tokens=12) == [want[1]]
    engine.cache.check()
    assert len(new_engine(setup, "bfloat16").generate(prompts, max_tokens=5)[2]) == 5


def test_a_preempted_request_is_recomputed(setups):
    setup = setups("Q")
    prompts = [tokens_of(90 + index, 40, CONFIGS["Q"]["vocab"]) for index in range(4)]
    want = [plain_generate_greedy(setup["raw"], setup["weights"], prompt, 20) for prompt in prompts]
    engine = new_engine(setup, "float32", max_tokens=176, max_requests=4)
    assert engine.generate(prompts, max_tokens=20, admit_partial=True) == want
    engine.cache.check()


@pytest.mark.parametrize("name,dtype", [("P", "float32"), ("R", "bfloat16"), ("S", "float32")])
def test_long_decoding_keeps_to_the_plain_implementation(setups, name, dtype):
    """A short prompt, then 200 tokens one by one: windows and chunks pass over decoded tokens many times, pages fill and
    (for windowed layers) go back to the pool while the request runs."""
    setup = setups(name)
    tokens = tokens_of(4, 205, CONFIGS[name]["vocab"])
    engine = new_engine(setup, dtype, max_tokens=256)
    got = run_cut(engine, "r", tokens, [5] + [1] * 200)
    assert_settled(got, setup, tokens, dtype, TOLERANCE[dtype], f"{name} {dtype}")
    engine.cache.check()


def test_the_command_line_and_the_replay_program_run_the_design(setups, tmp_path):
    import json
    import os
    import subprocess
    import sys
    import numpy
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    setup = setups("P")
    vocab = CONFIGS["P"]["vocab"]
    tokens, other = tokens_of(61, 40, vocab), tokens_of(62, 21, vocab)
    prompt = "ids:" + ",".join(str(token) for token in tokens[:9])
    cli = [sys.executable, os.path.join(root, "bin", "tinyllama_amd")]
    run = subprocess.run(cli + ["generate", setup["folder"], prompt, "6", "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert json.loads(run.stdout)["generated_tokens"] == plain_generate_greedy(setup["raw"], setup["weights"], tokens[:9], 6)
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
        read = lambda step: torch.from_numpy(numpy.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, vocab))
        assert_settled(read(0), setup, tokens, dtype, TOLERANCE[dtype], f"{dtype} step 0", places=[0, 29])
        assert_settled(read(1)[:1], setup, tokens, dtype, TOLERANCE[dtype], f"{dtype} step 1", places=[30])
        assert_settled(read(1)[1:], setup, other, dtype, TOLERANCE[dtype], f"{dtype} step 1, the other request", places=[20])
        assert_settled(read(3)[:1], setup, tokens, dtype, TOLERANCE[dtype], f"{dtype} step 3", places=[39])
        assert_settled(read(3)[1:], setup, other, dtype, TOLERANCE[dtype], f"{dtype} step 3, the other request", places=[20])


def drawn_configuration(seed):
    """A configuration drawn at random: every size, count, constant and option of the design, in ranges that the given
    configurations do not cover (odd widths and head sizes, up to eight streams, loops anywhere, one expert, all experts)."""
    rng = random.Random(seed)
    width = rng.choice([24, 36, 50, 64, 72, 100, 132])
    layers = []
    for _ in range(rng.randint(1, 4)):
        kind = rng.choice(["attention", "latent_attention", "attention_2"])
        groups = rng.choice([1, 2, 3])
        heads = groups * rng.choice([1, 2, 4])
        dim = rng.choice([4, 6, 10, 16, 24, 32, 48, 64])
        scale = rng.choice([0.1, 0.25, 0.4]) * (16.0 / dim) ** 0.5
        if kind == "attention":
            mixer = {"heads": heads, "kv_heads": groups, "dim": dim, "vdim": rng.choice([dim, dim, 5, 12, 40]), "scale": scale}
            if rng.random() < 0.6:
                mixer["softcap"] = rng.choice([0.5, 3.0, 25.0])
            if rng.random() < 0.6:
                mixer["q_temp"] = {"coef": rng.choice([0.2, 1.5]), "every": rng.choice([1, 3, 16, 2.5])}
        elif kind == "latent_attention":
            mixer = {"heads": heads, "dim": dim, "vdim": rng.choice([dim, 7, 20]), "kv_rank": rng.choice([8, 20, 48, 96, 136, 256]), "scale": scale}
            if rng.random() < 0.7:
                mixer["mask"] = {"size": rng.choice([1, 2, 5, 16, 17, 33, 64])}
        else:
            mixer = {"heads": heads, "kv_heads": groups, "dim": dim, "vdim": dim, "scale": scale}
            if rng.random() < 0.7:
                mixer["mask"] = {"size": rng.choice([1, 3, 8, 16, 31, 48])}
            if rng.random() < 0.7:
                mixer["rot"] = {"base": rng.choice([10.0, 1000.0, 500000.0]), "dims": rng.choice([d for d in (2, 4, dim - dim % 2) if d <= dim])}
        mlp = None
        if rng.random() < 0.8:
            experts = rng.choice([1, 2, 5, 9])
            mlp = {"kind": "moe", "expert": {"ff": rng.choice([3, 8, 20, 33]), "limit": rng.choice([0.5, 2.0, 7.0])},
                   "router": {"experts": experts, "top": rng.randint(1, experts)}}
            if rng.random() < 0.5:
                mlp["shared"] = {"ff": rng.choice([4, 10, 24]), "limit": rng.choice([0.7, 3.0])}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    raw = {"architecture": "Narolorn", "vocab": rng.choice([31, 100, 257]), "width": width, "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])},
           "layers": layers}
    if rng.random() < 0.75:
        raw["streams"] = rng.choice([1, 2, 3, 5, 8])
    if rng.random() < 0.6:
        raw["logit_softcap"] = rng.choice([2.0, 15.0, 50.0])
    if rng.random() < 0.6:
        start = rng.randrange(len(layers))
        raw["loop"] = {"start": start, "stop": rng.randint(start + 1, len(layers)), "times": rng.randint(1, 3)}
    return raw


@pytest.mark.parametrize("seed", range(16))
def test_drawn_configurations_in_32_bit(tmp_path, seed):
    """Sizes and constants nobody chose: whole, in portions of changing sizes beside a second request, and token by token,
    against the plain implementation, in 32-bit (where no close call of a router decides), pages of 16 or 32 rows."""
    from tlie_amd import Engine, StepEntry
    raw = drawn_configuration(seed)
    folder = make_model(tmp_path / "model", raw, seed=seed)
    config, weights = load_plain(folder)
    rng = random.Random(100 + seed)
    tokens, other = tokens_of(seed, rng.randint(40, 110), raw["vocab"]), tokens_of(seed + 50, rng.randint(1, 30), raw["vocab"])
    want, want_other = plain.forward(config, weights, tokens)[0], plain.forward(config, weights, other)[0]
    engine = Engine(folder, dtype="float32", max_tokens=256, page_size=rng.choice([16, 32]), max_requests=2)
    assert_rows(run_cut(engine, "w", tokens, [len(tokens)]), want, TOLERANCE["float32"], f"seed {seed} whole: {raw}")
    engine.admit("a")
    engine.admit("b")
    rows, at, fed = [], 0, 0
    while at < len(tokens):
        count = min(rng.choice([1, 1, 2, 3, 7, 20, 40]), len(tokens) - at)
        entries = [StepEntry("a", tokens[at:at + count], list(range(count)))]
        if fed < len(other):
            entries.append(StepEntry("b", other[fed:fed + 1], [0]))
        logits = engine.step(entries)
        rows.append(logits[:count].clone())
        if fed < len(other):
            assert_rows(logits[count:], want_other[fed:fed + 1], TOLERANCE["float32"], f"seed {seed}, the second request's token {fed}: {raw}")
            fed += 1
        at += count
    assert_rows(torch.cat(rows), want, TOLERANCE["float32"], f"seed {seed} in portions: {raw}")
    engine.finish("a")
    engine.finish("b")
    engine.cache.check()
    short = tokens[:24]
    assert_rows(run_cut(engine, "t", short, [1]), want[:24], TOLERANCE["float32"], f"seed {seed} token by token: {raw}")


@pytest.mark.parametrize("seed", range(16))
def test_drawn_configurations_in_bfloat16(tmp_path, seed):
    """The same configurations through the bfloat16 kernels (head sizes that the matrix cores take and others side by side):
    whole and with the last tokens decoded one by one, at the tokens without a router's close call."""
    from tlie_amd import Engine
    raw = drawn_configuration(seed)
    folder = make_model(tmp_path / "model", raw, seed=seed)
    config, weights = load_plain(folder)
    setup = {"raw": config, "weights": weights, "plain": {}, "margin": {}}
    tokens = tokens_of(seed, 70, raw["vocab"])
    engine = Engine(folder, dtype="bfloat16", max_tokens=128, page_size=16, max_requests=2)
    whole = run_cut(engine, "w", tokens, [len(tokens)])
    assert bool(torch.isfinite(whole).all())
    # (a drawn model may have many routers with many experts: however few tokens are without a close call, those are held)
    assert_settled(whole, setup, tokens, "bfloat16", TOLERANCE["bfloat16"], f"seed {seed} whole: {raw}", least=0.0)
    cut = run_cut(engine, "c", tokens, [50] + [1] * 20)
    assert_settled(cut, setup, tokens, "bfloat16", TOLERANCE["bfloat16"], f"seed {seed}, the last tokens one by one: {raw}", least=0.0)
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_latent_vector_wider_than_any_value_head(tmp_path, dtype):
    """A latent vector of 320 dims is beyond what the attention kernels take as a value head: the layer then expands and
    caches every head's keys and values; the results are the same function of the weights."""
    from tlie_amd import Engine
    raw = {"architecture": "Narolorn", "vocab": 90, "width": 72, "norm": {"eps": 1e-5}, "streams": 2,
           "layers": [{"type": "latent_attention", "mixer": {"heads": 3, "dim": 16, "vdim": 16, "kv_rank": 320, "scale": 0.25, "mask": {"size": 21}},
                       "mlp": None},
                      {"type": "latent_attention", "mixer": {"heads": 2, "dim": 8, "vdim": 24, "kv_rank": 272, "scale": 0.3}, "mlp": None}]}
    folder = make_model(tmp_path / "model", raw, seed=5)
    config, weights = load_plain(folder)
    tokens = tokens_of(9, 60, raw["vocab"])
    want = plain.forward(config, weights, tokens)[0]
    engine = Engine(folder, dtype=dtype, max_tokens=128, page_size=16, max_requests=2)
    for cuts in ([len(tokens)], [1], [7, 2, 30, 1]):
        assert_rows(run_cut(engine, "r", tokens, cuts), want, TOLERANCE[dtype], f"{dtype} cut {cuts}")
    engine.cache.check()
