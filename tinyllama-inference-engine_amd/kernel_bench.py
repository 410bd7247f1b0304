"""Times the engine's kernels one by one at a model's layer sizes: `python bench.py --kernels`.

reference: benchmarks/kernel_benchmarks.cu:127-163 times each of its kernels at TinyLlama's sizes
(warm-up, samples, median and p95).  Here every kernel of a decode step of `batch` requests at
`context` positions and of a prompt step of `prompt` tokens is launched through its face in
`ops`, as the parts launch it.  A kernel's launches are recorded into a HIP graph that walks
through copies of its weights (more than the chip's caches hold, so every launch reads its weights
from memory as it does inside a step), the graph is replayed `samples` times, and a launch's time is
a replay's time divided by its launches: what a kernel costs inside a replayed step, dependent
launch included.
"""
from __future__ import annotations

import math
import statistics
from types import SimpleNamespace

import numpy as np
import torch

from . import ops

COPIES_BYTES = 640 << 20          # a kernel's weights are cycled through copies of at least this many bytes together


def _timed(build, copies: int, samples: int, warmup: int = 3):
    """build(i) launches the kernel on copy i.  Returns per-launch microseconds, one per sample."""
    for index in range(copies):
        build(index)                                         # eager once: allocations and plans are made
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for index in range(copies):
            build(index)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    times = []
    for run in range(warmup + samples):
        start.record()
        graph.replay()
        stop.record()
        stop.synchronize()
        if run >= warmup:
            times.append(start.elapsed_time(stop) * 1e3 / copies)
    return times


def _row(name, times, read_bytes=0, flops=0):
    times = sorted(times)
    median = statistics.median(times)
    row = {"kernel": name, "median_us": round(median, 2), "p95_us": round(times[min(len(times) - 1, int(0.95 * len(times)))], 2)}
    if read_bytes:
        row["mb"] = round(read_bytes / 1e6, 2)
        row["gbs"] = round(read_bytes / median / 1e3, 0)
    if flops:
        row["tflops"] = round(flops / median / 1e6, 1)
    return row


def _copies(nbytes: int) -> int:
    return max(2, min(96, -(-COPIES_BYTES // max(nbytes, 1))))


def bench_kernels(cfg: dict, batch: int = 8, context: int = 2048, prompt: int = 2048, samples: int = 20, device="cuda:0",
                  only: str | None = None) -> list[dict]:
    """cfg: a config.json's keys (sizes of the layer and the vocabulary).  Returns one row per kernel."""
    device = torch.device(device)
    torch.cuda.set_device(device)
    hidden, inter, vocab = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or hidden // nq
    eps, theta = cfg["rms_norm_eps"], cfg.get("rope_theta", 10000.0)
    page_size = 16
    bf = torch.bfloat16
    rows = []

    def rand(*shape, scale=0.02, dtype=bf):
        return (torch.randn(shape, device=device, dtype=torch.float32) * scale).to(dtype)

    def want(name):
        return only is None or only in name
    inv_freq = torch.pow(torch.tensor(theta, dtype=torch.float32), -2.0 * torch.arange(d // 2, dtype=torch.float32) / d).to(device)
    norm_weight = rand(hidden, scale=1.0)
    blocks = (context + page_size - 1) // page_size
    pages = batch * blocks
    cache = rand(pages, 2, nkv, page_size * d, scale=0.5)
    table = torch.arange(pages, dtype=torch.int32, device=device).view(batch, blocks).contiguous()
    positions = torch.full((batch,), context - 1, dtype=torch.int32, device=device)
    slot_map = (table[:, -1] * page_size + (context - 1) % page_size).to(torch.int32).contiguous()
    few = ops.few_rows_route(batch, bf)

    # ---- a decode step's kernels --------------------------------------------------------------------
    def normed_rows(width):
        xg = rand(batch, width, scale=1.0)
        ssq = torch.rand(((width + 15) // 16, 16), device=device, dtype=torch.float32) * 16.0
        return ops.NormedRows(xg, ssq, eps)
    label = f"decode b{batch}"
    shapes = {"qkv": ((nq + 2 * nkv) * d, hidden), "o": (hidden, nq * d), "gate_up": (2 * inter, hidden), "down": (hidden, inter),
              "head": (vocab, hidden)}
    if few:
        for name, (n, k) in shapes.items():
            if not want(name):
                continue
            count = _copies(n * k * 2)
            weights = [rand(n, k) for _ in range(count)]
            x = normed_rows(k) if name in ("qkv", "gate_up", "head") else rand(batch, k, scale=1.0)
            residual = torch.zeros((batch, n), dtype=torch.float32, device=device)
            rope = ops.RopeTarget(positions, slot_map, inv_freq, d, cache, nq, nkv, d)
            if name == "qkv":
                launch = lambda i: ops.gemm_rows(x, weights[i], None, "rope", rope=rope)
            elif name == "gate_up":
                launch = lambda i: ops.gemm_rows(x, weights[i], None, "silu")
            elif name == "head":
                launch = lambda i: ops.gemm_rows(x, weights[i], None, "store")
            else:
                launch = lambda i: ops.gemm_rows(x, weights[i], None, "residual", residual=residual, next_norm=(norm_weight, eps))
            rows.append(_row(f"{label}: gemm_rows {name} [{n} x {k}]", _timed(launch, count, samples), read_bytes=n * k * 2))
            del weights
    else:
        for name, (n, k) in shapes.items():
            if not want(name):
                continue
            count = _copies(n * k * 2)
            weights = [rand(n, k) for _ in range(count)]
            x = rand(batch, k, scale=1.0)
            if batch <= ops.SKINNY_MAX_ROWS and name == "gate_up":
                launch, kind = (lambda i: ops.gemm_skinny(x, weights[i], None, gated=True)), "gemm_skinny (gated)"
            elif batch <= ops.SKINNY_MAX_ROWS:
                launch, kind = (lambda i: ops.gemm_skinny(x, weights[i], None)), "gemm_skinny"
            else:
                launch, kind = (lambda i: ops.library_mm(x, weights[i], torch.float32 if name == "head" else bf)), "library"
            rows.append(_row(f"{label}: {kind} {name} [{n} x {k}]", _timed(launch, count, samples), read_bytes=n * k * 2))
            del weights
    if want("attention"):
        ctx = SimpleNamespace(max_new=1, num_seqs=batch, num_tokens=batch, max_context=context, scratch={}, tile_owner=None,
                              compute_units=int(torch.cuda.get_device_properties(device).multi_processor_count), host={})
        tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, nq // nkv, nkv, d)
        kv_bytes = batch * context * 2 * nkv * d * 2
        count = _copies(kv_bytes)
        caches = [rand(pages, 2, nkv, page_size * d, scale=0.5) for _ in range(count)]
        q = rand(batch, nq * d, scale=1.0)
        launch = lambda i: ops.attention_mfma(q, caches[i], table, tiles, positions, nq, nkv, d, None, d ** -0.5, nsplit, split_len,
                                              col_tiles, waves, shared)
        rows.append(_row(f"{label}: attention + merge, {context} positions ({nsplit} parts x {waves} waves)",
                         _timed(launch, count, samples), read_bytes=kv_bytes))
        del caches
    if want("embed") and few:
        table_rows = rand(vocab, hidden)
        tokens = torch.randint(0, vocab, (batch,), dtype=torch.int32, device=device)
        rows.append(_row(f"{label}: embed_rows", _timed(lambda i: ops.embed_rows(tokens, table_rows, (norm_weight, eps)), 8, samples)))
    if want("sample"):
        logits = rand(batch, vocab, scale=1.0, dtype=torch.float32)
        rows.append(_row(f"{label}: sample (greedy) [{batch} x {vocab}]", _timed(lambda i: ops.sample(logits), 8, samples),
                         read_bytes=batch * vocab * 4))

    # ---- a prompt step's kernels ----------------------------------------------------------------------
    if prompt > 0:
        label = f"prompt {prompt}"
        x_by_width = {}
        for name, (n, k) in shapes.items():
            if name == "head" or not want(name):
                continue
            count = _copies(n * k * 2)
            weights = [rand(n, k) for _ in range(count)]
            x = x_by_width.setdefault(k, rand(prompt, k, scale=1.0))
            rows.append(_row(f"{label}: library product {name} [{prompt} x {n} x {k}]",
                             _timed(lambda i: ops.library_mm(x, weights[i]), count, samples), flops=2.0 * prompt * n * k))
            del weights
        if want("attention"):
            blocks_p = (prompt + page_size - 1) // page_size
            cache_p = rand(blocks_p, 2, nkv, page_size * d, scale=0.5)
            table_p = torch.arange(blocks_p, dtype=torch.int32, device=device).view(1, blocks_p)
            positions_p = torch.arange(prompt, dtype=torch.int32, device=device)
            host = {"seq_start": np.asarray([0, prompt], dtype=np.int32), "seq_len": np.asarray([prompt], dtype=np.int32)}
            ctx = SimpleNamespace(max_new=prompt, num_seqs=1, num_tokens=prompt, max_context=prompt, scratch={}, tile_owner=None,
                                  compute_units=int(torch.cuda.get_device_properties(device).multi_processor_count), host=host,
                                  tokens=positions_p)
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, nq // nkv, nkv, d)
            q = rand(prompt, nq * d, scale=1.0)
            launch = lambda i: ops.attention_mfma(q, cache_p, table_p, tiles, positions_p, nq, nkv, d, None, d ** -0.5, nsplit,
                                                  split_len, col_tiles, waves, shared)
            rows.append(_row(f"{label}: attention ({col_tiles} column groups, {waves} waves, shared {shared})",
                             _timed(launch, 4, samples), flops=4.0 * nq * d * prompt * (prompt + 1) / 2))
        if want("norm"):
            residual = rand(prompt, hidden, scale=1.0, dtype=torch.float32)
            delta = ops.Product(rand(prompt, hidden, scale=1.0), 1)
            rows.append(_row(f"{label}: add + rmsnorm [{prompt} x {hidden}]",
                             _timed(lambda i: ops.add_rmsnorm(residual, delta, norm_weight, eps, bf), 4, samples),
                             read_bytes=prompt * hidden * (4 + 2 + 4 + 2)))
        if want("silu"):
            gate_up = ops.Product(rand(prompt, 2 * inter, scale=1.0), 1)
            rows.append(_row(f"{label}: silu * up [{prompt} x {inter}]",
                             _timed(lambda i: ops.silu_mul(gate_up, bf, interleaved=True), 4, samples), read_bytes=prompt * inter * 6))
        if want("rope"):
            blocks_p = (prompt + page_size - 1) // page_size
            cache_p = rand(blocks_p, 2, nkv, page_size * d, scale=0.5)
            positions_p = torch.arange(prompt, dtype=torch.int32, device=device)
            qkv = ops.Product(rand(prompt, (nq + 2 * nkv) * d, scale=1.0), 1)
            rows.append(_row(f"{label}: rotation + cache write",
                             _timed(lambda i: ops.rope_cache(qkv, positions_p, positions_p, inv_freq, d, cache_p, nq, nkv, d, bf, paired=True),
                                    4, samples), read_bytes=prompt * (nq + 2 * nkv) * d * 4))
    return rows


def bench_design_kernels(sizes: dict, batch: int = 8, context: int = 2048, prompt: int = 2048, samples: int = 10, device="cuda:0",
                         hbm_gbs: float = 8000.0, mfma_tflops: float = 2500.0) -> list[dict]:
    """The kernels that the Fadutar decoder adds, each alone at a layer's sizes, for a decode step of `batch`
    requests at `context` positions and a prompt step of `prompt` tokens, each beside the like kernel of the
    Llama decoder at the same sizes; every row carries the fraction of the roofline its bytes or flops reach
    (`frac`: of `hbm_gbs` for rows with bytes, of `mfma_tflops` for rows with flops).
    sizes: width, ff, heads, kv_heads, dim (attention, keys and values alike), chunk; latent_heads, latent_dim,
    latent_rot, latent_vdim, rank; lru_width, lru_blocks, taps."""
    device = torch.device(device)
    torch.cuda.set_device(device)
    bf, f32 = torch.bfloat16, torch.float32
    width, ff = sizes["width"], sizes["ff"]
    nq, nkv, d, chunk = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["chunk"]
    lh, ldim, lrot, lv, rank = sizes["latent_heads"], sizes["latent_dim"], sizes["latent_rot"], sizes["latent_vdim"], sizes["rank"]
    lru, lru_blocks, taps = sizes["lru_width"], sizes["lru_blocks"], sizes["taps"]
    page_size, rows = 16, []
    units = int(torch.cuda.get_device_properties(device).multi_processor_count)

    def rand(*shape, scale=0.02, dtype=bf):
        return (torch.randn(shape, device=device, dtype=f32) * scale).to(dtype)

    def row(name, times, read_bytes=0, flops=0):
        entry = _row(name, times, read_bytes, flops)
        if read_bytes:
            entry["frac"] = round(entry["gbs"] / hbm_gbs, 3)
        elif flops:
            entry["frac"] = round(entry["tflops"] / mfma_tflops, 4)
        rows.append(entry)

    def ints(values):
        return torch.tensor(values, dtype=torch.int32, device=device)

    for label, tokens, seqs in ((f"decode b{batch}", batch, batch), (f"prompt {prompt}", prompt, 1)):
        if tokens <= 0:
            continue
        decode = seqs == tokens
        length = context if decode else prompt
        blocks = (length + page_size - 1) // page_size
        table = torch.arange(seqs * blocks, dtype=torch.int32, device=device).view(seqs, blocks).contiguous()
        if decode:
            positions = torch.full((tokens,), length - 1, dtype=torch.int32, device=device)
            token_seq, seq_start = ints(list(range(tokens))), ints(list(range(tokens + 1)))
            host = {"seq_start": np.arange(tokens + 1, dtype=np.int32), "seq_len": np.full(tokens, length, dtype=np.int32)}
        else:
            positions = torch.arange(tokens, dtype=torch.int32, device=device)
            token_seq, seq_start = torch.zeros(tokens, dtype=torch.int32, device=device), ints([0, tokens])
            host = {"seq_start": np.asarray([0, tokens], dtype=np.int32), "seq_len": np.asarray([tokens], dtype=np.int32)}
        slot_map = (table[token_seq.long(), (positions // page_size).long()] * page_size + positions % page_size).to(torch.int32).contiguous()
        seq_slot = ints(list(range(seqs)))
        token_slot = seq_slot[token_seq.long()].contiguous()
        ctx = SimpleNamespace(max_new=1 if decode else tokens, num_seqs=seqs, num_tokens=tokens, max_context=length, scratch={},
                              tile_owner=None, compute_units=units, host=host, tokens=positions)
        seen = min(length, chunk) if chunk else length            # keys a token of the chunked layers reads at most
        # ---- attention with a sink inside chunks, on the matrix cores, beside the plain causal one --------------
        cache = rand(seqs * blocks, 2, nkv, page_size * d, scale=0.5)
        q = rand(tokens, nq * d, scale=1.0)
        sink = rand(nq, scale=1.0, dtype=f32)
        tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, nq // nkv, nkv, d)
        for name, extra, keys in (("attention, causal (Llama's)", {}, length), (f"attention, sink + chunks of {chunk}", {"chunk": chunk, "sink": sink}, seen)):
            launch = lambda i: ops.attention_mfma(q, cache, table, tiles, positions, nq, nkv, d, None, d ** -0.5, nsplit, split_len,
                                                  col_tiles, waves, shared, **extra)
            if decode:
                row(f"{label}: {name}", _timed(launch, 4, samples), read_bytes=seqs * keys * 2 * nkv * d * 2)
            else:
                pairs = sum(p % chunk + 1 for p in range(tokens)) if extra and chunk else tokens * (tokens + 1) // 2
                row(f"{label}: {name}", _timed(launch, 4, samples), flops=4.0 * nq * d * pairs)
        # ---- latent attention: placement, the heads' products before and after, the attention over the latent cache ----
        key = rank + lrot
        fused = ops.Product(rand(tokens, lh * (ldim + lrot) + rank + lrot, scale=1.0), 1)
        latent_cache = rand(seqs * blocks, 2, 1, page_size * key, scale=0.5)       # values as wide as keys
        inv_freq = torch.pow(torch.tensor(10000.0), -2.0 * torch.arange(lrot // 2, dtype=f32) / lrot).to(device)
        norm_weight = rand(rank, scale=1.0)
        launch = lambda i: ops.latent_place(fused, positions, slot_map, inv_freq, norm_weight, 1e-5, latent_cache, lh, ldim, lrot, rank, bf,
                                            wide_values=True)
        row(f"{label}: latent placement (norm, rotation, cache write)", _timed(launch, 4, samples),
            read_bytes=tokens * (fused.cols * 2 + lh * (ldim + lrot) * 2 + (key + rank) * 2))
        q_plain, q_wide = launch(0)
        up_keys, up_values = rand(lh, ldim, rank), rand(lh, rank, lv)
        up_keys_rows, up_values_rows = up_keys.transpose(1, 2).contiguous(), up_values.transpose(1, 2).contiguous()
        launch = lambda i: ops.block_linear(q_plain, 0, lh * ldim, ldim, up_keys, None, q_wide, 0, lh * key, key, tokens, weight=up_keys_rows)
        row(f"{label}: heads' queries onto the latent space [{lh} x {ldim} x {rank}]", _timed(launch, 4, samples),
            **({"read_bytes": lh * ldim * rank * 2 + tokens * lh * (ldim + rank) * 2} if decode else {"flops": 2.0 * tokens * lh * ldim * rank}))
        latent_sink = rand(lh, scale=1.0, dtype=f32)
        ltiles, lcol_tiles, lnsplit, lsplit_len, lwaves, lshared = ops.attention_plan(ctx, lh, 1, key)
        launch = lambda i: ops.attention_mfma(q_wide, latent_cache, table, ltiles, positions, lh, 1, key, None, 0.1, lnsplit, lsplit_len,
                                              lcol_tiles, lwaves, lshared, sink=latent_sink)
        if decode:
            row(f"{label}: attention over the latent cache ({lh} heads, {key} key dims)", _timed(launch, 4, samples),
                read_bytes=seqs * length * (key + rank) * 2)
        else:
            row(f"{label}: attention over the latent cache ({lh} heads, {key} key dims)", _timed(launch, 2, samples),
                flops=2.0 * lh * (key + rank) * tokens * (tokens + 1) / 2)
        attended = rand(tokens, lh * key, scale=1.0)
        values = torch.empty((tokens, lh * lv), dtype=bf, device=device)
        launch = lambda i: ops.block_linear(attended, 0, lh * key, key, up_values, None, values, 0, lh * lv, lv, tokens, weight=up_values_rows)
        row(f"{label}: attended latent vectors onto the heads' values [{lh} x {rank} x {lv}]", _timed(launch, 4, samples),
            **({"read_bytes": lh * rank * lv * 2 + tokens * lh * (rank + lv) * 2} if decode else {"flops": 2.0 * tokens * lh * rank * lv}))
        # ---- the recurrence: convolution, gates, scan -------------------------------------------------------------
        inside = lru // lru_blocks
        both = ops.Product(rand(tokens, 2 * lru, scale=1.0), 1)
        state = torch.zeros((seqs, taps, lru), dtype=f32, device=device)
        conv, conv_bias = rand(lru, taps, scale=0.5), rand(lru)
        launch = lambda i: ops.causal_conv(both, lru, conv, conv_bias, state, token_seq, token_slot, seq_start)
        row(f"{label}: causal convolution [{lru} x {taps}]", _timed(launch, 4, samples), read_bytes=tokens * lru * (2 + 4) + seqs * taps * lru * 4)
        u = launch(0)
        gates_t, gate_bias = rand(lru_blocks, inside, 2 * inside), rand(lru_blocks, 2 * inside)
        gates = torch.empty((tokens, 2 * lru), dtype=f32, device=device)
        gates_rows = gates_t.transpose(1, 2).contiguous()
        launch = lambda i: ops.block_linear(u, 0, lru, inside, gates_t, gate_bias, gates, 0, 2 * lru, 2 * inside, tokens, weight=gates_rows)
        row(f"{label}: the recurrence's gates [{lru_blocks} x {inside} x {2 * inside}]", _timed(launch, 4, samples),
            **({"read_bytes": lru_blocks * inside * 2 * inside * 2 + tokens * lru * 12} if decode else {"flops": 4.0 * tokens * lru * inside}))
        lam = rand(lru, scale=1.0)
        launch = lambda i: ops.gated_recurrence(both, lru, 0, u, gates, lam, 8.0, state, seq_start, seq_slot, inside, bf, max_new=ctx.max_new)
        row(f"{label}: gated recurrence (scan, gate branch, state)", _timed(launch, 4, samples),
            read_bytes=tokens * lru * (4 + 8 + 4 + 2) + seqs * taps * lru * 8)
        # ---- the element-wise kernels beside Llama's ------------------------------------------------------------------
        residual = rand(tokens, width, scale=1.0, dtype=f32)
        delta = ops.Product(rand(tokens, width, scale=1.0), 1)
        weight, weight32 = rand(width, scale=1.0), rand(width, scale=1.0, dtype=f32)
        row(f"{label}: add + norm (Llama's) [{tokens} x {width}]",
            _timed(lambda i: ops.add_rmsnorm(residual, delta, weight, 1e-5, bf), 4, samples), read_bytes=tokens * width * (4 + 2 + 4 + 2))
        row(f"{label}: norm + add + norm [{tokens} x {width}]",
            _timed(lambda i: ops.norm_add_rmsnorm(residual, delta, weight32, 1e-5, weight32, 1e-5, bf), 4, samples),
            read_bytes=tokens * width * (4 + 2 + 4 + 2))
        gate_up = ops.Product(rand(tokens, 2 * ff, scale=1.0), 1)
        row(f"{label}: silu gate (Llama's) [{tokens} x {ff}]", _timed(lambda i: ops.silu_mul(gate_up, bf, interleaved=True), 4, samples),
            read_bytes=tokens * ff * 6)
        row(f"{label}: clamped gate [{tokens} x {ff}]",
            _timed(lambda i: ops.silu_mul(gate_up, bf, interleaved=True, gate="clamped_swish", alpha=1.702, limit=7.0), 4, samples),
            read_bytes=tokens * ff * 6)
        qkv = ops.Product(rand(tokens, (nq + 2 * nkv) * d, scale=1.0), 1)
        rot_freq = torch.pow(torch.tensor(10000.0), -2.0 * torch.arange(d // 2, dtype=f32) / d).to(device)
        row(f"{label}: rotation + cache write (Llama's)",
            _timed(lambda i: ops.rope_cache(qkv, positions, slot_map, rot_freq, d, cache, nq, nkv, d, bf, paired=True), 4, samples),
            read_bytes=tokens * (nq + 2 * nkv) * d * 4)
        row(f"{label}: placement of q, k, v (no rotation)",
            _timed(lambda i: ops.qkv_place(qkv, positions, slot_map, None, 0, cache, nq, nkv, d, d, bf), 4, samples),
            read_bytes=tokens * (nq + 2 * nkv) * d * 4)
    return rows


def bench_raketar_kernels(sizes: dict, batch: int = 8, context: int = 2048, prompt: int = 2048, samples: int = 10, device="cuda:0",
                          hbm_gbs: float = 8000.0, mfma_tflops: float = 2500.0) -> list[dict]:
    """The kernels that the Raketar decoder adds, each alone at a layer's sizes, for a decode step of `batch` requests at
    `context` positions and a prompt step of `prompt` tokens, each beside the like kernel of the Llama decoder at the
    same sizes; every row carries the fraction of the roofline its bytes or flops reach (`frac`: of `hbm_gbs` for rows
    with bytes, of `mfma_tflops` for rows with flops).
    sizes: width, ff, heads, kv_heads, dim, vdim (differential attention), llama_heads, llama_kv_heads; memory_heads,
    memory_dim, memory_vdim; experts, top, expert_ff, shared_ff; side."""
    device = torch.device(device)
    torch.cuda.set_device(device)
    bf, f32 = torch.bfloat16, torch.float32
    width, ff = sizes["width"], sizes["ff"]
    H, G, d, dv = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    lq, lkv = sizes["llama_heads"], sizes["llama_kv_heads"]
    mh, md, mv = sizes["memory_heads"], sizes["memory_dim"], sizes["memory_vdim"]
    experts, top, eff, sff, side = sizes["experts"], sizes["top"], sizes["expert_ff"], sizes["shared_ff"], sizes["side"]
    page_size, rows = 16, []
    units = int(torch.cuda.get_device_properties(device).multi_processor_count)

    def rand(*shape, scale=0.02, dtype=bf):
        return (torch.randn(shape, device=device, dtype=f32) * scale).to(dtype)

    def row(name, times, read_bytes=0, flops=0):
        entry = _row(name, times, read_bytes, flops)
        if read_bytes:
            entry["frac"] = round(entry["gbs"] / hbm_gbs, 3)
        elif flops:
            entry["frac"] = round(entry["tflops"] / mfma_tflops, 4)
        rows.append(entry)

    def ints(values):
        return torch.tensor(values, dtype=torch.int32, device=device)

    for label, tokens, seqs in ((f"decode b{batch}", batch, batch), (f"prompt {prompt}", prompt, 1)):
        if tokens <= 0:
            continue
        decode = seqs == tokens
        length = context if decode else prompt
        blocks = (length + page_size - 1) // page_size
        table = torch.arange(seqs * blocks, dtype=torch.int32, device=device).view(seqs, blocks).contiguous()
        if decode:
            positions = torch.full((tokens,), length - 1, dtype=torch.int32, device=device)
            token_seq, seq_start = ints(list(range(tokens))), ints(list(range(tokens + 1)))
            host = {"seq_start": np.arange(tokens + 1, dtype=np.int32), "seq_len": np.full(tokens, length, dtype=np.int32)}
        else:
            positions = torch.arange(tokens, dtype=torch.int32, device=device)
            token_seq, seq_start = torch.zeros(tokens, dtype=torch.int32, device=device), ints([0, tokens])
            host = {"seq_start": np.asarray([0, tokens], dtype=np.int32), "seq_len": np.asarray([tokens], dtype=np.int32)}
        slot_map = (table[token_seq.long(), (positions // page_size).long()] * page_size + positions % page_size).to(torch.int32).contiguous()
        seq_slot = ints(list(range(seqs)))
        ids = torch.randint(0, 1000, (tokens,), device=device, dtype=torch.int32)
        ctx = SimpleNamespace(max_new=1 if decode else tokens, num_seqs=seqs, num_tokens=tokens, max_context=length, scratch={},
                              tile_owner=None, compute_units=units, host=host, tokens=positions)
        keys_seen = length if decode else (length + 1) / 2            # keys a token sees on average
        # ---- attention: two maps a head over shared values, beside the plain causal one of as many query heads -------
        parts = dv // d
        cache = rand(seqs * blocks, 2, lkv, page_size * d, scale=0.5)
        q = rand(tokens, lq * d, scale=1.0)
        tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, lq // lkv, lkv, d)
        times = _timed(lambda i: ops.attention_mfma(q, cache, table, tiles, positions, lq, lkv, d, None, d ** -0.5, nsplit, split_len,
                                                    col_tiles, waves, shared), 8, samples)
        cache_bytes, flops = seqs * length * lkv * 2 * d * 2, 4.0 * tokens * lq * d * keys_seen
        row(f"{label}: attention, causal (Llama's), {lq} heads of {d} on {lkv}", times, cache_bytes if decode else 0, 0 if decode else flops)
        ctx.scratch = {}
        cache2 = rand(seqs * blocks, G, page_size * (2 * d + dv), scale=0.5)
        q2 = rand(tokens, 2 * H * d, scale=1.0)
        tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, H // G, 2 * G * parts, d)
        times = _timed(lambda i: ops.attention_mfma(q2, cache2, table, tiles, positions, 2 * H * parts, 2 * G * parts, d, None, d ** -0.5,
                                                    nsplit, split_len, col_tiles, waves, shared, planes=(parts, 2 * parts, parts),
                                                    float_out=True), 8, samples)
        cache_bytes = seqs * length * G * (2 * d + dv) * 2
        flops = 2.0 * tokens * 2 * H * (d + dv) * keys_seen             # scores once a map, values of dv
        row(f"{label}: attention, two maps of {H} heads of {d} on {G} groups, values of {dv}", times, cache_bytes if decode else 0,
            0 if decode else flops)
        attended = rand(tokens, 2 * H * dv, scale=1.0, dtype=f32)
        fused = ops.Product(rand(tokens, 2 * H * d + 2 * G * d + G * dv + H * dv, scale=1.0), 1)
        times = _timed(lambda i: ops.head_combine(attended, H, dv, 1e-5, bf, pair_group=H // G, pair_lambda=0.3, mult=0.5, gate=fused,
                                                  gate_col=fused.cols - H * dv, parts=parts), 8, samples)
        row(f"{label}: difference of the maps, norm and gate", times, tokens * H * dv * (8 + 2 + 2))
        times = _timed(lambda i: ops.qkv_place(fused, positions, slot_map, torch.ones(d // 2, device=device), d, cache2, 2 * H, 2 * G, d, dv,
                                               bf, value_heads=G, extra_cols=H * dv), 8, samples)
        row(f"{label}: placement of q, k, v (shared value heads)", times, tokens * (2 * H * d * 2 + 2 * G * d + G * dv) * 2 * 2)
        qkv = ops.Product(rand(tokens, (lq + 2 * lkv) * d, scale=1.0), 1)
        times = _timed(lambda i: ops.rope_cache(qkv, positions, slot_map, torch.ones(d // 2, device=device), d, cache, lq, lkv, d, bf), 8, samples)
        row(f"{label}: rotation + cache write (Llama's)", times, tokens * (lq * 2 + 2 * lkv) * d * 2 * 2)
        # ---- the matrix memory -------------------------------------------------------------------------------------
        memory_in = ops.Product(rand(tokens, 2 * mh * md + 2 * mh * mv, scale=1.0), 1)
        gates = rand(tokens, 2 * mh, scale=1.0, dtype=f32) + 3.0
        state = torch.zeros((seqs, *ops.mlstm_state_shape(mh, md, mv)), dtype=f32, device=device)
        times = _timed(lambda i: ops.mlstm_scan(memory_in, 0, mh * md, 2 * mh * md, gates, state, seq_start, seq_slot, mh, md, mv, 15.0,
                                                md ** -0.5, max_new=ctx.max_new), 8, samples)
        state_bytes = seqs * mh * md * mv * 4 * 2
        # a token: S = keep S + k v^T and S^T q, 4 flops an element of S (the sliced walk does the first half twice)
        row(f"{label}: matrix memory, {mh} heads of {md} x {mv} (gates, walk)", times, state_bytes if decode else 0,
            0 if decode else 4.0 * tokens * mh * md * mv)
        memory_out = rand(tokens, mh * mv, scale=1.0, dtype=f32)
        weight = rand(mh * mv, scale=1.0)
        times = _timed(lambda i: ops.head_combine(memory_out, mh, mv, 1e-5, bf, weight=weight, gate=memory_in, gate_col=2 * mh * md + mh * mv),
                       8, samples)
        row(f"{label}: the memory heads' norm and gate", times, tokens * mh * mv * (4 + 2 + 2))
        x = rand(tokens, width, scale=1.0)
        gate_w, gate_b = rand(2 * mh, width), rand(2 * mh)
        times = _timed(lambda i: ops.few_outputs(x, gate_w, gate_b), 8, samples)
        row(f"{label}: the gates' product, float sums ({2 * mh} outputs)", times, (tokens + 2 * mh) * width * 2)
        # ---- the routed feed-forward -------------------------------------------------------------------------------
        router = rand(experts, width)
        times = _timed(lambda i: ops.few_outputs(x, router, top=top), 8, samples)
        row(f"{label}: router, {top} of {experts}", times, (tokens + experts) * width * 2)
        inter = experts * eff + sff
        scale = ops.few_outputs(x, router, top=top)
        gate_up = ops.Product(rand(tokens, 2 * inter, scale=1.0), 1)
        times = _timed(lambda i: ops.routed_gate(gate_up, scale, eff, bf), 4, samples)
        row(f"{label}: gate of the routed feed-forward (all experts' columns)", times, tokens * inter * 6)
        dense_up = ops.Product(rand(tokens, 2 * ff, scale=1.0), 1)
        times = _timed(lambda i: ops.silu_mul(dense_up, bf, interleaved=True), 4, samples)
        row(f"{label}: SiLU gate (Llama's)", times, tokens * ff * 6)
        if not decode:
            from .parts.linear import Linear
            for name, out_features, in_features, useful in (
                    ("routed gate/up, all experts", 2 * inter, width, 2 * (top * eff + sff)), ("routed down, all experts", width, inter, None),
                    ("dense gate/up (Llama's)", 2 * ff, width, 2 * ff), ("dense down (Llama's)", width, ff, None)):
                linear = Linear(rand(out_features, in_features), None, bf)
                operand = rand(tokens, in_features, scale=1.0)
                times = _timed(lambda i: linear(operand), 4, samples)
                used = useful if useful is not None else out_features
                inner = in_features if useful is not None else (top * eff + sff if "routed" in name else ff)
                row(f"{label}: {name} (flops of the experts in use)", times, 0, 2.0 * tokens * used * inner)
        # ---- the residual and the token input ----------------------------------------------------------------------
        residual = rand(tokens, width, scale=1.0, dtype=f32)
        first, second = ops.Product(rand(tokens, width, scale=1.0), 1), ops.Product(rand(tokens, width, scale=1.0), 1)
        times = _timed(lambda i: ops.residual_update(residual, first, second, 0.5, copy_dtype=bf), 8, samples)
        row(f"{label}: residual += both sublayers, copy for the token input", times, tokens * width * (4 + 4 + 2 + 2 + 2))
        norm_w = rand(width, scale=1.0)
        times = _timed(lambda i: ops.norm_add_rmsnorm(residual, first, norm_w, 1e-5, norm_w, 1e-5, bf), 8, samples)
        row(f"{label}: token input normed, added, next norm", times, tokens * width * (4 + 4 + 2 + 2))
        times = _timed(lambda i: ops.add_rmsnorm(residual, first, norm_w, 1e-5, bf), 8, samples)
        row(f"{label}: add + norm (Llama's)", times, tokens * width * (4 + 4 + 2 + 2))
        pre = ops.Product(rand(tokens, side, scale=1.0), 1)
        side_table = rand(1000, 4 * side, scale=1.0)
        times = _timed(lambda i: ops.side_gate(pre, ids, side_table, side, bf), 8, samples)
        row(f"{label}: token input's gate", times, tokens * side * 6)
    return rows



def bench_narolorn_kernels(sizes: dict, batch: int = 8, context: int = 2048, prompt: int = 2048, samples: int = 10, device="cuda:0",
                           hbm_gbs: float = 8000.0, mfma_tflops: float = 2500.0) -> list[dict]:
    """The kernels that the Narolorn decoder adds or extends, each alone at a layer's sizes, for a decode step of `batch`
    requests at `context` positions and a prompt step of `prompt` tokens, each beside the like kernel of the Llama decoder at
    the same sizes; every row carries the fraction of the roofline its bytes or flops reach (`frac`: of `hbm_gbs` for rows
    with bytes, of `mfma_tflops` for rows with flops).
    sizes: width, ff, vocab, streams, heads, kv_heads, dim; softcap, chunk, window; latent_heads, latent_dim, latent_vdim, rank;
    experts, top, expert_ff, shared_ff."""
    device = torch.device(device)
    torch.cuda.set_device(device)
    bf, f32 = torch.bfloat16, torch.float32
    width, ff, vocab, count = sizes["width"], sizes["ff"], sizes["vocab"], sizes["streams"]
    H, G, d = sizes["heads"], sizes["kv_heads"], sizes["dim"]
    lh, ld, lv, rank = sizes["latent_heads"], sizes["latent_dim"], sizes["latent_vdim"], sizes["rank"]
    experts, top, eff, sff = sizes["experts"], sizes["top"], sizes["expert_ff"], sizes["shared_ff"]
    page_size, rows = 16, []
    units = int(torch.cuda.get_device_properties(device).multi_processor_count)

    def rand(*shape, scale=0.02, dtype=bf):
        return (torch.randn(shape, device=device, dtype=f32) * scale).to(dtype)

    def row(name, times, read_bytes=0, flops=0):
        entry = _row(name, times, read_bytes, flops)
        if read_bytes:
            entry["frac"] = round(entry["gbs"] / hbm_gbs, 3)
        elif flops:
            entry["frac"] = round(entry["tflops"] / mfma_tflops, 4)
        rows.append(entry)

    def ints(values):
        return torch.tensor(values, dtype=torch.int32, device=device)

    for label, tokens, seqs in ((f"decode b{batch}", batch, batch), (f"prompt {prompt}", prompt, 1)):
        if tokens <= 0:
            continue
        decode = seqs == tokens
        length = context if decode else prompt
        blocks = (length + page_size - 1) // page_size
        table = torch.arange(seqs * blocks, dtype=torch.int32, device=device).view(seqs, blocks).contiguous()
        if decode:
            positions = torch.full((tokens,), length - 1, dtype=torch.int32, device=device)
            token_seq = ints(list(range(tokens)))
            host = {"seq_start": np.arange(tokens + 1, dtype=np.int32), "seq_len": np.full(tokens, length, dtype=np.int32)}
        else:
            positions = torch.arange(tokens, dtype=torch.int32, device=device)
            token_seq = torch.zeros(tokens, dtype=torch.int32, device=device)
            host = {"seq_start": np.asarray([0, tokens], dtype=np.int32), "seq_len": np.asarray([tokens], dtype=np.int32)}
        slot_map = (table[token_seq.long(), (positions // page_size).long()] * page_size + positions % page_size).to(torch.int32).contiguous()
        ctx = SimpleNamespace(max_new=1 if decode else tokens, num_seqs=seqs, num_tokens=tokens, max_context=length, scratch={},
                              tile_owner=None, compute_units=units, host=host, tokens=positions)
        keys_seen = length if decode else (length + 1) / 2            # keys a token sees on average
        # ---- attention: capped scores; chunks; the window over the latent cache; beside the plain causal one --------
        cache = rand(seqs * blocks, 2, G, page_size * d, scale=0.5)
        q = rand(tokens, H * d, scale=1.0)
        cache_bytes, flops = seqs * length * G * 2 * d * 2, 4.0 * tokens * H * d * keys_seen
        for name, options in (("causal (Llama's)", {}), ("capped scores", {"softcap": sizes["softcap"]}), (f"chunks of {sizes['chunk']}", {"chunk": sizes["chunk"]})):
            ctx.scratch = {}
            tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, H // G, G, d)
            times = _timed(lambda i: ops.attention_mfma(q, cache, table, tiles, positions, H, G, d, None, d ** -0.5, nsplit, split_len,
                                                        col_tiles, waves, shared, **options), 8, samples)
            seen = min(keys_seen, sizes["chunk"] if decode else sizes["chunk"] / 2) if "chunk" in options else keys_seen
            row(f"{label}: attention, {name}, {H} heads of {d} on {G}", times, int(cache_bytes * seen / keys_seen) if decode else 0,
                0 if decode else 4.0 * tokens * H * d * seen)
        key = rank
        latent_cache = rand(seqs * blocks, 2, 1, page_size * key, scale=0.5)
        q_wide = rand(tokens, lh * key, scale=1.0)
        ctx.scratch = {}
        tiles, col_tiles, nsplit, split_len, waves, shared = ops.attention_plan(ctx, lh, 1, key)
        times = _timed(lambda i: ops.attention_mfma(q_wide, latent_cache, table, tiles, positions, lh, 1, key, sizes["window"], ld ** -0.5,
                                                    nsplit, split_len, col_tiles, waves, shared), 8, samples)
        seen = min(keys_seen, sizes["window"])
        row(f"{label}: attention over the latent cache, window of {sizes['window']}, {lh} heads on one key of {key}", times,
            int(seqs * seen * 2 * key * 2) if decode else 0, 0 if decode else 4.0 * tokens * lh * key * seen)
        # ---- placement ---------------------------------------------------------------------------------------------------
        inv_freq = torch.ones(d // 2, device=device)
        qkv = ops.Product(rand(tokens, (H + 2 * G) * d, scale=1.0), 1)
        times = _timed(lambda i: ops.rope_cache(qkv, positions, slot_map, inv_freq, d, cache, H, G, d, bf), 8, samples)
        row(f"{label}: rotation + cache write (Llama's)", times, tokens * (H * 2 + 2 * G) * d * 2 * 2)
        times = _timed(lambda i: ops.qkv_place(qkv, positions, slot_map, None, 0, cache, H, G, d, d, bf, q_temp=(0.1, 512.0)), 8, samples)
        row(f"{label}: placement of q, k, v with a query temperature", times, tokens * (H * 2 + 2 * G) * d * 2 * 2)
        qk = ops.Product(rand(tokens, (H + G) * d, scale=1.0), 1)
        q_norm, k_norm = rand(H * d, scale=1.0, dtype=f32), rand(G * d, scale=1.0, dtype=f32)
        times = _timed(lambda i: ops.qkv_place(qk, positions, slot_map, inv_freq, d, cache, H, G, d, d, bf, q_norm=q_norm, k_norm=k_norm,
                                               norm_eps=1e-5, values_are_keys=True), 8, samples)
        row(f"{label}: placement of q and k: norms over the whole projections, rotation, the projected keys as values", times,
            tokens * ((H + G) * d * 2 * 2 + G * d * 2))
        gate_cols = lh * lv
        fused = ops.Product(rand(tokens, lh * ld + rank + gate_cols, scale=1.0), 1)
        latent_norm = rand(rank, scale=1.0)
        times = _timed(lambda i: ops.latent_place(fused, positions, slot_map, None, latent_norm, 1e-5, latent_cache, lh, ld, 0, rank, bf,
                                                  wide_values=True, turn=0, extra_cols=gate_cols), 8, samples)
        row(f"{label}: latent placement (norm, cache write, queries apart)", times, tokens * (lh * ld * 2 + rank * 3) * 2)
        values = rand(tokens, gate_cols, scale=1.0)
        times = _timed(lambda i: ops.sigmoid_gate(values, fused, fused.cols - gate_cols), 8, samples)
        row(f"{label}: gate on the heads' results", times, tokens * gate_cols * 6)
        # ---- the residual of several streams ------------------------------------------------------------------------------
        streams = rand(count, tokens, width, scale=1.0, dtype=f32)
        update = ops.StreamUpdate(ops.Product(rand(tokens, width, scale=1.0), 1), rand(count, count, scale=0.3, dtype=f32),
                                  rand(count, scale=0.3, dtype=f32))
        read, norm_w = rand(count, scale=0.5, dtype=f32), rand(width, scale=1.0)
        times = _timed(lambda i: ops.stream_norm(streams, update, read, norm_w, 1e-5, bf), 8, samples)
        row(f"{label}: {count} streams take a result, are read and normed", times, tokens * width * (count * 8 + 2 + 2))
        times = _timed(lambda i: ops.stream_norm(streams, update, None, None, 0.0, bf, total=True), 8, samples)
        row(f"{label}: {count} streams take a result and are summed", times, tokens * width * (count * 8 + 2 + 4))
        residual = rand(tokens, width, scale=1.0, dtype=f32)
        times = _timed(lambda i: ops.add_rmsnorm(residual, update.product, norm_w, 1e-5, bf), 8, samples)
        row(f"{label}: add + norm (Llama's)", times, tokens * width * (4 + 4 + 2 + 2))
        # ---- the routed feed-forward --------------------------------------------------------------------------------------
        x = rand(tokens, width, scale=1.0)
        router, bias = rand(experts + 1, width), rand(experts + 1)
        times = _timed(lambda i: ops.few_outputs(x, router, bias, top=top, score="softmax_of_chosen", extra=1), 8, samples)
        row(f"{label}: router, softmax over the chosen {top} of {experts}, the shared expert's gate", times, (tokens + experts + 1) * width * 2)
        inter = experts * eff + sff
        scale = ops.few_outputs(x, router, bias, top=top, score="softmax_of_chosen", extra=1)
        gate_up = ops.Product(rand(tokens, 2 * inter, scale=1.0), 1)
        times = _timed(lambda i: ops.routed_gate(gate_up, scale, eff, bf, weigh="output", shared_scaled=True, gate="clamped_swish",
                                                 alpha=1.702, limit=7.0, shared_limit=7.0), 4, samples)
        row(f"{label}: clamped gate of the routed feed-forward, weighed results (all experts' columns)", times, tokens * inter * 6)
        dense_up = ops.Product(rand(tokens, 2 * ff, scale=1.0), 1)
        times = _timed(lambda i: ops.silu_mul(dense_up, bf, interleaved=True), 4, samples)
        row(f"{label}: SiLU gate (Llama's)", times, tokens * ff * 6)
        # ---- capped logits (the wanted rows: every row of a decode step, one of a prompt) ------------------------------
        logits = rand(tokens if decode else 1, vocab, scale=5.0, dtype=f32)
        times = _timed(lambda i: ops.softcap(logits, 30.0), 8, samples)
        row(f"{label}: capped logits", times, logits.numel() * 8)
    return rows

def bench_tugalix_kernels(sizes: dict, batch: int = 8, context: int = 2048, prompt: int = 2048, samples: int = 10, device="cuda:0",
                          hbm_gbs: float = 8000.0, mfma_tflops: float = 2500.0) -> list[dict]:
    """The kernels that the Tugalix decoder adds, each alone at a layer's sizes, for a decode step of `batch` requests at
    `context` positions and a prompt step of `prompt` tokens, each beside the like kernel of the closest model (the
    matrix memory's walk and its heads' norm of the memory layers at the same head sizes, the recurrent layers'
    convolution, Llama's add + norm, rotation and gate); every row carries the fraction of the roofline its bytes or
    flops reach (`frac`: of `hbm_gbs` for rows with bytes, of `mfma_tflops` for rows with flops).
    sizes: width, ff, llama_ff, heads, kv_heads, dim (the attention beside the token-shift mixing); ret_heads, ret_dim,
    ret_vdim; gla_heads, gla_dim, gla_vdim; shift_heads, shift_dim; rank; taps."""
    device = torch.device(device)
    torch.cuda.set_device(device)
    bf, f32 = torch.bfloat16, torch.float32
    width, ff, lff, taps, rank = sizes["width"], sizes["ff"], sizes["llama_ff"], sizes["taps"], sizes["rank"]
    lq, lkv, d = sizes["heads"], sizes["kv_heads"], sizes["dim"]
    rows = []

    def rand(*shape, scale=0.02, dtype=bf):
        return (torch.randn(shape, device=device, dtype=f32) * scale).to(dtype)

    def row(name, times, read_bytes=0, flops=0):
        entry = _row(name, times, read_bytes, flops)
        if read_bytes:
            entry["frac"] = round(entry["gbs"] / hbm_gbs, 3)
        elif flops:
            entry["frac"] = round(entry["tflops"] / mfma_tflops, 4)
        rows.append(entry)

    def ints(values):
        return torch.tensor(values, dtype=torch.int32, device=device)

    for label, tokens, seqs in ((f"decode b{batch}", batch, batch), (f"prompt {prompt}", prompt, 1)):
        if tokens <= 0:
            continue
        decode = seqs == tokens
        if decode:
            positions = torch.full((tokens,), context - 1, dtype=torch.int32, device=device)
            token_seq, seq_start = ints(list(range(tokens))), ints(list(range(tokens + 1)))
        else:
            positions = torch.arange(tokens, dtype=torch.int32, device=device)
            token_seq, seq_start = torch.zeros(tokens, dtype=torch.int32, device=device), ints([0, tokens])
        seq_slot = ints(list(range(seqs)))
        token_slot = seq_slot[token_seq.long()].contiguous()
        ctx = SimpleNamespace(max_new=1 if decode else tokens, token_seq=token_seq, token_slot=token_slot, seq_start=seq_start, seq_slot=seq_slot)
        # ---- the scans: state [dim x vdim] a head; a token costs 4 flops an element of S ---------------------------
        scans = (("retention", sizes["ret_heads"], sizes["ret_dim"], sizes["ret_vdim"], "head"),
                 ("gated linear attention", sizes["gla_heads"], sizes["gla_dim"], sizes["gla_vdim"], "channel"),
                 ("token-shift mixing", sizes["shift_heads"], sizes["shift_dim"], sizes["shift_dim"], "bonus"))
        for name, heads, dim, vdim, kind in scans:
            fused = ops.Product(rand(tokens, 2 * heads * dim + 2 * heads * vdim, scale=1.0, dtype=f32 if kind == "head" else bf), 1)
            state = torch.zeros((seqs, *ops.decay_scan_state_shape(heads, dim, vdim)), dtype=f32, device=device)
            options = {}
            if kind == "head":
                options["head_decay"] = torch.full((heads,), 0.97, dtype=f32, device=device)
            else:
                options["decay"] = torch.rand(tokens, heads * dim, device=device) * 0.1 + 0.9
            if kind == "bonus":
                options["bonus"] = rand(heads * dim, scale=1.0, dtype=f32)
            times = _timed(lambda i: ops.decay_scan((fused, 0), (fused, heads * dim), (fused, 2 * heads * dim), state, seq_start, seq_slot,
                                                    heads, dim, vdim, max_new=ctx.max_new, **options), 8, samples)
            state_bytes = seqs * heads * dim * vdim * 4 * 2
            row(f"{label}: scan of {name}, {heads} heads of {dim} x {vdim}", times, state_bytes if decode else 0,
                0 if decode else 4.0 * tokens * heads * dim * vdim)
            # the like kernel: the memory layers' walk at the same head sizes (it also carries a normaliser and a maximum)
            memory_in = ops.Product(rand(tokens, 2 * heads * dim + 2 * heads * vdim, scale=1.0), 1)
            gates = rand(tokens, 2 * heads, scale=1.0, dtype=f32) + 3.0
            memory = torch.zeros((seqs, *ops.mlstm_state_shape(heads, dim, vdim)), dtype=f32, device=device)
            times = _timed(lambda i: ops.mlstm_scan(memory_in, 0, heads * dim, 2 * heads * dim, gates, memory, seq_start, seq_slot, heads, dim,
                                                    vdim, 15.0, dim ** -0.5, max_new=ctx.max_new), 8, samples)
            row(f"{label}: matrix memory's walk at these sizes (the memory layers')", times, state_bytes if decode else 0,
                0 if decode else 4.0 * tokens * heads * dim * vdim)
            scanned = rand(tokens, heads * vdim, scale=1.0, dtype=f32)
            weight = rand(heads * vdim, scale=1.0)
            times = _timed(lambda i: ops.head_combine(scanned, heads, vdim, 1e-5, bf, weight=None if kind == "head" else weight, gate=fused,
                                                      gate_col=2 * heads * dim + heads * vdim, gate_kind="silu"), 8, samples)
            row(f"{label}: heads of {name}: norm and gate", times, tokens * heads * vdim * (4 + 2 + 2))
            if kind == "head":
                inv_freq = torch.ones(dim // 2, device=device)
                product = ops.Product(rand(tokens, 2 * heads * dim + 2 * heads * vdim, scale=1.0), 1)
                times = _timed(lambda i: ops.rotate_heads(product, 0, positions, inv_freq, dim, 2 * heads, heads, dim, 1.0, dim ** -0.5,
                                                          tail=heads * vdim), 8, samples)
                row(f"{label}: rotation of q and k on their way into the scan (floats out)", times, tokens * (2 * heads * dim + heads * vdim) * (2 + 4))
            else:
                low = rand(tokens, rank, scale=1.0, dtype=f32)
                up, bias = rand(heads * dim, rank, scale=0.3), rand(heads * dim, scale=1.0)
                times = _timed(lambda i: ops.low_rank_decay(low, up, bias, "sigmoid_root" if kind == "channel" else "exp_neg_exp", tau=16.0,
                                                            inner_tanh=kind == "bonus"), 8, samples)
                row(f"{label}: decays of {name} from rank {rank}", times, tokens * (rank * 4 + heads * dim * 4) + heads * dim * rank * 2)
        x = rand(tokens, width, scale=1.0)
        from .parts.linear import Linear
        down = Linear(rand(rank, width), None, bf)
        times = _timed(lambda i: down(x, out_dtype=f32), 8, samples)
        row(f"{label}: the decays' inner product, float sums ({rank} outputs)", times, (tokens + rank) * width * 2)
        gate_w = rand(rank, width)
        times = _timed(lambda i: ops.few_outputs(x, gate_w), 8, samples)
        row(f"{label}: a product of {rank} outputs with float sums (the memory layers' gates')", times, (tokens + rank) * width * 2)
        # ---- rotation + cache write of the attention beside the token-shift mixing is Llama's own kernel -------------
        # ---- around a sublayer -------------------------------------------------------------------------------------
        residual = rand(tokens, width, scale=1.0, dtype=f32)
        first, second = ops.Product(rand(tokens, width, scale=1.0), 1), ops.Product(rand(tokens, width, scale=1.0), 1)
        norm_w, norm_b = rand(width, scale=1.0), rand(width, scale=1.0)
        times = _timed(lambda i: ops.layer_norm(residual, first, norm_w, norm_b, 1e-5, f32), 8, samples)
        row(f"{label}: add + layer norm, floats out", times, tokens * width * (4 + 4 + 2 + 4))
        times = _timed(lambda i: ops.layer_norm(residual, ops.ScaledSum(first, 1.0, second, 1.0), norm_w, norm_b, 1e-5, f32), 8, samples)
        row(f"{label}: add of both sides + layer norm, floats out", times, tokens * width * (4 + 4 + 2 + 2 + 4))
        history = rand(6, tokens, width, scale=1.0, dtype=f32)
        mix = rand(4, scale=1.0)
        times = _timed(lambda i: ops.layer_norm(history[3], first, norm_w, norm_b, 1e-5, f32, history=history, history_count=4,
                                                history_weight=mix, mixed=history[4]), 8, samples)
        row(f"{label}: add + sum over four results + layer norm, floats out", times, tokens * width * (4 * 4 + 4 + 2 + 4 + 4))
        times = _timed(lambda i: ops.add_rmsnorm(residual, first, norm_w, 1e-5, bf), 8, samples)
        row(f"{label}: add + norm (Llama's)", times, tokens * width * (4 + 4 + 2 + 2))
        normed = rand(tokens, width, scale=1.0, dtype=f32)
        tap_w = rand(width, taps, scale=0.3)
        conv_state = torch.zeros(seqs, max(taps - 1, 1), width, dtype=f32, device=device)
        times = _timed(lambda i: ops.input_conv(normed, tap_w, conv_state, ctx, bf), 8, samples)
        row(f"{label}: h + conv(h), {taps} taps", times, tokens * width * (4 + 2) + (seqs * (taps - 1) * width * 8 if decode else 0))
        conv_in = ops.Product(rand(tokens, width, scale=1.0), 1)
        lru_state = torch.zeros(seqs, taps, width, dtype=f32, device=device)
        times = _timed(lambda i: ops.causal_conv(conv_in, 0, tap_w, None, lru_state, token_seq, token_slot, seq_start), 8, samples)
        row(f"{label}: convolution of {taps} taps (the recurrent layers')", times, tokens * width * (2 + 4) + (seqs * (taps - 1) * width * 8 if decode else 0))
        mu = torch.rand(5, width, device=device).to(bf)
        shift_state = torch.zeros(seqs, width, dtype=f32, device=device)
        times = _timed(lambda i: ops.token_shift(x, mu, shift_state, ctx), 8, samples)
        row(f"{label}: five blends with the token before", times, tokens * width * (2 + 5 * 2))
        pre = ops.Product(rand(tokens, ff, scale=1.0), 1)
        numbers = rand(2, scale=1.0)
        times = _timed(lambda i: ops.xielu(pre, numbers, bf), 4, samples)
        row(f"{label}: xIELU", times, tokens * ff * 4)
        dense_up = ops.Product(rand(tokens, 2 * lff, scale=1.0), 1)
        times = _timed(lambda i: ops.silu_mul(dense_up, bf, interleaved=True), 4, samples)
        row(f"{label}: SiLU gate (Llama's)", times, tokens * lff * 6)
    return rows
