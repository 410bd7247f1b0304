"""Python faces of the HIP kernels.

Every function checks on the host that operand shapes, types and index ranges are what the kernel
and its grid assume, raises `EngineError` when they are not, and only then launches on torch's
current stream.  Nothing here computes anything in torch: without the compiled library (and a
GPU) these functions fail.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

import torch

from .csrc import build as _build
from .errors import EngineError, ErrorCode, invalid_argument, invalid_shape

F32, BF16 = 0, 1
ROWS_MAX = 16          # the most rows the products take that fold in the layer's neighbouring arithmetic
ATTENTION_MAX_HEAD_DIM = 256   # the largest head size that both attention kernels take
GENERIC_TILED_MIN_TOKENS = 4   # a sequence's tokens in a step from which the plain attention shares its reads of the keys
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dtype: torch.dtype) -> int:
    if dtype not in _CODES:
        raise EngineError(ErrorCode.INVALID_DTYPE, f"kernels take float32 or bfloat16, not {dtype}")
    return _CODES[dtype]


def library() -> ctypes.CDLL:
    return _build.load()


def _ptr(tensor: torch.Tensor | None):
    return ctypes.c_void_p(tensor.data_ptr()) if tensor is not None else ctypes.c_void_p(0)


def _stream():
    # the current stream of the current device, by the accessors that cost no Python (a step of
    # prompt portions makes some two hundred launches, and torch.cuda.current_stream() alone took
    # a quarter of the time the host needs for them)
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def _check(status: int, what: str) -> None:
    if status == 0:
        return
    if status == -1:
        raise invalid_argument(f"{what}: the kernel does not take these sizes or types")
    raise EngineError(ErrorCode.HIP, f"{what}: the launch failed (status {status})")


def _device_tensor(tensor: torch.Tensor, name: str, dtype: torch.dtype | tuple | None = None) -> None:
    if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda:
        raise invalid_argument(f"{name} must be a tensor on the GPU")
    if not tensor.is_contiguous():
        raise invalid_argument(f"{name} must be contiguous")
    if dtype is not None:
        allowed = dtype if isinstance(dtype, tuple) else (dtype,)
        if tensor.dtype not in allowed:
            raise EngineError(ErrorCode.INVALID_DTYPE, f"{name} has dtype {tensor.dtype}, expected one of {allowed}")


@dataclass
class Product:
    """The result of a matrix product: [rows, cols], or `nsplit` float partial sums
    [nsplit, rows, cols] of a split-K kernel that the consumer adds up."""
    data: torch.Tensor
    nsplit: int = 1

    @property
    def rows(self) -> int:
        return self.data.shape[-2]

    @property
    def cols(self) -> int:
        return self.data.shape[-1]

    @property
    def split_stride(self) -> int:
        return self.rows * self.cols

    def dense(self, dtype: torch.dtype | None = None) -> torch.Tensor:
        """The summed result as one tensor (for parts that do not fuse the sum)."""
        if self.nsplit == 1:
            out = self.data.view(self.rows, self.cols)        # nothing to add up: no kernel runs
        else:
            out = self.data.view(self.nsplit, self.rows, self.cols).sum(0)
        return out if dtype is None or out.dtype == dtype else out.to(dtype)


@dataclass
class NormedDelta:
    """A sublayer's result that is normed before it joins the residual: the product, and the weight and
    eps of that RMS norm.  Whoever norms the residual next does both in one kernel (`norm_add_rmsnorm`)."""
    product: Product
    weight: torch.Tensor
    eps: float


def as_product(value) -> Product:
    if isinstance(value, Product):
        return value
    if isinstance(value, torch.Tensor) and value.dim() == 2:
        return Product(value.contiguous(), 1)
    if hasattr(value, "first_scale"):                     # a ScaledSum: added up here for whoever does not fuse it
        return Product(value.dense(torch.float32).contiguous(), 1)
    raise invalid_argument("a part must return a [tokens, width] tensor or a Product")


def _check_product(product: Product, name: str) -> None:
    _device_tensor(product.data, name, (torch.float32, torch.bfloat16))
    if product.nsplit < 1 or product.data.numel() != product.nsplit * product.rows * product.cols:
        raise invalid_shape(f"{name}: {product.nsplit} splits do not fit a tensor of shape {list(product.data.shape)}")
    if product.nsplit > 1 and product.data.dtype != torch.float32:
        raise EngineError(ErrorCode.INVALID_DTYPE, f"{name}: partial sums must be float32")


# ---------------------------------------------------------------------------------------------
def embed_gather(tokens: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """float32 residual[t, :] = table[tokens[t], :].  The caller has checked 0 <= token < vocab."""
    _device_tensor(tokens, "tokens", torch.int32)
    _device_tensor(table, "embedding table", (torch.float32, torch.bfloat16))
    if tokens.dim() != 1 or table.dim() != 2:
        raise invalid_shape("embed_gather takes tokens [T] and a table [vocab, hidden]")
    out = torch.empty((tokens.shape[0], table.shape[1]), dtype=torch.float32, device=table.device)
    _check(library().tlie_embed_gather(_ptr(tokens), _ptr(table), dtype_code(table.dtype), _ptr(out),
                                       tokens.shape[0], table.shape[1], _stream()), "embed_gather")
    return out


def add_rmsnorm(residual: torch.Tensor, delta: Product | None, weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: torch.Tensor | None = None, want_out: bool = True) -> torch.Tensor | None:
    """residual += delta (all rows, in place) and out = RMSNorm(residual) * weight.

    With `rows` (int32 indices) only those rows are normed, from residual + delta, and the
    residual is left as it was.  `delta` may be None (norm only)."""
    _device_tensor(residual, "residual", torch.float32)
    _device_tensor(weight, "norm weight", (torch.float32, torch.bfloat16))
    if residual.dim() != 2 or weight.shape != (residual.shape[1],):
        raise invalid_shape(f"add_rmsnorm: residual {list(residual.shape)} and weight {list(weight.shape)} do not fit")
    if not eps > 0.0:
        raise EngineError(ErrorCode.NUMERICAL, "RMSNorm requires a positive epsilon")
    tokens, hidden = residual.shape
    delta_code, nsplit, stride = F32, 1, 0
    if delta is not None:
        _check_product(delta, "delta")
        if (delta.rows, delta.cols) != (tokens, hidden):
            raise invalid_shape(f"add_rmsnorm: delta [{delta.rows}, {delta.cols}] does not fit residual {list(residual.shape)}")
        delta_code, nsplit, stride = dtype_code(delta.data.dtype), delta.nsplit, delta.split_stride
    count = tokens
    if rows is not None:
        _device_tensor(rows, "rows", torch.int32)
        count = rows.shape[0]
        if count == 0:
            return torch.empty((0, hidden), dtype=out_dtype, device=residual.device)
    out = torch.empty((count, hidden), dtype=out_dtype, device=residual.device) if want_out else None
    _check(library().tlie_add_rmsnorm(_ptr(residual), _ptr(delta.data if delta is not None else None), delta_code, nsplit,
                                      ctypes.c_longlong(stride), _ptr(weight), dtype_code(weight.dtype),
                                      ctypes.c_float(eps), _ptr(out), dtype_code(out_dtype), _ptr(rows), count, hidden,
                                      _stream()), "add_rmsnorm")
    return out


GATES = {"silu": 0, "clamped_swish": 1}


def silu_mul(gate_up: Product, out_dtype: torch.dtype, interleaved: bool = False, gate: str = "silu", alpha: float = 1.0,
             limit: float = 0.0) -> torch.Tensor:
    """out[t, i] = silu(gate[t, i]) * up[t, i], with gate_up = [gate | up] side by side or, interleaved,
    g0 u0 g1 u1 ...  gate "clamped_swish": g = min(gate, limit), u = clamp(up, -limit, limit),
    out = g * sigmoid(alpha * g) * (u + 1)."""
    _check_product(gate_up, "gate_up")
    if gate not in GATES:
        raise invalid_argument(f"silu_mul: unknown gate '{gate}'")
    if gate == "clamped_swish" and not limit > 0.0:
        raise invalid_argument("silu_mul: the clamped gate needs a positive limit")
    if gate_up.cols % 2 != 0:
        raise invalid_shape("silu_mul: the input holds gate and up side by side, its width must be even")
    rows, inter = gate_up.rows, gate_up.cols // 2
    out = torch.empty((rows, inter), dtype=out_dtype, device=gate_up.data.device)
    _check(library().tlie_silu_mul(_ptr(gate_up.data), dtype_code(gate_up.data.dtype), gate_up.nsplit,
                                   ctypes.c_longlong(gate_up.split_stride), _ptr(out), dtype_code(out_dtype), rows, inter,
                                   1 if interleaved else 0, GATES[gate], ctypes.c_float(alpha), ctypes.c_float(limit),
                                   _stream()), "silu_mul")
    return out


def _check_cache(cache: torch.Tensor, num_kv_heads: int, head_dim: int, what: str, value_dim: int | None = None,
                 value_heads: int | None = None) -> int:
    """cache: [pages, 2, nkv, page_size * d]; per page and kv head the keys lie as [row][dim] and
    the values transposed, [dim][row].  With a value size dv of its own a page is
    [nkv, page_size * (d + dv)] instead: the nkv planes of keys, then the nkv planes of values
    (the same order of bytes when dv = d).  With fewer value heads than key heads (nkv / nv key heads in a
    row read one value head) a page is [nv, page_size * (nkv / nv * d + dv)]: the nkv planes of keys, then
    the nv planes of values.  Returns the page size."""
    if value_heads is not None and value_heads != num_kv_heads:
        dv = head_dim if value_dim is None else value_dim
        if value_heads <= 0 or num_kv_heads % value_heads != 0:
            raise invalid_shape(f"{what}: {num_kv_heads} key heads do not share {value_heads} value heads evenly")
        per = num_kv_heads // value_heads * head_dim + dv
        if cache.dim() != 3 or cache.shape[1] != value_heads or cache.shape[2] % per != 0:
            raise invalid_shape(f"{what}: cache {list(cache.shape)} is not [pages, nv, page_size * (nkv / nv * d + dv)]")
        return cache.shape[2] // per
    if value_dim is None or value_dim == head_dim:
        if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[2] != num_kv_heads or cache.shape[3] % head_dim != 0:
            raise invalid_shape(f"{what}: cache {list(cache.shape)} is not [pages, 2, nkv, page_size * d]")
        return cache.shape[3] // head_dim
    if cache.dim() != 3 or cache.shape[1] != num_kv_heads or cache.shape[2] % (head_dim + value_dim) != 0:
        raise invalid_shape(f"{what}: cache {list(cache.shape)} is not [pages, nkv, page_size * (d + dv)]")
    return cache.shape[2] // (head_dim + value_dim)


def paired_rows(num_heads: int, num_kv_heads: int, head_dim: int, rot_dim: int) -> torch.Tensor:
    """The order in which the rows of a fused q/k/v weight are stored when rotation pairs are to sit
    side by side: within each q and k head, element i of the rotated part goes to 2i and element
    i + rot_dim / 2 to 2i + 1; everything else stays.  Returns the source row of each stored row."""
    half = rot_dim // 2
    inside = []
    for i in range(half):
        inside += [i, i + half]
    inside += list(range(rot_dim, head_dim))
    order = []
    for head in range(num_heads + num_kv_heads):
        order += [head * head_dim + e for e in inside]
    order += list(range((num_heads + num_kv_heads) * head_dim, (num_heads + 2 * num_kv_heads) * head_dim))
    return torch.tensor(order, dtype=torch.long)


def rope_cache(qkv: Product, positions: torch.Tensor, slot_map: torch.Tensor, inv_freq: torch.Tensor | None,
               rot_dim: int, cache: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
               act_dtype: torch.dtype, paired: bool = False) -> torch.Tensor:
    """Rotates q and k, returns q [T, nq * d], writes k and v into the cache rows of `slot_map`.
    paired: qkv's columns are in the order of `paired_rows`.

    slot_map[t] = page * page_size + row, or -1 to skip.  The slot map comes from the cache
    manager, which hands out only rows of pages it owns."""
    _check_product(qkv, "qkv")
    _device_tensor(positions, "positions", torch.int32)
    _device_tensor(slot_map, "slot_map", torch.int32)
    _device_tensor(cache, "cache", act_dtype)
    tokens = qkv.rows
    if qkv.cols != (num_heads + 2 * num_kv_heads) * head_dim:
        raise invalid_shape(f"rope_cache: qkv width {qkv.cols} is not (nq + 2 nkv) * d")
    if positions.shape != (tokens,) or slot_map.shape != (tokens,):
        raise invalid_shape("rope_cache: positions and slot_map need one entry per token")
    page_size = _check_cache(cache, num_kv_heads, head_dim, "rope_cache")
    if inv_freq is not None:
        _device_tensor(inv_freq, "inv_freq", torch.float32)
        if rot_dim % 2 != 0 or not 0 < rot_dim <= head_dim or inv_freq.shape != (rot_dim // 2,):
            raise invalid_shape("rope_cache: inv_freq needs rot_dim / 2 entries, rot_dim even and at most d")
    else:
        rot_dim = 0
    q_out = torch.empty((tokens, num_heads * head_dim), dtype=act_dtype, device=cache.device)
    _check(library().tlie_rope_cache(_ptr(qkv.data), dtype_code(qkv.data.dtype), qkv.nsplit,
                                     ctypes.c_longlong(qkv.split_stride), _ptr(positions), _ptr(slot_map), _ptr(inv_freq),
                                     rot_dim, _ptr(q_out), _ptr(cache), dtype_code(act_dtype), tokens, num_heads,
                                     num_kv_heads, head_dim, page_size, 1 if paired else 0, _stream()), "rope_cache")
    return q_out


def attention_generic(q: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor, token_seq: torch.Tensor,
                      positions: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                      window: int | None, scale: float, tiled: bool | int = False, seq_start: torch.Tensor | None = None,
                      min_tokens: int = GENERIC_TILED_MIN_TOKENS, value_dim: int | None = None, chunk: int | None = None,
                      sink: torch.Tensor | None = None, value_heads: int | None = None, float_out: bool = False,
                      softcap: float | None = None) -> torch.Tensor:
    """Causal attention of every token over its sequence's cached keys; any number of tokens per
    sequence.  block_table: [sequences, max_blocks] pages; token_seq[t]: the token's row of it.
    tiled 1 (True): the step's sequences bring several tokens each (consecutive in the step, at
    consecutive positions): neighbouring tokens then share each read of the keys (head sizes up to
    64; the result has the same bits either way).  tiled 2: both kernels are launched and every token
    is served by one of them: by the tiled one if its sequence brings `min_tokens` tokens or more
    (seq_start: the step's cumulative token counts [sequences + 1], on the device), by the plain one
    otherwise: for steps that mix portions of prompts with single tokens.
    value_dim: the size of a value head when it is not the key heads' (see `_check_cache`); the result is
    [tokens, nq * value_dim].  chunk: a token sees only the keys of its own chunk of so many positions
    (counted from position 0).  sink: float32 [nq], a number per head whose exponential joins the
    softmax's denominator.  value_heads: fewer value heads than key heads (num_kv_heads / value_heads key heads in
    a row read one value head; see `_check_cache`).  float_out: the result is float32 whatever q's type.
    softcap: a scaled score s enters the softmax as softcap * tanh(s / softcap)."""
    _device_tensor(q, "q", (torch.float32, torch.bfloat16))
    if softcap is not None and not float(softcap) > 0.0:
        raise invalid_argument("attention: a cap of the scores must be positive")
    value_dim = head_dim if value_dim is None else int(value_dim)
    value_heads = num_kv_heads if value_heads is None else int(value_heads)
    if sink is not None:
        _device_tensor(sink, "sink", torch.float32)
        if sink.shape != (num_heads,):
            raise invalid_shape("attention: the sink needs one entry per query head")
    if chunk is not None and int(chunk) <= 0:
        raise invalid_argument("attention: a chunk must be a positive count of positions")
    if not 0 < value_dim <= ATTENTION_MAX_HEAD_DIM:
        raise invalid_argument(f"attention: the plain kernel takes value heads of 1 to {ATTENTION_MAX_HEAD_DIM} dims")
    _device_tensor(cache, "cache", q.dtype)
    _device_tensor(block_table, "block_table", torch.int32)
    _device_tensor(token_seq, "token_seq", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    tokens = q.shape[0]
    if q.shape != (tokens, num_heads * head_dim):
        raise invalid_shape(f"attention: q {list(q.shape)} is not [tokens, nq * d]")
    page_size = _check_cache(cache, num_kv_heads, head_dim, "attention", value_dim, value_heads)
    if block_table.dim() != 2 or token_seq.shape != (tokens,) or positions.shape != (tokens,):
        raise invalid_shape("attention: block_table must be [sequences, max_blocks], token_seq and positions [tokens]")
    if num_heads % num_kv_heads != 0:
        raise invalid_shape("attention: the number of heads must be a multiple of the number of kv heads")
    tiled = int(tiled)
    if tiled == 2:
        _device_tensor(seq_start, "seq_start", torch.int32)
        if seq_start.dim() != 1 or seq_start.shape[0] != block_table.shape[0] + 1 or min_tokens < 1:
            raise invalid_shape("attention: seq_start needs one entry more than the block table has rows, min_tokens at least 1")
    elif tiled not in (0, 1):
        raise invalid_argument("attention: tiled is 0, 1 or 2")
    out = torch.empty((tokens, num_heads * value_dim), dtype=torch.float32 if float_out else q.dtype, device=q.device)
    _check(library().tlie_attention_generic(_ptr(q), _ptr(cache), dtype_code(q.dtype), _ptr(block_table),
                                            block_table.shape[1], _ptr(token_seq), _ptr(positions), _ptr(out), tokens,
                                            num_heads, num_kv_heads, head_dim, value_dim, page_size,
                                            int(window) if window else 0, int(chunk) if chunk else 0, _ptr(sink),
                                            ctypes.c_float(scale), tiled,
                                            _ptr(seq_start if tiled == 2 else None), int(min_tokens),
                                            num_kv_heads // value_heads, 1 if float_out else 0,
                                            ctypes.c_float(float(softcap) if softcap else 0.0), _stream()),
           "attention_generic")
    return out


def attention_generic_plan(ctx, head_dim: int, value_dim: int | None = None) -> int:
    """Which form of the plain attention kernel a step takes (the `tiled` of `attention_generic`): the
    one that shares each read of the keys among a sequence's tokens pays from a few tokens a
    sequence on, and costs dearly where a workgroup's 32 columns belong to many sequences of one
    token (it walks each one's context in turn).  A launched step is decided from its host arrays;
    a recorded step of portions, whose cut changes from replay to replay, launches both and lets
    each sequence's token count on the device decide."""
    if max(head_dim, value_dim or head_dim) > 64 or ctx.max_new < GENERIC_TILED_MIN_TOKENS:
        return 0
    if ctx.tile_owner is not None:
        return 2
    starts = ctx.host["seq_start"]
    counts = starts[1:] - starts[:-1]
    many = int((counts >= GENERIC_TILED_MIN_TOKENS).sum())
    return 1 if many == len(counts) else (2 if many else 0)


def norm_add_rmsnorm(residual: torch.Tensor, delta: Product, post_weight: torch.Tensor, post_eps: float,
                     weight: torch.Tensor | None, eps: float, out_dtype: torch.dtype,
                     rows: torch.Tensor | None = None) -> torch.Tensor | None:
    """residual += RMSNorm(delta) * post_weight (all rows, in place), then out = RMSNorm(residual) * weight:
    a sublayer's result is normed before it joins the residual, and the residual before the next
    sublayer, in one pass.  weight None: only the residual is brought up to date (returns None).  With
    `rows` only those rows are computed, and the residual is left as it was."""
    _device_tensor(residual, "residual", torch.float32)
    _check_product(delta, "delta")
    _device_tensor(post_weight, "post norm weight", (torch.float32, torch.bfloat16))
    tokens, hidden = residual.shape
    if (delta.rows, delta.cols) != (tokens, hidden) or post_weight.shape != (hidden,):
        raise invalid_shape(f"norm_add_rmsnorm: delta [{delta.rows}, {delta.cols}] or the weight do not fit residual {list(residual.shape)}")
    if weight is not None:
        _device_tensor(weight, "norm weight", post_weight.dtype)
        if weight.shape != (hidden,):
            raise invalid_shape("norm_add_rmsnorm: the norm's weight needs one entry per column")
    if not (post_eps > 0.0 and eps > 0.0):
        raise EngineError(ErrorCode.NUMERICAL, "RMSNorm requires a positive epsilon")
    count = tokens
    if rows is not None:
        _device_tensor(rows, "rows", torch.int32)
        count = rows.shape[0]
    out = torch.empty((count, hidden), dtype=out_dtype, device=residual.device) if weight is not None else None
    if count == 0:
        return out
    _check(library().tlie_norm_add_rmsnorm(_ptr(residual), _ptr(delta.data), dtype_code(delta.data.dtype), delta.nsplit,
                                           ctypes.c_longlong(delta.split_stride), _ptr(post_weight), ctypes.c_float(post_eps),
                                           _ptr(weight), dtype_code(post_weight.dtype), ctypes.c_float(eps), _ptr(out),
                                           dtype_code(out_dtype), _ptr(rows), count, hidden, _stream()), "norm_add_rmsnorm")
    return out


def qkv_place(qkv: Product, positions: torch.Tensor, slot_map: torch.Tensor | None, inv_freq: torch.Tensor | None,
              rot_dim: int, cache: torch.Tensor | None, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
              act_dtype: torch.dtype, value_heads: int | None = None, extra_cols: int = 0,
              q_norm: torch.Tensor | None = None, k_norm: torch.Tensor | None = None, norm_eps: float = 0.0,
              values_are_keys: bool = False, q_temp: tuple[float, float] | None = None) -> torch.Tensor:
    """`rope_cache` for any sizes: value heads of `value_dim` dims (a page is then nkv planes of keys and
    after them nkv planes of transposed values), and num_kv_heads 0 for a layer that reads another
    layer's cache: only its queries [T, nq * d] are rotated and returned, nothing is written.
    value_heads: fewer value heads than key heads (see `_check_cache`).  extra_cols: columns that the product
    has after q, k and v, which are someone else's to read.
    q_norm, k_norm (float32 [nq * d], [nkv * d]): all of a token's query columns together, and all of its key columns
    together, are RMS-normed (norm_eps inside the root) and multiplied by the weight before the rotation.
    values_are_keys: the product holds no value columns; a key head as projected, before norm and rotation, is also its
    value head (value_dim = head_dim).  q_temp (coef, every): a query at position p is multiplied by
    1 + coef * ln(floor((p + 1) / every) + 1)."""
    _check_product(qkv, "qkv")
    if values_are_keys and (value_dim != head_dim or (value_heads is not None and value_heads != num_kv_heads) or num_kv_heads == 0):
        raise invalid_shape("qkv_place: values that are the keys have the keys' heads and size")
    for name, weight, count in (("q_norm", q_norm, num_heads * head_dim), ("k_norm", k_norm, num_kv_heads * head_dim)):
        if weight is not None:
            _device_tensor(weight, name, torch.float32)
            if weight.shape != (count,) or not norm_eps > 0.0:
                raise invalid_shape(f"qkv_place: {name} needs {count} entries and a positive eps")
    if q_temp is not None and not float(q_temp[1]) > 0.0:
        raise invalid_argument("qkv_place: the query temperature's period must be positive")
    _device_tensor(positions, "positions", torch.int32)
    tokens = qkv.rows
    value_heads = num_kv_heads if value_heads is None else int(value_heads)
    if extra_cols < 0 or qkv.cols != (num_heads + num_kv_heads) * head_dim + (0 if values_are_keys else value_heads * value_dim) + extra_cols:
        raise invalid_shape(f"qkv_place: qkv width {qkv.cols} is not (nq + nkv) * d + nv * dv + {extra_cols}")
    if positions.shape != (tokens,):
        raise invalid_shape("qkv_place: positions need one entry per token")
    page_size = 1
    if num_kv_heads > 0:
        _device_tensor(slot_map, "slot_map", torch.int32)
        _device_tensor(cache, "cache", act_dtype)
        if slot_map.shape != (tokens,):
            raise invalid_shape("qkv_place: slot_map needs one entry per token")
        page_size = _check_cache(cache, num_kv_heads, head_dim, "qkv_place", value_dim, value_heads)
    if inv_freq is not None:
        _device_tensor(inv_freq, "inv_freq", torch.float32)
        if rot_dim % 2 != 0 or not 0 < rot_dim <= head_dim or inv_freq.shape != (rot_dim // 2,):
            raise invalid_shape("qkv_place: inv_freq needs rot_dim / 2 entries, rot_dim even and at most d")
    else:
        rot_dim = 0
    q_out = torch.empty((tokens, num_heads * head_dim), dtype=act_dtype, device=qkv.data.device)
    _check(library().tlie_qkv_place(_ptr(qkv.data), dtype_code(qkv.data.dtype), qkv.nsplit, ctypes.c_longlong(qkv.split_stride),
                                    _ptr(positions), _ptr(slot_map if num_kv_heads > 0 else None), _ptr(inv_freq), rot_dim,
                                    _ptr(q_out), _ptr(cache if num_kv_heads > 0 else None), dtype_code(act_dtype), tokens,
                                    num_heads, num_kv_heads, value_heads, head_dim, value_dim, page_size, qkv.cols,
                                    _ptr(q_norm), _ptr(k_norm), ctypes.c_float(norm_eps), 1 if values_are_keys else 0,
                                    ctypes.c_float(float(q_temp[0]) if q_temp else 0.0),
                                    ctypes.c_float(float(q_temp[1]) if q_temp else 0.0), _stream()),
           "qkv_place")
    return q_out


BLOCK_LINEAR_MANY_ROWS = 16    # rows beyond which the block-diagonal product goes to the matrix cores (where it can)


def block_linear(x: torch.Tensor, x_offset: int, x_row: int, x_block: int, weight_t: torch.Tensor, bias: torch.Tensor | None,
                 out: torch.Tensor, out_offset: int, out_row: int, out_block: int, rows: int,
                 weight: torch.Tensor | None = None) -> None:
    """Block-diagonal product: for each of weight_t's blocks b, rows of `inner` values that lie in the flat
    array x at x_offset + row * x_row + b * x_block are multiplied by weight_t[b] ([inner, outer], the
    block's matrix transposed) and, plus bias[b], written to the flat array `out` at out_offset + row *
    out_row + b * out_block.  Sums are float.
    weight: the same matrices as they are stored, [blocks, outer, inner], in bfloat16: with it a step of more than
    BLOCK_LINEAR_MANY_ROWS rows goes to the matrix cores (x, if float, is rounded to bfloat16 as an operand), when
    inner is a multiple of 32 and x's offset and strides are multiples of 8."""
    _device_tensor(x, "x", (torch.float32, torch.bfloat16))
    _device_tensor(weight_t, "weight", (torch.float32, torch.bfloat16))
    _device_tensor(out, "out", (torch.float32, torch.bfloat16))
    if weight_t.dim() != 3:
        raise invalid_shape("block_linear: the weight must be [blocks, inner, outer]")
    blocks, inner, outer = weight_t.shape
    if bias is not None:
        _device_tensor(bias, "bias", weight_t.dtype)
        if bias.shape != (blocks, outer):
            raise invalid_shape("block_linear: the bias must be [blocks, outer]")
    if rows <= 0:
        return
    if min(x_offset, x_row, x_block, out_offset, out_row, out_block) < 0:
        raise invalid_argument("block_linear: offsets and strides must not be negative")
    if x_offset + (rows - 1) * x_row + (blocks - 1) * x_block + inner > x.numel():
        raise invalid_shape("block_linear: the strides reach beyond x")
    if out_offset + (rows - 1) * out_row + (blocks - 1) * out_block + outer > out.numel():
        raise invalid_shape("block_linear: the strides reach beyond out")
    x_address = x.data_ptr() + x_offset * x.element_size()
    out_address = out.data_ptr() + out_offset * out.element_size()
    if (weight is not None and rows > BLOCK_LINEAR_MANY_ROWS and weight.dtype == torch.bfloat16 and inner % 32 == 0
            and x_offset % 8 == 0 and x_row % 8 == 0 and x_block % 8 == 0 and x_address % 32 == 0):
        _device_tensor(weight, "weight (as stored)", torch.bfloat16)
        if weight.shape != (blocks, outer, inner):
            raise invalid_shape("block_linear: the stored weight must be [blocks, outer, inner]")
        if bias is not None and bias.dtype != torch.bfloat16:
            raise EngineError(ErrorCode.INVALID_DTYPE, "block_linear: on the matrix cores the bias is bfloat16")
        _check(library().tlie_block_linear_mfma(ctypes.c_void_p(x_address), dtype_code(x.dtype), ctypes.c_longlong(x_row),
                                                ctypes.c_longlong(x_block), _ptr(weight), _ptr(bias), ctypes.c_void_p(out_address),
                                                dtype_code(out.dtype), ctypes.c_longlong(out_row), ctypes.c_longlong(out_block),
                                                rows, blocks, inner, outer, _stream()), "block_linear_mfma")
        return
    _check(library().tlie_block_linear(ctypes.c_void_p(x_address), dtype_code(x.dtype), ctypes.c_longlong(x_row),
                                       ctypes.c_longlong(x_block), _ptr(weight_t), dtype_code(weight_t.dtype), _ptr(bias),
                                       ctypes.c_void_p(out_address), dtype_code(out.dtype), ctypes.c_longlong(out_row),
                                       ctypes.c_longlong(out_block), rows, blocks, inner, outer, _stream()), "block_linear")


def latent_place(fused: Product, positions: torch.Tensor, slot_map: torch.Tensor, inv_freq: torch.Tensor | None,
                 norm_weight: torch.Tensor, eps: float, cache: torch.Tensor, heads: int, plain: int, rot: int, rank: int,
                 act_dtype: torch.dtype, wide_values: bool = False, turn: int | None = None,
                 extra_cols: int = 0) -> tuple[torch.Tensor, torch.Tensor]:
    """Latent attention between its first product and the attention kernel.  fused: [T, heads * (plain +
    rot) + rank + rot].  The rank dims are RMS-normed (weight, eps) and written to the cache rows of
    `slot_map` as keys [row][rank + rot] beside the rotated shared key part, and once more, transposed, as
    values; returns (q_plain [T, heads * plain], q_wide [T, heads, rank + rot] of which only each head's
    last rot dims, the rotated ones, are filled: the per-head product of q_plain fills the rest).
    wide_values: the value side of a page has rank + rot rows, as many as a key has dims (the cache is then
    [pages, 2, 1, page_size * (rank + rot)], what an attention kernel with one head size reads); its last rot
    rows are never written.  turn: how many of the rot dims are rotated (the first ones; default all), inv_freq
    then has turn / 2 entries.  extra_cols: columns that the product has after these, which are someone else's to read."""
    _check_product(fused, "fused")
    _device_tensor(positions, "positions", torch.int32)
    _device_tensor(slot_map, "slot_map", torch.int32)
    _device_tensor(cache, "cache", act_dtype)
    _device_tensor(norm_weight, "latent norm weight", (torch.float32, torch.bfloat16))
    tokens = fused.rows
    if extra_cols < 0 or fused.cols != heads * (plain + rot) + rank + rot + extra_cols or norm_weight.shape != (rank,):
        raise invalid_shape(f"latent_place: width {fused.cols} is not heads * (plain + rot) + rank + rot")
    if positions.shape != (tokens,) or slot_map.shape != (tokens,):
        raise invalid_shape("latent_place: positions and slot_map need one entry per token")
    turn = rot if turn is None else int(turn)
    if rot < 0 or not 0 <= turn <= rot or turn % 2 != 0 or (turn > 0 and (inv_freq is None or inv_freq.shape != (turn // 2,))):
        raise invalid_shape("latent_place: inv_freq needs one entry for every two rotated dims, an even number of them, at most rot")
    if inv_freq is not None:
        _device_tensor(inv_freq, "inv_freq", torch.float32)
    if not eps > 0.0:
        raise EngineError(ErrorCode.NUMERICAL, "RMSNorm requires a positive epsilon")
    page_size = _check_cache(cache, 1, rank + rot, "latent_place", rank + rot if wide_values else rank)
    q_plain = torch.empty((tokens, heads * plain), dtype=act_dtype, device=cache.device)
    q_wide = torch.empty((tokens, heads * (rank + rot)), dtype=act_dtype, device=cache.device)
    _check(library().tlie_latent_place(_ptr(fused.data), dtype_code(fused.data.dtype), fused.nsplit,
                                       ctypes.c_longlong(fused.split_stride), _ptr(positions), _ptr(slot_map), _ptr(inv_freq),
                                       _ptr(norm_weight), dtype_code(norm_weight.dtype), ctypes.c_float(eps), _ptr(q_plain),
                                       _ptr(q_wide), _ptr(cache), dtype_code(act_dtype), tokens, heads, plain, rot, turn, rank,
                                       rank + rot if wide_values else rank, page_size, fused.cols, _stream()), "latent_place")
    return q_plain, q_wide


def causal_conv(fused: Product, x_col: int, taps: torch.Tensor, bias: torch.Tensor | None, state: torch.Tensor,
                token_seq: torch.Tensor, token_slot: torch.Tensor, seq_start: torch.Tensor) -> torch.Tensor:
    """A causal convolution per channel over each sequence's tokens of the step: columns x_col .. x_col +
    channels - 1 of `fused` are its inputs, taps [channels, n] (the last tap is the current token's), what came
    before the step is read from state [slots, n, channels] (rows 0 .. n-2: the last inputs, oldest first).
    Returns float32 [T, channels]; rows of tokens whose slot is negative are left unwritten."""
    _check_product(fused, "fused")
    _device_tensor(taps, "taps", (torch.float32, torch.bfloat16))
    _device_tensor(state, "state", torch.float32)
    for name, tensor in (("token_seq", token_seq), ("token_slot", token_slot), ("seq_start", seq_start)):
        _device_tensor(tensor, name, torch.int32)
    if taps.dim() != 2:
        raise invalid_shape("causal_conv: taps must be [channels, n]")
    channels, count = taps.shape
    tokens = fused.rows
    if bias is not None:
        _device_tensor(bias, "bias", taps.dtype)
        if bias.shape != (channels,):
            raise invalid_shape("causal_conv: the bias needs one entry per channel")
    if state.dim() != 3 or state.shape[1:] != (count, channels) or not 0 <= x_col <= fused.cols - channels:
        raise invalid_shape(f"causal_conv: state {list(state.shape)} is not [slots, {count}, {channels}], or the columns do not fit")
    if token_seq.shape != (tokens,) or token_slot.shape != (tokens,) or seq_start.dim() != 1:
        raise invalid_shape("causal_conv: token_seq and token_slot need one entry per token")
    u = torch.empty((tokens, channels), dtype=torch.float32, device=state.device)
    _check(library().tlie_causal_conv(_ptr(fused.data), dtype_code(fused.data.dtype), fused.nsplit,
                                      ctypes.c_longlong(fused.split_stride), fused.cols, x_col, _ptr(taps), _ptr(bias),
                                      dtype_code(taps.dtype), _ptr(state), _ptr(token_seq), _ptr(token_slot), _ptr(seq_start),
                                      _ptr(u), tokens, channels, count, _stream()), "causal_conv")
    return u


RECURRENCE_SLICE = 32          # tokens of a slice of the sliced recurrence (the kernel's kSlice)
RECURRENCE_SLICED_FROM = 64    # tokens a sequence brings from which the sliced form pays (three launches' worth of work)


def gated_recurrence(fused: Product, x_col: int, y_col: int, u: torch.Tensor, gates: torch.Tensor, lam: torch.Tensor,
                     decay: float, state: torch.Tensor, seq_start: torch.Tensor, seq_slot: torch.Tensor, block_width: int,
                     out_dtype: torch.dtype, max_new: int = 1) -> torch.Tensor:
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with a_t = exp(-decay * r_t * softplus(lam)), r and i the
    sigmoids of `gates` [T, blocks, 2 * block_width] (a block's r before its i), per channel and sequence,
    from and to row n-1 of state [slots, n, channels]; out = S * gelu_tanh(y), y in columns y_col .. of
    `fused`; the state's other rows get the step's last inputs of the convolution (columns x_col ..).
    Sequences whose slot is negative are skipped.  max_new: the most tokens any sequence brings in this step
    (the caller knows it on the host); beyond RECURRENCE_SLICED_FROM the sequences' tokens are taken in slices
    that run side by side (each from the carry that the slices before it leave), else a thread walks a
    sequence's tokens in order."""
    _check_product(fused, "fused")
    _device_tensor(u, "u", torch.float32)
    _device_tensor(gates, "gates", torch.float32)
    _device_tensor(lam, "lambda", (torch.float32, torch.bfloat16))
    _device_tensor(state, "state", torch.float32)
    _device_tensor(seq_start, "seq_start", torch.int32)
    _device_tensor(seq_slot, "seq_slot", torch.int32)
    tokens, channels = u.shape
    seqs = seq_slot.shape[0]
    if (fused.rows != tokens or gates.numel() != tokens * 2 * channels or lam.shape != (channels,) or state.dim() != 3
            or state.shape[2] != channels or seq_start.shape != (seqs + 1,) or block_width <= 0 or channels % block_width != 0):
        raise invalid_shape("gated_recurrence: the operands do not fit each other")
    if not (0 <= x_col <= fused.cols - channels and 0 <= y_col <= fused.cols - channels):
        raise invalid_shape("gated_recurrence: the columns do not fit the product")
    out = torch.empty((tokens, channels), dtype=out_dtype, device=u.device)
    slices, parts = 0, None
    if max_new > RECURRENCE_SLICED_FROM:
        slices = (min(int(max_new), tokens) + RECURRENCE_SLICE - 1) // RECURRENCE_SLICE
        parts = torch.empty((seqs, 2 * slices + 1, channels), dtype=torch.float32, device=u.device)
    _check(library().tlie_gated_recurrence(_ptr(fused.data), dtype_code(fused.data.dtype), fused.nsplit,
                                           ctypes.c_longlong(fused.split_stride), fused.cols, x_col, y_col, _ptr(u), _ptr(gates),
                                           _ptr(lam), dtype_code(lam.dtype), ctypes.c_float(decay), _ptr(state), _ptr(seq_start),
                                           _ptr(seq_slot), _ptr(out), dtype_code(out_dtype), seqs, channels, block_width,
                                           state.shape[1], slices, _ptr(parts), _stream()), "gated_recurrence")
    return out


HEAD_GATES = {"sigmoid": 0, "silu": 1}      # what a head's gate becomes: sigmoid(z), or z * sigmoid(z)


def head_combine(a: torch.Tensor, heads: int, value_dim: int, eps: float, out_dtype: torch.dtype, pair_group: int = 0,
                 pair_lambda: float = 0.0, weight: torch.Tensor | None = None, mult: float = 1.0,
                 gate: Product | None = None, gate_col: int = 0, parts: int = 1, gate_kind: str = "sigmoid") -> torch.Tensor:
    """Each head's result normed by itself, on its way to the output product:
    out[t, h, :] = o / sqrt(mean(o^2) + eps) * weight[h] * mult * f(gate[t, h]) (f: `gate_kind`), with o = a[t, h] or, for two maps
    of attention a head (pair_group > 0: the query heads of one key head lie side by side in `a`, pair_group of them,
    first all first maps' key heads ... see the kernel), o = first - pair_lambda * second.  a: float32
    [tokens, heads (or 2 * heads) * value_dim]; weight (or None): [heads * value_dim]; gate (or None): a product whose
    columns gate_col .. gate_col + heads * value_dim hold the gate's pre-activations.  parts > 1 (with pair_group): a
    map's result lies in `parts` pieces of value_dim / parts dims, each a head of its own of the attention kernel: the
    pieces of a key head's query heads follow each other piece by piece (key head, piece, query head of the key head)."""
    _device_tensor(a, "a", torch.float32)
    if parts < 1 or value_dim % parts != 0 or (parts > 1 and pair_group <= 0):
        raise invalid_argument("head_combine: the pieces of a result must divide the value size (and go with two maps)")
    maps = 2 if pair_group > 0 else 1
    if a.dim() != 2 or a.shape[1] != maps * heads * value_dim:
        raise invalid_shape(f"head_combine: a {list(a.shape)} is not [tokens, {maps} * heads * value_dim]")
    if pair_group < 0 or (pair_group > 0 and heads % pair_group != 0):
        raise invalid_shape("head_combine: the heads of a key head must divide the heads")
    if not eps > 0.0:
        raise EngineError(ErrorCode.NUMERICAL, "a norm requires a positive epsilon")
    tokens = a.shape[0]
    weight_code = F32
    if weight is not None:
        _device_tensor(weight, "weight", (torch.float32, torch.bfloat16))
        if weight.shape != (heads * value_dim,):
            raise invalid_shape("head_combine: the weight needs one entry per head and dim")
        weight_code = dtype_code(weight.dtype)
    gate_code, gate_nsplit, gate_stride, gate_row = F32, 1, 0, 0
    if gate is not None:
        _check_product(gate, "gate")
        if gate.rows != tokens or gate_col < 0 or gate_col + heads * value_dim > gate.cols:
            raise invalid_shape("head_combine: the gate's columns do not lie in the product")
        gate_code, gate_nsplit, gate_stride, gate_row = dtype_code(gate.data.dtype), gate.nsplit, gate.split_stride, gate.cols
    out = torch.empty((tokens, heads * value_dim), dtype=out_dtype, device=a.device)
    if tokens == 0:
        return out
    _check(library().tlie_head_combine(_ptr(a), tokens, heads, value_dim, pair_group, int(parts), ctypes.c_float(pair_lambda),
                                       ctypes.c_float(eps), _ptr(weight), weight_code, ctypes.c_float(mult),
                                       _ptr(gate.data if gate is not None else None), gate_code, gate_nsplit,
                                       ctypes.c_longlong(gate_stride), gate_row, gate_col, HEAD_GATES[gate_kind], _ptr(out), dtype_code(out_dtype),
                                       _stream()), "head_combine")
    return out


MLSTM_MAX_DIM = 256            # the largest query/key size of a head that the matrix-memory kernel keeps in registers
MLSTM_SLICE = 32               # tokens of a slice of the sliced walk (the kernel's kMlstmSlice)
MLSTM_SLICED_FROM = 96         # tokens a sequence brings from which the sliced walk pays (two walks of a slice and a carry)


def mlstm_state_shape(heads: int, dim: int, value_dim: int) -> tuple[int, ...]:
    """A request's state row for `mlstm_scan`: per head and tile of 64 value columns, S as [dim][64], n and m."""
    return (heads, (value_dim + 63) // 64, dim * 64 + dim + 1)


def mlstm_scan(fused: Product, q_col: int, k_col: int, v_col: int, gates: torch.Tensor, state: torch.Tensor,
               seq_start: torch.Tensor, seq_slot: torch.Tensor, heads: int, dim: int, value_dim: int, cap: float,
               q_scale: float, max_new: int = 1) -> torch.Tensor:
    """The matrix memory of an mLSTM layer over the step's tokens, sequence by sequence (see csrc/mlstm.hip): reads
    q, k, v from the product's columns, the gates' pre-activations from `gates` (float32 [tokens, 2 * heads]: input
    gates, then forget gates), carries `state` (float32 [slots, *mlstm_state_shape]) for sequences whose slot is not
    negative, and returns float32 [tokens, heads * value_dim], the heads' results before their norm.  max_new: the
    most tokens any sequence brings in this step (the caller knows it on the host); from MLSTM_SLICED_FROM on the
    sequences' tokens are taken in slices of MLSTM_SLICE that run side by side, each from the start that the slices
    before it leave; else every sequence's tokens are walked in order."""
    _check_product(fused, "fused")
    _device_tensor(gates, "gates", torch.float32)
    _device_tensor(state, "state", torch.float32)
    _device_tensor(seq_start, "seq_start", torch.int32)
    _device_tensor(seq_slot, "seq_slot", torch.int32)
    tokens = fused.rows
    if not 0 < dim <= MLSTM_MAX_DIM or heads <= 0 or value_dim <= 0:
        raise invalid_argument(f"mlstm_scan: heads of 1 to {MLSTM_MAX_DIM} query dims")
    if gates.shape != (tokens, 2 * heads):
        raise invalid_shape("mlstm_scan: the gates need two numbers a head and token")
    if state.dim() != 4 or tuple(state.shape[1:]) != mlstm_state_shape(heads, dim, value_dim):
        raise invalid_shape(f"mlstm_scan: state {list(state.shape)} is not [slots, {mlstm_state_shape(heads, dim, value_dim)}]")
    sequences = seq_slot.shape[0]
    if seq_start.shape != (sequences + 1,):
        raise invalid_shape("mlstm_scan: seq_start needs one entry more than there are sequences")
    for col, size in ((q_col, heads * dim), (k_col, heads * dim), (v_col, heads * value_dim)):
        if col < 0 or col + size > fused.cols:
            raise invalid_shape("mlstm_scan: q, k or v do not lie in the product's columns")
    out = torch.empty((tokens, heads * value_dim), dtype=torch.float32, device=state.device)
    if tokens == 0 or sequences == 0:
        return out
    values = torch.empty((tokens, heads, 4), dtype=torch.float32, device=state.device)
    slices, parts = 0, None
    if max_new >= MLSTM_SLICED_FROM:
        slices = (min(int(max_new), tokens) + MLSTM_SLICE - 1) // MLSTM_SLICE
        parts = torch.empty((sequences, slices, *state.shape[1:]), dtype=torch.float32, device=state.device)
    _check(library().tlie_mlstm_scan(_ptr(fused.data), dtype_code(fused.data.dtype), fused.nsplit,
                                     ctypes.c_longlong(fused.split_stride), fused.cols, q_col, k_col, v_col, _ptr(gates),
                                     _ptr(values), _ptr(state), _ptr(seq_start), _ptr(seq_slot), _ptr(out), sequences, heads,
                                     dim, value_dim, ctypes.c_float(cap), ctypes.c_float(q_scale), slices, _ptr(parts),
                                     _stream()), "mlstm_scan")
    return out


@dataclass
class ScaledSum:
    """What a mixer of two branches hands on: first * first_scale + second * second_scale, not added up yet.  A norm
    that knows it (`layer_norm`) adds both into the residual in its own kernel; anyone else asks for `dense()`."""
    first: Product
    first_scale: float
    second: Product
    second_scale: float

    def dense(self, dtype: torch.dtype | None = None) -> torch.Tensor:
        out = self.first.dense(torch.float32) * self.first_scale + self.second.dense(torch.float32) * self.second_scale
        return out if dtype is None else out.to(dtype)


def layer_norm(residual: torch.Tensor, delta, weight: torch.Tensor | None, bias: torch.Tensor | None, eps: float,
               out_dtype: torch.dtype, rows: torch.Tensor | None = None, history: torch.Tensor | None = None,
               history_count: int = 0, history_weight: torch.Tensor | None = None, mixed: torch.Tensor | None = None,
               want_out: bool = True) -> torch.Tensor | None:
    """residual += delta (a Product, a ScaledSum or None; all rows, in place), then out = (x - mean) / sqrt(var + eps)
    * weight + bias of every row, means and variances float.  With `history` (float32 [entries, tokens, hidden] of which
    the first history_count are read, the last of them being `residual` itself) what is normed is the weighted sum
    sum_j history_weight[j] * history[j], which is also written to `mixed`.  With `rows` (int32 indices) only those
    rows are normed and nothing but the result is written.  want_out False: only the sums."""
    _device_tensor(residual, "residual", torch.float32)
    if residual.dim() != 2:
        raise invalid_shape("layer_norm: the residual is [tokens, hidden]")
    tokens, hidden = residual.shape
    if hidden > 16000:
        raise invalid_argument("layer_norm: rows of at most 16000 values")
    w_code = F32
    if want_out:
        _device_tensor(weight, "norm weight", (torch.float32, torch.bfloat16))
        w_code = dtype_code(weight.dtype)
        if weight.shape != (hidden,) or (bias is not None and (bias.shape != (hidden,) or bias.dtype != weight.dtype)):
            raise invalid_shape("layer_norm: weight and bias need one entry per column, of one type")
        if not eps > 0.0:
            raise EngineError(ErrorCode.NUMERICAL, "a norm requires a positive epsilon")
    parts = []
    if isinstance(delta, ScaledSum):
        parts = [(delta.first, delta.first_scale), (delta.second, delta.second_scale)]
    elif delta is not None:
        parts = [(as_product(delta), 1.0)]
    for product, _ in parts:
        _check_product(product, "delta")
        if (product.rows, product.cols) != (tokens, hidden):
            raise invalid_shape(f"layer_norm: delta [{product.rows}, {product.cols}] does not fit residual {list(residual.shape)}")
    while len(parts) < 2:
        parts.append((None, 0.0))
    if history_count > 0:
        _device_tensor(history, "history", torch.float32)
        _device_tensor(history_weight, "history weight", (torch.float32, torch.bfloat16))
        if want_out and history_weight.dtype != weight.dtype:
            raise invalid_shape("layer_norm: the history's weights are of the norm's type")
        w_code = dtype_code(history_weight.dtype)
        if (history.dim() != 3 or tuple(history.shape[1:]) != (tokens, hidden) or history_count > history.shape[0]
                or history_weight.shape != (history_count,)
                or history[history_count - 1].data_ptr() != residual.data_ptr()):
            raise invalid_shape("layer_norm: the history is [entries, tokens, hidden], its last entry read the residual itself")
        if rows is None:
            _device_tensor(mixed, "mixed", torch.float32)
            if mixed.shape != residual.shape:
                raise invalid_shape("layer_norm: the weighted sum has the residual's shape")
    count = tokens
    if rows is not None:
        _device_tensor(rows, "rows", torch.int32)
        count = rows.shape[0]
    out = torch.empty((count, hidden), dtype=out_dtype, device=residual.device) if want_out else None
    if count == 0 or tokens == 0:
        return out

    def code(product):
        return dtype_code(product.data.dtype) if product is not None else F32
    (d1, s1), (d2, s2) = parts
    _check(library().tlie_layer_norm(
        _ptr(residual), _ptr(d1.data if d1 is not None else None), code(d1), d1.nsplit if d1 is not None else 1,
        ctypes.c_longlong(d1.split_stride if d1 is not None else 0), ctypes.c_float(s1),
        _ptr(d2.data if d2 is not None else None), code(d2), d2.nsplit if d2 is not None else 1,
        ctypes.c_longlong(d2.split_stride if d2 is not None else 0), ctypes.c_float(s2),
        _ptr(history if history_count > 0 else None), ctypes.c_longlong(tokens * hidden), int(history_count),
        _ptr(history_weight if history_count > 0 else None), _ptr(mixed if history_count > 0 and rows is None else None),
        _ptr(weight if want_out else None), _ptr(bias if want_out else None), w_code, ctypes.c_float(eps if want_out else 1.0),
        _ptr(out), dtype_code(out_dtype), _ptr(rows), count, hidden, _stream()), "layer_norm")
    return out


INPUT_CONV_MAX_TAPS = 8


def input_conv(h: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, ctx, out_dtype: torch.dtype) -> torch.Tensor:
    """out = h + conv(h): a causal convolution per channel over each sequence's tokens of the step.  h: float32
    [tokens, channels]; taps [channels, n], tap j weighs the input n - 1 - j tokens back; state: float32
    [slots, max(n - 1, 1), channels] (the slots may lie apart: a part of a wider area), a request's last n - 1 inputs, oldest first, read for what came before the step and
    brought up to the step's last token.  Rows of tokens whose slot is negative are left unwritten."""
    _device_tensor(h, "h", torch.float32)
    _device_tensor(taps, "taps", (torch.float32, torch.bfloat16))
    if not isinstance(state, torch.Tensor) or not state.is_cuda or state.dtype != torch.float32:
        raise invalid_argument("input_conv: the state is a float32 tensor on the GPU")
    if h.dim() != 2 or taps.dim() != 2 or taps.shape[0] != h.shape[1] or not 1 <= taps.shape[1] <= INPUT_CONV_MAX_TAPS:
        raise invalid_shape(f"input_conv: h {list(h.shape)} and taps {list(taps.shape)} do not fit (1 to {INPUT_CONV_MAX_TAPS} taps)")
    tokens, channels = h.shape
    count = taps.shape[1]
    if state.dim() != 3 or tuple(state.shape[1:]) != (max(count - 1, 1), channels) or state.stride()[1:] != (channels, 1):
        raise invalid_shape(f"input_conv: state {list(state.shape)} is not [slots, {max(count - 1, 1)}, {channels}] with rows side by side")
    sequences = ctx.seq_slot.shape[0]
    if ctx.token_seq.shape != (tokens,) or ctx.token_slot.shape != (tokens,) or ctx.seq_start.shape != (sequences + 1,):
        raise invalid_shape("input_conv: the step's arrays do not fit the tokens")
    out = torch.empty((tokens, channels), dtype=out_dtype, device=h.device)
    if tokens == 0 or sequences == 0:
        return out
    _check(library().tlie_input_conv(_ptr(h), _ptr(taps), dtype_code(taps.dtype), _ptr(state), _ptr(ctx.token_seq),
                                     _ptr(ctx.token_slot), _ptr(ctx.seq_start), _ptr(ctx.seq_slot), _ptr(out),
                                     dtype_code(out_dtype), tokens, sequences, channels, count,
                                     ctypes.c_longlong(state.stride(0)), _stream()), "input_conv")
    return out


def token_shift(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, ctx) -> torch.Tensor:
    """out[m, t] = x_t + (x_(t-1) - x_t) * mu[m]: blends of a token's input with that of the token before it in its
    sequence (zeros before the first).  x: [tokens, width] in the activation type; mu: [mixes, width]; state: float32
    [slots, width], the last token's input of the step before, read and brought up to date.  Returns [mixes, tokens, width]."""
    _device_tensor(x, "x", (torch.float32, torch.bfloat16))
    _device_tensor(mu, "mu", (torch.float32, torch.bfloat16))
    if not isinstance(state, torch.Tensor) or not state.is_cuda or state.dtype != torch.float32:
        raise invalid_argument("token_shift: the state is a float32 tensor on the GPU")
    if (x.dim() != 2 or mu.dim() != 2 or mu.shape[1] != x.shape[1] or state.dim() != 2 or state.shape[1] != x.shape[1]
            or state.stride(1) != 1):
        raise invalid_shape("token_shift: x [tokens, width], mu [mixes, width], state [slots, width] (the slots may lie apart)")
    tokens, width = x.shape
    sequences = ctx.seq_slot.shape[0]
    if ctx.token_seq.shape != (tokens,) or ctx.token_slot.shape != (tokens,) or ctx.seq_start.shape != (sequences + 1,):
        raise invalid_shape("token_shift: the step's arrays do not fit the tokens")
    out = torch.empty((mu.shape[0], tokens, width), dtype=x.dtype, device=x.device)
    if tokens == 0 or sequences == 0:
        return out
    _check(library().tlie_token_shift(_ptr(x), dtype_code(x.dtype), _ptr(mu), dtype_code(mu.dtype), _ptr(state),
                                      _ptr(ctx.token_seq), _ptr(ctx.token_slot), _ptr(ctx.seq_start), _ptr(ctx.seq_slot),
                                      _ptr(out), tokens, sequences, width, mu.shape[0], ctypes.c_longlong(state.stride(0)),
                                      _stream()), "token_shift")
    return out


def xielu(pre: Product, numbers: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """softplus(p) z^2 + z / 2 for z > 0, (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2 otherwise, (p, q) = numbers."""
    _check_product(pre, "pre")
    _device_tensor(numbers, "numbers", (torch.float32, torch.bfloat16))
    if numbers.shape != (2,):
        raise invalid_shape("xielu: two numbers")
    out = torch.empty((pre.rows, pre.cols), dtype=out_dtype, device=pre.data.device)
    if out.numel() == 0:
        return out
    _check(library().tlie_xielu(_ptr(pre.data), dtype_code(pre.data.dtype), pre.nsplit, ctypes.c_longlong(pre.split_stride),
                                _ptr(numbers), dtype_code(numbers.dtype), _ptr(out), dtype_code(out_dtype),
                                ctypes.c_longlong(pre.rows * pre.cols), _stream()), "xielu")
    return out


def rotate_heads(fused: Product, col: int, positions: torch.Tensor, inv_freq: torch.Tensor | None, rot_dim: int, heads: int,
                 heads_a: int, dim: int, scale_a: float, scale_b: float, tail: int = 0) -> torch.Tensor:
    """Columns col .. of a product as floats on their way into a scan: `heads` heads of `dim` whose first rot_dim dims
    turn by the token's position (dim i with dim i + rot_dim / 2, angle position * inv_freq[i]), the first heads_a of
    them times scale_a afterwards and the others times scale_b, and `tail` more columns as they are."""
    _check_product(fused, "fused")
    _device_tensor(positions, "positions", torch.int32)
    if rot_dim > 0:
        _device_tensor(inv_freq, "inv_freq", torch.float32)
        if inv_freq.shape != (rot_dim // 2,):
            raise invalid_shape("rotate_heads: one frequency a pair")
    if (rot_dim < 0 or rot_dim % 2 or rot_dim > dim or col < 0 or tail < 0 or col + heads * dim + tail > fused.cols
            or positions.shape != (fused.rows,)):
        raise invalid_shape("rotate_heads: the heads do not lie in the product's columns")
    out = torch.empty((fused.rows, heads * dim + tail), dtype=torch.float32, device=fused.data.device)
    if fused.rows == 0:
        return out
    _check(library().tlie_rotate_heads(_ptr(fused.data), dtype_code(fused.data.dtype), fused.nsplit,
                                       ctypes.c_longlong(fused.split_stride), fused.cols, int(col), _ptr(positions),
                                       _ptr(inv_freq if rot_dim > 0 else None), int(rot_dim), heads, heads_a, dim,
                                       ctypes.c_float(scale_a), ctypes.c_float(scale_b), int(tail), _ptr(out), fused.rows,
                                       _stream()), "rotate_heads")
    return out


LOW_RANK_DECAYS = {"sigmoid_root": 0, "exp_neg_exp": 1}


def low_rank_decay(low, weight: torch.Tensor, bias: torch.Tensor | None, kind: str, tau: float = 1.0,
                   inner_tanh: bool = False) -> torch.Tensor:
    """Decays per token and channel from a low-rank product: z = bias + weight . f(low) (f: tanh or the identity), then
    "sigmoid_root": sigmoid(z)^(1 / tau); "exp_neg_exp": exp(-exp(z)).  low: a float32 product [tokens, rank] (a tensor,
    or a `Product` of float partial sums); weight [channels, rank].  Float throughout; returns float32 [tokens, channels]."""
    low = as_product(low)
    _check_product(low, "low")
    _device_tensor(weight, "weight", (torch.float32, torch.bfloat16))
    if low.data.dtype != torch.float32 or weight.dim() != 2 or weight.shape[1] != low.cols or low.cols > 1024:
        raise invalid_shape("low_rank_decay: low float32 [tokens, rank], weight [channels, rank], rank up to 1024")
    if bias is not None:
        _device_tensor(bias, "bias", weight.dtype)
        if bias.shape != (weight.shape[0],):
            raise invalid_shape("low_rank_decay: one bias a channel")
    if kind not in LOW_RANK_DECAYS or (kind == "sigmoid_root" and not tau > 0.0):
        raise invalid_argument("low_rank_decay: an unknown kind, or a root that is not positive")
    out = torch.empty((low.rows, weight.shape[0]), dtype=torch.float32, device=low.data.device)
    if low.rows == 0:
        return out
    _check(library().tlie_low_rank_decay(_ptr(low.data), low.nsplit, ctypes.c_longlong(low.split_stride), int(inner_tanh), _ptr(weight),
                                         _ptr(bias), dtype_code(weight.dtype), LOW_RANK_DECAYS[kind], ctypes.c_float(tau), _ptr(out),
                                         low.rows, weight.shape[0], low.cols, _stream()), "low_rank_decay")
    return out


SCAN_MAX_DIM = 256             # the largest query/key size of a head that the scan keeps in registers
SCAN_SLICE = 32                # tokens of a slice of the sliced walk (the kernel's kScanSlice)
SCAN_SLICED_FROM = 96          # tokens a sequence brings from which the sliced walk pays


def decay_scan_state_shape(heads: int, dim: int, value_dim: int) -> tuple[int, ...]:
    """A request's state row for `decay_scan`: per head and tile of 64 value columns, S as [dim][64]."""
    return (heads, (value_dim + 63) // 64, dim * 64)


def decay_scan(q: tuple[Product, int], k: tuple[Product, int], v: tuple[Product, int], state: torch.Tensor, seq_start: torch.Tensor,
               seq_slot: torch.Tensor, heads: int, dim: int, value_dim: int, decay: torch.Tensor | None = None,
               head_decay: torch.Tensor | None = None, bonus: torch.Tensor | None = None, q_scale: float = 1.0,
               k_scale: float = 1.0, max_new: int = 1) -> torch.Tensor:
    """Linear attention with a decaying matrix state over the step's tokens, sequence by sequence (see
    csrc/decay_scan.hip): S' = diag(w) S + k v^T, o = S'^T q per head; with `bonus` (float32 [heads * dim]) the result is
    read before the token joins the state, o = (S + diag(bonus) k v^T)^T q.  q, k, v: (product, first column), of one
    type; the decays w either `head_decay` (float32 [heads], one a head) or `decay` (float32 [tokens, heads * dim], one a
    token and key channel).  Carries `state` (float32 [slots, *decay_scan_state_shape]) for sequences whose slot is not
    negative (or [slots, floats] rows that begin with that shape's floats); returns float32 [tokens, heads * value_dim].  max_new: the most tokens any sequence brings in this step;
    from SCAN_SLICED_FROM on the tokens are taken in slices of SCAN_SLICE that run side by side."""
    for name, (product, _) in (("q", q), ("k", k), ("v", v)):
        _check_product(product, name)
    _device_tensor(state, "state", torch.float32)
    _device_tensor(seq_start, "seq_start", torch.int32)
    _device_tensor(seq_slot, "seq_slot", torch.int32)
    tokens = q[0].rows
    code = dtype_code(q[0].data.dtype)
    if k[0].rows != tokens or v[0].rows != tokens or dtype_code(k[0].data.dtype) != code or dtype_code(v[0].data.dtype) != code:
        raise invalid_shape("decay_scan: q, k and v have one row a token and one type")
    if not 0 < dim <= SCAN_MAX_DIM or heads <= 0 or value_dim <= 0:
        raise invalid_argument(f"decay_scan: heads of 1 to {SCAN_MAX_DIM} query dims")
    shape = decay_scan_state_shape(heads, dim, value_dim)
    if state.dim() == 2:                # a row that holds more than the scan's part, which comes first
        if state.shape[1] < shape[0] * shape[1] * shape[2]:
            raise invalid_shape(f"decay_scan: state rows of {state.shape[1]} floats do not hold {shape}")
    elif state.dim() != 4 or tuple(state.shape[1:]) != shape:
        raise invalid_shape(f"decay_scan: state {list(state.shape)} is not [slots, {shape}]")
    sequences = seq_slot.shape[0]
    if seq_start.shape != (sequences + 1,):
        raise invalid_shape("decay_scan: seq_start needs one entry more than there are sequences")
    for (product, col), size in ((q, heads * dim), (k, heads * dim), (v, heads * value_dim)):
        if col < 0 or col + size > product.cols:
            raise invalid_shape("decay_scan: q, k or v do not lie in their product's columns")
    if (decay is None) == (head_decay is None):
        raise invalid_argument("decay_scan: decays come either one a head or one a token and channel")
    kind = 0
    if decay is not None:
        _device_tensor(decay, "decay", torch.float32)
        if decay.shape != (tokens, heads * dim):
            raise invalid_shape("decay_scan: one decay a token and key channel")
        kind = 1
    else:
        _device_tensor(head_decay, "head_decay", torch.float32)
        if head_decay.shape != (heads,):
            raise invalid_shape("decay_scan: one decay a head")
    if bonus is not None:
        _device_tensor(bonus, "bonus", torch.float32)
        if kind != 1 or bonus.shape != (heads * dim,):
            raise invalid_shape("decay_scan: a bonus goes with decays per channel and has one entry a key channel")
        kind = 2
    out = torch.empty((tokens, heads * value_dim), dtype=torch.float32, device=state.device)
    if tokens == 0 or sequences == 0:
        return out
    slices, parts = 0, None
    if max_new >= SCAN_SLICED_FROM:
        slices = (min(int(max_new), tokens) + SCAN_SLICE - 1) // SCAN_SLICE
        parts = torch.empty((sequences, slices, shape[0], shape[1], shape[2] + dim), dtype=torch.float32, device=state.device)

    def columns(pair):
        product, col = pair
        return (_ptr(product.data), product.nsplit, ctypes.c_longlong(product.split_stride), product.cols, int(col))
    _check(library().tlie_decay_scan(*columns(q), *columns(k), *columns(v), code, kind, _ptr(decay), _ptr(head_decay), _ptr(bonus),
                                     ctypes.c_float(q_scale), ctypes.c_float(k_scale), _ptr(state), _ptr(seq_start),
                                     _ptr(seq_slot), _ptr(out), sequences, heads, dim, value_dim, slices, _ptr(parts),
                                     ctypes.c_longlong(state.stride(0)), _stream()), "decay_scan")
    return out


ROUTER_SCORES = {"sigmoid": 0, "softmax_of_chosen": 1}


def few_outputs(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, top: int = 0,
                score: str = "sigmoid", extra: int = 0) -> torch.Tensor:
    """A product with few outputs and float sums: float32 [tokens, outputs] = x . weight^T + bias.  top > 0: as a
    router: score "sigmoid": the sigmoids of the sums, of which each token's `top` largest keep their value and the rest
    become 0; score "softmax_of_chosen": each token's `top` largest sums are chosen and keep their softmax over the
    chosen ones only (at most 64), the rest become 0.  extra: the last `extra` outputs stand outside the choice and become
    their own sigmoids (gates of something every token uses)."""
    if score not in ROUTER_SCORES:
        raise invalid_argument(f"few_outputs: unknown score '{score}'")
    if extra < 0 or (top == 0 and (extra or score != "sigmoid")):
        raise invalid_argument("few_outputs: scores and extra outputs go with a router (top > 0)")
    _device_tensor(x, "x", (torch.float32, torch.bfloat16))
    _device_tensor(weight, "weight", (torch.float32, torch.bfloat16))
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise invalid_shape(f"few_outputs: x {list(x.shape)} does not fit weight {list(weight.shape)}")
    outputs = weight.shape[0]
    if outputs > 4096:
        raise invalid_argument("few_outputs: at most 4096 outputs")
    if bias is not None:
        _device_tensor(bias, "bias", weight.dtype)
        if bias.shape != (outputs,):
            raise invalid_shape("few_outputs: the bias needs one entry per output")
    if top < 0 or top > outputs - extra or (score == "softmax_of_chosen" and top > 64):
        raise invalid_argument("few_outputs: a router picks between 1 and all of its outputs (a softmax over at most 64)")
    out = torch.empty((x.shape[0], outputs), dtype=torch.float32, device=x.device)
    if x.shape[0] == 0:
        return out
    _check(library().tlie_few_outputs(_ptr(x), dtype_code(x.dtype), _ptr(weight), _ptr(bias), dtype_code(weight.dtype),
                                      _ptr(out), x.shape[0], x.shape[1], outputs, int(top), ROUTER_SCORES[score], int(extra),
                                      _stream()), "few_outputs")
    return out


def routed_gate(gate_up: Product, scale: torch.Tensor, block: int, out_dtype: torch.dtype, weigh: str = "input",
                shared_scaled: bool = False, gate: str = "silu", alpha: float = 1.0, limit: float = 0.0,
                shared_limit: float | None = None) -> torch.Tensor:
    """hidden[t, c] = silu(s g) * (s u): g and u side by side in gate_up (g0 u0 g1 u1 ...), s = scale[t, c // block]
    for the columns of the experts (scale: float32 [tokens, experts], 0 for an expert the token does not use) and 1
    for the columns after them (an expert that every token uses).
    weigh "output": hidden[t, c] = s * act(g, u), the score weighs what the expert gives (the product that follows is
    linear); the gate may then be any of `GATES` with its alpha and limit (shared_limit: the limit of the columns after
    the experts', default the same).  shared_scaled: scale has one column more, which the columns after the experts'
    take in the place of 1."""
    _check_product(gate_up, "gate_up")
    _device_tensor(scale, "scale", torch.float32)
    if gate_up.cols % 2 != 0:
        raise invalid_shape("routed_gate: gate and up lie side by side, the width must be even")
    rows, inter = gate_up.rows, gate_up.cols // 2
    if weigh not in ("input", "output") or gate not in GATES or (weigh == "input" and gate != "silu"):
        raise invalid_argument("routed_gate: a score weighs the input (SiLU gate) or the output (any gate)")
    if gate == "clamped_swish" and not (limit > 0.0 and (shared_limit is None or shared_limit > 0.0)):
        raise invalid_argument("routed_gate: the clamped gate needs positive limits")
    experts = scale.shape[1] - (1 if shared_scaled else 0) if scale.dim() == 2 else -1
    if scale.dim() != 2 or scale.shape[0] != rows or block <= 0 or experts < 0 or experts * block > inter:
        raise invalid_shape("routed_gate: the scale matrix does not fit the columns")
    out = torch.empty((rows, inter), dtype=out_dtype, device=gate_up.data.device)
    if rows == 0:
        return out
    _check(library().tlie_routed_gate(_ptr(gate_up.data), dtype_code(gate_up.data.dtype), gate_up.nsplit,
                                      ctypes.c_longlong(gate_up.split_stride), _ptr(scale), experts, int(block),
                                      _ptr(out), dtype_code(out_dtype), rows, inter, 1 if weigh == "output" else 0,
                                      scale.shape[1], 1 if shared_scaled else 0, GATES[gate], ctypes.c_float(alpha),
                                      ctypes.c_float(limit), ctypes.c_float(limit if shared_limit is None else shared_limit),
                                      _stream()), "routed_gate")
    return out



def sigmoid_gate(values: torch.Tensor, pre: Product, col: int) -> torch.Tensor:
    """values[t, c] *= sigmoid(pre[t, col + c]), in place: a gate on a mixer's heads whose pre-activations are columns
    of a wider product; the sigmoid and the product are float."""
    _device_tensor(values, "values", (torch.float32, torch.bfloat16))
    _check_product(pre, "pre")
    if values.dim() != 2 or values.shape[0] != pre.rows or col < 0 or col + values.shape[1] > pre.cols:
        raise invalid_shape(f"sigmoid_gate: columns {col} .. of a product [{pre.rows}, {pre.cols}] do not fit values {list(values.shape)}")
    if values.shape[0] == 0:
        return values
    _check(library().tlie_sigmoid_gate(_ptr(values), dtype_code(values.dtype), _ptr(pre.data), dtype_code(pre.data.dtype), pre.nsplit,
                                       ctypes.c_longlong(pre.split_stride), int(col), pre.cols, values.shape[0], values.shape[1],
                                       _stream()), "sigmoid_gate")
    return values


def softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap * tanh(x / cap), in place, on floats."""
    _device_tensor(x, "x", torch.float32)
    if not cap > 0.0:
        raise invalid_argument("softcap: the cap must be positive")
    if x.numel() > 0:
        _check(library().tlie_softcap(_ptr(x), ctypes.c_longlong(x.numel()), ctypes.c_float(cap), _stream()), "softcap")
    return x


MAX_STREAMS = 8        # the most streams a residual of several may have


@dataclass
class StreamUpdate:
    """What a residual of several streams still lacks: a sublayer's result and how it joins, `mix` float32 [S, S]
    ([from, to]) and `write` float32 [S]: x_t <- sum_s mix[s, t] x_s + write[t] * result.  Whoever reads the streams next
    brings them up to date in the same kernel (`stream_norm`)."""
    product: Product
    mix: torch.Tensor
    write: torch.Tensor


def stream_spread(first: torch.Tensor, count: int) -> torch.Tensor:
    """float32 [count, tokens, hidden]: `count` copies of `first` [tokens, hidden]."""
    _device_tensor(first, "first", torch.float32)
    if first.dim() != 2 or not 0 < count <= MAX_STREAMS:
        raise invalid_shape(f"stream_spread: [tokens, hidden] floats into 1 to {MAX_STREAMS} streams")
    out = torch.empty((count, *first.shape), dtype=torch.float32, device=first.device)
    if first.numel() > 0:
        _check(library().tlie_stream_spread(_ptr(first), _ptr(out), int(count), ctypes.c_longlong(first.numel()), _stream()), "stream_spread")
    return out


def stream_norm(streams: torch.Tensor, update: StreamUpdate | None, read: torch.Tensor | None, weight: torch.Tensor | None,
                eps: float, out_dtype: torch.dtype, total: bool = False):
    """Between two sublayers of a residual of several streams (float32 [S, tokens, hidden], changed in place): the
    streams are brought up to date with `update` (or left, None); then, with `read` (float32 [S]), u = sum_s read[s] x_s is
    RMS-normed with `weight` and `eps` and returned in `out_dtype`; with `total` the sum of the streams is returned too
    (float32 [tokens, hidden]).  Returns (normed or None, total or None)."""
    _device_tensor(streams, "streams", torch.float32)
    if streams.dim() != 3 or not 0 < streams.shape[0] <= MAX_STREAMS:
        raise invalid_shape(f"stream_norm: the streams must be [1 to {MAX_STREAMS}, tokens, hidden]")
    count, tokens, hidden = streams.shape
    delta = None
    if update is not None:
        delta = update.product
        _check_product(delta, "delta")
        _device_tensor(update.mix, "mix", torch.float32)
        _device_tensor(update.write, "write", torch.float32)
        if (delta.rows, delta.cols) != (tokens, hidden) or update.mix.shape != (count, count) or update.write.shape != (count,):
            raise invalid_shape("stream_norm: the result, mix [S, S] and write [S] do not fit the streams")
    out = None
    if read is not None:
        _device_tensor(read, "read", torch.float32)
        _device_tensor(weight, "norm weight", (torch.float32, torch.bfloat16))
        if read.shape != (count,) or weight.shape != (hidden,):
            raise invalid_shape("stream_norm: read [S] and the norm's weight [hidden] do not fit the streams")
        if not eps > 0.0:
            raise EngineError(ErrorCode.NUMERICAL, "RMSNorm requires a positive epsilon")
        out = torch.empty((tokens, hidden), dtype=out_dtype, device=streams.device)
    summed = torch.empty((tokens, hidden), dtype=torch.float32, device=streams.device) if total else None
    if tokens == 0 or (update is None and read is None and not total):
        return out, summed
    _check(library().tlie_stream_norm(_ptr(streams), count, _ptr(delta.data if delta is not None else None),
                                      dtype_code(delta.data.dtype) if delta is not None else F32, delta.nsplit if delta is not None else 1,
                                      ctypes.c_longlong(delta.split_stride if delta is not None else 0),
                                      _ptr(update.mix if update is not None else None), _ptr(update.write if update is not None else None),
                                      _ptr(read), _ptr(weight), dtype_code(weight.dtype) if weight is not None else F32,
                                      ctypes.c_float(eps if read is not None else 1.0), _ptr(out), dtype_code(out_dtype) if out is not None else F32,
                                      _ptr(summed), tokens, hidden, _stream()), "stream_norm")
    return out, summed

def residual_update(residual: torch.Tensor, first: Product, second: Product | None, mult: float,
                    copy_dtype: torch.dtype | None = None) -> torch.Tensor | None:
    """residual += mult * (first + second), in place.  copy_dtype: the residual as it is afterwards comes back once
    more in that type (what a product that reads the residual takes as its input)."""
    _device_tensor(residual, "residual", torch.float32)
    _check_product(first, "first")
    rows, width = residual.shape
    for product in [first] + ([second] if second is not None else []):
        _check_product(product, "second")
        if (product.rows, product.cols) != (rows, width) or product.data.dtype != first.data.dtype:
            raise invalid_shape("residual_update: the sublayers' results do not fit the residual (or differ in type)")
    copy = torch.empty((rows, width), dtype=copy_dtype, device=residual.device) if copy_dtype is not None else None
    if rows == 0:
        return copy
    _check(library().tlie_residual_update(_ptr(residual), _ptr(first.data), first.nsplit, ctypes.c_longlong(first.split_stride),
                                          _ptr(second.data if second is not None else None),
                                          second.nsplit if second is not None else 1,
                                          ctypes.c_longlong(second.split_stride if second is not None else 0),
                                          dtype_code(first.data.dtype), ctypes.c_float(mult), ctypes.c_longlong(rows * width),
                                          _ptr(copy), dtype_code(copy_dtype) if copy_dtype is not None else F32, _stream()),
           "residual_update")
    return copy


def side_gate(pre: Product, tokens: torch.Tensor, table: torch.Tensor, offset: int, out_dtype: torch.dtype) -> torch.Tensor:
    """g[t, j] = gelu_tanh(pre[t, j]) * table[tokens[t], offset + j], for the pre.cols columns of the table from `offset` on."""
    _check_product(pre, "pre")
    _device_tensor(tokens, "tokens", torch.int32)
    _device_tensor(table, "table", (torch.float32, torch.bfloat16))
    rows, dim = pre.rows, pre.cols
    if tokens.shape != (rows,) or table.dim() != 2 or offset < 0 or offset + dim > table.shape[1]:
        raise invalid_shape("side_gate: the table's columns or the tokens do not fit")
    out = torch.empty((rows, dim), dtype=out_dtype, device=table.device)
    if rows == 0:
        return out
    _check(library().tlie_side_gate(_ptr(pre.data), dtype_code(pre.data.dtype), pre.nsplit, ctypes.c_longlong(pre.split_stride),
                                    _ptr(tokens), _ptr(table), dtype_code(table.dtype), table.shape[1], int(offset), dim, _ptr(out),
                                    dtype_code(out_dtype), rows, _stream()), "side_gate")
    return out


def residual_inject(residual: torch.Tensor, tokens: torch.Tensor | None, table: torch.Tensor | None,
                    vector: torch.Tensor | None, accumulate: bool = True) -> None:
    """residual[t, :] (+)= table[tokens[t], :] + vector, in place; table and vector are optional and of one type."""
    _device_tensor(residual, "residual", torch.float32)
    rows, width = residual.shape
    given = [tensor for tensor in (table, vector) if tensor is not None]
    if not given:
        if not accumulate:
            residual.zero_()
        return
    code = dtype_code(given[0].dtype)
    if table is not None:
        _device_tensor(table, "table", given[0].dtype)
        _device_tensor(tokens, "tokens", torch.int32)
        if table.dim() != 2 or table.shape[1] != width or tokens.shape != (rows,):
            raise invalid_shape("residual_inject: the table's rows are not the residual's, or tokens are missing")
    if vector is not None:
        _device_tensor(vector, "vector", given[0].dtype)
        if vector.shape != (width,):
            raise invalid_shape("residual_inject: the vector needs one entry per column")
    if rows == 0:
        return
    _check(library().tlie_residual_inject(_ptr(residual), _ptr(tokens), _ptr(table), _ptr(vector), code, rows, width,
                                          1 if accumulate else 0, _stream()), "residual_inject")


def gemm_generic(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, out_dtype: torch.dtype) -> Product:
    """y = x . W^T (+ bias), every product and sum in true 32-bit.  W is [out, in]."""
    _device_tensor(x, "x", (torch.float32, torch.bfloat16))
    _device_tensor(weight, "weight", (torch.float32, torch.bfloat16))
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise invalid_shape(f"gemm: x {list(x.shape)} and weight {list(weight.shape)} do not fit")
    if bias is not None:
        _device_tensor(bias, "bias", weight.dtype)
        if bias.shape != (weight.shape[0],):
            raise invalid_shape("gemm: bias needs one entry per output")
    out = torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=x.device)
    if x.shape[0] == 0:
        return Product(out, 1)
    _check(library().tlie_gemm_generic(_ptr(x), dtype_code(x.dtype), _ptr(weight), dtype_code(weight.dtype), _ptr(bias),
                                       _ptr(out), dtype_code(out_dtype), x.shape[0], weight.shape[0], x.shape[1],
                                       _stream()), "gemm_generic")
    return Product(out, 1)


# state: None (not tried), True, False (not there); fallbacks: products that took this library's plain kernel instead
_library_gemm = {"state": None, "workspace": {}, "fallbacks": 0, "warned": set(), "no_bias_epilogue": set()}
LIBRARY_WORKSPACE_BYTES = 32 << 20


def library_mm(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
               bias: torch.Tensor | None = None) -> torch.Tensor:
    """y = x . W^T of bfloat16 operands through the vendor's library (hipBLASLt), for steps of many
    rows; y in bfloat16, or in float32 (the output head's logits).  The library is called
    directly, with its plan for the shape kept (half the host time of torch.mm, which a step of
    prompt portions calls four times a layer); where that is not possible (the library's file
    is not beside torch, or it has no algorithm for the shape) this library's plain kernel makes the
    product.  bias (bfloat16, one entry per row of W): joins the float sums in the library's own kernel; where
    the library offers nothing for that, the product is made without it and a kernel of this library adds it to
    the float result (either way the sum is rounded once)."""
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise EngineError(ErrorCode.INVALID_DTYPE, f"library_mm gives bfloat16 or float32, not {out_dtype}")
    _device_tensor(x, "x", torch.bfloat16)
    _device_tensor(weight, "weight", torch.bfloat16)
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise invalid_shape(f"library_mm: x {list(x.shape)} and weight {list(weight.shape)} do not fit")
    state = _library_gemm
    if state["state"] is None:
        import os
        path = os.path.join(os.path.dirname(torch.__file__), "lib", "libhipblaslt.so")
        torch.mm(x[:1], weight[:1].t())                       # torch loads and sets up its copy of the library first
        state["state"] = os.path.isfile(path) and library().tlie_library_gemm_init(path.encode()) == 0
    if bias is not None:
        _device_tensor(bias, "bias", torch.bfloat16)
        if bias.shape != (weight.shape[0],):
            raise invalid_shape("library_mm: the bias needs one entry per row of W")
        if state["state"] and x.dim() == 2 and x.shape[0] > 0 and (tuple(x.shape), tuple(weight.shape)) not in state["no_bias_epilogue"]:
            _device_tensor(x, "x", torch.bfloat16)
            _device_tensor(weight, "weight", torch.bfloat16)
            if weight.dim() != 2 or x.shape[1] != weight.shape[1]:
                raise invalid_shape(f"library_mm: x {list(x.shape)} and weight {list(weight.shape)} do not fit")
            index = x.device.index or 0
            if index not in state["workspace"]:
                state["workspace"][index] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
            workspace = state["workspace"][index]
            out = torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=x.device)
            status = library().tlie_library_gemm_bias(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), int(out_dtype == torch.float32),
                                                      x.shape[0], weight.shape[0], x.shape[1], _ptr(workspace),
                                                      ctypes.c_size_t(workspace.numel()), _stream())
            if status == 0:
                return out
            if status != -3:
                _check(status, "library_gemm_bias")
            state["no_bias_epilogue"].add((tuple(x.shape), tuple(weight.shape)))       # (not asked for again)
        return add_bias(library_mm(x, weight, torch.float32), bias, out_dtype)
    if state["state"] and x.shape[0] > 0:
        index = x.device.index or 0
        if index not in state["workspace"]:
            state["workspace"][index] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
        workspace = state["workspace"][index]
        out = torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=x.device)
        status = library().tlie_library_gemm(_ptr(x), _ptr(weight), _ptr(out), int(out_dtype == torch.float32), x.shape[0],
                                             weight.shape[0], x.shape[1], _ptr(workspace), ctypes.c_size_t(workspace.numel()),
                                             _stream())
        if status == 0:
            return out
        if status != -3:
            _check(status, "library_gemm")
    # where the library cannot be called directly (its file is not beside torch, or it has no
    # algorithm for the shape) this library's own kernels make the product: the tiled one on the matrix
    # cores (some two thirds of the vendor's speed) for sizes it takes, else the plain 32-bit one (many
    # times slower); one route, recorded or not, so that a step gives the same bits replayed and launched
    # (and safe inside a recording, where a library call that has not been tried may clear a workspace
    # with a memset node)
    if x.shape[0] > 0:
        state["fallbacks"] += 1
        shape = (x.shape[0], weight.shape[0], weight.shape[1])
        if shape not in state["warned"]:
            # said once per shape: nothing else shows why a prompt step is ten times slower than it should be
            state["warned"].add(shape)
            import warnings
            why = "has no algorithm within its workspace for" if state["state"] else "is not available for"
            how = ("this library's tiled kernel, at some two thirds of the speed" if gemm_tiles_takes(weight)
                   else "this library's plain 32-bit kernel, which is many times slower")
            warnings.warn(f"the vendor's matrix library {why} the bfloat16 product {shape[0]} x {shape[1]} x {shape[2]}; "
                          f"it takes {how}", stacklevel=2)
    if gemm_tiles_takes(weight):
        return gemm_tiles(x, weight, out_dtype)
    return gemm_generic(x, weight, None, out_dtype).data


def gemm_tiles_takes(weight: torch.Tensor) -> bool:
    return weight.dtype == torch.bfloat16 and weight.shape[1] % 64 == 0 and weight.shape[0] % 4 == 0


def gemm_tiles(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """y = x . W^T of bfloat16 operands on this library's own tiled kernel for many rows (tiles of 128
    rows of W by 128 tokens on the matrix cores): what `library_mm` runs where the vendor's library
    cannot be called.  The inner size a multiple of 64, W's rows a multiple of 4; y bfloat16 or float32."""
    _device_tensor(x, "x", torch.bfloat16)
    _device_tensor(weight, "weight", torch.bfloat16)
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise invalid_shape(f"gemm_tiles: x {list(x.shape)} and weight {list(weight.shape)} do not fit")
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise EngineError(ErrorCode.INVALID_DTYPE, f"gemm_tiles gives bfloat16 or float32, not {out_dtype}")
    if not gemm_tiles_takes(weight):
        raise invalid_argument("gemm_tiles takes an inner size that is a multiple of 64 and a multiple of 4 of rows of W")
    out = torch.empty((x.shape[0], weight.shape[0]), dtype=out_dtype, device=x.device)
    if x.shape[0] == 0:
        return out
    _check(library().tlie_gemm_tiles(_ptr(x), _ptr(weight), _ptr(out), int(out_dtype == torch.float32), x.shape[0],
                                     weight.shape[0], x.shape[1], _stream()), "gemm_tiles")
    return out


def library_fallbacks() -> int:
    """How many products `library_mm` has made with this library's own kernels because the vendor's
    library was not there or offered nothing for the shape (each slower, some many times)."""
    return _library_gemm["fallbacks"]


def add_bias(product: torch.Tensor, bias: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """out = product + bias (one entry per column) for a float32 product that came without its bias;
    the sum is float32 and rounded once to `out_dtype` (float32: in place)."""
    _device_tensor(product, "product", torch.float32)
    _device_tensor(bias, "bias", (torch.float32, torch.bfloat16))
    if product.dim() != 2 or bias.shape != (product.shape[1],):
        raise invalid_shape(f"add_bias: product {list(product.shape)} and bias {list(bias.shape)} do not fit")
    out = product if out_dtype == torch.float32 else torch.empty(product.shape, dtype=out_dtype, device=product.device)
    if product.shape[0] == 0:
        return out
    _check(library().tlie_add_bias(_ptr(product), _ptr(bias), dtype_code(bias.dtype), _ptr(out), dtype_code(out_dtype),
                                   product.shape[0], product.shape[1], _stream()), "add_bias")
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor | None = None, top_p: torch.Tensor | None = None,
           seed: torch.Tensor | None = None, counter: torch.Tensor | None = None,
           out: torch.Tensor | None = None) -> torch.Tensor:
    """One token per row of float32 logits: the first maximum when the row's temperature is not
    positive (or none is given), else a draw from the top-p part of softmax(logits / T) with the
    uniform number of (seed, counter).  A row with a NaN or an infinity gives -1.  `out`: int32
    [rows] to write into (else a new tensor)."""
    _device_tensor(logits, "logits", torch.float32)
    if logits.dim() != 2:
        raise invalid_shape("sample takes logits [rows, vocab]")
    rows = logits.shape[0]
    for name, tensor, dtype in (("temperature", temperature, torch.float32), ("top_p", top_p, torch.float32),
                                ("seed", seed, torch.int64), ("counter", counter, torch.int64)):
        if tensor is not None:
            _device_tensor(tensor, name, dtype)
            if tensor.shape != (rows,):
                raise invalid_shape(f"sample: {name} needs one entry per row")
    if out is None:
        out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    else:
        _device_tensor(out, "out", torch.int32)
        if out.shape != (rows,):
            raise invalid_shape("sample: out needs one entry per row")
    if rows == 0:
        return out
    _check(library().tlie_sample(_ptr(logits), rows, logits.shape[1], _ptr(temperature), _ptr(top_p), _ptr(seed),
                                 _ptr(counter), _ptr(out), _stream()), "sample")
    return out


def feed_tokens(tokens: torch.Tensor, source: torch.Tensor, sampled: torch.Tensor, vocab: int) -> None:
    """tokens[i] = sampled[source[i]] wherever source[i] >= 0, on the device, brought into the
    vocabulary's range 0 .. vocab - 1 (a sample of -1 marks a row of logits that held a NaN or an
    infinity: the host raises when it reads it, and the step that is already launched takes token 0).
    The caller has checked on the host that every such source is a row of `sampled`."""
    for name, tensor in (("tokens", tokens), ("source", source), ("sampled", sampled)):
        _device_tensor(tensor, name, torch.int32)
    if tokens.dim() != 1 or source.shape != tokens.shape or sampled.dim() != 1 or sampled.shape[0] == 0:
        raise invalid_shape("feed_tokens takes tokens [T], source [T] and sampled [rows]")
    if vocab <= 0:
        raise invalid_argument("feed_tokens: the vocabulary's size must be positive")
    if tokens.shape[0] == 0:
        return
    _check(library().tlie_feed_tokens(_ptr(tokens), _ptr(source), _ptr(sampled), tokens.shape[0], int(vocab), _stream()),
           "feed_tokens")


# ---- bfloat16 kernels on the matrix cores ---------------------------------------------------------
SKINNY_MAX_ROWS = 64
def skinny_split_len(rows: int, out_features: int, in_features: int) -> int:
    """How many k values one split takes when the matrix has work for many workgroups per compute
    unit.  Measured on the MI355X inside whole decode steps: the gated feed-forward's first product
    (11264 rows and more) with 512, and 1024 once the step has more than 32 rows of x, because each
    partial sum is a write and a read of rows x outputs; a long inner size (4096 and more) with 1024
    up to 32 rows and 512 beyond; the others with 256."""
    strips = (out_features + 15) // 16
    if strips >= 512:
        length = 1024 if rows > 32 else 512
    else:
        length = 256
    if in_features >= 4096:
        length = max(length, 1024 if rows <= 32 else 512)
    return min(length, (in_features + 63) // 64 * 64)


_SKINNY_PLANS: dict = {}
_COMPUTE_UNITS: dict = {}


def _compute_units(device: torch.device) -> int:
    index = device.index or 0
    if index not in _COMPUTE_UNITS:
        _COMPUTE_UNITS[index] = int(torch.cuda.get_device_properties(device).multi_processor_count)
    return _COMPUTE_UNITS[index]


def skinny_plan(rows: int, out_features: int, in_features: int, compute_units: int = 256) -> tuple[int, int, int]:
    """The launch shape of `gemm_skinny`: (k values per split, waves a workgroup, strips of 16 rows
    of W a wave).  A compute unit draws some 20 GB/s from memory whatever its waves ask for, so a
    matrix of up to 64 MB is cut into as many equal workgroups as there are compute units, or just
    fewer (the product takes as long as the unit with the most bytes: TinyLlama's q/k/v matrix at 64
    rows 7.4 -> 6.4 us, the output projection 6.9 -> 5.7, gate/up 17.9 -> 16.9, down 11.0 -> 10.3),
    by the number of waves (each takes 16 rows of W) and the number of splits, each split costing a
    write and a read of rows x outputs partial sums (a decode step of the TinyLlama shape at batch
    64 2.10 -> 2.01 ms, at 32 1.69 -> 1.63).  Larger matrices keep many workgroups per compute unit
    (several at once hide each other's waits, which counts for more there)."""
    key = (rows, out_features, in_features, compute_units)
    if key in _SKINNY_PLANS:
        return _SKINNY_PLANS[key]
    plan = (skinny_split_len(rows, out_features, in_features), 4, 2 if rows > 32 else 1)
    if out_features * in_features * 2 <= (64 << 20):
        best = None
        for waves in range(4, 17):
            blocks = -(-out_features // (16 * waves))
            for nsplit in range(1, 33):
                split_len = (-(-in_features // nsplit) + 63) // 64 * 64
                if -(-in_features // split_len) != nsplit:
                    continue
                rounds = -(-blocks * nsplit // compute_units)
                # microseconds: a workgroup's bytes at 20 GB/s and half a microsecond per round; the partial sums at 6 TB/s
                # (the coefficients that gave the fastest whole decode steps at 20, 32 and 64 rows)
                cost = rounds * (16 * waves * split_len * 2 / 20e3 + 0.5) + nsplit * rows * out_features * 8 / 6e6
                if best is None or cost < best[0]:
                    best = (cost, split_len, waves, 1)
        plan = best[1:]
    _SKINNY_PLANS[key] = plan
    return plan


def gemm_skinny_takes(x: torch.Tensor, weight: torch.Tensor) -> bool:
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and 0 < x.shape[0] <= SKINNY_MAX_ROWS
            and weight.shape[1] % 8 == 0)


def skinny_gated_plan(rows: int, out_features: int, in_features: int, compute_units: int = 256) -> tuple[int, int]:
    """(waves a workgroup, strips a wave) of `gemm_skinny` when it keeps all of K in a workgroup and applies
    the SiLU gate itself: as many equal workgroups as compute units, or just fewer (see `skinny_plan`); a
    workgroup's time is its rows of W from memory and all of x from the caches."""
    best = None
    for strips in ((1, 2) if rows > 32 else (1,)):
        for waves in range(3, (8 if strips == 2 else 16) + 1):
            blocks = -(-out_features // (16 * waves * strips))
            rounds = -(-blocks // compute_units)
            cost = rounds * (16 * waves * strips * in_features * 2 / 20e3 + 0.5)
            if best is None or cost < best[0]:
                best = (cost, waves, strips)
    return best[1], best[2]


def _gate_args(gate) -> tuple:
    """(kind, alpha, limit) as the kernels take them, from None (the SiLU gate) or (name, alpha, limit)."""
    if gate is None:
        return 0, ctypes.c_float(1.0), ctypes.c_float(0.0)
    name, alpha, limit = gate
    if name not in GATES or (name == "clamped_swish" and not limit > 0.0):
        raise invalid_argument(f"unknown gate {gate!r}")
    return GATES[name], ctypes.c_float(alpha), ctypes.c_float(limit)


def gemm_skinny(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, split_len: int | None = None,
                waves: int | None = None, strips: int | None = None, gated: bool = False, gate=None):
    """y = x . W^T (+ bias) for at most 64 rows of bfloat16 x: float partial sums [nsplit, M, N].
    split_len, waves, strips: the launch shape (see `skinny_plan`, which chooses it when they are not given).
    gated: W's rows alternate gate and up; K is not split, and the kernel stores bfloat16
    silu(gate) * up [M, N / 2], which is returned as a tensor (no partial sums, no activation kernel).
    gate: (name, alpha, limit) of another gate than SiLU (see `silu_mul`)."""
    _device_tensor(x, "x", torch.bfloat16)
    _device_tensor(weight, "weight", torch.bfloat16)
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise invalid_shape(f"gemm_skinny: x {list(x.shape)} and weight {list(weight.shape)} do not fit")
    rows, (out_features, in_features) = x.shape[0], weight.shape
    if not 0 < rows <= SKINNY_MAX_ROWS or in_features % 8 != 0:
        raise invalid_argument(f"gemm_skinny takes 1..{SKINNY_MAX_ROWS} rows and an inner size that is a multiple of 8")
    if bias is not None:
        _device_tensor(bias, "bias", torch.bfloat16)
        if bias.shape != (out_features,):
            raise invalid_shape("gemm_skinny: bias needs one entry per output")
    if gated:
        if out_features % 2 != 0:
            raise invalid_shape("gemm_skinny: the gated product needs an even number of rows of W")
        if split_len is not None and split_len < in_features:
            raise invalid_argument("gemm_skinny: the gated product does not split K")
        split_len = (in_features + 63) // 64 * 64
        if waves is None or strips is None:
            waves, strips = skinny_gated_plan(rows, out_features, in_features, _compute_units(x.device))
    elif split_len is None:
        split_len, waves, strips = skinny_plan(rows, out_features, in_features, _compute_units(x.device))
    elif waves is None or strips is None:
        waves, strips = waves or 4, strips or (2 if rows > 32 else 1)
    if split_len <= 0 or split_len % 64 != 0:
        raise invalid_argument("gemm_skinny: a split's length must be a positive multiple of 64")
    if not 3 <= waves <= 16 or strips not in (1, 2) or (strips == 2 and (rows <= 32 or waves > 8)):
        raise invalid_argument("gemm_skinny: 3 to 16 waves; two strips a wave only for more than 32 rows and up to 8 waves")
    nsplit = (in_features + split_len - 1) // split_len
    if gated:
        act = torch.empty((rows, out_features // 2), dtype=torch.bfloat16, device=x.device)
        _check(library().tlie_gemm_skinny(_ptr(x), _ptr(weight), _ptr(bias), _ptr(None), _ptr(act), rows, out_features, in_features,
                                          split_len, waves, strips, *_gate_args(gate), _stream()), "gemm_skinny")
        return act
    out = torch.empty((nsplit, rows, out_features), dtype=torch.float32, device=x.device)
    _check(library().tlie_gemm_skinny(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), _ptr(None), rows, out_features, in_features,
                                      split_len, waves, strips, *_gate_args(None), _stream()), "gemm_skinny")
    return Product(out, nsplit)


def attention_col_tiles(head_dim: int) -> int:
    """How many groups of 16 columns a wave of the tiled attention kernel serves in a step that
    brings prompt portions.  The registers hold 4 for head sizes up to 64; 2 measured faster there
    (a prompt of 2048 tokens: 70 us against 92 with 4 waves a tile), the softmax arithmetic of one
    wave then overlapping the products of another."""
    return 2 if head_dim <= 128 else 1


def attention_max_waves(head_dim: int, col_tiles: int = 1) -> int:
    """How many waves of a workgroup of the tiled attention kernel may share a tile's keys."""
    fit, cap = 1024 // (col_tiles * head_dim), 4 if col_tiles * head_dim > 128 else 8
    return max(1, min(fit, cap))


def attention_tiles(seq_start, groups_per_kv: int, col_tiles: int = 1, seq_len=None):
    """The work list of the tiled attention kernel for a step, on the host: for every sequence,
    tiles of 16 * col_tiles columns, a column being a (token, query head of one group) pair.
    seq_start: the step's cumulative token counts [S + 1].  seq_len: the sequences' lengths after
    the step [S]; with it the tiles are ordered by the number of keys they see, most first, so
    that the longest are not the last to start.  Returns an int32 array [tiles, 4]:
    (sequence, its first token's index in the step, its number of tokens, the tile's first column)."""
    import numpy as np
    step = 16 * col_tiles
    parts, keys = [], []
    for seq in range(len(seq_start) - 1):                  # (a sequence's tiles at once: a prompt has thousands)
        first, count = int(seq_start[seq]), int(seq_start[seq + 1] - seq_start[seq])
        if count <= 0:
            continue
        col0 = np.arange(0, count * groups_per_kv, step, dtype=np.int64)
        block = np.empty((col0.shape[0], 4), dtype=np.int32)
        block[:, 0], block[:, 1], block[:, 2], block[:, 3] = seq, first, count, col0
        parts.append(block)
        if seq_len is not None:
            last_token = np.minimum(count - 1, (col0 + step - 1) // groups_per_kv)
            keys.append(int(seq_len[seq]) - count + last_token + 1)
    rows = np.concatenate(parts) if parts else np.zeros((0, 4), dtype=np.int32)
    if seq_len is not None and rows.shape[0] > 1:
        rows = rows[np.argsort(-np.concatenate(keys), kind="stable")]
    return np.ascontiguousarray(rows)


def few_rows_route(rows: int, dtype: torch.dtype) -> bool:
    """Whether a step of `rows` tokens may take the route on which the products of few rows fold in
    the norm before them and the add (or gate, or rotation) after them: bfloat16, at most 16 rows."""
    return dtype == torch.bfloat16 and 0 < rows <= ROWS_MAX


def attention_plan(ctx, groups_per_kv: int, num_kv_heads: int, head_dim: int):
    """How the tiled attention kernel is launched for the step `ctx` describes: its work list (made
    once per step and group size, kept in `ctx.scratch`; None for a decode step, whose tiles the
    kernel derives itself), and how the keys are cut: into as many parts as it takes to give a step
    of few tiles about a thousand waves (measured: at batch 64 and 2048 positions 4 parts reach
    5 TB/s, 16 parts 4 TB/s, and merging more than 16 costs more than it gains), each part a
    multiple of 32 positions and at least 64.  The policy is this kernel's own and measured on the
    MI355X; the step's context only supplies the host arrays, the number of compute units, and, in a
    recorded step, the owner of work lists at fixed addresses.
    Returns (tiles, col_tiles, nsplit, split_len, waves, shared): `waves` of a workgroup share a
    tile's keys, or with `shared` take columns of their own and get the keys through LDS."""
    decode = ctx.max_new == 1 and ctx.num_seqs == ctx.num_tokens
    col_tiles, shared = 1, False
    if decode:
        tiles, count = None, ctx.num_tokens * ((groups_per_kv + 15) // 16)
    else:
        col_tiles = attention_col_tiles(head_dim)
        # sequences of some length with portions of many columns: 4 waves take columns of their own
        # of one tile and every block of keys is brought once for all of them, through LDS (a
        # prompt of 1536 tokens: 34 us against 42; of 8192: 450 against 780; of 512: 15 against
        # 13).  Each wave takes 32 columns, or 16 while that leaves no more tiles than two and a
        # half for every compute unit: the smaller ones then fill the chip better, four
        # workgroups a compute unit (2048 tokens: 51 us against 63; 2560: 74 against 81; 3072:
        # 100 against 98; 4096: 162 against 150)
        shared = (col_tiles == 2 and head_dim <= 128 and ctx.max_context >= 768
                  and ctx.num_tokens * groups_per_kv >= 64 * ctx.num_seqs)

        def tiles_of(groups):
            key = ("attention_tiles", groups_per_kv, groups)
            if key not in ctx.scratch:
                def make(host):
                    return attention_tiles(host["seq_start"], groups_per_kv, groups, host["seq_len"])
                if ctx.tile_owner is not None:
                    # a sequence of n tokens has ceil(n * G / (16 * groups)) tiles
                    capacity = (ctx.num_tokens * groups_per_kv + 16 * groups - 1) // (16 * groups) + ctx.num_seqs
                    ctx.scratch[key] = ctx.tile_owner.tiles_for(key, make, capacity)
                else:
                    ctx.scratch[key] = torch.from_numpy(make(ctx.host)).to(ctx.tokens.device)
            return ctx.scratch[key]
        tiles = tiles_of(col_tiles * (4 if shared else 1))
        if shared and 2 * tiles.shape[0] * num_kv_heads <= 5 * ctx.compute_units:
            col_tiles = 1
            tiles = tiles_of(4)
        count = tiles.shape[0] * (4 if shared else 1)
    tiles_all = count * num_kv_heads
    if not decode:
        # a step of prompt portions has tiles enough; cutting their keys would only add merging,
        # unless few tiles see many keys (a short portion late in a long sequence): then into parts of
        # 256 keys or more (parts of 64 and more made prompts of 64 to 256 tokens 3 to 4% slower: 2.50 ->
        # 2.43 ms at 256 tokens).
        # Up to 4 waves share a tile's keys, each with 128 or more: a tile that sees the whole of
        # a long sequence then takes a quarter of the time, and it is the longest tiles that
        # the step waits for (a prompt of 2048 tokens: 70 us against 87 with one wave a tile)
        nsplit = max(1, min((512 + tiles_all - 1) // tiles_all, 16, ctx.max_context // 256))
        waves = 4 if shared else 1
        while (not shared and waves < 4 and waves * 2 <= attention_max_waves(head_dim, col_tiles)
               and ctx.max_context >= nsplit * waves * 2 * 128):
            waves *= 2
    else:
        # workgroups share a tile's keys until there is one for every compute unit (their sums
        # meet in the merge kernel); then the waves of a workgroup share them, which costs no
        # launch, while a wave keeps 128 keys or more and the step has 2048 waves at most
        # (measured inside whole steps at 2048 positions: batch 1 16 parts x 1 wave, batch 8
        # 8 x 2, batch 64 1 x 8)
        nsplit = max(1, min((256 + tiles_all - 1) // tiles_all, 16, (ctx.max_context + 63) // 64))
        waves = 1
        while (waves * 2 <= attention_max_waves(head_dim) and tiles_all * nsplit * waves * 2 <= 2048
               and ctx.max_context >= nsplit * waves * 2 * 128):
            waves *= 2
        if nsplit > 1 and ctx.max_context <= 256 and attention_max_waves(head_dim) >= 2:
            # up to 256 positions there is nothing to cut: two waves of one workgroup share the keys and the
            # merge launch goes (batch 1 at 200 positions 0.902 ms a step against 0.919, batch 8 0.998
            # against 1.017; at 450 positions the parts win again: 0.928 against 0.944 with 1 x 4)
            nsplit, waves = 1, 2
    if nsplit == 1:
        return tiles, col_tiles, 1, 0, waves, shared
    split_len = ((ctx.max_context + nsplit - 1) // nsplit + 31) // 32 * 32
    nsplit = (ctx.max_context + split_len - 1) // split_len
    return tiles, col_tiles, nsplit, split_len, waves, shared


def attention_mfma_takes(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 0 < head_dim <= ATTENTION_MAX_HEAD_DIM and page_size >= 16
            and page_size & (page_size - 1) == 0)


def attention_mfma(q: torch.Tensor, cache: torch.Tensor, block_table: torch.Tensor, tiles: torch.Tensor | None,
                   positions: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, window: int | None,
                   scale: float, nsplit: int = 1, split_len: int = 0, col_tiles: int = 1, waves: int = 1,
                   shared: bool = False, chunk: int | None = None, sink: torch.Tensor | None = None,
                   planes: tuple[int, int, int] | None = None, float_out: bool = False,
                   softcap: float | None = None) -> torch.Tensor:
    """Causal attention of every token of the step over its sequence's cache, bfloat16.

    tiles: int32 [n, 4] from `attention_tiles` (built from the same step as block_table and
    positions: every tile's sequence is a row of block_table, its tokens are rows of q); None for
    a decode step, in which token i is the one token of sequence i.  nsplit > 1 cuts the keys into
    that many parts of split_len positions (a multiple of 32; nsplit * split_len must reach the
    longest sequence) that run side by side and are merged.  col_tiles: the value the tiles were
    made with.  waves (a power of two up to `attention_max_waves`): so many waves of a
    workgroup share each tile's (or part's) keys and merge their results before writing.
    shared (prompt portions; col_tiles 1 or 2, head size up to 128, 4 or 8 waves): the tiles were made
    with col_tiles * waves column groups, every wave takes col_tiles of them, and each block of keys
    and values is brought once for the whole workgroup.
    chunk: a token sees only the keys of its own chunk of so many positions (counted from position 0).
    sink: float32 [nq], a number per head whose exponential joins the softmax's denominator.
    planes (key_share, value_group, value_planes): kv heads share planes of a page: key_share kv heads in a row read
    one key plane, and q holds one query head for them ([tokens, nq / key_share * d]); of every value_group kv heads in
    a row the i-th reads value plane i % value_planes of that group's value_planes.  A page then holds
    nkv / key_share planes of keys and after them nkv / value_group * value_planes planes of values, each
    page_size * d (cache: [pages, ...] with so many values a page).  The result has all nq heads.
    float_out (with planes): the result is float32.
    softcap (without planes): a scaled score s enters the softmax as softcap * tanh(s / softcap)."""
    _device_tensor(q, "q", torch.bfloat16)
    if softcap is not None and (not float(softcap) > 0.0 or planes is not None):
        raise invalid_argument("attention: a cap of the scores must be positive, and does not go with shared planes")
    if planes is not None:
        key_share, value_group, value_planes = (int(v) for v in planes)
        if (min(key_share, value_group, value_planes) <= 0 or max(key_share, value_group) > 255 or value_planes > value_group
                or num_kv_heads % key_share != 0 or num_kv_heads % value_group != 0):
            raise invalid_argument("attention: kv heads do not share planes that way")
    elif float_out:
        raise invalid_argument("attention: float results go with shared planes only")
    if sink is not None:
        _device_tensor(sink, "sink", torch.float32)
        if sink.shape != (num_heads,):
            raise invalid_shape("attention: the sink needs one entry per query head")
    if chunk is not None and int(chunk) <= 0:
        raise invalid_argument("attention: a chunk must be a positive count of positions")
    _device_tensor(cache, "cache", torch.bfloat16)
    _device_tensor(block_table, "block_table", torch.int32)
    _device_tensor(positions, "positions", torch.int32)
    tokens = q.shape[0]
    if num_kv_heads <= 0 or num_heads % num_kv_heads != 0:
        raise invalid_shape("attention: the number of heads must be a multiple of the number of kv heads")
    if planes is None:
        if q.shape != (tokens, num_heads * head_dim):
            raise invalid_shape(f"attention: q {list(q.shape)} is not [tokens, nq * d]")
        page_size = _check_cache(cache, num_kv_heads, head_dim, "attention")
    else:
        if q.shape != (tokens, num_heads // key_share * head_dim):
            raise invalid_shape(f"attention: q {list(q.shape)} is not [tokens, nq / key_share * d]")
        per_row = (num_kv_heads // key_share + num_kv_heads // value_group * value_planes) * head_dim
        per_page = cache[0].numel() if cache.dim() >= 2 and cache.shape[0] > 0 else 0
        if per_page == 0 or per_page % per_row != 0:
            raise invalid_shape(f"attention: cache {list(cache.shape)} does not hold pages of {per_row} values a position")
        page_size = per_page // per_row
    if block_table.dim() != 2 or positions.shape != (tokens,):
        raise invalid_shape("attention: block_table must be [sequences, max_blocks], positions [tokens]")
    if num_heads % num_kv_heads != 0:
        raise invalid_shape("attention: the number of heads must be a multiple of the number of kv heads")
    if not scale > 0:
        raise invalid_argument(f"attention: the scale {scale} of the scores is not positive")
    if tiles is not None:
        _device_tensor(tiles, "tiles", torch.int32)
        if tiles.dim() != 2 or tiles.shape[1] != 4 or tiles.shape[0] == 0:
            raise invalid_shape("attention: tiles must be [n, 4]")
        num_tiles = tiles.shape[0]
        if col_tiles not in (1, 2, 4) or col_tiles > (4 if head_dim <= 64 else (2 if head_dim <= 128 else 1)):
            raise invalid_argument(f"attention: {col_tiles} column groups a wave do not fit head size {head_dim}")
    else:
        col_tiles = 1
        if block_table.shape[0] < tokens:
            raise invalid_shape("attention: a decode step needs a block table row per token")
        num_tiles = tokens * ((num_heads // num_kv_heads + 15) // 16)
    if nsplit > 1 and (split_len <= 0 or split_len % 32 != 0):
        raise invalid_argument("attention: split_len must be a positive multiple of 32")
    if shared:
        if tiles is None or col_tiles not in (1, 2) or head_dim > 128 or waves not in (4, 8):
            raise invalid_argument("attention: sharing through LDS takes tiles, 1 or 2 column groups a wave, a head size up to 128 and 4 or 8 waves")
    elif waves not in (1, 2, 4, 8) or waves > attention_max_waves(head_dim, col_tiles):
        raise invalid_argument(f"attention: waves must be a power of two up to {attention_max_waves(head_dim, col_tiles)}")
    if not attention_mfma_takes(q.dtype, head_dim, page_size):
        raise invalid_argument("attention_mfma takes bfloat16, head sizes in steps of 16 up to 256, pages of a power of two of rows (at least 16)")
    out = torch.empty((tokens, num_heads * head_dim), dtype=torch.float32 if float_out else torch.bfloat16, device=q.device)
    part_o = part_ml = None
    if nsplit > 1:
        part_o = torch.empty((tokens * num_heads * nsplit, head_dim), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((tokens * num_heads * nsplit, 2), dtype=torch.float32, device=q.device)
    if planes is not None:
        _check(library().tlie_attention_mfma_planes(_ptr(q), _ptr(cache), _ptr(block_table), block_table.shape[1], _ptr(tiles),
                                                    num_tiles, col_tiles, _ptr(positions), _ptr(out), _ptr(part_o), _ptr(part_ml),
                                                    nsplit, split_len, tokens, num_heads, num_kv_heads, head_dim, page_size,
                                                    int(window) if window else 0, int(chunk) if chunk else 0, _ptr(sink),
                                                    ctypes.c_float(scale), waves, int(bool(shared)), key_share, value_group,
                                                    value_planes, 1 if float_out else 0, _stream()), "attention_mfma")
        return out
    if softcap is not None:
        _check(library().tlie_attention_mfma_capped(_ptr(q), _ptr(cache), _ptr(block_table), block_table.shape[1], _ptr(tiles),
                                                    num_tiles, col_tiles, _ptr(positions), _ptr(out), _ptr(part_o), _ptr(part_ml),
                                                    nsplit, split_len, tokens, num_heads, num_kv_heads, head_dim, page_size,
                                                    int(window) if window else 0, int(chunk) if chunk else 0, _ptr(sink),
                                                    ctypes.c_float(scale), waves, int(bool(shared)), ctypes.c_float(softcap),
                                                    _stream()), "attention_mfma")
        return out
    _check(library().tlie_attention_mfma(_ptr(q), _ptr(cache), _ptr(block_table), block_table.shape[1], _ptr(tiles),
                                         num_tiles, col_tiles, _ptr(positions), _ptr(out), _ptr(part_o), _ptr(part_ml), nsplit,
                                         split_len, tokens, num_heads, num_kv_heads, head_dim, page_size,
                                         int(window) if window else 0, int(chunk) if chunk else 0, _ptr(sink),
                                         ctypes.c_float(scale), waves, int(bool(shared)), _stream()),
           "attention_mfma")
    return out


# ---- at most 16 rows: products with the layer's neighbouring arithmetic folded in --------------------


@dataclass
class NormedRows:
    """The input of a product, not yet normed: xg = bfloat16(residual * norm weight) [T, width] and
    partial sums of squares of the residual's rows, ssq [parts, 16] (each part covers some of the
    columns; their sum over the parts is the row's sum of squares).  The product applies
    rsqrt(sum(ssq) / width + eps) to its result's rows, which is the same as having normed the
    input."""
    xg: torch.Tensor
    ssq: torch.Tensor
    eps: float

    @property
    def shape(self):
        return self.xg.shape


@dataclass
class ResidualUpdated:
    """A product's result was added into the residual by the kernel that computed it; `normed`
    is the residual as the next norm's product wants it, when that was asked for."""
    normed: NormedRows | None


def gemm_rows_takes(rows: int, weight: torch.Tensor, dtype: torch.dtype) -> bool:
    return (dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and 0 < rows <= ROWS_MAX
            and weight.shape[1] % 8 == 0)


def gemm_rows_shape(out_features: int, in_features: int, epilogue: str = "store", compute_units: int = 256,
                    rows: int = 1) -> tuple[int, int]:
    """(waves that share K, rows of W per workgroup), measured inside whole decode steps on the
    TinyLlama shapes: about four thousand waves in all, 4 to 16 a workgroup (11264 rows: 4 waves a
    strip of 16, 1.15 ms a step against 1.25 with 8; 2560 rows: 16 waves, against 8 another 0.03 ms
    less); strips of 8 rows where 16 waves on strips of 16 are still too few and K is long
    (2048 rows, K = 5632).  Two strips a workgroup and 2 waves gained nothing at these sizes.
    Where strips of 16 rows leave compute units without a workgroup and the product's result feeds
    no norm (whose partial sums would grow in number with the workgroups), the rows are shared out
    evenly over the units instead: 2560 rows on 256 workgroups of 10 rather than 160 of 16, 0.7%
    of a step at batch 1 and 8; the same for the output projection (residual and norm sums) measured
    0.5% slower.
    With 8 rows of x and more, a workgroup's part of x weighs half as much as its 16 rows of W and
    more (both come through the L2): large matrices then take two strips a workgroup, which halves
    that share (Llama-3-8B's output head at 8 rows 239 -> 209 us, at 16 rows 269 -> 229; its gate/up
    61 -> 58, its q/k/v with 8 waves 17.7 -> 16.6; TinyLlama's head at 16 rows 37.6 -> 34.0)."""
    strips = (out_features + 15) // 16
    waves = 4
    while waves < 16 and strips * waves * 2 <= 4096 and in_features >= waves * 2 * 64:
        waves *= 2
    rows_per_block = 8 if (waves == 16 and strips * 16 < 3072 and in_features > 4096) else 16
    if waves == 16 and rows_per_block == 16 and epilogue in ("store", "rope") and compute_units // 2 < strips < compute_units:
        rows_per_block = max(8, (-(-out_features // compute_units) + 1) // 2 * 2)
    if rows >= 8 and ((waves == 4 and strips * rows >= 14336) or (waves == 8 and in_features >= 4096 and strips >= compute_units)):
        rows_per_block = 32
    return waves, rows_per_block


@dataclass
class RopeTarget:
    """What the rotation and cache write need besides the q/k/v product: see `rope_cache`."""
    positions: torch.Tensor
    slot_map: torch.Tensor
    inv_freq: torch.Tensor | None
    rot_dim: int
    cache: torch.Tensor
    num_heads: int
    num_kv_heads: int
    head_dim: int


def gemm_rows(x, weight: torch.Tensor, bias: torch.Tensor | None, epilogue: str = "store",
              residual: torch.Tensor | None = None, next_norm: tuple | None = None, waves: int | None = None,
              rows_per_block: int | None = None, rope: RopeTarget | None = None, gate=None):
    """y = x . W^T (+ bias) for at most 16 rows.  x: bfloat16 [M, K], or `NormedRows` (then the
    result's rows are scaled as the norm would have scaled the input).
    epilogue "store": float32 [M, N] as a `Product`.  "silu": W's rows alternate gate and up;
    returns bfloat16 silu(gate) * up [M, N / 2] (gate: (name, alpha, limit) of another gate, see `silu_mul`).  "residual": residual [M, N] += y in place, returns
    a `ResidualUpdated`, with the next norm's inputs when next_norm = (weight [N], eps) is given.
    "rope": W is a fused q/k/v weight with rows in the order of `paired_rows`; q and k are rotated,
    k and v written to the cache (as `rope_cache` does), bfloat16 q [M, nq * d] is returned."""
    scale = x if isinstance(x, NormedRows) else None
    data = scale.xg if scale is not None else x
    _device_tensor(data, "x", torch.bfloat16)
    _device_tensor(weight, "weight", torch.bfloat16)
    if data.dim() != 2 or weight.dim() != 2 or data.shape[1] != weight.shape[1]:
        raise invalid_shape(f"gemm_rows: x {list(data.shape)} and weight {list(weight.shape)} do not fit")
    rows, (out_features, in_features) = data.shape[0], weight.shape
    if not gemm_rows_takes(rows, weight, data.dtype):
        raise invalid_argument(f"gemm_rows takes 1..{ROWS_MAX} rows of bfloat16 and an inner size that is a multiple of 8")
    if bias is not None:
        _device_tensor(bias, "bias", torch.bfloat16)
        if bias.shape != (out_features,):
            raise invalid_shape("gemm_rows: bias needs one entry per output")
    ssq_in, strips_in, eps = None, 0, 0.0
    if scale is not None:
        _device_tensor(scale.ssq, "ssq", torch.float32)
        if scale.ssq.dim() != 2 or scale.ssq.shape[1] != 16 or scale.ssq.shape[0] == 0:
            raise invalid_shape(f"gemm_rows: ssq {list(scale.ssq.shape)} is not [parts, 16]")
        ssq_in, strips_in, eps = scale.ssq, scale.ssq.shape[0], float(scale.eps)
    default_waves, default_rows = gemm_rows_shape(out_features, in_features, epilogue, _compute_units(data.device), rows)
    waves, rows_per_block = waves or default_waves, rows_per_block or default_rows
    if epilogue == "silu" and rows_per_block % 2 != 0:
        raise invalid_argument("gemm_rows: a gate and its up must fall into one block")
    device = data.device
    y = act = xg = ssq_out = next_weight = None
    next_code = BF16
    if epilogue == "store":
        code = 0
        y = torch.empty((rows, out_features), dtype=torch.float32, device=device)
    elif epilogue == "silu":
        code = 1
        if out_features % 2 != 0:
            raise invalid_shape("gemm_rows: the gated product needs an even number of rows of W")
        act = torch.empty((rows, out_features // 2), dtype=torch.bfloat16, device=device)
    elif epilogue == "residual":
        code = 2
        _device_tensor(residual, "residual", torch.float32)
        if residual.shape != (rows, out_features):
            raise invalid_shape(f"gemm_rows: residual {list(residual.shape)} is not [{rows}, {out_features}]")
        if next_norm is not None:
            next_weight = next_norm[0]
            _device_tensor(next_weight, "next norm weight", (torch.bfloat16, torch.float32))
            if next_weight.shape != (out_features,):
                raise invalid_shape("gemm_rows: the next norm's weight needs one entry per output")
            next_code = dtype_code(next_weight.dtype)
            xg = torch.empty((rows, out_features), dtype=torch.bfloat16, device=device)
            parts = (out_features + rows_per_block - 1) // rows_per_block * max(1, rows_per_block // 16)
            ssq_out = torch.empty((parts, 16), dtype=torch.float32, device=device)
    elif epilogue == "rope":
        code = 3
        if rope is None:
            raise invalid_argument("gemm_rows: the rotation epilogue needs a RopeTarget")
        _device_tensor(rope.positions, "positions", torch.int32)
        _device_tensor(rope.slot_map, "slot_map", torch.int32)
        _device_tensor(rope.cache, "cache", torch.bfloat16)
        if out_features != (rope.num_heads + 2 * rope.num_kv_heads) * rope.head_dim:
            raise invalid_shape(f"gemm_rows: {out_features} rows of W are not (nq + 2 nkv) * d")
        if rope.positions.shape != (rows,) or rope.slot_map.shape != (rows,):
            raise invalid_shape("gemm_rows: positions and slot_map need one entry per token")
        page_size = _check_cache(rope.cache, rope.num_kv_heads, rope.head_dim, "gemm_rows")
        rot_dim = rope.rot_dim if rope.inv_freq is not None else 0
        if rope.inv_freq is not None:
            _device_tensor(rope.inv_freq, "inv_freq", torch.float32)
            if rot_dim % 2 != 0 or not 0 < rot_dim <= rope.head_dim or rope.inv_freq.shape != (rot_dim // 2,):
                raise invalid_shape("gemm_rows: inv_freq needs rot_dim / 2 entries, rot_dim even and at most d")
        if rope.head_dim % 2 != 0:
            raise invalid_shape("gemm_rows: the rotation epilogue needs an even head size")
        q_out = torch.empty((rows, rope.num_heads * rope.head_dim), dtype=torch.bfloat16, device=device)
    else:
        raise invalid_argument(f"gemm_rows: unknown epilogue '{epilogue}'")
    if rope is None or epilogue != "rope":
        rope_args = (_ptr(None), _ptr(None), _ptr(None), 0, 0, 0, 0, 0, _ptr(None), _ptr(None))
    else:
        rope_args = (_ptr(rope.positions), _ptr(rope.slot_map), _ptr(rope.inv_freq), rot_dim, rope.num_heads,
                     rope.num_kv_heads, rope.head_dim, page_size, _ptr(q_out), _ptr(rope.cache))
    _check(library().tlie_gemm_rows(_ptr(data), _ptr(weight), _ptr(bias), rows, out_features, in_features, _ptr(ssq_in),
                                    strips_in, in_features, ctypes.c_float(eps), code, _ptr(y), _ptr(act), _ptr(residual),
                                    _ptr(next_weight), next_code, _ptr(xg), _ptr(ssq_out), *rope_args, waves, rows_per_block,
                                    *_gate_args(gate if epilogue == "silu" else None), _stream()), "gemm_rows")
    if epilogue == "rope":
        return q_out
    if epilogue == "store":
        return Product(y, 1)
    if epilogue == "silu":
        return act
    return ResidualUpdated(NormedRows(xg, ssq_out, float(next_norm[1])) if next_norm is not None else None)


def embed_rows(tokens: torch.Tensor, table: torch.Tensor, next_norm: tuple):
    """The embedding for at most 16 tokens with the first norm's inputs: returns (float32
    residual [T, hidden], NormedRows)."""
    _device_tensor(tokens, "tokens", torch.int32)
    _device_tensor(table, "embedding table", (torch.float32, torch.bfloat16))
    next_weight, next_eps = next_norm
    _device_tensor(next_weight, "next norm weight", (torch.bfloat16, torch.float32))
    if tokens.dim() != 1 or table.dim() != 2 or next_weight.shape != (table.shape[1],) or not 0 < tokens.shape[0] <= ROWS_MAX:
        raise invalid_shape("embed_rows takes 1..16 tokens, a table [vocab, hidden] and a norm weight [hidden]")
    count, hidden = tokens.shape[0], table.shape[1]
    residual = torch.empty((count, hidden), dtype=torch.float32, device=table.device)
    xg = torch.empty((count, hidden), dtype=torch.bfloat16, device=table.device)
    ssq = torch.empty(((hidden + 15) // 16, 16), dtype=torch.float32, device=table.device)
    _check(library().tlie_embed_rows(_ptr(tokens), _ptr(table), dtype_code(table.dtype), _ptr(residual), _ptr(next_weight),
                                     dtype_code(next_weight.dtype), _ptr(xg), _ptr(ssq), count, hidden, _stream()),
           "embed_rows")
    return residual, NormedRows(xg, ssq, float(next_eps))


# ---- the machine's own ceilings ---------------------------------------------------------------------
def measured_peaks(device="cuda:0", repeats: int = 5) -> dict:
    """What this GPU delivers to kernels that do nothing else: GB/s of a streaming read of 2 GiB
    (workgroups of 512 threads, four a compute unit, eight 16-byte loads in flight a thread) and
    TFLOP/s of chains of bfloat16 matrix instructions (32 x 32 x 16, eight independent chains a wave,
    eight waves a compute unit); the best of `repeats` timed launches each, after one warm-up."""
    device = torch.device(device)
    units = int(torch.cuda.get_device_properties(device).multi_processor_count)
    sink = torch.zeros(4, dtype=torch.float32, device=device)
    data = torch.empty(1 << 31, dtype=torch.uint8, device=device)
    data.fill_(1)
    blocks = 4 * units
    lib = library()
    lib.tlie_probe_stream_read_bytes.restype = ctypes.c_ulonglong
    read_bytes = lib.tlie_probe_stream_read_bytes(ctypes.c_ulonglong(data.numel()), blocks)
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best_read = best_mfma = None
    iterations, mfma_blocks = 4096, 2 * units
    for run in range(repeats + 1):
        start.record()
        _check(lib.tlie_probe_stream_read(_ptr(data), ctypes.c_ulonglong(data.numel()), blocks, _ptr(sink), _stream()), "probe_stream_read")
        stop.record()
        stop.synchronize()
        seconds = start.elapsed_time(stop) / 1e3
        if run > 0:
            best_read = seconds if best_read is None else min(best_read, seconds)
        start.record()
        _check(lib.tlie_probe_mfma_bf16(iterations, mfma_blocks, _ptr(sink), _stream()), "probe_mfma_bf16")
        stop.record()
        stop.synchronize()
        seconds = start.elapsed_time(stop) / 1e3
        if run > 0:
            best_mfma = seconds if best_mfma is None else min(best_mfma, seconds)
    flops = mfma_blocks * 4 * 8 * iterations * 32768.0
    return {"stream_read_gbs": read_bytes / best_read / 1e9, "mfma_bf16_tflops": flops / best_mfma / 1e12}
