"""A plain implementation of the Narolorn decoder, for tests: one function per mechanism, float64, whole
sequences at once (no cache, no state carried between calls, no batching), written from the design's
equations and sharing nothing with the engine.

A model is (config, weights): `config` is the config.json dict, `weights` a dict of float64 tensors by the
checkpoint's names.  `forward(config, weights, tokens)` returns the logits of every position and the residual
stream (the sum of the streams) after every layer run.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


# ---- who sees whom --------------------------------------------------------------------------------------
def visible(T, window=None, chunk=None):
    """[T, T] booleans: row i sees column j.  Causal; with a window only the last `window` positions, itself
    included; with chunks only positions of its own chunk, counted from position 0."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    mask = j <= i
    if window is not None:
        mask &= (i - j) < window
    if chunk is not None:
        mask &= (i // chunk) == (j // chunk)
    return mask


def softmax_attention(q, k, v, scale, mask, softcap=None):
    """q, k: [T, dim], v: [T, vdim]; scores scaled, capped by softcap * tanh(score / softcap) if asked, masked."""
    scores = (q @ k.T) * scale
    if softcap is not None:
        scores = softcap * torch.tanh(scores / softcap)
    scores = scores.masked_fill(~mask, -math.inf)
    return torch.softmax(scores, dim=-1) @ v


# ---- positions ------------------------------------------------------------------------------------------
def rotate_halves(x, positions, dims, base):
    """x: [T, heads, dim].  Of every head's first `dims` dims, dim i turns with dim i + dims / 2 by the angle
    position * base^(-2i / dims); the rest pass."""
    out = x.clone()
    half = dims // 2
    for i in range(half):
        angle = positions.to(F64) * base ** (-2.0 * i / dims)
        cos, sin = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * cos - v * sin
        out[..., i + half] = v * cos + u * sin
    return out


def query_temperature(positions, coef, every):
    """What a query at each position is multiplied by: 1 + coef * ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * torch.log(torch.floor((positions.to(F64) + 1.0) / every) + 1.0)


# ---- mixers ---------------------------------------------------------------------------------------------
def attention(mixer, w, prefix, h, positions, eps):
    """Grouped causal attention without positions in the keys; a capped score; a query temperature."""
    H, G, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    q = (h @ w[prefix + "q"].T).reshape(T, H, dim)
    k = (h @ w[prefix + "k"].T).reshape(T, G, dim)
    v = (h @ w[prefix + "v"].T).reshape(T, G, vdim)
    temp = mixer.get("q_temp")
    if temp is not None:
        q = q * query_temperature(positions, float(temp["coef"]), float(temp["every"]))[:, None, None]
    mask = visible(T)
    cap = mixer.get("softcap")
    heads = [softmax_attention(q[:, head], k[:, head // (H // G)], v[:, head // (H // G)], float(mixer["scale"]), mask,
                               float(cap) if cap is not None else None) for head in range(H)]
    return torch.cat(heads, dim=-1) @ w[prefix + "o"].T


def latent_attention(mixer, w, prefix, h, positions, eps):
    """Keys and values of every head from one normed low-rank vector a position; a sliding window; a gate on
    the heads' results."""
    H, dim, vdim, rank = mixer["heads"], mixer["dim"], mixer["vdim"], mixer["kv_rank"]
    T = h.shape[0]
    q = (h @ w[prefix + "q"].T).reshape(T, H, dim)
    c = rms_norm(h @ w[prefix + "dkv"].T, w[prefix + "dkv.norm"], eps)
    assert c.shape[1] == rank
    k = (c @ w[prefix + "uk"].T).reshape(T, H, dim)
    v = (c @ w[prefix + "uv"].T).reshape(T, H, vdim)
    size = (mixer.get("mask") or {}).get("size")
    mask = visible(T, window=int(size) if size is not None else None)
    heads = [softmax_attention(q[:, head], k[:, head], v[:, head], float(mixer["scale"]), mask) for head in range(H)]
    gated = torch.cat(heads, dim=-1) * torch.sigmoid(h @ w[prefix + "g"].T)
    return gated @ w[prefix + "o"].T


def attention_2(mixer, w, prefix, h, positions, eps):
    """Values are the keys as projected; q and k are normed over their whole width, then turned; chunks."""
    H, G, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    q = h @ w[prefix + "q"].T
    k = h @ w[prefix + "k"].T
    v = k.reshape(T, G, dim)
    assert vdim == dim
    q = rms_norm(q, w[prefix + "q.norm"], eps).reshape(T, H, dim)
    k = rms_norm(k, w[prefix + "k.norm"], eps).reshape(T, G, dim)
    rot = mixer.get("rot")
    if rot is not None:
        q = rotate_halves(q, positions, int(rot["dims"]), float(rot["base"]))
        k = rotate_halves(k, positions, int(rot["dims"]), float(rot["base"]))
    size = (mixer.get("mask") or {}).get("size")
    mask = visible(T, chunk=int(size) if size is not None else None)
    heads = [softmax_attention(q[:, head], k[:, head // (H // G)], v[:, head // (H // G)], float(mixer["scale"]), mask)
             for head in range(H)]
    return torch.cat(heads, dim=-1) @ w[prefix + "o"].T


MIXERS = {"attention": attention, "latent_attention": latent_attention, "attention_2": attention_2}


# ---- feed-forward ---------------------------------------------------------------------------------------
def expert(w, prefix, h, limit):
    g = torch.clamp(h @ w[prefix + "gate"].T, max=limit)
    u = torch.clamp(h @ w[prefix + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[prefix + "down"].T


def router_choice(z, top):
    """z: [T, experts] logits -> (chosen [T, top], weights [T, top]): the largest logits, softmax over them only."""
    values, chosen = torch.topk(z, top, dim=-1)
    return chosen, torch.softmax(values, dim=-1)


def router_margin(z, top):
    """How far each token's choice is from another one: the gap between its `top`-th and its next logit ([T]; infinite
    when all experts are chosen)."""
    if top >= z.shape[-1]:
        return torch.full(z.shape[:-1], math.inf, dtype=z.dtype)
    ordered = torch.sort(z, dim=-1, descending=True).values
    return ordered[..., top - 1] - ordered[..., top]


def mixture(mlp, w, prefix, h, margins=None):
    """margins: a list that takes, per call, every token's `router_margin`."""
    experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h @ w[prefix + "router"].T + w[prefix + "router.b"]
    chosen, weights = router_choice(z, top)
    if margins is not None:
        margins.append(router_margin(z, top))
    out = torch.zeros_like(h)
    for e in range(experts):
        y = expert(w, f"{prefix}e{e}.", h, float(mlp["expert"]["limit"]))
        share = ((chosen == e).to(F64) * weights).sum(dim=-1, keepdim=True)
        out = out + share * y
    shared = mlp.get("shared")
    if shared is not None:
        gate = torch.sigmoid(h @ w[prefix + "shared.sg"].T)          # [T, 1]
        out = out + gate * expert(w, prefix + "shared.", h, float(shared["limit"]))
    return out


# ---- the model ------------------------------------------------------------------------------------------
def run_order(config):
    count = len(config["layers"])
    loop = config.get("loop")
    if loop is None:
        return list(range(count))
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, count))


def hyper_sublayer(streams, w, prefix, sublayer):
    """streams: [S, T, width].  The sublayer reads a weighted sum of the streams; the streams are mixed among
    themselves (mix[from, to]) and each takes its own multiple of the result."""
    u = torch.einsum("s,std->td", w[prefix + "in"], streams)
    y = sublayer(u)
    return torch.einsum("sr,std->rtd", w[prefix + "mix"], streams) + w[prefix + "out"][:, None, None] * y[None]


def forward(config, weights, tokens, margins=None):
    """margins: a list that takes every router's margins, one tensor [T] per feed-forward that runs."""
    w = weights
    eps = float(config["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.shape[0])
    x = w["embed"][tokens]
    count = config.get("streams")
    streams = torch.stack([x] * int(count)) if count is not None else None
    residuals = []
    for index in run_order(config):
        layer = config["layers"][index]
        prefix = f"l{index}."

        def mix(u, layer=layer, prefix=prefix):
            return MIXERS[layer["type"]](layer["mixer"], w, prefix + "mix.", rms_norm(u, w[prefix + "norm1"], eps), positions, eps)

        def feed(u, layer=layer, prefix=prefix):
            return mixture(layer["mlp"], w, prefix + "mlp.", rms_norm(u, w[prefix + "norm2"], eps), margins)
        if streams is not None:
            streams = hyper_sublayer(streams, w, prefix + "hc1.", mix)
            if layer.get("mlp") is not None:
                streams = hyper_sublayer(streams, w, prefix + "hc2.", feed)
            residuals.append(streams.sum(dim=0))
        else:
            x = x + mix(x)
            if layer.get("mlp") is not None:
                x = x + feed(x)
            residuals.append(x)
    x = streams.sum(dim=0) if streams is not None else x
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    cap = config.get("logit_softcap")
    if cap is not None:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits, torch.stack(residuals)
