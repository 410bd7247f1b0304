"""A plain implementation of the Tugalix decoder, for tests: one function per mechanism, float64, whole
sequences at once (no cache, no state carried between calls, no batching), written from the design's
equations and sharing nothing with the engine.

A model is (config, weights): `config` is the config.json dict, `weights` a dict of float64 tensors by the
checkpoint's names.  `forward(config, weights, tokens)` returns the logits of every position and the residual
stream after every layer.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.nn.functional.softplus(torch.as_tensor(z, dtype=F64))


def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x, weight, bias, eps):
    mean = x.mean(dim=-1, keepdim=True)
    variance = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) / torch.sqrt(variance + eps) * weight + bias


def input_convolution(h, taps_weight):
    """h: [T, width], taps_weight: [width, taps].  h + conv(h); tap j of a channel weighs the input
    taps - 1 - j tokens back, and what lies before the sequence is zero."""
    T, taps = h.shape[0], taps_weight.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            source = t - taps + 1 + j
            if source >= 0:
                out[t] += taps_weight[:, j] * h[source]
    return out


def rotate_halves(x, positions, dims, base):
    """x: [T, heads, dim].  Of the first `dims` dims of every head, dim i turns with dim i + dims / 2 by the
    angle position * base^(-2i / dims); the rest pass."""
    out = x.clone()
    half = dims // 2
    for i in range(half):
        angle = positions.to(F64) * base ** (-2.0 * i / dims)
        cos, sin = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * cos - v * sin
        out[..., i + half] = v * cos + u * sin
    return out


def xielu(z, p, q):
    """For z > 0: softplus(p) z^2 + z / 2; else (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2."""
    positive = softplus(p) * z * z + 0.5 * z
    negative = (0.5 + softplus(q)) * (torch.expm1(z) - z) + 0.5 * z
    return torch.where(z > 0, positive, negative)


def dense_feed_forward(w, prefix, h):
    act = w[prefix + "act"]
    return xielu(h @ w[prefix + "up"].T, act[0], act[1]) @ w[prefix + "down"].T


# ---- linear attention with a decaying matrix state ------------------------------------------------------
def decayed_state_walk(q, k, v, decay, bonus=None):
    """One head.  q, k, decay: [T, dim] (decay per key channel and token), v: [T, vdim].
    Without bonus: S_t = diag(decay_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.
    With bonus u [dim]: o_t = (S_(t-1) + diag(u) k_t v_t^T)^T q_t, and then the same update of S."""
    T, dim = q.shape
    S = torch.zeros(dim, v.shape[1], dtype=F64)
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for t in range(T):
        outer = k[t][:, None] * v[t][None, :]
        if bonus is not None:
            out[t] = (S + bonus[:, None] * outer).T @ q[t]
            S = decay[t][:, None] * S + outer
        else:
            S = decay[t][:, None] * S + outer
            out[t] = S.T @ q[t]
    return out


def retention(mixer, w, prefix, h, positions, eps):
    H, dim, vdim = mixer["heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    q = (h @ w[prefix + "q"].T).reshape(T, H, dim)
    k = (h @ w[prefix + "k"].T).reshape(T, H, dim)
    v = (h @ w[prefix + "v"].T).reshape(T, H, vdim)
    rot = mixer["rot"]
    q = rotate_halves(q, positions, int(rot["dims"]), float(rot["base"]))
    k = rotate_halves(k, positions, int(rot["dims"]), float(rot["base"])) * dim ** -0.5
    heads = []
    for head in range(H):
        decay = torch.full((T, dim), float(mixer["decay"][head]), dtype=F64)
        heads.append(unit_rms(decayed_state_walk(q[:, head], k[:, head], v[:, head], decay), eps))
    joined = torch.cat(heads, dim=-1) * silu(h @ w[prefix + "g"].T)
    return joined @ w[prefix + "o"].T


def gated_linear_attention(mixer, w, prefix, h, eps):
    H, dim, vdim, tau = mixer["heads"], mixer["dim"], mixer["vdim"], float(mixer["tau"])
    T = h.shape[0]
    q = (h @ w[prefix + "q"].T).reshape(T, H, dim) * dim ** -0.5
    k = (h @ w[prefix + "k"].T).reshape(T, H, dim)
    v = (h @ w[prefix + "v"].T).reshape(T, H, vdim)
    z = (h @ w[prefix + "a1"].T) @ w[prefix + "a2"].T + w[prefix + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / tau)).reshape(T, H, dim)
    heads = []
    for head in range(H):
        o = decayed_state_walk(q[:, head], k[:, head], v[:, head], alpha[:, head])
        heads.append(unit_rms(o, eps) * w[prefix + "norm"])
    joined = torch.cat(heads, dim=-1) * silu(h @ w[prefix + "g"].T)
    return joined @ w[prefix + "o"].T


def softmax_attention(mixer, w, prefix, h, positions):
    """Grouped causal softmax attention with value heads of their own size."""
    H, G, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    q = (h @ w[prefix + "q"].T).reshape(T, H, dim)
    k = (h @ w[prefix + "k"].T).reshape(T, G, dim)
    v = (h @ w[prefix + "v"].T).reshape(T, G, vdim)
    rot = mixer["rot"]
    q = rotate_halves(q, positions, int(rot["dims"]), float(rot["base"]))
    k = rotate_halves(k, positions, int(rot["dims"]), float(rot["base"]))
    visible = torch.ones(T, T, dtype=torch.bool).tril()
    heads = []
    for head in range(H):
        group = head // (H // G)
        scores = (q[:, head] @ k[:, group].T) * float(mixer["scale"])
        scores = scores.masked_fill(~visible, -math.inf)
        heads.append(torch.softmax(scores, dim=-1) @ v[:, group])
    return torch.cat(heads, dim=-1) @ w[prefix + "o"].T


def token_shift_mixing(mixer, w, prefix, h, eps):
    """Time mixing with a token shift: every projection reads its own blend of a token's input and the one before."""
    H, dim = mixer["heads"], mixer["dim"]
    T = h.shape[0]
    before = torch.cat([torch.zeros(1, h.shape[1], dtype=F64), h[:-1]], dim=0)

    def blend(name):
        return h + (before - h) * w[prefix + "mu." + name]
    r = (blend("r") @ w[prefix + "r"].T).reshape(T, H, dim)
    k = (blend("k") @ w[prefix + "k"].T).reshape(T, H, dim)
    v = (blend("v") @ w[prefix + "v"].T).reshape(T, H, dim)
    gate = silu(blend("g") @ w[prefix + "g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(blend("w") @ w[prefix + "w1"].T) @ w[prefix + "w2"].T + w[prefix + "w0"])).reshape(T, H, dim)
    heads = []
    for head in range(H):
        o = decayed_state_walk(r[:, head], k[:, head], v[:, head], decay[:, head], bonus=w[prefix + "u"][head])
        heads.append(unit_rms(o, eps))
    joined = torch.cat(heads, dim=-1) * w[prefix + "norm"] * gate
    return joined @ w[prefix + "o"].T


def side_by_side(mixer, w, prefix, h, positions, eps):
    left = softmax_attention(mixer["left"], w, prefix + "left.", h, positions)
    right = token_shift_mixing(mixer["right"], w, prefix + "right.", h, eps)
    return float(mixer["left_scale"]) * left + float(mixer["right_scale"]) * right


def mixer_output(layer, w, prefix, h, positions, eps):
    kind, mixer = layer["type"], layer["mixer"]
    if kind == "retention":
        return retention(mixer, w, prefix, h, positions, eps)
    if kind == "gla":
        return gated_linear_attention(mixer, w, prefix, h, eps)
    if kind == "parallel":
        return side_by_side(mixer, w, prefix, h, positions, eps)
    raise ValueError(kind)


def forward(config, w, tokens):
    """tokens: a list of ids.  Returns (logits [T, vocab], [the residual stream after every layer, each [T, width]])."""
    eps = float(config["norm"]["eps"])
    positions = torch.arange(len(tokens))
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = layer_norm(x, w["embed.norm"], w["embed.norm.b"], eps)
    results = [x]               # the embedding's output, then every layer's own result
    after = []
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}."
        h = input_convolution(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps), w[p + "canon1"])
        x = x + mixer_output(layer, w, p + "mix.", h, positions, eps)
        if layer.get("mlp") is not None:
            h = input_convolution(layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps), w[p + "canon2"])
            x = x + dense_feed_forward(w, p + "mlp.", h)
        results.append(x)
        x = sum(w[p + "dwa"][j] * results[j] for j in range(index + 2))
        after.append(x)
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return (x @ w["head"].T) * float(config["logit_scale"]), after
