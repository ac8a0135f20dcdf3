"""Bonerax computed plainly: whole sequences, float64, no cache, one function a mechanism.

This file shares no code with `llmx_amd`; it reads a configuration (a dict with config.json's keys) and a dict of numpy
arrays by the model folder's tensor names.  Notation: T tokens, E the model's width, H heads, G key heads, D key
width, V value width; weights are [out, in] and applied as x @ W.T.

A layer:      x <- x + LN(mixer(x)) ; x <- x + LN(ff(x))       (the sublayers read x itself; LN has a weight, no bias)
Mixers:       "gla" (gated linear attention), "channel_delta" (delta rule with a decay a key channel),
              "parallel" (windowed softmax attention and a delta rule side by side, a weighted sum of both)
Feed-forward: dense SwiGLU, or top-k routed SwiGLU experts with softmax weights over the picked logits
Output:       LN, head, logits * scale, cap * tanh(logits / cap)
"""

from __future__ import annotations

import math

import numpy as np


# ---------------------------------------------------------------------------- small pieces
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * w over the last axis."""
    mu = x.mean(axis=-1, keepdims=True)
    dev = x - mu
    return dev / np.sqrt((dev * dev).mean(axis=-1, keepdims=True) + eps) * w


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


# ---------------------------------------------------------------------------- rotation
def rotary_frequencies(dims, base, scaling):
    """(frequency of each of the dims/2 pairs, the factor on cos and sin).  Pair i turns by base^(-2i/dims) a position;
    with scaling {factor, original, fast, slow} slow pairs are slowed down by `factor`, fast ones kept, and a ramp over
    the pair index blends between the two."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = float(base) ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def pair_that_turns(times):
        return dims * math.log(original / (2.0 * math.pi * times)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_that_turns(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_that_turns(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, dims, base, scaling):
    """x [T, heads, D]: dims (2i, 2i+1), i < dims/2, of every head turn by positions * f_i; the rest pass."""
    if dims == 0:
        return x
    f, magnitude = rotary_frequencies(dims, base, scaling)
    angle = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]          # [T, dims/2]
    c, s = np.cos(angle)[:, None, :] * magnitude, np.sin(angle)[:, None, :] * magnitude
    out = x.copy()
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ---------------------------------------------------------------------------- windowed softmax attention
def window_attention(h, w, m, eps, positions=None):
    """h [T, E]; w: tensors by their short names (q, q.b, k, k.b, v, v.b, q.norm, k.norm, o, o.b); m: the mixer's sizes."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = np.arange(T) if positions is None else np.asarray(positions)
    q = (h @ w["q"].T + w["q.b"]).reshape(T, H, D)
    k = (h @ w["k"].T + w["k.b"]).reshape(T, G, D)
    v = (h @ w["v"].T + w["v.b"]).reshape(T, G, V)
    q = rms_unit(q, eps) * w["q.norm"]
    k = rms_unit(k, eps) * w["k.norm"]
    rot = m["rot"]
    q = rotate_pairs(q, pos, rot["dims"], rot["base"], rot.get("scaling"))
    k = rotate_pairs(k, pos, rot["dims"], rot["base"], rot.get("scaling"))
    size = m["mask"]["size"]
    out = np.zeros((T, H, V))
    for head in range(H):
        g = head // (H // G)
        for t in range(T):
            lo = max(0, t - size + 1)
            s = (k[lo:t + 1, g] @ q[t, head]) * m["scale"]
            p = np.exp(s - s.max())
            out[t, head] = (p / p.sum()) @ v[lo:t + 1, g]
    return out.reshape(T, H * V) @ w["o"].T + w["o.b"]


# ---------------------------------------------------------------------------- recurrences
def short_conv_silu(x, taps_w):
    """x [T, C]; taps_w [C, taps], the last column weighs the current token; zeros before the start; then silu."""
    T, C = x.shape
    taps = taps_w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), x], axis=0)
    y = np.zeros((T, C))
    for j in range(taps):
        y += padded[j:j + T] * taps_w[:, j]
    return silu(y)


def delta_rule_scan(q, k, v, decay, beta):
    """q, k [T, H, D], v [T, H, V], decay [T, H, D], beta [T, H] -> o [T, H, V].
    S <- decay * S (rows are key channels); u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, D = q.shape
    V = v.shape[2]
    S = np.zeros((H, D, V))
    o = np.zeros((T, H, V))
    for t in range(T):
        for head in range(H):
            S[head] *= decay[t, head][:, None]
            u = beta[t, head] * (v[t, head] - S[head].T @ k[t, head])
            S[head] += np.outer(k[t, head], u)
            o[t, head] = S[head].T @ q[t, head]
    return o


def channel_delta(h, w, m, eps):
    """The delta-rule mixer.  w: q, q.conv, k, k.conv, v, v.conv, b, A_log, norm, a1, a2, dt_bias, g1, g2, o."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(h @ w["q"].T, w["q.conv"]).reshape(T, G, D)
    k = short_conv_silu(h @ w["k"].T, w["k.conv"]).reshape(T, G, D)
    v = short_conv_silu(h @ w["v"].T, w["v.conv"]).reshape(T, H, V)
    q = q / np.sqrt((q * q).sum(axis=-1, keepdims=True) + 1e-6) * D ** -0.5
    k = k / np.sqrt((k * k).sum(axis=-1, keepdims=True) + 1e-6)
    share = H // G
    q = np.repeat(q, share, axis=1)
    k = np.repeat(k, share, axis=1)
    beta = sigmoid(h @ w["b"].T)                                                            # [T, H]
    step = softplus((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).reshape(T, H, D)
    decay = np.exp(-np.exp(w["A_log"])[None, :, None] * step)
    o = delta_rule_scan(q, k, v, decay, beta)
    gate = sigmoid((h @ w["g1"].T) @ w["g2"].T).reshape(T, H, V)
    o = rms_unit(o, eps) * w["norm"] * gate
    return o.reshape(T, H * V) @ w["o"].T


def gla(h, w, m, eps):
    """Gated linear attention.  w: q, k, v, g, o, norm, a1, a2, a2.b.  S_t = diag(alpha_t) S_(t-1) + k_t v_t^T; o_t = S_t^T q_t."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ w["k"].T).reshape(T, H, D)
    v = (h @ w["v"].T).reshape(T, H, V)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, D)
    S = np.zeros((H, D, V))
    o = np.zeros((T, H, V))
    for t in range(T):
        S = S * alpha[t][:, :, None] + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    o = rms_unit(o, eps) * w["norm"]
    return (o.reshape(T, H * V) * silu(h @ w["g"].T)) @ w["o"].T


def parallel_mixer(h, w, m, eps):
    left = window_attention(h, {k[len("left."):]: v for k, v in w.items() if k.startswith("left.")}, m["left"], eps)
    right = channel_delta(h, {k[len("right."):]: v for k, v in w.items() if k.startswith("right.")}, m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


# ---------------------------------------------------------------------------- feed-forward
def glu(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def routed_experts(h, w, mlp, picks_out=None, picks_in=None):
    """w: router, router.b, e<i>.gate / up / down.  The `top` largest logits pick; weights are their softmax.
    `picks_in` [T, top] replaces the choice (not the weights): a comparison with an implementation that rounds elsewhere
    hands its picks over, so that a near tie that fell the other way does not count as a difference."""
    z = h @ w["router"].T + w["router.b"]
    top = mlp["router"]["top"]
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        ids = sorted(range(z.shape[1]), key=lambda e: (-z[t, e], e))[:top] if picks_in is None else [int(e) for e in picks_in[t]]
        p = np.exp(z[t, ids] - z[t, ids].max())
        p /= p.sum()
        if picks_out is not None:
            picks_out.append(ids)
        for weight, e in zip(p, ids):
            out[t] += weight * glu(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    return out


# ---------------------------------------------------------------------------- the model
def under(tensors, prefix):
    return {k[len(prefix):]: np.asarray(v, dtype=np.float64) for k, v in tensors.items() if k.startswith(prefix)}


def forward(config, tensors, tokens, residuals=None, picks=None):
    """Logits [T, vocab] of one sequence.  `residuals`, a list, receives x after every layer run; `picks`, a list with one
    [T, top] array for every routed layer run in order, replaces the routers' choices."""
    picks = list(picks) if picks is not None else None
    eps = config["norm"]["eps"]
    x = np.asarray(tensors["embed"], dtype=np.float64)[np.asarray(tokens)]
    for i, layer in enumerate(config["layers"]):
        src = layer.get("weights_of", i)
        p = f"l{src}."
        mix = under(tensors, p + "mix.")
        kind = layer["type"]
        if kind == "gla":
            y = gla(x, mix, layer["mixer"], eps)
        elif kind == "channel_delta":
            y = channel_delta(x, mix, layer["mixer"], eps)
        elif kind == "parallel":
            y = parallel_mixer(x, mix, layer["mixer"], eps)
        else:
            raise ValueError(f"layer type {kind!r}")
        x = x + layer_norm(y, np.asarray(tensors[p + "norm1"], dtype=np.float64), eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            ff = under(tensors, p + "mlp.")
            if mlp["kind"] == "dense":
                y = glu(x, ff["gate"], ff["up"], ff["down"])
            else:
                y = routed_experts(x, ff, mlp, picks_in=picks.pop(0) if picks is not None else None)
            x = x + layer_norm(y, np.asarray(tensors[p + "norm2"], dtype=np.float64), eps)
        if residuals is not None:
            residuals.append(x.copy())
    x = layer_norm(x, np.asarray(tensors["final.norm"], dtype=np.float64), eps)
    logits = x @ np.asarray(tensors["head"], dtype=np.float64).T * config["logit_scale"]
    cap = config.get("logit_softcap")
    return cap * np.tanh(logits / cap) if cap else logits
