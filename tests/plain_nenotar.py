"""The plain implementation of the Nenotar design: whole sequences, no cache, no batching, one function a mechanism.

torch on the CPU as a calculator, float64 by default.  It shares no code with llmx_amd: config.json is read with `json`
and the weights with the `safetensors` package.  Notation: T tokens, E the model's width, a linear weight W is stored
[out, in] and applied as x @ W^T.

`round_to=torch.bfloat16` rounds the inputs of weight products and what the serving path keeps in bfloat16 (the cached
latent and rotated key part, the queries, the attention output); norms, scores, softmax, the recurrence, gates of the
recurrence and the residual stay in `dtype`.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def load_folder(folder):
    """(config dict, {name: tensor}) of a model folder."""
    from safetensors import safe_open
    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    weights = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name)
    return config, weights


def _r(x, round_to):
    return x if round_to is None else x.to(round_to).to(x.dtype)


def linear(x, w, round_to=None):
    return _r(x, round_to) @ w.to(x.dtype).T


# ---------------------------------------------------------------------------
def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(x):
    return torch.log1p(torch.exp(-x.abs())) + torch.clamp(x, min=0.0)


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2; z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def rotary_frequencies(rot: dict):
    """(frequencies [dims/2] float64, factor on cos and sin) with the YaRN blend when rot has `scaling`."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x, positions, rot: dict):
    """x [T, ..., D]: dims (2i, 2i+1), i < dims/2, of the last axis turn by positions[t] * f_i; the rest pass."""
    dims = int(rot["dims"])
    f, mag = rotary_frequencies(rot)
    angle = (torch.as_tensor(positions, dtype=torch.float32)[:, None] * f.float()[None, :]).double()   # 32-bit angles
    cos, sin = (torch.cos(angle) * mag).to(x.dtype), (torch.sin(angle) * mag).to(x.dtype)
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    cos, sin = cos.view(shape), sin.view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ---------------------------------------------------------------------------
def mingru(h, w, prefix, m, round_to=None, state=None):
    """S_t = (1 - z_t) S_(t-1) + z_t c_t from S_(-1) = state or 0; out = W_o (S_t * silu(W_g h_t))."""
    z = torch.sigmoid(linear(h, w[prefix + "z"], round_to) + w[prefix + "z.b"].to(h.dtype))
    u = linear(h, w[prefix + "x"], round_to) + w[prefix + "x.b"].to(h.dtype)
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(int(m["width"]), dtype=h.dtype) if state is None else state.clone()
    rows = []
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        rows.append(S)
    S_all = torch.stack(rows)
    g = linear(h, w[prefix + "g"], round_to)
    return linear(S_all * (g * torch.sigmoid(g)), w[prefix + "o"], round_to), S


def latent_attention(h, w, prefix, m, eps, positions, round_to=None):
    """Causal softmax attention whose keys and values are expanded from one cached latent a token."""
    T = h.shape[0]
    H, D, R, V, C = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    q = linear(h, w[prefix + "q"], round_to).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], rotate_interleaved(q[..., D:], positions, m["rot"])
    down = linear(h, w[prefix + "dkv"], round_to)
    c = _r(rms(down[:, :C], eps) * w[prefix + "dkv.norm"].to(h.dtype), round_to)
    k_rot = _r(rotate_interleaved(down[:, C:], positions, m["rot"]), round_to)          # one for all heads
    k_plain = linear(c, w[prefix + "uk"]).view(T, H, D)
    v = linear(c, w[prefix + "uv"]).view(T, H, V)
    q_plain, q_rot = _r(q_plain, round_to), _r(q_rot, round_to)
    scores = (torch.einsum("thd,shd->hts", q_plain, k_plain) + torch.einsum("thr,sr->hts", q_rot, k_rot)) * float(m["scale"])
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    scores = scores.masked_fill(~mask, float("-inf"))
    p = torch.softmax(scores, dim=-1)
    o = torch.einsum("hts,shv->thv", p, v)
    gate = torch.sigmoid(linear(h, w[prefix + "g"], round_to))                            # [T, H]
    o = o * gate[:, :, None]
    return linear(o.reshape(T, H * V), w[prefix + "o"], round_to)


def dense_ff(h, w, prefix, round_to=None):
    a = w[prefix + "act"].to(h.dtype)
    return linear(xielu(linear(h, w[prefix + "up"], round_to), a[0], a[1]), w[prefix + "down"], round_to)


def token_side(x, tokens, w, layer, dim, eps, round_to=None):
    """x + rms(side.proj(gelu_tanh(side.gate x) * e)) * side.norm, e the layer's part of the side table's row."""
    p = f"l{layer}.side."
    e = w["side.embed"][tokens][:, layer * dim:(layer + 1) * dim].to(x.dtype)
    g = gelu_tanh(linear(x, w[p + "gate"], round_to)) * e
    y = linear(g, w[p + "proj"], round_to)
    return x + rms(y, eps) * w[p + "norm"].to(x.dtype)


def forward(config, w, tokens, dtype=torch.float64, round_to=None, layers_out=None):
    """Logits [T, vocab] of one sequence from position 0; `layers_out` (a list) receives the residual after every layer."""
    eps = float(config["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = list(range(len(tokens)))
    x = w["embed"][tokens].to(dtype) * float(config["embedding"]["scale"])
    side = config.get("token_side")
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h1 = rms(x, eps) * w[p + "norm1"].to(dtype)
        if layer["type"] == "mingru":
            y, _ = mingru(h1, w, p + "mix.", layer["mixer"], round_to)
        elif layer["type"] == "latent_attention":
            y = latent_attention(h1, w, p + "mix.", layer["mixer"], eps, positions, round_to)
        else:
            raise ValueError(layer["type"])
        y = y * w[p + "ls1"].to(dtype)
        if layer.get("mlp"):
            h2 = rms(x, eps) * w[p + "norm2"].to(dtype)
            y = y + dense_ff(h2, w, p + "mlp.", round_to) * w[p + "ls2"].to(dtype)
        x = x + y
        if side:
            x = token_side(x, tokens, w, i, int(side["dim"]), eps, round_to)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms(x, eps) * w["final.norm"].to(dtype)
    return linear(x, w["head"], round_to)


def greedy(config, w, prompt, n_new, dtype=torch.float64):
    tokens = list(prompt)
    out = []
    for _ in range(n_new):
        logits = forward(config, w, tokens, dtype)
        t = int(torch.argmax(logits[-1]))
        out.append(t)
        tokens.append(t)
    return out
