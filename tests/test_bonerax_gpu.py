"""Bonerax in the engine against the plain implementation (tests/plain_bonerax.py), mechanism by mechanism and whole.

Kernels alone (layer norm and its join, the join of two mixers, logit scale and cap, the delta rule's row preparation with
its convolution tail, the matrix-state scan with and without the delta correction, the gated head norm, the router with a
bias in its logits, the attention step with a norm a head) against the plain functions; then the engine under every way of
cutting the same tokens into steps, which must agree bit for bit with each other in both dtypes, with the plain
implementation within F32_TOL in float32 and within BF16_TOL in bfloat16 (the engine's expert picks handed over); pages and state slots
that are used again; long decoding; weights made so that single keys at a window's edge, or tokens hundreds of steps back,
carry the result; greedy generation through `generate`; the trace replay tool and the command line.
"""

from __future__ import annotations

import copy
import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_bonerax as plain
from bonerax_cases import CONFIGS, PAGES, SEEDS, greedy, load_plain, model_folder, plain_logits, portions, tokens_for, write_folder

pytestmark = pytest.mark.gpu

F32_TOL = 3e-5      # |engine - plain| over all logits relative to the largest |logit|: float32 sums in another order
BF16_TOL = 4e-2     # the serving path against the plain implementation (float64, nothing rounded), with the engine's expert picks
BF16_RMS = 2.5e-2   # ... and the root mean square of all differences relative to that of the logits
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def ops():
    from llmx_amd import ops as o
    return o


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a)).to(device="cuda", dtype=dtype).contiguous()


def close(got, want, tol, what=""):
    got, want = torch.as_tensor(np.asarray(got.cpu() if isinstance(got, torch.Tensor) else got)).double(), torch.as_tensor(np.asarray(want.cpu() if isinstance(want, torch.Tensor) else want)).double()
    err = float((got - want).abs().max()) / max(float(want.abs().max()), 1e-30)
    assert err <= tol, f"{what}: relative error {err:.3e} above {tol:.1e}"
    return err


# ---------------------------------------------------------------------------
# kernels alone
@pytest.mark.parametrize("rows,n", [(1, 8), (5, 54), (3, 1030), (2, 4100)])
def test_layer_norm_its_join_and_the_rounded_copy(rows, n):
    rng = np.random.default_rng(rows * n)
    x, y, w = rng.normal(size=(rows, n)) * 3 + 1.5, rng.normal(size=(rows, n)) * 2 - 0.7, rng.normal(size=n)
    o = ops()
    out, out32 = torch.empty(rows, n, device="cuda", dtype=torch.bfloat16), torch.empty(rows, n, device="cuda")
    o.layernorm(dev(x), dev(w), 1e-5, out, out32)
    close(out32, plain.layer_norm(x, w, 1e-5), 3e-6, "layernorm")
    assert torch.equal(out, out32.to(torch.bfloat16))
    pick = torch.tensor([rows - 1, 0], device="cuda", dtype=torch.int32)
    picked = torch.empty(2, n, device="cuda")
    o.layernorm(dev(x), dev(w), 1e-5, None, picked, pick)
    assert torch.equal(picked, out32[[rows - 1, 0]])
    xd, copy_ = dev(x), torch.empty(rows, n, device="cuda", dtype=torch.bfloat16)
    o.layernorm_add(xd, dev(y), dev(w), 1e-5, copy_)
    close(xd, x + plain.layer_norm(y, w, 1e-5), 3e-6, "layernorm_add")
    assert torch.equal(copy_, xd.to(torch.bfloat16))
    cast = torch.empty(rows, n, device="cuda", dtype=torch.bfloat16)
    o.cast_rows(xd, cast)
    assert torch.equal(cast, copy_)


def test_join_of_two_results_and_logit_cap():
    rng = np.random.default_rng(7)
    a, b, bias = rng.normal(size=(5, 37)), rng.normal(size=(5, 37)), rng.normal(size=37)
    o = ops()
    out = torch.full((5, 37), 2.0, device="cuda")
    o.combine_rows(out, dev(a), 0.8, dev(bias), dev(b), -1.5)
    close(out, 0.8 * (a + bias) - 1.5 * b, 1e-6)
    o.combine_rows(out, dev(a), 1.0, None, None, 1.0, accumulate=True)
    close(out, 0.8 * (a + bias) - 1.5 * b + a, 1e-6)
    z = dev(rng.normal(size=(3, 50)) * 40)
    want = 9.0 * np.tanh(z.cpu().double().numpy() * 0.7 / 9.0)
    o.scale_softcap(z, 0.7, 9.0)
    close(z, want, 1e-6)
    z2 = dev(np.ones((2, 4)))
    o.scale_softcap(z2, 3.0, 0.0)           # no cap
    assert torch.equal(z2, torch.full((2, 4), 3.0, device="cuda"))


def _delta_case(seed, H, G, D, V, taps, entries, slots_read, slots_write, n_slots=6, max_rows=0):
    """Runs delta_prep + state_scan + head_norm_gate over a step whose entries have `entries` rows each, from random
    states; returns everything the plain functions need and what the kernels gave."""
    rng = np.random.default_rng(seed)
    o = ops()
    T = sum(entries)
    C = 2 * G * D + H * V
    ld = C + H + 3                       # beta's columns after the channels, then columns that belong to no one
    pre = rng.normal(size=(T, ld))
    conv = rng.normal(size=(C, taps)) * 0.6
    step_pre, dt_bias, a_log = rng.normal(size=(T, H * D)), rng.normal(size=H * D), rng.normal(size=H) * 0.5 - 1.0
    matrix = o.state_matrix_size(H, D, V)       # the kernel keeps S in tiles of value channels
    state = rng.normal(size=(n_slots, H * D * V + (taps - 1) * C)) * 0.5
    state_d = torch.cat([o.state_matrix_tiled(dev(state[:, :H * D * V]).reshape(n_slots, H, D, V)), dev(state[:, H * D * V:])], dim=1).contiguous()
    before = state_d.clone()
    row_entry = np.repeat(np.arange(len(entries)), entries)
    entry_rows = np.array([[sum(entries[:i]), n] for i, n in enumerate(entries)])
    q, k = torch.empty(T, G * D, device="cuda"), torch.empty(T, G * D, device="cuda")
    v, decay, beta = torch.empty(T, H * V, device="cuda"), torch.empty(T, H * D, device="cuda"), torch.empty(T, H, device="cuda")
    sr, sw = dev(slots_read, torch.int32), dev(slots_write, torch.int32)
    pre_d = dev(pre)
    o.delta_prep(pre_d, dev(conv), dev(step_pre), dev(dt_bias), dev(a_log), state_d, matrix, sr, dev(row_entry, torch.int32),
                 dev(entry_rows, torch.int32), q, k, v, decay, beta, G, H, D, V, C)
    out = torch.empty(T, H * V, device="cuda")
    tail = (pre_d[:, :C], taps, matrix) if taps > 1 else None
    o.state_scan(q, k, v, decay, beta, state_d, sr, sw, dev(entry_rows, torch.int32), out, D ** -0.5, H, G, D, V, tail=tail, max_rows=max_rows)
    # the plain way, entry by entry, from the slot each entry reads
    for e, n in enumerate(entries):
        r0 = entry_rows[e, 0]
        S0 = state[slots_read[e], :H * D * V].reshape(H, D, V)
        old_tail = state[slots_read[e], H * D * V:].reshape(taps - 1, C)
        x = np.concatenate([old_tail, pre[r0:r0 + n, :C]], axis=0)
        y = np.zeros((n, C))
        for j in range(taps):
            y += x[j:j + n] * conv[:, j]
        y = plain.silu(y)
        qq, kk, vv = y[:, :G * D].reshape(n, G, D), y[:, G * D:2 * G * D].reshape(n, G, D), y[:, 2 * G * D:].reshape(n, H, V)
        qq = qq / np.sqrt((qq * qq).sum(-1, keepdims=True) + 1e-6) * D ** -0.5
        kk = kk / np.sqrt((kk * kk).sum(-1, keepdims=True) + 1e-6)
        qq, kk = np.repeat(qq, H // G, axis=1), np.repeat(kk, H // G, axis=1)
        g = np.exp(-np.exp(a_log)[None, :, None] * plain.softplus(step_pre[r0:r0 + n] + dt_bias).reshape(n, H, D))
        b = plain.sigmoid(pre[r0:r0 + n, C:C + H])
        S = S0.copy()
        want = np.zeros((n, H, V))
        for t in range(n):
            for h in range(H):
                S[h] *= g[t, h][:, None]
                u = b[t, h] * (vv[t, h] - S[h].T @ kk[t, h])
                S[h] += np.outer(kk[t, h], u)
                want[t, h] = S[h].T @ qq[t, h]
        close(out[r0:r0 + n], want.reshape(n, H * V), 2e-5, f"read-out of entry {e}")
        close(o.state_matrix_plain(state_d[slots_write[e]], H, D, V), S, 2e-5, f"state of entry {e}")
        if taps > 1:
            got_tail = state_d[slots_write[e], matrix:].cpu().double().numpy()
            assert np.array_equal(got_tail.reshape(taps - 1, C), x[n:].astype(np.float32).astype(np.float64)), f"tail of entry {e}"
    untouched = [s for s in range(n_slots) if s not in slots_write]
    assert torch.equal(state_d[untouched], before[untouched])
    return out


@pytest.mark.parametrize("sizes", [(4, 2, 16, 24, 4), (3, 3, 5, 7, 1), (1, 1, 9, 3, 3), (2, 1, 72, 8, 5), (2, 2, 132, 20, 2), (2, 1, 256, 17, 2)])
def test_delta_rule_rows_states_slots_and_the_convolution_tail(sizes):
    """Entries of 1, 2 (fewer than the taps: the tail is shifted), 9 and 40 rows read their state and tail at one slot and
    write them at another (and in place); slots of no entry are untouched."""
    H, G, D, V, taps = sizes
    whole = _delta_case(1, H, G, D, V, taps, [9, 1, 2, 40], [0, 2, 4, 5], [1, 3, 4, 0])
    # steps of one or two rows an entry take smaller chunks: the same bits as the rows get in the larger ones
    short = _delta_case(2, H, G, D, V, taps, [1, 2, 1], [0, 2, 4], [1, 3, 4], max_rows=2)
    assert torch.equal(short, _delta_case(2, H, G, D, V, taps, [1, 2, 1], [0, 2, 4], [1, 3, 4]))


def test_matrix_state_without_the_delta_correction_and_strided_operands():
    """Gated linear attention's recurrence: q, k and v are columns of one wide projection."""
    rng = np.random.default_rng(3)
    o = ops()
    H, D, V, entries = 3, 16, 40, [5, 1, 33]
    T = sum(entries)
    wide = rng.normal(size=(T, 2 * H * D + H * V + 5))
    z, bias = rng.normal(size=(T, H * D)) * 2, rng.normal(size=H * D)
    decay = torch.empty(T, H * D, device="cuda")
    o.sigmoid_root(dev(z), dev(bias), 8.0, decay)
    alpha = plain.sigmoid(z + bias) ** (1.0 / 8.0)
    close(decay, alpha, 1e-6)
    state = rng.normal(size=(4, H * D * V))
    state_d, wide_d = o.state_matrix_tiled(dev(state).reshape(4, H, D, V)).contiguous(), dev(wide)
    entry_rows = np.array([[sum(entries[:i]), n] for i, n in enumerate(entries)])
    out = torch.empty(T, H * V, device="cuda")
    o.state_scan(wide_d[:, :H * D], wide_d[:, H * D:2 * H * D], wide_d[:, 2 * H * D:2 * H * D + H * V], decay, None, state_d,
                 dev([0, 1, 3], torch.int32), dev([0, 2, 3], torch.int32), dev(entry_rows, torch.int32), out, 0.25, H, H, D, V)
    for e, (r0, n) in enumerate(entry_rows):
        S = state[[0, 1, 3][e]].reshape(H, D, V).copy()
        q, k = wide[r0:r0 + n, :H * D].reshape(n, H, D), wide[r0:r0 + n, H * D:2 * H * D].reshape(n, H, D)
        v = wide[r0:r0 + n, 2 * H * D:2 * H * D + H * V].reshape(n, H, V)
        for t in range(n):
            S = S * alpha[r0 + t].reshape(H, D)[:, :, None] + k[t][:, :, None] * v[t][:, None, :]
            close(out[r0 + t], 0.25 * np.einsum("hdv,hd->hv", S, q[t]).reshape(-1), 2e-5)
        close(o.state_matrix_plain(state_d[[0, 2, 3][e]], H, D, V), S, 2e-5)


@pytest.mark.parametrize("gate", ["sigmoid", "silu"])
def test_gated_head_norm(gate):
    rng = np.random.default_rng(5)
    o = ops()
    T, H, V = 6, 3, 70
    x, w, z = rng.normal(size=(T, H, V)) * 4, rng.normal(size=V), rng.normal(size=(T, H * V + 3)) * 2
    out = torch.empty(T, H * V, device="cuda")
    o.head_norm_gate(dev(x.reshape(T, H * V)), dev(w), dev(z)[:, :H * V], out, 1e-5, H, V, o.GATE_SIGMOID if gate == "sigmoid" else o.GATE_SILU)
    g = plain.sigmoid(z[:, :H * V]) if gate == "sigmoid" else plain.silu(z[:, :H * V])
    close(out, (plain.rms_unit(x, 1e-5) * w).reshape(T, H * V) * g, 3e-6)


@pytest.mark.parametrize("experts,top", [(16, 2), (3, 1), (5, 5), (300, 7)])
def test_router_with_a_bias_in_its_logits(experts, top):
    rng = np.random.default_rng(experts)
    o = ops()
    rows = 9
    z, bias = rng.normal(size=(rows, experts)), rng.normal(size=experts) * 3
    ids, weights = torch.empty(rows, top, dtype=torch.int32, device="cuda"), torch.empty(rows, top, device="cuda")
    zd = dev(z)
    o.route_topk(zd, None, ids, weights, top, o.SCORE_SOFTMAX, "always", 1.0, logit_bias=dev(bias))
    full = (z + bias).astype(np.float32).astype(np.float64)
    for r in range(rows):
        want = sorted(range(experts), key=lambda e: (-full[r, e], e))[:top]
        assert ids[r].tolist() == want
        p = np.exp(full[r, want] - full[r, want].max())
        close(weights[r], p / p.sum(), 2e-6)
    close(zd, full, 1e-6)       # the logits a hook sees hold the bias


def _attention_case(dtype, H, G, D, VD, R, scaling, window, page, length, sharp=None):
    """One attention part alone through its two kernels (the step with a norm a head, then the attention over pages) for a
    prompt of `length` rows over shuffled pages, against the plain function.  sharp = (row, key): the row's query is made
    to fit that key alone."""
    from llmx_amd.parts.position import scaled_table
    rng = np.random.default_rng(H * 1000 + D + length)
    o = ops()
    E = 24
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": VD, "scale": 0.3, "mask": {"size": window},
         "rot": {"base": 500.0, "dims": R, "scaling": dict(zip(("factor", "original", "fast", "slow"), scaling)) if scaling else None}}
    w = {n: rng.normal(size=s) * 0.5 for n, s in (("q", (H * D, E)), ("k", (G * D, E)), ("v", (G * VD, E)), ("q.b", (H * D,)), ("k.b", (G * D,)),
                                                  ("v.b", (G * VD,)), ("q.norm", (D,)), ("k.norm", (D,)))}
    w["o"], w["o.b"] = np.eye(H * VD), np.zeros(H * VD)
    h = rng.normal(size=(length, E))
    if sharp is not None:
        # the key row's input is far from all others, and the query row's input is made the same: after the norm a head
        # both point the same way, so that key's score stands out as far as the rotation lets it
        row, key = sharp
        h[key] = h[key] * 6
        h[row] = h[key]
        w["q"][:] = 0.0
        w["q"][:, :] = np.tile(w["k"][:D], (H, 1))
        w["q.b"][:] = np.tile(w["k.b"][:D], H)
        w["q.norm"], w["k.norm"] = np.full(D, 6.0), np.full(D, 6.0)
    want = plain.window_attention(h, w, m, 1e-6)
    qkv = np.concatenate([h @ w["q"].T, h @ w["k"].T, h @ w["v"].T], axis=1)
    bias = np.concatenate([w["q.b"], w["k.b"], w["v.b"]])
    n_pages = -(-length // page)
    order = list(range(n_pages + 3))
    random.Random(length).shuffle(order)
    tables = dev(np.array([order[:n_pages] + [-1] * 5]), torch.int32)
    kc = torch.zeros(n_pages + 3, G, page, D, device="cuda", dtype=dtype)
    vc = torch.zeros(n_pages + 3, G, VD, page, device="cuda", dtype=dtype)
    cos_sin = dev(scaled_table(length, R, 500.0, m["rot"]["scaling"]))
    pos, ent = dev(np.arange(length), torch.int32), dev(np.zeros(length), torch.int32)
    q = torch.empty(length, H * D, device="cuda", dtype=dtype)
    o.head_norm_rope_kvwrite(dev(qkv), dev(bias), dev(w["q.norm"]), dev(w["k.norm"]), cos_sin, pos, ent, tables, q, kc, vc, 1e-6, H, G, D, R,
                             o.QKNORM_HEAD, pairing=o.ROPE_INTERLEAVED)
    out = torch.empty(length, H * VD, device="cuda", dtype=dtype)
    plan = None
    if VD == D and o.attention_mfma_ok(dtype, D, page):
        plan = o.attention_plan([length], [length], H, G, torch.device("cuda"), window)
    o.paged_attention(q, kc, vc, pos, ent, tables, out, 0.3, H, window=window, plan=plan)
    return out.float().cpu(), torch.as_tensor(want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(4, 2, 32, 32, 16, (4.0, 64, 16.0, 2.0), 40, 16), (3, 1, 10, 6, 6, None, 5, 4), (2, 2, 16, 48, 16, (2.0, 32, 8.0, 1.0), 4096, 16),
                                   (6, 3, 48, 16, 8, None, 17, 16), (1, 1, 64, 64, 0, None, 1, 16)])
def test_attention_with_a_norm_a_head_over_shuffled_pages(dtype, sizes):
    H, G, D, VD, R, scaling, window, page = sizes
    got, want = _attention_case(dtype, H, G, D, VD, R, scaling, window, page, 150)
    close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("back", [0, 1, 15, 16, 38, 39, 40, 41, 64])
def test_attention_keeps_the_window_to_the_key(dtype, back):
    """A row whose query fits one key `back` positions before it: inside the window of 40 (back <= 39) that key's value
    carries the result, outside it the key must not be seen.  Values as wide as keys (the matrix cores run in bfloat16) and
    of their own width."""
    for VD in (32, 24):
        row = 130
        got, want = _attention_case(dtype, 2, 1, 32, VD, 0, None, 40, 16, 150, sharp=(row, row - back))
        close(got[row], want[row], 2e-5 if dtype == torch.float32 else 2e-2, f"{back} back, values of {VD}")


# ---------------------------------------------------------------------------
# the engine
def make_engine(name, dtype, kv_tokens=1024, max_requests=4, graphs=True, folder=None):
    from llmx_amd.engine import Engine
    return Engine.load(folder or model_folder(name), dtype=dtype, kv_tokens=kv_tokens, page_tokens=PAGES[name], max_requests=max_requests, graphs=graphs)


@pytest.fixture(scope="module", params=[(n, d) for n in CONFIGS for d in ("float32", "bfloat16")], ids=lambda p: f"{p[0]}-{p[1]}")
def setup(request):
    name, dtype = request.param
    return name, dtype, make_engine(name, dtype)


def run_cut(engine, rid, tokens, cuts):
    from llmx_amd.engine import StepEntry
    engine.add_request(rid)
    rows = [engine.step([StepEntry(rid, tokens[a:b], list(range(b - a)))]).clone() for a, b in cuts]
    engine.end_request(rid)
    return torch.cat(rows).cpu()


def same_rows(got, whole, what):
    """Two cuttings of the same tokens give every row the same bits, in both number formats."""
    assert torch.equal(got, whole), f"{what}: rows differ, first at row {int((got != whole).any(1).nonzero()[0])}"


def run_whole_with_picks(engine, tokens):
    """(rows, picks): a whole prompt's logits and, for every routed layer run in order, the experts the engine picked
    [T, top], each row's picks checked against the engine's own float32 router logits (the `top` largest, lower ids first)."""
    shown = []
    engine.observer = lambda step, kind, **t: shown.append((t["ids"].cpu().numpy().copy(), t["logits"].cpu().numpy().copy())) if kind == "routing" else None
    try:
        rows = run_cut(engine, "picks", tokens, [(0, len(tokens))])
    finally:
        engine.observer = None
    for ids, z in shown:
        for t in range(ids.shape[0]):
            assert list(ids[t]) == sorted(range(z.shape[1]), key=lambda e: (-z[t, e], e))[:ids.shape[1]]
    return rows, [ids for ids, _ in shown]


def reference_rows(name, dtype, length, seed, got, engine=None, folder=None, tol=None):
    """float32 against the plain implementation.  bfloat16 too, within BF16_TOL, with the engine's own expert picks handed
    to the plain implementation (a near tie of two router logits may fall the other way after rounding, and then another
    expert runs); `got` must be the bits of the whole prompt that was run to see the picks."""
    tokens = tokens_for(name, length, seed)
    if dtype == "float32":
        want = plain_logits(name, length, seed) if folder is None else plain.forward(*load_plain(folder), tokens)
        # configuration B's heads of a handful of values turn a last-bit difference into more than the others' do
        close(got, want, tol or (F32_TOL if name != "B" else 3 * F32_TOL), "against the plain implementation")
        return
    rows, picks = run_whole_with_picks(engine, tokens)
    assert torch.equal(rows, got), "the whole prompt run again gives other bits"
    config, tensors = load_plain(folder or model_folder(name))
    want = torch.as_tensor(plain.forward(config, tensors, tokens, picks=picks))
    # heads of a handful of values (configuration B: unit vectors of five dims, a norm over three) turn one rounding into
    # several percent of a logit now and then: the single worst logit gets three times the room, the mean none
    close(got, want, tol or (BF16_TOL if name != "B" else 3 * BF16_TOL), "against the plain implementation with the engine's picks")
    rms = float((got.double() - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt())
    assert rms <= BF16_RMS, f"root mean square of the differences {rms:.3e} of the logits' above {BF16_RMS:.1e}"


LENGTHS = (1, 2, 9, 33, 75, 130)


def test_whole_prompts_and_every_layer(setup):
    name, dtype, engine = setup
    for seed, length in enumerate(LENGTHS):
        reference_rows(name, dtype, length, seed, run_cut(engine, ("w", seed), tokens_for(name, length, seed), [(0, length)]), engine)
    if dtype != "float32":
        return
    config, tensors = load_plain(model_folder(name))
    tokens = tokens_for(name, 21, 99)
    layers = []
    plain.forward(config, tensors, tokens, layers)
    seen = []
    engine.observer = lambda step, kind, **t: seen.append(t["residual"].clone()) if kind == "layer" else None
    try:
        run_cut(engine, "layers", tokens, [(0, 21)])
    finally:
        engine.observer = None
    assert len(seen) == len(layers) == len(config["layers"])
    for i, (got, want) in enumerate(zip(seen, layers)):
        close(got, want, F32_TOL, f"residual after layer {i}")


def test_prompt_against_token_by_token_and_portions(setup):
    """Every cutting gives every row the same bits: whole, token by token from the first token, most of it whole and the
    rest one by one, portions of changing size down to two tokens and to one, pairs."""
    name, dtype, engine = setup
    length, seed = 130, 5
    tokens = tokens_for(name, length, seed)
    whole = run_cut(engine, "whole", tokens, [(0, length)])
    reference_rows(name, dtype, length, seed, whole, engine)
    cuttings = {
        "one by one": [(i, i + 1) for i in range(length)],
        "decoded tail": [(0, length - 50)] + [(i, i + 1) for i in range(length - 50, length)],
        "portions": portions(length, 1),
        "portions of one": portions(length, 2, smallest=1),
        "pairs": [(i, min(i + 2, length)) for i in range(0, length, 2)],
    }
    for what, cuts in cuttings.items():
        same_rows(run_cut(engine, what, tokens, cuts), whole, what)


def test_unequal_requests_in_one_batch_and_reused_pages_and_slots(setup):
    """Eight requests of unequal length through four seats, portions of some beside single tokens of others, in an engine
    with so few pages that ended requests' pages and slots are taken again by later ones; every row has the bits it has
    when its request runs alone in a fresh engine."""
    from llmx_amd.engine import StepEntry
    name, dtype, _ = setup
    lengths = [70, 23, 1, 96, 40, 17, 64, 5]
    alone_engine = make_engine(name, dtype)
    alone = {i: run_cut(alone_engine, i, tokens_for(name, n, 20 + i), [(0, n)]) for i, n in enumerate(lengths)}
    engine = make_engine(name, dtype, kv_tokens=4 * 112, max_requests=4)
    rng = random.Random(3)
    waiting = list(range(len(lengths)))
    live, fed, got = [], {}, {i: [] for i in range(len(lengths))}
    while waiting or live:
        while waiting and len(live) < 4:
            i = waiting.pop(0)
            engine.add_request(i)
            live.append(i)
            fed[i] = 0
        entries, taken = [], []
        for i in live:
            if rng.random() < 0.2 and len(live) > 1:
                continue                                     # a request may be left out of a step
            left = lengths[i] - fed[i]
            n = 1 if rng.random() < 0.4 else min(left, rng.choice([2, 3, 8, 16, 31]))
            entries.append(StepEntry(i, tokens_for(name, lengths[i], 20 + i)[fed[i]:fed[i] + n], list(range(n))))
            taken.append((i, n))
        if not entries:
            continue
        out = engine.step(entries).clone().cpu()
        at = 0
        for i, n in taken:
            got[i].append(out[at:at + n])
            at += n
            fed[i] += n
            if fed[i] == lengths[i]:
                engine.end_request(i)
                live.remove(i)
    for i in range(len(lengths)):
        same_rows(torch.cat(got[i]), alone[i], f"request {i} in batches against its whole prompt alone")
    assert all(engine.cache.pages_in_use(g) == 0 for g in range(len(engine.cache.groups)))
    assert engine.cache.slots.in_use == 0


def test_long_decoding_and_graph_replays(setup):
    """A short prompt, then 230 tokens one by one over many pages and past every window: the rows of the whole sequence, from
    an engine that replays decode steps as graphs and from one that does not."""
    name, dtype, engine = setup
    length, seed = 250, 8
    tokens = tokens_for(name, length, seed)
    cuts = [(0, 20)] + [(i, i + 1) for i in range(20, length)]
    before = engine.graph_replays
    got = run_cut(engine, "long", tokens, cuts)
    assert engine.graphs and engine.graph_replays - before > 150
    eager = make_engine(name, dtype, graphs=False)
    assert torch.equal(run_cut(eager, "long", tokens, cuts), got)
    whole = run_cut(eager, "whole", tokens, [(0, length)])
    same_rows(got, whole, "decoded against whole")
    reference_rows(name, dtype, length, seed, whole, eager)


def test_which_kernels_a_serving_step_takes():
    """The launch witness: at sizes the matrix cores take (configuration A), a bfloat16 step runs the design's own kernels
    and the matrix-core attention and products, never the universal ones; a float32 engine never launches a bfloat16
    product.  A dispatch that fell back silently fails here, not only in a benchmark."""
    from llmx_amd.engine import StepEntry
    o = ops()
    tokens = tokens_for("A", 70, 2)
    for dtype in ("bfloat16", "float32"):
        engine = make_engine("A", dtype, graphs=False)
        engine.add_request("r")
        seen = {}
        for entry in (StepEntry("r", tokens[:69], [68]), StepEntry("r", tokens[69:], [0])):       # a prompt's portion, then one token
            o.take_launches()
            engine.step([entry])
            for name, count in o.take_launches().items():
                seen[name] = seen.get(name, 0) + count
        for name in ("state_scan", "delta_prep", "head_norm_gate", "sigmoid_root", "layernorm_add", "layernorm", "head_norm_rope_kvwrite",
                     "combine_rows", "scale_softcap", "route_topk", "moe_combine"):
            assert seen.get(name), f"{dtype}: no launch of {name} ({sorted(seen)})"
        if dtype == "bfloat16":
            assert not any(n.startswith(("gemm_generic", "attention.generic")) for n in seen), sorted(seen)
            assert any(n.startswith("attention.") for n in seen) and any(n.startswith("gemm_skinny") or n.startswith("gemm_tile") for n in seen)
            assert seen.get("cast_rows") == 2        # the first layer's copy of x, once a step; later layers get theirs from the joins
        else:
            assert not any(n.startswith(("gemm_skinny", "gemm_tile", "attention.tiles", "attention.split", "attention.direct")) for n in seen), sorted(seen)


def test_a_failed_step_leaves_states_and_pages_as_they_were():
    from llmx_amd.cache import OutOfPages
    from llmx_amd.engine import StepEntry
    name = "A"
    tokens = tokens_for(name, 60, 1)
    engine = make_engine(name, "float32", kv_tokens=64, max_requests=2)
    engine.add_request("a")
    engine.add_request("b")
    first = engine.step([StepEntry("a", tokens[:20], [19])]).clone()
    with pytest.raises(OutOfPages):
        engine.step([StepEntry("a", tokens[20:40], [19]), StepEntry("b", tokens[:60], [])])
    rest = engine.step([StepEntry("a", tokens[20:60], list(range(40)))]).clone().cpu()
    whole = run_cut(make_engine(name, "float32"), "w", tokens, [(0, 60)])
    assert torch.equal(first.cpu()[0], whole[19]) and torch.equal(rest, whole[20:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_and_long_memory(dtype, tmp_path):
    """Query and key weights made larger let the softmax pick single keys, so a key lost at a window's or a page's edge
    shows; decays close to one let tokens hundreds of steps back stay in the states, so a state lost or reset shows.  Whole,
    portions and decoding agree bit for bit, and float32 with the plain model."""
    def edit(tensors):
        for k in tensors:
            if k.endswith("left.q.norm") or k.endswith("left.k.norm"):
                tensors[k] = (tensors[k].float() * 3.0).to(tensors[k].dtype)
            if k.endswith("A_log"):
                tensors[k] = torch.full_like(tensors[k], -5.0)
            if k.endswith("a2.b"):
                tensors[k] = torch.full_like(tensors[k], 6.0)
    folder = write_folder(CONFIGS["A"], 17, str(tmp_path / "sharp"), edit)
    engine = make_engine("A", dtype, folder=folder)
    length = 420
    tokens = tokens_for("A", length, 4)
    whole = run_cut(engine, "w", tokens, [(0, length)])
    config, tensors = load_plain(folder)
    if dtype == "float32":
        want = plain.forward(config, tensors, tokens)
        close(whole, want, 1e-4, "against the plain implementation")
        # the memory is long indeed: another first token changes the last row
        other = plain.forward(config, tensors, [(tokens[0] + 1) % 200] + tokens[1:])
        assert float(np.abs(other[-1] - want[-1]).max()) > 1e-3 * float(np.abs(want).max())
    else:
        rows, picks = run_whole_with_picks(engine, tokens)
        assert torch.equal(rows, whole)
        close(whole, plain.forward(config, tensors, tokens, picks=picks), 8e-2, "against the plain implementation with the engine's picks")
    same_rows(run_cut(engine, "p", tokens, portions(length, 9)), whole, "portions")
    same_rows(run_cut(engine, "pairs", tokens, [(i, i + 2) for i in range(0, length, 2)]), whole, "pairs")
    same_rows(run_cut(engine, "d", tokens, [(0, length - 90)] + [(i, i + 1) for i in range(length - 90, length)]), whole, "decoded")


def test_greedy_generation_through_the_scheduler():
    """`generate` (scheduler, step function, device sampler) with prompts of unequal length and a small step budget, so
    that prompts are cut into portions beside decoding requests; float32 picks the plain implementation's tokens."""
    from llmx_amd import SamplingParams, generate
    name = "A"
    config, tensors = load_plain(model_folder(name))
    prompts = [tokens_for(name, n, 40 + n) for n in (3, 29, 11, 1, 18)]
    engine = make_engine(name, "float32", kv_tokens=512, max_requests=3)
    got = generate(engine, prompts, SamplingParams(max_tokens=10, temp=0.0), max_seqs=3, max_step_tokens=16)
    for p, g in zip(prompts, got):
        assert g == greedy(config, tensors, p, 10)
    engine16 = make_engine(name, "bfloat16", kv_tokens=512, max_requests=3)
    got16 = generate(engine16, prompts, SamplingParams(max_tokens=10, temp=0.0), max_seqs=3, max_step_tokens=16)
    for p, g in zip(prompts, got16):
        # bfloat16 may take another of two nearly equal logits: each token it chose is among the plain model's best within rounding
        rows = plain.forward(config, tensors, p + g[:-1])[len(p) - 1:]
        for i, tok in enumerate(g):
            assert float(rows[i, tok]) >= float(rows[i].max()) - BF16_TOL * float(np.abs(rows[i]).max())


def test_trace_replay_and_command_line(tmp_path):
    """bin/trace_run as a subprocess on a model folder: a prompt portion beside decoded tokens, requests that end and
    whose slots are taken again; the logits files are the plain model's rows.  `llmx logits` reads the same folder."""
    name = "B"
    a, b, c = tokens_for(name, 40, 1), tokens_for(name, 9, 2), tokens_for(name, 30, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": [0, 32]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[33:34], "want": [0]}, {"id": "b", "tokens": b, "want": [8]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "c", "tokens": c[:2], "want": []}], "end": []},
        {"step": 3, "entries": [{"id": "c", "tokens": c[2:], "want": [27]}, {"id": "a", "tokens": a[34:], "want": [5]}], "end": ["a", "c"]},
    ]
    out = tmp_path / "out"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folder(name), "--dtype", "float32", "--out", str(out),
                          "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    V = CONFIGS[name]["vocab"]
    want = {"a": plain_logits(name, 40, 1), "b": plain_logits(name, 9, 2), "c": plain_logits(name, 30, 3)}
    rows = {0: [("a", 0), ("a", 32)], 1: [("a", 33), ("b", 8)], 3: [("c", 29), ("a", 39)]}
    assert not (out / "2.f32").exists()
    for step, places in rows.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, V))
        assert got.shape[0] == len(places)
        for r, (rid, p) in enumerate(places):
            close(got[r], want[rid][p], F32_TOL)
    cli = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "llmx"), "logits", model_folder(name), " ".join(map(str, b)), "--dtype", "f32", "--top", "1"],
                         capture_output=True, text=True, timeout=600)
    assert cli.returncode == 0, cli.stderr[-2000:]
    assert int(cli.stdout.splitlines()[-1].split()[0]) == int(torch.argmax(want["b"][8]))


def test_command_line_generates_from_a_configuration_with_random_weights(tmp_path):
    """`llmx generate --config JSON --random SEED` for this design (the configuration states the inner widths that a model
    folder's tensors would give): weights generated on the device, the scheduler's loop, the device sampler."""
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(CONFIGS["C"]))
    outs = []
    for extra in (["--temp", "0"], ["--temp", "0"]):
        run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "llmx"), "generate", "--config", str(cfg), "--random", "5", "--std", "0.06",
                              "3 1 4 1 5 9 2 6", "-n", "9"] + extra, capture_output=True, text=True, timeout=600)
        assert run.returncode == 0, run.stderr[-2000:]
        ids = [int(t) for t in run.stdout.split()]
        assert len(ids) == 9 and all(0 <= t < CONFIGS["C"]["vocab"] for t in ids)
        outs.append(ids)
    assert outs[0] == outs[1]
