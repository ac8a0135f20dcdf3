"""Nenotar in the engine against the plain implementation (tests/plain_nenotar.py), mechanism by mechanism and whole.

Kernels alone (the norm pass with two gains, the scaled join, the normed join, xIELU, the gated table slice, the gated
recurrence, the step before the latent attention, the attention over paged latents, the head gate) against the plain
functions; then the engine under every way of cutting the same tokens into steps, which must agree bit for bit with each
other in both dtypes and with the plain implementation within F32_TOL / BF16_TOL; pages and state slots that are used
again; long decoding; weights made so that one far key carries the result; greedy generation through `generate`.
"""

from __future__ import annotations

import math
import os
import random

import pytest
import torch

import plain_nenotar as plain
from nenotar_cases import CONFIGS, PAGES, SEEDS, model_folder, plain_logits, portions, tokens_for, write_folder

pytestmark = pytest.mark.gpu

F32_TOL = 2e-5      # |engine - plain| over all logits relative to the largest |logit|, float32 sums in another order
BF16_TOL = 2.5e-2   # both round at the same places; single bfloat16 roundings flip on last-bit differences of the sums
CUT_TOL = 1.5e-2    # bfloat16, one cutting against another: see same_rows


def ops():
    from llmx_amd import ops as o
    return o


def dev(t, dtype=None):
    return t.to(device="cuda", dtype=dtype or t.dtype).contiguous()


def close(got, want, tol):
    got, want = got.double().cpu(), want.double().cpu()
    err = float((got - want).abs().max()) / max(float(want.abs().max()), 1e-30)
    assert err <= tol, f"relative error {err:.3e} above {tol:.1e}"
    return err


# ---------------------------------------------------------------------------
# kernels alone
@pytest.mark.parametrize("rows,n", [(1, 8), (5, 80), (3, 1030), (2, 9001)])
def test_norm_pass_with_two_gains(rows, n):
    g = torch.Generator().manual_seed(rows * n)
    x = torch.randn(rows, n, generator=g) * 3
    w1, w2 = torch.randn(n, generator=g), torch.randn(n, generator=g)
    for dtype in (torch.float32, torch.bfloat16):
        o1, o2 = torch.empty(rows, n, dtype=dtype, device="cuda"), torch.empty(rows, n, dtype=dtype, device="cuda")
        ops().rmsnorm_pair(dev(x), dev(w1), dev(w2), 1e-5, o1, o2)
        want = plain.rms(x.double(), 1e-5)
        close(o1, want * w1.double(), 1e-6 if dtype == torch.float32 else 5e-3)
        close(o2, want * w2.double(), 1e-6 if dtype == torch.float32 else 5e-3)
        # each output has the bits of the norm kernel with that gain
        single = torch.empty_like(o2)
        ops().rmsnorm(dev(x), dev(w2), 1e-5, single)
        assert torch.equal(single, o2)
    only = torch.empty(rows, n, dtype=torch.float32, device="cuda")
    ops().rmsnorm_pair(dev(x), dev(w1), None, 1e-5, only, None)
    close(only, plain.rms(x.double(), 1e-5) * w1.double(), 1e-6)


def test_scaled_join_and_normed_join():
    g = torch.Generator().manual_seed(1)
    T, n = 7, 83
    x, y1, y2 = (torch.randn(T, n, generator=g) for _ in range(3))
    s1, s2, w = (torch.randn(n, generator=g) for _ in range(3))
    xd, copy = dev(x), torch.empty(T, n, dtype=torch.bfloat16, device="cuda")
    ops().scale_add(xd, dev(y1), dev(s1), dev(y2), dev(s2), copy)
    want = x.double() + (y1.double() * s1.double() + y2.double() * s2.double())
    close(xd, want, 1e-6)
    assert torch.equal(copy, xd.to(torch.bfloat16))
    xd = dev(x)
    ops().scale_add(xd, dev(y1), None)
    close(xd, x.double() + y1.double(), 1e-6)
    xd = dev(x)
    ops().rmsnorm_add(xd, dev(y1), dev(w), 1e-6)
    close(xd, x.double() + plain.rms(y1.double(), 1e-6) * w.double(), 1e-6)


def test_xielu_both_branches_and_the_gated_table_slice():
    z = torch.cat([torch.linspace(-30, 30, 601), torch.tensor([0.0, -0.0, 1e-8, -1e-8, -80.0])]).reshape(1, -1)
    for p, q in ((0.3, -1.1), (-2.0, 4.0), (0.0, 0.0)):
        pq = torch.tensor([p, q])
        out = torch.empty_like(z, device="cuda")
        ops().act_xielu(dev(z), dev(pq), out)
        want = plain.xielu(z.double(), pq[0].double(), pq[1].double())
        assert float((out.cpu().double() - want).abs().max() / want.abs().max()) < 1e-6
    g = torch.Generator().manual_seed(2)
    T, n, L = 9, 5, 4
    pre = torch.randn(T, n, generator=g) * 3
    table = torch.randn(40, n * L, generator=g).to(torch.bfloat16)
    ids = torch.randint(0, 40, (T,), generator=g, dtype=torch.int32)
    for layer in range(L):
        out = torch.empty(T, n, dtype=torch.float32, device="cuda")
        ops().act_gelu_gather(dev(pre), dev(table), dev(ids), out, layer * n)
        want = plain.gelu_tanh(pre.double()) * table[ids.long()][:, layer * n:(layer + 1) * n].double()
        close(out, want, 1e-6)


@pytest.mark.parametrize("M,N,K,dtype", [(1, 48, 64, "bf16"), (3, 200, 256, "bf16"), (40, 4096, 256, "bf16"), (40, 130, 512, "bf16"), (300, 96, 128, "bf16"),
                                         (2048, 3072, 256, "bf16"), (5, 33, 54, "bf16"), (70, 50, 48, "f32")])
def test_activation_in_the_products_epilogue(M, N, K, dtype):
    """A storing product with xIELU gives the bits of the product followed by the activation's kernel, in every form of the
    product (weight streaming, two strips, tiles, wide tiles, K's runs apart, the universal kernel), and the plain values."""
    o = ops()
    g = torch.Generator().manual_seed(M + N + K)
    t = torch.bfloat16 if dtype == "bf16" else torch.float32
    a, w = dev(torch.randn(M, K, generator=g), t), dev(torch.randn(N, K, generator=g) * 0.3, t)
    pq = dev(torch.tensor([0.4, -0.9]))
    held = {}
    scratch = lambda name, shape, dt: held.setdefault((name, tuple(shape), dt), torch.empty(shape, dtype=dt, device="cuda"))
    for with_scratch in (False, True):
        fused = torch.empty(M, N, dtype=t, device="cuda")
        o.take_launches()
        o.gemm(a, w, fused, act=(o.ACT_XIELU, pq), scratch=scratch if with_scratch else None)
        ran = o.take_launches()
        assert "act.xielu" not in ran
        pre = torch.empty(M, N, dtype=torch.float32, device="cuda")
        o.gemm(a, w, pre, scratch=scratch if with_scratch else None)
        apart = torch.empty(M, N, dtype=t, device="cuda")
        o.act_xielu(pre, pq, apart)
        assert torch.equal(fused, apart), sorted(ran)
        want = plain.xielu(a.double().cpu() @ w.double().cpu().T, pq[0].double().cpu(), pq[1].double().cpu())
        close(fused, want, 1e-5 if dtype == "f32" else 1e-2)
    with pytest.raises(o.KernelError):
        o.gemm(a, w, torch.zeros(M, N, dtype=torch.float32, device="cuda"), o.EPI_ADD, act=(o.ACT_XIELU, pq))


@pytest.mark.parametrize("W", [1, 40, 131])
def test_gated_recurrence_rows_state_and_slots(W):
    """Three requests of 1, 2 and 19 rows in one launch, states read from one slot and written to another; then each
    request goes on from what was written; against the plain recurrence over the whole sequence."""
    g = torch.Generator().manual_seed(W)
    lengths = [(1, 6), (2, 1), (19, 14)]                     # rows in the first launch, in the second
    E = 24
    w = {"m.z": torch.randn(W, E, generator=g), "m.x": torch.randn(W, E, generator=g) * 2, "m.g": torch.randn(W, E, generator=g),
         "m.z.b": torch.randn(W, generator=g), "m.x.b": torch.randn(W, generator=g), "m.o": torch.eye(W)}
    hs = [torch.randn(a + b, E, generator=g) for a, b in lengths]
    want = [plain.mingru(h.double(), w, "m.", {"width": W})[0] for h in hs]
    w_in = torch.cat([w["m.z"], w["m.x"], w["m.g"]])
    state = torch.full((8, W), 7.0, device="cuda")           # slots that are not read hold rubbish
    read1, write1, write2 = [5, 0, 3], [1, 6, 2], [5, 0, 3]
    state[read1] = 0.0
    got = [[] for _ in lengths]
    for rnd, (reads, writes) in enumerate(((read1, write1), (write1, write2))):
        parts = [h[:lengths[i][0]] if rnd == 0 else h[lengths[i][0]:] for i, h in enumerate(hs)]
        pre = torch.cat(parts) @ w_in.T
        rows, at = [], 0
        for p in parts:
            rows.append([at, p.shape[0]])
            at += p.shape[0]
        out = torch.empty(at, W, dtype=torch.float32, device="cuda")
        ops().mingru_scan(dev(pre), dev(w["m.z.b"]), dev(w["m.x.b"]), state, dev(torch.tensor(reads, dtype=torch.int32)),
                          dev(torch.tensor(writes, dtype=torch.int32)), dev(torch.tensor(rows, dtype=torch.int32)), out)
        for i, (r0, n) in enumerate(rows):
            got[i].append(out[r0:r0 + n].cpu())
    for i in range(len(lengths)):
        close(torch.cat(got[i]), want[i], 2e-5)
    assert float(state[7].min()) == 7.0 and float(state[4].max()) == 7.0      # slots of no request are untouched


def test_gated_recurrence_in_chunks():
    """Long runs of rows take the three-launch form (chunks of 64 rows): two requests of 700 and 3 rows beside one of 257,
    from given states, against the plain recurrence and against the one-launch form."""
    g = torch.Generator().manual_seed(9)
    W, E = 70, 16
    w = {"m.z": torch.randn(W, E, generator=g), "m.x": torch.randn(W, E, generator=g) * 2, "m.g": torch.randn(W, E, generator=g),
         "m.z.b": torch.randn(W, generator=g), "m.x.b": torch.randn(W, generator=g), "m.o": torch.eye(W)}
    lengths = [700, 3, 257]
    hs = [torch.randn(n, E, generator=g) for n in lengths]
    starts = torch.rand(3, W, generator=g)
    want = [plain.mingru(h.double(), w, "m.", {"width": W}, state=starts[i].double()) for i, h in enumerate(hs)]
    pre = dev(torch.cat(hs) @ torch.cat([w["m.z"], w["m.x"], w["m.g"]]).T)
    rows = dev(torch.tensor([[0, 700], [700, 3], [703, 257]], dtype=torch.int32))
    reads, writes = dev(torch.tensor([0, 1, 2], dtype=torch.int32)), dev(torch.tensor([5, 4, 3], dtype=torch.int32))
    outs = []
    for chunked in (True, False):
        state = torch.zeros(6, W, device="cuda")
        state[:3] = dev(starts)
        out = torch.empty(960, W, dtype=torch.float32, device="cuda")
        plan = ops().scan_plan(lengths, "cuda") if chunked else None
        assert (plan is not None) == chunked
        ops().take_launches()
        ops().mingru_scan(pre, dev(w["m.z.b"]), dev(w["m.x.b"]), state, reads, writes, rows, out, plan=plan)
        assert ("gated_scan.chunks" in ops().take_launches()) == chunked
        at = 0
        for i, n in enumerate(lengths):
            close(out[at:at + n], want[i][0], 2e-5)
            close(state[5 - i], want[i][1], 2e-5)
            at += n
        assert torch.equal(state[:3].cpu(), starts)
        outs.append(out)
    close(outs[0], outs[1], 1e-5)
    assert ops().scan_plan([255, 1, 30], "cuda") is None


def _latent_case(seed, H, D, R, V, C, dims, scaling, positions, page, dtype, sharp=None, tiles=True):
    """One latent-attention layer on the kernels (products by torch) for rows at `positions` of one request whose earlier
    tokens are already cached in shuffled pages, against plain.latent_attention over the whole sequence."""
    from llmx_amd.parts.position import scaled_table
    g = torch.Generator().manual_seed(seed)
    n_ctx = max(positions) + 1
    E = 32
    m = {"heads": H, "dim": D, "rot_dim": R, "vdim": V, "kv_rank": C, "scale": 0.3, "rot": {"base": 300.0, "dims": dims}}
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    w = {"a.q": torch.randn(H * (D + R), E, generator=g) * 0.3, "a.dkv": torch.randn(C + R, E, generator=g) * 0.3,
         "a.dkv.norm": 1 + 0.3 * torch.randn(C, generator=g), "a.uk": torch.randn(H * D, C, generator=g) * 0.3,
         "a.uv": torch.randn(H * V, C, generator=g), "a.g": torch.randn(H, E, generator=g), "a.o": torch.eye(H * V)}
    w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    h = torch.randn(n_ctx, E, generator=g).to(torch.bfloat16).float()
    if sharp is not None:
        # row sharp[0] looks for key sharp[1] alone: W_q = gain * W_uk,n W_dkv P with P taking the query row's input to the
        # far row's input, so that the query's unrotated part is the far key's (before its norm) and no other's
        h_q, h_far = h[sharp[0]], h[sharp[1]]
        P = torch.outer(h_far, h_q) / float(h_q @ h_q)
        w["a.q"][:, :] = 0.0
        for n in range(H):
            w["a.q"][n * (D + R):n * (D + R) + D] = (8.0 * w["a.uk"][n * D:(n + 1) * D] @ w["a.dkv"][:C] @ P).to(torch.bfloat16).float()
    rounded = torch.bfloat16 if dtype == torch.bfloat16 else None
    want = plain.latent_attention(h.double(), w, "a.", m, 1e-6, list(range(n_ctx)), rounded)
    o = ops()
    n_pages = -(-n_ctx // page) + 3
    order = list(range(n_pages))
    random.Random(seed).shuffle(order)
    tables = torch.full((2, 64 * (-(-n_pages // 64))), -1, dtype=torch.int32)
    tables[1, :n_pages] = torch.tensor(order, dtype=torch.int32)           # the request is entry 1 of its steps
    tables = dev(tables)
    cache = torch.zeros(n_pages, page, C + R, dtype=dtype, device="cuda")
    # where the matrix cores take the sizes they run (with the latents' second, transposed copy and a plan of work items)
    cores = o.latent_attention_mfma_ok(dtype, C, R, page)
    cache_t = torch.zeros(n_pages, C, page, dtype=dtype, device="cuda") if cores else None
    cos_sin = dev(torch.from_numpy(scaled_table(n_ctx, dims, 300.0, m["rot"].get("scaling"))))
    w_in = torch.cat([w["a.q"], w["a.dkv"], w["a.g"]])
    uk_t = dev(w["a.uk"].view(H, D, C).transpose(1, 2), dtype)
    uv = dev(w["a.uv"].view(H, V, C), dtype)
    got = {}
    first = [p for p in range(n_ctx) if p not in positions]
    for rows in (first, list(positions)):                                  # the earlier tokens in one step, then the asked rows
        if not rows:
            continue
        T = len(rows)
        proj = dev(h[rows].to(dtype).float() @ w_in.T)
        pos = dev(torch.tensor(rows, dtype=torch.int32))
        entry = dev(torch.ones(T, dtype=torch.int32))
        q_plain, q_rot = torch.empty(H, T, D, dtype=dtype, device="cuda"), torch.empty(H, T, R, dtype=dtype, device="cuda")
        o.latent_prep(proj, dev(w["a.dkv.norm"]), cos_sin, pos, entry, tables, q_plain, q_rot, cache, 1e-6, H, D, R, C, cache_t=cache_t)
        q_lat = torch.bmm(q_plain.float(), uk_t.float().transpose(1, 2)).to(dtype).contiguous()
        mixed = torch.empty(H, T, C, dtype=dtype, device="cuda")
        o.take_launches()
        o.latent_attention(q_lat, q_rot, cache, pos, entry, tables, mixed, 0.3, cache_t=cache_t,
                           plan=o.latent_plan([0, T], H, "cuda", contexts=[0, max(rows) + 1], tiles=tiles) if cores else None)
        ran = o.take_launches()
        assert any(k in ran for k in ("latent_attention.mfma", "latent_attention.tiles", "latent_attention.rows")) == cores
        assert not cores or tiles or set(ran) <= {"latent_attention.mfma", "latent_attention.merge"}
        assert ("latent_attention.merge" in ran) == (cores and T == 1 and max(rows) >= o.LATENT_SPLIT_KEYS)
        values = torch.bmm(mixed.float(), uv.float().transpose(1, 2)).contiguous()
        joined = torch.empty(T, H * V, dtype=dtype, device="cuda")
        o.head_gate(values, proj[:, H * (D + R) + C + R:], joined)
        for i, p in enumerate(rows):
            got[p] = joined[i].float().cpu()
    return torch.stack([got[p] for p in positions]), want[list(positions)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(3, 24, 16, 40, 48, 16, (8.0, 64, 16.0, 2.0)), (1, 5, 6, 3, 10, 4, None), (17, 8, 0, 8, 16, 0, None),
                                   (2, 16, 8, 24, 130, 8, (2.0, 16, 4.0, 1.5)), (20, 16, 32, 8, 96, 32, None), (16, 8, 64, 8, 512, 64, None)],
                         ids=["even", "ragged", "no_rotation", "wide_latent", "twenty_heads", "real_latent"])
def test_latent_attention_rows_at_page_borders_and_first_tokens(dtype, sizes):
    H, D, R, V, C, dims, scaling = sizes
    positions = [0, 1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 200]
    got, want = _latent_case(11, H, D, R, V, C, dims, scaling, positions, 16, dtype)
    close(got, want, 3e-5 if dtype == torch.float32 else 3e-2)
    if ops().latent_attention_mfma_ok(dtype, C, R, 16):
        # the workgroups of four waves give every column the bits of the one-wave form
        assert torch.equal(_latent_case(11, H, D, R, V, C, dims, scaling, positions, 16, dtype, tiles=False)[0], got)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
@pytest.mark.parametrize("far", [0, 15, 16, 63, 64, 255, 256, 300])
def test_latent_attention_finds_one_far_key(dtype, far):
    """The last row's query is made to fit one key hundreds of tokens back (the first key, keys on both sides of page and
    tile borders): its result is that key's values, which a key lost or shifted by one would not give."""
    n = 700
    got, want = _latent_case(5 + far, 2, 16, 32, 12, 32, 4, None, [n - 2, n - 1], 16, dtype, sharp=(n - 1, far))
    close(got, want, 1e-4 if dtype == torch.float32 else 3e-2)
    # the same row decoded alone: in bfloat16 its context is shared out over work items and joined
    got, want = _latent_case(5 + far, 2, 16, 32, 12, 32, 4, None, [n - 1], 16, dtype, sharp=(n - 1, far))
    close(got, want, 1e-4 if dtype == torch.float32 else 3e-2)
    if dtype == torch.bfloat16:
        assert torch.equal(_latent_case(5 + far, 2, 16, 32, 12, 32, 4, None, [n - 1], 16, dtype, sharp=(n - 1, far), tiles=False)[0], got)


# ---------------------------------------------------------------------------
# the engine
def make_engine(name, dtype, kv_tokens=1024, max_requests=4, graphs=True):
    from llmx_amd.engine import Engine
    return Engine.load(model_folder(name), dtype=dtype, kv_tokens=kv_tokens, page_tokens=PAGES[name], max_requests=max_requests, graphs=graphs)


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


def same_rows(got, whole, dtype, what, tol=CUT_TOL):
    """Two cuttings of the same tokens.  float32: the same bits.  bfloat16: the same bits except that a token decoded alone
    shares out its context over work items of the matrix-core latent attention, whose partial sums are joined in another
    order than a prompt portion's row walks its keys: such rows agree within rounding."""
    if dtype == "float32":
        assert torch.equal(got, whole), f"{what}: rows differ, first at row {int((got != whole).any(1).nonzero()[0])}"
    else:
        close(got, whole, tol)


def against_plain(name, dtype, length, seed, got):
    want = plain_logits(name, length, seed, dtype == "bfloat16")
    close(got, want, F32_TOL if dtype == "float32" else BF16_TOL)


LENGTHS = (1, 2, 9, 33, 75, 130)


def test_whole_prompts_and_every_layer(setup):
    name, dtype, engine = setup
    for seed, length in enumerate(LENGTHS):
        tokens = tokens_for(name, length, seed)
        got = run_cut(engine, ("w", seed), tokens, [(0, length)])
        against_plain(name, dtype, length, seed, got)
    # the residual after every layer, for one prompt
    cfg, w = plain.load_folder(model_folder(name))
    tokens = tokens_for(name, 21, 99)
    layers = []
    plain.forward(cfg, w, tokens, torch.float64, torch.bfloat16 if dtype == "bfloat16" else None, layers)
    seen = []
    engine.observer = lambda step, kind, **t: seen.append(t["residual"].clone()) if kind == "layer" else None
    try:
        run_cut(engine, "layers", tokens, [(0, 21)])
    finally:
        engine.observer = None
    assert len(seen) == len(layers)
    for got, want in zip(seen, layers):
        close(got, want, F32_TOL if dtype == "float32" else BF16_TOL)


def test_prompt_against_token_by_token_and_portions(setup):
    """Every cutting gives every row the same values: whole, token by token from the first token, most of it whole and the
    rest one by one, and portions of changing size down to two tokens and to one (same_rows says what "the same" is)."""
    name, dtype, engine = setup
    length, seed = 130, 5
    tokens = tokens_for(name, length, seed)
    whole = run_cut(engine, "whole", tokens, [(0, length)])
    against_plain(name, dtype, length, seed, whole)
    cuttings = {
        "one by one": [(i, i + 1) for i in range(length)],
        "decoded tail": [(0, length - 40)] + [(i, i + 1) for i in range(length - 40, length)],
        "portions": portions(length, 1),
        "portions of one": portions(length, 2, smallest=1),
        "pairs": [(i, min(i + 2, length)) for i in range(0, length, 2)],
    }
    for what, cuts in cuttings.items():
        same_rows(run_cut(engine, what, tokens, cuts), whole, dtype, what)
    # portions of at least two tokens walk their keys as the whole prompt does: the same bits in bfloat16 too
    assert torch.equal(run_cut(engine, "pairs", tokens, cuttings["pairs"]), whole)


def test_unequal_requests_in_one_batch_and_reused_pages_and_slots(setup):
    """Four requests of unequal length advance together, portions of some beside single tokens of others, in an engine
    with four seats and so few pages that ended requests' pages and slots are taken again by later ones; every row has
    the bits it has when its request runs alone, cut the same way, in a fresh engine, and the whole prompt's rows."""
    from llmx_amd.engine import StepEntry
    name, dtype, _ = setup
    lengths = [70, 23, 1, 96, 40, 17, 64, 5]
    alone_engine = make_engine(name, dtype)
    alone = {i: run_cut(alone_engine, i, tokens_for(name, n, 20 + i), [(0, n)]) for i, n in enumerate(lengths)}
    engine = make_engine(name, dtype, kv_tokens=4 * 112, max_requests=4)
    rng = random.Random(3)
    waiting = list(range(len(lengths)))
    live, fed, got, cuts = [], {}, {i: [] for i in range(len(lengths))}, {i: [] for i in range(len(lengths))}
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
            cuts[i].append((fed[i], fed[i] + n))
            at += n
            fed[i] += n
            if fed[i] == lengths[i]:
                engine.end_request(i)
                live.remove(i)
    for i in range(len(lengths)):
        same_rows(torch.cat(got[i]), alone[i], dtype, f"request {i} against its whole prompt")
        again = run_cut(alone_engine, ("again", i), tokens_for(name, lengths[i], 20 + i), cuts[i])
        assert torch.equal(torch.cat(got[i]), again), f"request {i} differs from its run alone"
    assert engine.cache.pages_in_use(0) == 0 if engine.cache.groups else True
    assert engine.cache.slots.in_use == 0


def test_long_decoding_and_graph_replays(setup):
    """A short prompt, then 150 tokens one by one over many pages: the rows of the whole sequence, from an engine that
    replays decode steps as graphs and from one that does not."""
    name, dtype, engine = setup
    length, seed = 170, 8
    tokens = tokens_for(name, length, seed)
    cuts = [(0, 20)] + [(i, i + 1) for i in range(20, length)]
    before = engine.graph_replays
    got = run_cut(engine, "long", tokens, cuts)
    assert engine.graphs and engine.graph_replays - before > 100
    against_plain(name, dtype, length, seed, got)
    eager = make_engine(name, dtype, graphs=False)
    assert torch.equal(run_cut(eager, "long", tokens, cuts), got)
    same_rows(got, run_cut(eager, "whole", tokens, [(0, length)]), dtype, "decoded against whole")


def test_a_long_prompt_in_one_step(setup):
    """600 tokens in one step: the recurrence runs in chunks and the attention walks many segments; against the plain model,
    against portions of at most 100 rows (the one-launch recurrence) and against decoding the last 40 tokens."""
    name, dtype, engine = setup
    length, seed = 600, 12
    tokens = tokens_for(name, length, seed)
    whole = run_cut(engine, "long whole", tokens, [(0, length)])
    against_plain(name, dtype, length, seed, whole)
    tol = 2e-5 if dtype == "float32" else CUT_TOL
    close(run_cut(engine, "long portions", tokens, [(i, min(i + 100, length)) for i in range(0, length, 100)]), whole, tol)
    close(run_cut(engine, "long decoded", tokens, [(0, 300), (300, length - 40)] + [(i, i + 1) for i in range(length - 40, length)]), whole, tol)


def test_a_failed_step_leaves_the_state_as_it_was():
    """A step that is refused for want of pages changes neither pages nor recurrent state: the request goes on with the
    bits of an engine that never failed."""
    from llmx_amd.cache import OutOfPages
    from llmx_amd.engine import StepEntry
    name = "P"
    tokens = tokens_for(name, 60, 1)
    engine = make_engine(name, "float32", kv_tokens=64, max_requests=2)
    engine.add_request("a")
    engine.add_request("b")
    first = engine.step([StepEntry("a", tokens[:20], [19])]).clone()
    with pytest.raises(OutOfPages):
        engine.step([StepEntry("a", tokens[20:40], [19]), StepEntry("b", tokens[:40], [])])
    rest = engine.step([StepEntry("a", tokens[20:60], list(range(40)))]).clone().cpu()
    whole = run_cut(make_engine(name, "float32"), "w", tokens, [(0, 60)])
    assert torch.equal(first.cpu()[0], whole[19]) and torch.equal(rest, whole[20:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_hundreds_of_tokens(dtype, tmp_path):
    """Query and key weights eight times larger make the softmax pick single keys far back; a key lost, shifted by one or
    read from another page shows in the logits.  Whole, portions and decoding agree bit for bit and with the plain model."""
    def sharper(tensors):
        for k in tensors:
            if k.endswith("mix.q") or k.endswith("mix.dkv"):
                tensors[k] = (tensors[k].float() * 4.0).to(tensors[k].dtype)
    folder = write_folder(CONFIGS["R"], 17, str(tmp_path / "sharp"), sharper)
    from llmx_amd.engine import Engine
    engine = Engine.load(folder, dtype=dtype, kv_tokens=1024, page_tokens=16, max_requests=2)
    length = 520
    tokens = tokens_for("R", length, 4)
    cfg, w = plain.load_folder(folder)
    want = plain.forward(cfg, w, tokens, torch.float64, torch.bfloat16 if dtype == "bfloat16" else None)
    whole = run_cut(engine, "w", tokens, [(0, length)])
    close(whole, want, 1e-4 if dtype == "float32" else 6e-2)
    same_rows(run_cut(engine, "p", tokens, portions(length, 9)), whole, dtype, "portions", 6e-2)
    assert torch.equal(run_cut(engine, "pairs", tokens, [(i, i + 2) for i in range(0, length, 2)]), whole)
    same_rows(run_cut(engine, "d", tokens, [(0, length - 50)] + [(i, i + 1) for i in range(length - 50, length)]), whole, dtype, "decoded", 6e-2)


def test_greedy_generation_through_the_scheduler():
    """`generate` (scheduler, step function, device sampler) with prompts of unequal length and a small step budget, so
    that prompts are cut into portions beside decoding requests; float32 picks the plain implementation's tokens."""
    from llmx_amd import SamplingParams, generate
    name = "P"
    cfg, w = plain.load_folder(model_folder(name))
    prompts = [tokens_for(name, n, 40 + n) for n in (3, 29, 11, 1, 18)]
    engine = make_engine(name, "float32", kv_tokens=512, max_requests=3)
    got = generate(engine, prompts, SamplingParams(max_tokens=12, temp=0.0), max_seqs=3, max_step_tokens=16)
    for p, g in zip(prompts, got):
        assert g == plain.greedy(cfg, w, p, 12)
    engine16 = make_engine(name, "bfloat16", kv_tokens=512, max_requests=3)
    got16 = generate(engine16, prompts, SamplingParams(max_tokens=12, temp=0.0), max_seqs=3, max_step_tokens=16)
    for p, g in zip(prompts, got16):
        # bfloat16 may take another of two nearly equal logits: each token it chose is among the plain model's best within rounding
        rows = plain.forward(cfg, w, p + g[:-1], torch.float64, torch.bfloat16)[len(p) - 1:]
        for i, tok in enumerate(g):
            assert float(rows[i, tok]) >= float(rows[i].max()) - 3e-2 * float(rows[i].abs().max())


def test_trace_replay_and_command_line(tmp_path):
    """bin/trace_run as a subprocess on a model folder: a prompt portion beside decoded tokens, requests that end and
    whose slots are taken again; the logits files are the engine's own rows.  `llmx logits` reads the same folder."""
    import json
    import subprocess
    import sys
    import numpy as np
    name = "P"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b, c = tokens_for(name, 40, 1), tokens_for(name, 9, 2), tokens_for(name, 30, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": [0, 32]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[33:34], "want": [0]}, {"id": "b", "tokens": b, "want": [8]}], "end": ["b"]},
        {"step": 2, "entries": [{"id": "c", "tokens": c[:2], "want": []}], "end": []},
        {"step": 3, "entries": [{"id": "c", "tokens": c[2:], "want": [27]}, {"id": "a", "tokens": a[34:], "want": [5]}], "end": ["a", "c"]},
    ]
    out = tmp_path / "out"
    run = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", model_folder(name), "--dtype", "float32", "--out", str(out),
                          "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    V = CONFIGS[name]["vocab"]
    want = {"a": plain_logits(name, 40, 1, False), "b": plain_logits(name, 9, 2, False), "c": plain_logits(name, 30, 3, False)}
    rows = {0: [("a", 0), ("a", 32)], 1: [("a", 33), ("b", 8)], 3: [("c", 29), ("a", 39)]}
    assert not (out / "2.f32").exists()
    for step, places in rows.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(-1, V))
        assert got.shape[0] == len(places)
        for r, (rid, p) in enumerate(places):
            close(got[r], want[rid][p], F32_TOL)
    cli = subprocess.run([sys.executable, os.path.join(root, "bin", "llmx"), "logits", model_folder(name), " ".join(map(str, b)), "--dtype", "f32", "--top", "1"],
                         capture_output=True, text=True, timeout=600)
    assert cli.returncode == 0, cli.stderr[-2000:]
    assert int(cli.stdout.splitlines()[-1].split()[0]) == int(torch.argmax(want["b"][8]))


def test_command_line_generates_from_a_configuration_with_random_weights(tmp_path):
    """`llmx generate --config JSON --random SEED` for this design: weights generated on the device, the scheduler's loop,
    the device sampler; the same seed gives the same tokens, greedy or drawn."""
    import json
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(CONFIGS["P"]))
    outs = []
    for extra in (["--temp", "0"], ["--temp", "0"], ["--temp", "0.8", "--topk", "20", "--seed", "7"], ["--temp", "0.8", "--topk", "20", "--seed", "7"]):
        run = subprocess.run([sys.executable, os.path.join(root, "bin", "llmx"), "generate", "--config", str(cfg), "--random", "5", "--std", "0.06",
                              "3 1 4 1 5 9 2 6", "-n", "9"] + extra, capture_output=True, text=True, timeout=600)
        assert run.returncode == 0, run.stderr[-2000:]
        ids = [int(t) for t in run.stdout.split()]
        assert len(ids) == 9 and all(0 <= t < CONFIGS["P"]["vocab"] for t in ids)
        outs.append(ids)
    assert outs[0] == outs[1] and outs[2] == outs[3]
