"""Bonerax on the CPU: the plain implementation's functions against cases with known answers, the configuration reader's
refusals, and the assembly's tensor list and run order."""

from __future__ import annotations

import copy
import math

import numpy as np
import pytest

import plain_bonerax as plain
from bonerax_cases import CONFIGS, CONFIG_A, model_folder


def test_layer_norm_centres_and_scales():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(3, 17)) * 5 + 2
    y = plain.layer_norm(x, np.ones(17), 0.0)
    assert np.allclose(y.mean(-1), 0.0, atol=1e-12) and np.allclose((y * y).mean(-1), 1.0)
    # a large eps shrinks, the weight multiplies coordinate by coordinate
    w = rng.normal(size=17)
    assert np.allclose(plain.layer_norm(x, w, 3.0), (x - x.mean(-1, keepdims=True)) / np.sqrt(x.var(-1, keepdims=True) + 3.0) * w)


def test_rotation_keeps_lengths_scaled_and_composes():
    rng = np.random.default_rng(1)
    x = rng.normal(size=(5, 2, 12))
    scaling = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}
    y = plain.rotate_pairs(x, [0, 1, 7, 100, 1000], 8, 10000.0, scaling)
    magnitude = 0.1 * math.log(4.0) + 1.0
    assert np.allclose(y[..., 8:], x[..., 8:]) and np.allclose(y[0, :, :8], x[0, :, :8] * magnitude)
    assert np.allclose(np.linalg.norm(y[..., :8], axis=-1), np.linalg.norm(x[..., :8], axis=-1) * magnitude)
    # scores depend on the distance only
    q, k = rng.normal(size=(1, 1, 8)), rng.normal(size=(1, 1, 8))
    at = lambda v, p: plain.rotate_pairs(v, [p], 8, 500.0, scaling)[0, 0]
    assert np.isclose(at(q, 9) @ at(k, 4), at(q, 105) @ at(k, 100))
    # without scaling pair i turns by base^(-2i/dims); the blend keeps fast pairs and slows slow ones by the factor
    f, one = plain.rotary_frequencies(8, 10000.0, None)
    assert one == 1.0 and np.allclose(f, 10000.0 ** (-np.arange(4) / 4.0))
    g, _ = plain.rotary_frequencies(8, 10000.0, {"factor": 4.0, "original": 64, "fast": 1e9, "slow": 1e8})
    assert np.allclose(g[1:], f[1:] / 4.0) and g[0] == f[0]      # the ramp starts at pair 0: every later pair counts as slow
    g, _ = plain.rotary_frequencies(8, 10000.0, {"factor": 4.0, "original": 64, "fast": 1e-9, "slow": 1e-10})
    assert np.allclose(g, f)            # every pair counts as fast


def test_short_convolution_is_causal_and_starts_from_zeros():
    x = np.arange(1.0, 6.0)[:, None] * np.ones((1, 2))
    w = np.array([[0.0, 0.0, 1.0], [1.0, 0.0, 0.0]])     # channel 0 takes the current input, channel 1 the one two back
    y = plain.short_conv_silu(x, w)
    assert np.allclose(y[:, 0], plain.silu(x[:, 0])) and np.allclose(y[:, 1], plain.silu(np.array([0, 0, 1.0, 2, 3])))


def test_delta_rule_against_its_closed_forms():
    rng = np.random.default_rng(2)
    T, H, D, V = 6, 2, 3, 4
    q, k, v = rng.normal(size=(T, H, D)), rng.normal(size=(T, H, D)), rng.normal(size=(T, H, V))
    # no decay and beta 0: nothing is ever written
    assert np.allclose(plain.delta_rule_scan(q, k, v, np.ones((T, H, D)), np.zeros((T, H))), 0.0)
    # orthonormal keys, beta 1, no decay: every key returns the value last written under it
    k = np.zeros((3, 1, 3))
    k[[0, 1, 2], 0, [0, 1, 0]] = 1.0
    v = rng.normal(size=(3, 1, 2))
    o = plain.delta_rule_scan(k, k, v, np.ones((3, 1, 3)), np.ones((3, 1)))
    assert np.allclose(o[:, 0], v[:, 0])
    o2 = plain.delta_rule_scan(np.array([[[0, 1.0, 0]], [[1.0, 0, 0]]]), k[:2], v[:2], np.ones((2, 1, 3)), np.ones((2, 1)))
    assert np.allclose(o2[0, 0], 0.0) and np.allclose(o2[1, 0], v[0, 0])
    # a decay of one channel only fades what lies under that channel
    o3 = plain.delta_rule_scan(np.array([[[1.0, 0, 0]], [[1.0, 1.0, 0]]]), k[:2], v[:2], np.array([[[1.0, 1, 1]], [[0.5, 1, 1]]]), np.ones((2, 1)))
    assert np.allclose(o3[1, 0], 0.5 * v[0, 0] + v[1, 0])


def test_gated_linear_attention_with_no_decay_is_a_running_sum():
    rng = np.random.default_rng(3)
    T, E, H, D, V = 5, 6, 2, 3, 2
    w = {n: rng.normal(size=s) for n, s in (("q", (H * D, E)), ("k", (H * D, E)), ("v", (H * V, E)), ("g", (H * V, E)), ("o", (E, H * V)),
                                            ("a1", (2, E)), ("a2", (H * D, 2)))}
    w["a2"] *= 0.0
    w["a2.b"] = np.full(H * D, 50.0)          # sigmoid(50) is 1 to the last bit: no decay
    w["norm"] = np.ones(V)
    h = rng.normal(size=(T, E))
    m = {"heads": H, "dim": D, "vdim": V, "tau": 3.0}
    got = plain.gla(h, w, m, 1e-6)
    q, k, v = (h @ w["q"].T).reshape(T, H, D) * D ** -0.5, (h @ w["k"].T).reshape(T, H, D), (h @ w["v"].T).reshape(T, H, V)
    o = np.stack([sum((q[t, :, None, :] @ k[s, :, :, None])[:, 0, 0, None] * v[s] for s in range(t + 1)) for t in range(T)])
    want = (plain.rms_unit(o, 1e-6).reshape(T, H * V) * plain.silu(h @ w["g"].T)) @ w["o"].T
    assert np.allclose(got, want)


def test_window_attention_sees_exactly_its_window():
    rng = np.random.default_rng(4)
    T, E = 12, 8
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 3, "scale": 0.5, "mask": {"size": 4}, "rot": {"base": 100.0, "dims": 2}}
    w = {n: rng.normal(size=s) for n, s in (("q", (8, E)), ("k", (4, E)), ("v", (3, E)), ("o", (E, 6)), ("q.b", (8,)), ("k.b", (4,)),
                                            ("v.b", (3,)), ("o.b", (E,)), ("q.norm", (4,)), ("k.norm", (4,)))}
    h = rng.normal(size=(T, E))
    full = plain.window_attention(h, w, m, 1e-6)
    changed = h.copy()
    changed[3] += 1.0                                     # position 3 is inside the windows of rows 3..6 only
    again = plain.window_attention(changed, w, m, 1e-6)
    differs = np.abs(again - full).max(axis=1) > 1e-12
    assert list(np.nonzero(differs)[0]) == [3, 4, 5, 6]
    # a suffix run with its own positions matches the whole run once the window has forgotten the prefix
    tail = plain.window_attention(h[5:], w, m, 1e-6, positions=range(5, T))
    assert np.allclose(tail[3:], full[8:])


def test_router_softmax_over_the_picks_alone():
    rng = np.random.default_rng(5)
    h = rng.normal(size=(4, 6))
    w = {"router": rng.normal(size=(5, 6)), "router.b": rng.normal(size=5) * 3}
    for e in range(5):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = rng.normal(size=(3, 6)), rng.normal(size=(3, 6)), rng.normal(size=(6, 3))
    picks = []
    one = plain.routed_experts(h, w, {"router": {"experts": 5, "top": 1}}, picks)
    z = h @ w["router"].T + w["router.b"]
    assert [p[0] for p in picks] == list(z.argmax(1))     # the bias is part of the logits
    for t in range(4):
        e = picks[t][0]
        assert np.allclose(one[t], plain.glu(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0])   # one pick weighs 1
    every = plain.routed_experts(h, w, {"router": {"experts": 5, "top": 5}})
    p = np.exp(z - z.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    want = sum(p[:, e:e + 1] * plain.glu(h, w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"]) for e in range(5))
    assert np.allclose(every, want)


def test_configuration_reads_writes_and_refuses():
    from llmx_amd.config import BoneraxConfig, ConfigError
    from llmx_amd.models import read_config
    for config in CONFIGS.values():
        cfg = read_config(copy.deepcopy(config))
        assert isinstance(cfg, BoneraxConfig) and read_config(cfg.to_json()) == cfg
    def refused(change, text):
        bad = copy.deepcopy(CONFIG_A)
        change(bad)
        with pytest.raises(ConfigError, match=text):
            read_config(bad)
    refused(lambda c: c["layers"][0]["mixer"]["left"].pop("scale"), r"missing key layers\[0\].mixer.left.scale")
    refused(lambda c: c["layers"][1]["mixer"].update(extra=1), r"layers\[1\].mixer.extra is not one this engine reads")
    refused(lambda c: c["layers"][2].update(type="conv"), r"layers\[2\].type")
    refused(lambda c: c["layers"][3].update(weights_of=3), r"layers\[3\].weights_of")
    refused(lambda c: c["layers"][3].update(weights_of=1), r"layers\[3\].weights_of")
    refused(lambda c: c["layers"][0]["mlp"]["router"].update(top=7), r"layers\[0\].mlp.router.top")
    refused(lambda c: c["layers"][0]["mixer"]["right"].update(kv_heads=3), r"layers\[0\].mixer.right.kv_heads")
    refused(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=34), r"layers\[0\].mixer.left.rot.dims")
    refused(lambda c: c.update(tie_embeddings=True), r"key tie_embeddings is not one this engine reads")
    # keys that say nothing about the arithmetic are let through
    named = copy.deepcopy(CONFIG_A)
    named.update(name="a", seed=3, dtype="bfloat16")
    assert read_config(named) == read_config(copy.deepcopy(CONFIG_A))
    # without the inner widths a configuration cannot be assembled; a model folder's tensor shapes give them
    from llmx_amd.models import assemble, read_model_dir
    bare = {k: v for k, v in CONFIG_A.items() if k != "ranks"}
    with pytest.raises(ConfigError, match="inner width"):
        assemble(read_config(copy.deepcopy(bare)))
    cfg, spec = read_model_dir(model_folder("A"))
    assert cfg.ranks == {0: {"decay": 8, "gate": 16}, 1: {"decay": 24}, 2: {"decay": 16, "gate": 8}}
    # layers that name another's tensors are further run-order entries of that layer's block, each with its own cache
    assert len(spec.blocks) == 3 and [(e.layer, e.cache) for e in spec.run_order] == [(0, 0), (1, 1), (2, 2), (0, 3), (1, 4)]


def test_tensor_list_and_cache_needs():
    import torch
    from llmx_amd.engine.model import BuiltModel
    from llmx_amd.models import read_model_dir
    from llmx_amd.parts import BuildContext, CompositeNeed, PagedNeed, StateNeed
    cfg, spec = read_model_dir(model_folder("A"))
    model = BuiltModel(spec, BuildContext(torch.bfloat16, torch.device("cpu"), 64, 16))
    names = {s.name for s in model.tensor_specs()}
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.mix.left.q.b", "l0.mix.left.k.norm", "l0.mix.right.q.conv", "l0.mix.right.A_log",
            "l0.mlp.router.b", "l0.mlp.e5.down", "l1.mix.a2.b", "l1.mlp.gate", "l2.mix.dt_bias", "l2.mix.g2"} <= names
    assert not any(n.startswith(("l3.", "l4.", "l2.mlp", "l2.norm2")) for n in names)
    needs = model.cache_needs()
    assert len(needs) == 5 and needs[0] == needs[3] and isinstance(needs[0], CompositeNeed)
    paged, state = needs[0].members
    assert isinstance(paged, PagedNeed) and paged.window == 40 and isinstance(state, StateNeed)
    assert state.shape == (4 * 16 * 24 + 3 * (2 * 2 * 16 + 4 * 24),) and needs[1].shape == (3 * 16 * 40,)
    assert needs[2].shape == (2 * 24 * 16 + 1 * (2 * 24 + 2 * 16),)
