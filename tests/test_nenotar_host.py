"""Nenotar on the host: its configuration reader, its assembly from parts, and pins of the plain implementation."""

from __future__ import annotations

import copy
import math

import numpy as np
import pytest
import torch

import plain_nenotar as plain
from nenotar_cases import CONFIGS, CONFIG_P, model_folder


def test_configuration_round_trip_and_refusals():
    from llmx_amd import ConfigError, NenotarConfig
    from llmx_amd.models import read_config
    for name, config in CONFIGS.items():
        cfg = read_config(copy.deepcopy(config))
        assert isinstance(cfg, NenotarConfig) and cfg.to_json() == config
        assert read_config(cfg.to_json()) == cfg
    for path, value, word in ((("width",), None, "missing key width"), (("layers", 1, "mixer", "kv_rank"), None, "missing key layers[1].mixer.kv_rank"),
                              (("layers", 0, "type"), "lstm", "layers[0].type"), (("layers", 1, "mixer", "rot", "dims"), 15, "rot.dims"),
                              (("layers", 1, "mixer", "rot", "dims"), 18, "rot.dims"), (("layers", 0, "mlp", "kind"), "routed", "mlp.kind"),
                              (("norm", "eps"), "tiny", "norm.eps"), (("layers", 1, "mixer", "scale"), 0.0, "scale")):
        bad = copy.deepcopy(CONFIG_P)
        at = bad
        for k in path[:-1]:
            at = at[k]
        if value is None:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        with pytest.raises(ConfigError, match=word.replace("[", r"\[").replace("]", r"\]")):
            read_config(bad)
    extra = copy.deepcopy(CONFIG_P)
    extra["layers"][1]["mixer"]["window"] = 64
    with pytest.raises(ConfigError, match="window is not one this engine reads"):
        read_config(extra)
    with pytest.raises(ConfigError, match="unsupported architecture"):
        read_config({"architecture": "Nenotar2"})


def test_assembly_names_every_tensor_once_with_its_shape():
    from llmx_amd.models import read_config
    from llmx_amd.weights.folder import model_tensor_specs
    specs = {s.name: s for s in model_tensor_specs(read_config(copy.deepcopy(CONFIG_P)))}
    E, L, side = 80, 5, 16
    assert specs["embed"].shape == (304, E) and specs["side.embed"].shape == (304, L * side) and specs["head"].shape == (304, E)
    assert specs["final.norm"].shape == () and specs["l0.norm1"].shape == () and specs["l0.ls1"].shape == (E,)
    assert specs["l1.mix.q"].shape == (3 * (24 + 16), E) and specs["l1.mix.dkv"].shape == (48 + 16, E) and specs["l1.mix.g"].shape == (3, E)
    assert specs["l1.mix.uk"].shape == (3 * 24, 48) and specs["l1.mix.uv"].shape == (3 * 40, 48) and specs["l1.mix.o"].shape == (E, 3 * 40)
    assert specs["l0.mix.z"].shape == (72, E) and specs["l0.mix.x.b"].shape == (72,) and specs["l0.mix.o"].shape == (E, 72)
    assert specs["l0.mlp.up"].shape == (112, E) and specs["l0.mlp.act"].shape == (2,) and specs["l4.side.proj"].shape == (E, side)
    # a layer without a feed-forward has neither its norm nor its scale
    assert "l2.norm2" not in specs and "l2.ls2" not in specs and "l2.mlp.up" not in specs and "l3.norm2" not in specs
    # ... unless the file holds them all the same: then they are taken (and never applied) rather than refused
    from llmx_amd.engine.model import BuiltModel
    from llmx_amd.models import registry
    from llmx_amd.parts.base import BuildContext
    model = BuiltModel(registry.assemble(read_config(copy.deepcopy(CONFIG_P))), BuildContext(torch.float32, torch.device("cpu"), 1))
    held = {s.name for s in model.tensor_specs({"l2.norm2", "l2.ls2"})}
    assert {"l2.norm2", "l2.ls2"} <= held and "l3.norm2" not in held
    # the folder written from these specs is what the plain implementation reads
    cfg, w = plain.load_folder(model_folder("P"))
    assert set(w) == set(specs) and all(tuple(w[n].shape) == tuple(specs[n].shape) for n in specs)


def test_rotary_table_follows_the_blend_of_frequencies():
    from llmx_amd.parts.position import blended_frequencies, scaled_table
    for rot in ({"base": 10000.0, "dims": 16, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}},
                {"base": 500.0, "dims": 4}, {"base": 250000.0, "dims": 32, "scaling": {"factor": 3.0, "original": 4096, "fast": 32.0, "slow": 0.5}}):
        f, mag = blended_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        pf, pmag = plain.rotary_frequencies(rot)
        assert np.allclose(f, pf.numpy(), rtol=1e-12) and math.isclose(mag, pmag, rel_tol=1e-12)
        table = scaled_table(300, rot["dims"], rot["base"], rot.get("scaling"))
        x = torch.randn(300, 2, rot["dims"] + 3, dtype=torch.float64)
        want = plain.rotate_interleaved(x, list(range(300)), rot)
        half = rot["dims"] // 2
        cos, sin = torch.from_numpy(table[:, :half]).double()[:, None, :], torch.from_numpy(table[:, half:]).double()[:, None, :]
        u, v = x[..., 0:rot["dims"]:2], x[..., 1:rot["dims"]:2]
        assert torch.allclose(want[..., 0:rot["dims"]:2], u * cos - v * sin, atol=1e-6) and torch.allclose(want[..., 1:rot["dims"]:2], v * cos + u * sin, atol=1e-6)
        assert torch.equal(want[..., rot["dims"]:], x[..., rot["dims"]:])
    # with scaling the fastest pairs keep their frequency and the slowest are divided by the factor
    f, _ = blended_frequencies(16, 10000.0, {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0})
    plain_f, _ = blended_frequencies(16, 10000.0, None)
    assert f[0] == plain_f[0] and math.isclose(f[-1], plain_f[-1] / 8.0)


def test_plain_pins():
    """Special cases of the plain functions that reduce to library routines or to each other."""
    z = torch.linspace(-6, 6, 1001, dtype=torch.float64)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"), atol=1e-12)
    assert torch.allclose(plain.softplus(z * 20), torch.nn.functional.softplus(z * 20, threshold=1e9), atol=1e-12)
    p, q = torch.tensor(0.3, dtype=torch.float64), torch.tensor(-0.7, dtype=torch.float64)
    y = plain.xielu(torch.tensor([-1e-9, 0.0, 1e-9], dtype=torch.float64), p, q)
    assert abs(float(y[0])) < 1e-8 and float(y[1]) == 0.0 and abs(float(y[2])) < 1e-8          # continuous at 0, slope 1/2 on both sides
    assert math.isclose(float(plain.xielu(torch.tensor(2.0, dtype=torch.float64), p, q)), math.log1p(math.exp(0.3)) * 4 + 1)
    # the recurrence carried over a cut equals the whole
    g = torch.Generator().manual_seed(0)
    W, E = 6, 9
    w = {k: torch.randn(*s, generator=g, dtype=torch.float64) for k, s in (("z", (W, E)), ("x", (W, E)), ("g", (W, E)), ("o", (E, W)), ("z.b", (W,)), ("x.b", (W,)))}
    h = torch.randn(11, E, generator=g, dtype=torch.float64)
    whole, S = plain.mingru(h, w, "", {"width": W})
    a, Sa = plain.mingru(h[:4], w, "", {"width": W})
    b, Sb = plain.mingru(h[4:], w, "", {"width": W}, state=Sa)
    assert torch.allclose(torch.cat([a, b]), whole, atol=1e-13) and torch.allclose(Sb, S, atol=1e-13)
    # a gate of one half: z = 1/2 everywhere and a candidate of u + 1/2 give the running mean the closed form
    w0 = {k: torch.zeros_like(v) for k, v in w.items()}
    w0["o"] = torch.eye(E, W, dtype=torch.float64)
    w0["g"] = w["g"]
    _, S0 = plain.mingru(h[:3], w0, "", {"width": W})
    assert torch.allclose(S0, torch.full((W,), 0.5 * (1 - 0.5 ** 3), dtype=torch.float64))


def test_latent_attention_equals_the_form_over_cached_latents():
    """score = (W_uk^T q_plain) . c + q_rot . k_rot and result = W_uv (sum of weights * c): the form the engine computes
    over cached latents is the plain attention with expanded keys and values."""
    g = torch.Generator().manual_seed(4)
    H, D, R, V, C, E, T = 3, 5, 4, 6, 7, 10, 12
    m = {"heads": H, "dim": D, "rot_dim": R, "vdim": V, "kv_rank": C, "scale": 0.4, "rot": {"base": 50.0, "dims": 4}}
    w = {"q": torch.randn(H * (D + R), E, generator=g), "dkv": torch.randn(C + R, E, generator=g), "dkv.norm": torch.rand(C, generator=g) + 0.5,
         "uk": torch.randn(H * D, C, generator=g), "uv": torch.randn(H * V, C, generator=g), "g": torch.randn(H, E, generator=g),
         "o": torch.randn(E, H * V, generator=g)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.randn(T, E, generator=g).double()
    want = plain.latent_attention(h, w, "", m, 1e-6, list(range(T)))
    q = (h @ w["q"].T).view(T, H, D + R)
    down = h @ w["dkv"].T
    c = plain.rms(down[:, :C], 1e-6) * w["dkv.norm"]
    k_rot = plain.rotate_interleaved(down[:, C:], list(range(T)), m["rot"])
    q_rot = plain.rotate_interleaved(q[..., D:], list(range(T)), m["rot"])
    q_lat = torch.einsum("thd,hdc->thc", q[..., :D], w["uk"].view(H, D, C))
    out = torch.zeros(T, H, V, dtype=torch.float64)
    for t in range(T):
        s = (torch.einsum("hc,sc->hs", q_lat[t], c[:t + 1]) + torch.einsum("hr,sr->hs", q_rot[t], k_rot[:t + 1])) * 0.4
        mixed = torch.softmax(s, dim=-1) @ c[:t + 1]
        out[t] = torch.einsum("hc,hvc->hv", mixed, w["uv"].view(H, V, C))
    out = out * torch.sigmoid(h @ w["g"].T)[:, :, None]
    assert torch.allclose(out.reshape(T, H * V) @ w["o"].T, want, atol=1e-12)
