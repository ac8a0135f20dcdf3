"""Bonerax assembled from parts.

Embedding; per layer the "outnorm" arrangement (x += LN(mixer(x)); x += LN(ff(x)), the sublayers reading the residual
itself) with a mixer among gated linear attention, the channel-wise gated delta rule, and "parallel": windowed softmax
attention (biases, a norm a head on q and k, interleaved partial rotation with a YaRN blend, values of their own width)
side by side with such a delta rule, joined by two constant weights; a dense SwiGLU, routed SwiGLU experts (softmax over
the picked logits, a bias in the router's logits) or no feed-forward; a final layer norm and an untied head whose logits
are scaled and soft-capped.  A layer that names another's weights becomes a second run-order entry of that layer's block
with its own cache number.  Tensor names: embed, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*, final.norm, head.
"""

from __future__ import annotations

from ..config.bonerax import ARCHITECTURE, BoneraxConfig
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, RunEntry
from .registry import register_architecture

NO_POSITION_LIMIT = 1 << 30     # the design states no longest context: the cache's size is the limit

_ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "q_bias": "q.b", "k_bias": "k.b",
                    "v_bias": "v.b", "o_bias": "o.b"}
_EXPERT_NAMES = {"router": "router", "logit_bias": "router.b", "expert_gate": "e{e}.gate", "expert_up": "e{e}.up", "expert_down": "e{e}.down",
                 "fused_gate_up": "gate_up", "fused_down": "down"}
_GLU_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def _delta(c: BoneraxConfig, i: int, m, prefix: str) -> PartSpec:
    return PartSpec("channel_delta_rule", {"hidden": c.width, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
                                           "conv": m.conv, "eps": c.norm_eps, "decay_rank": c.rank(i, "decay"), "gate_rank": c.rank(i, "gate")},
                    prefix)


def _mixer(c: BoneraxConfig, i: int) -> PartSpec:
    layer = c.layers[i]
    m, p = layer.mixer, f"l{i}.mix."
    if layer.type == "gla":
        return PartSpec("gated_linear_attention", {"hidden": c.width, "heads": m.heads, "dim": m.dim, "vdim": m.vdim, "tau": m.tau,
                                                   "eps": c.norm_eps, "rank": c.rank(i, "decay")}, p)
    if layer.type == "channel_delta":
        return _delta(c, i, m, p)
    a = m.left
    s = a.rot_scaling
    position = PartSpec("rotary_scaled", {"dims": a.rot_dims, "base": a.rot_base, "pairing": "interleaved",
                                          "scaling": None if s is None else {"factor": s.factor, "original": s.original, "fast": s.fast,
                                                                             "slow": s.slow}})
    left = PartSpec("attention", {"hidden": c.width, "heads": a.heads, "kv_heads": a.kv_heads, "head_dim": a.dim, "v_dim": a.vdim,
                                  "qk_norm": "head", "eps": c.norm_eps, "window": a.window, "scale": a.scale, "bias": True,
                                  "position": position, "names": _ATTENTION_NAMES}, p + "left.")
    return PartSpec("side_by_side", {"hidden": c.width, "members": [
        {"name": "left", "scale": m.left_scale, "mixer": left},
        {"name": "right", "scale": m.right_scale, "mixer": _delta(c, i, m.right, p + "right.")}]}, p)


def assemble(c: BoneraxConfig) -> ModelSpec:
    E = c.width

    def norm(name):
        return PartSpec("layernorm", {"width": E, "eps": c.norm_eps, "tensor": ""}, name)

    blocks, block_of, run_order = [], {}, []
    for i, layer in enumerate(c.layers):
        if layer.weights_of is None:
            p = f"l{i}."
            ffn = ffn_norm = None
            if layer.mlp is not None:
                ffn_norm = norm(p + "norm2")
                if layer.mlp.kind == "dense":
                    ffn = PartSpec("dense_glu", {"hidden": E, "intermediate": layer.mlp.ff, "names": _GLU_NAMES}, p + "mlp.")
                else:
                    ffn = PartSpec("routed_experts", {"hidden": E, "experts": layer.mlp.experts, "top_k": layer.mlp.top,
                                                      "intermediate": layer.mlp.ff, "score": "softmax", "normalize": "always", "logit_bias": True,
                                                      "names": _EXPERT_NAMES, "files": "per_expert"}, p + "mlp.")
            block_of[i] = len(blocks)
            blocks.append(BlockSpec(mixer_norm=norm(p + "norm1"), mixer=_mixer(c, i), ffn_norm=ffn_norm, ffn=ffn, arrangement="outnorm"))
    for i in range(len(c.layers)):
        run_order.append(RunEntry(layer=block_of[c.owner(i)], cache=i))
    return ModelSpec(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab,
        hidden_size=E,
        max_positions=NO_POSITION_LIMIT,
        embedding=PartSpec("token_embedding", {"vocab": c.vocab, "hidden": E, "tensor": ""}, "embed"),
        blocks=blocks,
        run_order=run_order,
        final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab": c.vocab, "hidden": E, "tied": False, "tensor": "", "logit_scale": c.logit_scale,
                                 "softcap": c.logit_softcap}, "head"),
    )


register_architecture(ARCHITECTURE, BoneraxConfig, assemble, replace=True)
