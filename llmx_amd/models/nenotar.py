"""Nenotar assembled from parts.

Embedding times a scale; per layer the "parallel" arrangement: one RMS norm pass with two scalar gains, a mixer (latent
attention or minGRU) and a dense xIELU feed-forward on the same input, each result scaled a coordinate and summed into
the residual, then the layer's gated token input from its slice of a second token table; a final scalar-gain RMS norm and
an untied head.  Tensor names: embed, side.embed, l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*, l<i>.ls1, l<i>.ls2,
l<i>.side.*, final.norm, head.
"""

from __future__ import annotations

from ..config.nenotar import ARCHITECTURE, NenotarConfig
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, RunEntry
from .registry import register_architecture

SIDE_TABLE = "side.embed"
NO_POSITION_LIMIT = 1 << 30     # the design states no longest context: the cache's size is the limit


def assemble(c: NenotarConfig) -> ModelSpec:
    E = c.width
    n_layers = len(c.layers)
    side_width = (c.token_side_dim or 0) * n_layers

    def norm(name, optional=False):
        return PartSpec("rmsnorm", {"width": E, "eps": c.norm_eps, "gain": "scalar", "tensor": "", "optional": optional}, name)

    blocks = []
    for i, layer in enumerate(c.layers):
        p = f"l{i}."
        m = layer.mixer
        if layer.type == "latent_attention":
            s = m.rot_scaling
            position = PartSpec("rotary_scaled", {
                "dims": m.rot_dims, "base": m.rot_base, "pairing": "interleaved",
                "scaling": None if s is None else {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}})
            mixer = PartSpec("latent_attention", {
                "hidden": E, "heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
                "eps": c.norm_eps, "gate": "head_sigmoid", "position": position, "window": None}, p + "mix.")
        else:
            mixer = PartSpec("mingru", {"hidden": E, "width": m.width}, p + "mix.")
        extra = {"mixer_scale": ("scale", PartSpec("layer_scale", {"width": E}, p + "ls1"))}
        ffn = ffn_norm = None
        if layer.ff is not None:
            ffn = PartSpec("dense_act", {"hidden": E, "intermediate": layer.ff, "activation": "xielu"}, p + "mlp.")
            ffn_norm = norm(p + "norm2")
            extra["ffn_scale"] = ("scale", PartSpec("layer_scale", {"width": E}, p + "ls2"))
        else:   # a file may hold the second norm and scale of a layer without a feed-forward: taken, never applied
            ffn_norm = norm(p + "norm2", optional=True)
            extra["ffn_scale"] = ("scale", PartSpec("layer_scale", {"width": E, "optional": True}, p + "ls2"))
        if c.token_side_dim:
            extra["token_input"] = ("token_input", PartSpec("gated_table", {
                "hidden": E, "dim": c.token_side_dim, "column0": i * c.token_side_dim, "table": SIDE_TABLE, "table_width": side_width,
                "eps": c.norm_eps}, p + "side."))
        blocks.append(BlockSpec(mixer_norm=norm(p + "norm1"), mixer=mixer, ffn_norm=ffn_norm, ffn=ffn, arrangement="parallel", extra=extra))
    return ModelSpec(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab,
        hidden_size=E,
        max_positions=NO_POSITION_LIMIT,
        embedding=PartSpec("token_embedding", {"vocab": c.vocab, "hidden": E, "scale": c.embedding_scale, "tensor": "",
                                               "side_tables": {SIDE_TABLE: side_width} if side_width else {}}, "embed"),
        blocks=blocks,
        run_order=[RunEntry(layer=i, cache=i) for i in range(n_layers)],
        final_norm=norm("final.norm"),
        head=PartSpec("linear", {"vocab": c.vocab, "hidden": E, "tied": False, "tensor": ""}, "head"),
    )


register_architecture(ARCHITECTURE, NenotarConfig, assemble, replace=True)
