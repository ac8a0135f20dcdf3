"""Causal softmax attention over one cached latent a token (keys and values are low-rank expansions of it).

Per row, from the normed input h:  q = W_q h, head by head [dim unrotated | rot_dim rotated];  W_dkv h = [latent of
kv_rank | one key part of rot_dim]: the latent is RMS-normed (weight `dkv.norm`) and is, with the rotated key part that
all heads share, all that is cached.  Head n's key for a token is [W_uk,n c | k_rot], its value W_uv,n c;
score = (q_plain . W_uk,n c + q_rot . k_rot) * scale, softmax over the request's keys up to the row, and the head's
result is multiplied by sigmoid(W_g h)_n before the output projection.

Neither keys nor values are ever expanded: q_lat = W_uk,n^T q_plain (a grouped product, one group a head) turns the
score into (q_lat . c + q_rot . k_rot) * scale over the cached rows themselves, the attention returns the weighted sum of
latents, and W_uv,n is applied to that (a second grouped product).
"""

from __future__ import annotations

import torch

from .. import ops
from .base import BuildContext, LayerCache, Mixer, build_part, register
from .spec import CacheTensor, PagedNeed, PartSpec, TensorSpec

MAX_LATENT = 2048          # the attention kernels keep a row's weighted sum of latents in a wave's registers
MAX_LATENT_KEY = 4096      # latent + rotated key part: a query row in a workgroup's LDS


class LatentAttention(Mixer):
    """params: hidden, heads, dim (unrotated query/key dims a head), rot_dim (rotated dims a head), vdim, kv_rank, scale (the
    factor on the scores), eps (of the latent's norm), gate ("head_sigmoid" | None), position (PartSpec of a rotary encoding
    whose dims are at most rot_dim), window (None).  Tensors <prefix>q, dkv, dkv.norm, uk, uv, g, o."""
    graph_safe = True

    def __init__(self, params, prefix, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        p = params
        self.hidden = int(p["hidden"])
        self.heads = int(p["heads"])
        self.dim = int(p["dim"])
        self.rot_dim = int(p["rot_dim"])
        self.vdim = int(p["vdim"])
        self.rank = int(p["kv_rank"])
        self.eps = float(p["eps"])
        self.scale = float(p["scale"])
        self.window = p.get("window")
        self.gate = p.get("gate", "head_sigmoid")
        if self.gate not in ("head_sigmoid", None):
            raise ValueError(f"latent attention: gate {self.gate!r} is not 'head_sigmoid' or None")
        if min(self.heads, self.dim, self.vdim, self.rank) < 1 or self.rot_dim < 0:
            raise ValueError("latent attention: heads, dim, vdim and kv_rank are at least 1 and rot_dim is not negative")
        if self.rank > MAX_LATENT or self.rank + self.rot_dim > MAX_LATENT_KEY:
            raise ValueError(f"latent attention: kv_rank {self.rank} with rot_dim {self.rot_dim}; the attention kernels take a latent of at "
                             f"most {MAX_LATENT} and at most {MAX_LATENT_KEY} with the rotated part")
        if not self.scale > 0.0:
            raise ValueError(f"latent attention: the softmax scale must be positive, not {self.scale}")
        self.position = build_part("position", p.get("position") or PartSpec("none"), ctx)
        if getattr(self.position, "pairing", "interleaved") != "interleaved":
            raise ValueError("latent attention: the rotated parts turn as interleaved pairs")
        if self.position.rotation()[1] > self.rot_dim:
            raise ValueError(f"latent attention: {self.position.rotation()[1]} rotated dims do not fit the rotated part of {self.rot_dim}")
        self.q_width = self.heads * (self.dim + self.rot_dim)
        self.down_width = self.rank + self.rot_dim
        self.gate_width = self.heads if self.gate else 0
        self.w_in = self.w_o = self.latent_norm = self.w_uk_t = self.w_uv = None

    def _matrix_cores(self) -> bool:
        """Whether this engine's steps run the attention on the matrix cores, which read the latents once more, transposed."""
        page = self.ctx.page_tokens
        return bool(page) and self.window is None and self.ctx.device.type == "cuda" \
            and ops.latent_attention_mfma_ok(self.ctx.act_dtype, self.rank, self.rot_dim, page)

    def cache_need(self):
        tensors = [CacheTensor("latent", (self.down_width,), None, 0)]       # a page: [tokens, kv_rank + rot_dim]
        if self._matrix_cores():
            tensors.append(CacheTensor("latent_t", (self.rank,), None, 1))     # the latents once more: [kv_rank, tokens]
        return PagedNeed(tuple(tensors), self.window)

    def tensor_specs(self, available):
        E, q, d, g = self.hidden, self.q_width, self.down_width, self.gate_width
        fused, shape = self.name("in"), (q + d + g, E)      # one product for the projections that read h: q | dkv | g
        specs = [TensorSpec(self.name("q"), (q, E), into=(fused, shape, (slice(0, q),))),
                 TensorSpec(self.name("dkv"), (d, E), into=(fused, shape, (slice(q, q + d),))),
                 TensorSpec(self.name("dkv.norm"), (self.rank,), "norm"),
                 TensorSpec(self.name("uk"), (self.heads * self.dim, self.rank)),
                 TensorSpec(self.name("uv"), (self.heads * self.vdim, self.rank)),
                 TensorSpec(self.name("o"), (E, self.heads * self.vdim))]
        if g:
            specs.append(TensorSpec(self.name("g"), (g, E), into=(fused, shape, (slice(q + d, q + d + g),))))
        return specs

    def load(self, tensors):
        self.w_in = tensors[self.name("in")]
        self.w_o = tensors[self.name("o")]
        self.latent_norm = tensors[self.name("dkv.norm")]
        # q_lat = W_uk,n^T q_plain: the grouped product wants each head's matrix as [out = kv_rank, in = dim]
        self.w_uk_t = tensors[self.name("uk")].view(self.heads, self.dim, self.rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[self.name("uv")].view(self.heads, self.vdim, self.rank)

    def _groups(self, step):
        return ops.head_groups(self.heads, step.rows, step.device)

    def _plan(self, step):
        if not self._matrix_cores():
            return None
        return step.shared(("latent.plan", self.heads), lambda: ops.latent_plan([e.n for e in step.entries], self.heads, step.device,
                                                                                 contexts=[e.past + e.n for e in step.entries]))

    def graph_key(self, step):
        # a recorded step reads the groups' lists and the plan's items; the key keeps them alive
        return self._groups(step), self._plan(step)

    def forward(self, step, h, out, accumulate, cache: LayerCache, h32=None):
        T, H, act = step.rows, self.heads, step.act_dtype
        proj = step.buf("latent.proj", (T, self.q_width + self.down_width + self.gate_width), torch.float32)
        ops.gemm(h, self.w_in, proj, scratch=step.buf)
        q_plain = step.buf("latent.q_plain", (H, T, self.dim), act)
        q_rot = step.buf("latent.q_rot", (H, T, self.rot_dim), act)
        latents = cache.tensors["latent"]
        tables = step.tables(cache.group)
        ops.latent_prep(proj, self.latent_norm, self.position.rotation()[0], step.positions, step.row_entry, tables, q_plain, q_rot,
                        latents, self.eps, H, self.dim, self.rot_dim, self.rank, write_cache=cache.writes, cache_t=cache.tensors.get("latent_t"))
        offsets, pairs, active, n_active = self._groups(step)
        q_lat = step.buf("latent.q_lat", (H, T, self.rank), act)
        ops.grouped_gemm(q_plain.view(H * T, self.dim), self.w_uk_t, q_lat.view(H * T, self.rank), offsets, pairs, 1, ops.EPI_STORE,
                         active, n_active, token_rows=T)
        mixed = step.buf("latent.mixed", (H, T, self.rank), act)
        ops.latent_attention(q_lat, q_rot, latents, step.positions, step.row_entry, tables, mixed, self.scale, window=int(self.window or 0),
                             scratch=step.buf, cache_t=cache.tensors.get("latent_t"), plan=self._plan(step))
        values = step.buf("latent.values", (H, T, self.vdim), torch.float32)
        ops.grouped_gemm(mixed.view(H * T, self.rank), self.w_uv, values.view(H * T, self.vdim), offsets, pairs, 1, ops.EPI_STORE,
                         active, n_active, token_rows=T)
        joined = step.buf("latent.joined", (T, H * self.vdim), act)
        gate = proj[:, self.q_width + self.down_width:] if self.gate else None
        ops.head_gate(values, gate, joined)
        ops.gemm(joined, self.w_o, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


register("mixer", "latent_attention", LatentAttention)
