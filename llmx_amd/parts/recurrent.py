"""Mixers that carry a fixed-size float32 state from token to token.

minGRU: the gates read only the current row, so everything but the recurrence itself is a product over all rows:
    z = sigmoid(W_z h + b_z),  u = W_x h + b_x,  cand = u + 1/2 where u >= 0, sigmoid(u) where u < 0,
    S_t = (1 - z) S_(t-1) + z cand   (element by element, S = 0 before a request's first token),
    result = W_o (S_t * silu(W_g h)).
The recurrence, its gates and the state are float32; the state lives in the request's slot.
"""

from __future__ import annotations

import torch

from .. import ops
from .base import LayerCache, Mixer, register
from .spec import StateNeed, TensorSpec


class MinGRU(Mixer):
    """params: hidden, width.  Tensors <prefix>z, z.b, x, x.b, g, o."""
    graph_safe = True
    steps_between_slots = True      # reads the state at step.entry_held_slots, writes it at step.entry_slots

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.hidden = int(params["hidden"])
        self.width = int(params["width"])
        if self.width < 1:
            raise ValueError("mingru: the width is at least 1")
        self.w_in = self.w_o = self.b_z = self.b_x = None

    def cache_need(self):
        return StateNeed((self.width,), "float32")

    def tensor_specs(self, available):
        W, E = self.width, self.hidden
        fused, shape = self.name("in"), (3 * W, E)        # one product for gate | candidate | output gate
        return [TensorSpec(self.name("z"), (W, E), into=(fused, shape, (slice(0, W),))),
                TensorSpec(self.name("x"), (W, E), into=(fused, shape, (slice(W, 2 * W),))),
                TensorSpec(self.name("g"), (W, E), into=(fused, shape, (slice(2 * W, 3 * W),))),
                TensorSpec(self.name("z.b"), (W,), "bias"),
                TensorSpec(self.name("x.b"), (W,), "bias"),
                TensorSpec(self.name("o"), (E, W))]

    def load(self, tensors):
        self.w_in = tensors[self.name("in")]
        self.w_o = tensors[self.name("o")]
        self.b_z = tensors[self.name("z.b")]
        self.b_x = tensors[self.name("x.b")]

    def forward(self, step, h, out, accumulate, cache: LayerCache, h32=None):
        T, W = step.rows, self.width
        pre = step.buf("mingru.pre", (T, 3 * W), torch.float32)
        ops.gemm(h, self.w_in, pre, scratch=step.buf)
        gated = step.buf("mingru.gated", (T, W), step.act_dtype)
        # long runs of rows (a prompt's portion) are worked on in chunks; a decode step's entries never are (nothing for a graph to hold)
        plan = step.shared("scan.plan", lambda: ops.scan_plan([e.n for e in step.entries], step.device))
        ops.mingru_scan(pre, self.b_z, self.b_x, cache.state, step.entry_held_slots, step.entry_slots, step.entry_rows, gated,
                        plan=plan, scratch=step.buf)
        ops.gemm(gated, self.w_o, out, ops.EPI_ADD if accumulate else ops.EPI_STORE, scratch=step.buf)


register("mixer", "mingru", MinGRU)
