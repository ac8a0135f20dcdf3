"""A mixer made of mixers that read the same rows side by side; the result is their weighted sum.

    result = sum_i scale_i * member_i(h)

Every member is a mixer of the registry with its own tensors (under <prefix><member's name>.) and its own cache need: the
pages of a softmax attention beside the state of a recurrence, for instance.  The engine sees one composite need and
hands each member its own part of the cache.
"""

from __future__ import annotations

import torch

from .. import ops
from .base import LayerCache, Mixer, build_part, register
from .spec import CompositeNeed, PartSpec


class SideBySide(Mixer):
    """params: hidden; members: a list of {name, scale, mixer (PartSpec)}.  A member's tensors start with its own prefix
    (its PartSpec's); a built model lists the members as parts of their own after this one (`members()`), so each names
    and takes its tensors and has its say in a recorded step's key itself."""

    steps_between_slots = True      # every member with state says so itself; the engine asks the members

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.hidden = int(params["hidden"])
        listed = list(params["members"])
        if not listed:
            raise ValueError("side by side: at least one member")
        self.names = [str(m["name"]) for m in listed]
        self.scales = [float(m["scale"]) for m in listed]
        self._members = [build_part("mixer", m["mixer"], ctx) for m in listed]
        self.graph_safe = all(getattr(m, "graph_safe", False) for m in self._members)
        self.wants_f32_input = any(m.wants_f32_input for m in self._members)

    def members(self):
        return list(self._members)

    def cache_need(self):
        return CompositeNeed(tuple(m.cache_need() for m in self._members))

    def forward(self, step, h, out, accumulate, cache: LayerCache, h32=None):
        T = step.rows
        caches = cache.members if cache.members is not None else [None] * len(self._members)
        results, biases = [], []
        for i, (m, c) in enumerate(zip(self._members, caches)):
            y = step.buf(f"side_by_side.y{i}", (T, self.hidden), torch.float32)
            # a member that would add a bias to its result leaves that to the join, where it costs nothing
            later = getattr(m, "output_bias", None)
            bias = later() if later is not None else None
            if bias is not None:
                m.forward(step, h, y, False, c, h32 if m.wants_f32_input else None, add_output_bias=False)
            else:
                m.forward(step, h, y, False, c, h32 if m.wants_f32_input else None)
            results.append(y)
            biases.append(bias)
        # two members a launch, in the members' order
        first = True
        i = 0
        while i < len(results):
            pair = i + 1 < len(results) and biases[i + 1] is None
            ops.combine_rows(out, results[i], self.scales[i], biases[i], results[i + 1] if pair else None, self.scales[i + 1] if pair else 1.0,
                             accumulate or not first)
            first = False
            i += 2 if pair else 1


register("mixer", "side_by_side", SideBySide)
