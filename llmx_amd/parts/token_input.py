"""Per-layer token input: what a layer adds to the residual from a table row of the token itself.

"gated_table": e = a slice [column0, column0 + dim) of the token's row in a table the embedding holds;
g = gelu_tanh(W_gate x) * e;  y = W_proj g;  x += RMSNorm(y) * norm (a weight a coordinate), with x the residual after the
layer's sum.  gelu_tanh(z) = z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
"""

from __future__ import annotations

import torch

from .. import ops
from .base import Part, register
from .spec import TensorSpec


class TokenInput(Part):
    def forward(self, step, x: torch.Tensor, x_act: torch.Tensor) -> None:
        """x (float32 [T, hidden]) += the part's result; x_act holds the same rows in the activation type."""
        raise NotImplementedError


class GatedTableInput(TokenInput):
    """params: hidden, dim, column0, table (the full name of the token table, which the embedding lists), table_width,
    eps.  Tensors <prefix>gate (dim, hidden), proj (hidden, dim), norm (hidden,)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.hidden = int(params["hidden"])
        self.dim = int(params["dim"])
        self.column0 = int(params["column0"])
        self.table_name = str(params["table"])
        self.table_width = int(params["table_width"])
        self.eps = float(params["eps"])
        if self.dim < 1 or self.column0 < 0 or self.column0 + self.dim > self.table_width:
            raise ValueError(f"token input: columns {self.column0}..{self.column0 + self.dim} do not lie in a table of width {self.table_width}")
        self.w_gate = self.w_proj = self.norm = self.table = None

    def tensor_specs(self, available):
        return [TensorSpec(self.name("gate"), (self.dim, self.hidden)), TensorSpec(self.name("proj"), (self.hidden, self.dim)),
                TensorSpec(self.name("norm"), (self.hidden,), "norm")]

    def load(self, tensors):
        self.w_gate = tensors[self.name("gate")]
        self.w_proj = tensors[self.name("proj")]
        self.norm = tensors[self.name("norm")]
        self.table = tensors[self.table_name]
        if tuple(self.table.shape[1:]) != (self.table_width,):
            raise ValueError(f"token input: table {self.table_name} has rows of {tuple(self.table.shape[1:])}, expected ({self.table_width},)")

    def forward(self, step, x, x_act):
        T = step.rows
        pre = step.buf("token_input.pre", (T, self.dim), torch.float32)
        ops.gemm(x_act, self.w_gate, pre, scratch=step.buf)
        gated = step.buf("token_input.gated", (T, self.dim), step.act_dtype)
        ops.act_gelu_gather(pre, self.table, step.token_ids, gated, self.column0)
        y = step.buf("token_input.y", (T, self.hidden), torch.float32)
        ops.gemm(gated, self.w_proj, y, scratch=step.buf)
        ops.rmsnorm_add(x, y, self.norm, self.eps)


register("token_input", "gated_table", GatedTableInput)
