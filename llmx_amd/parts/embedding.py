"""Token embedding and the language-model head.

x[t] = table[id[t]] widened to float32, times the embedding's scale where the model has one (/root/reference/src/model/arch/blocks.hpp:95-97); logits = rows . W^T in
float32 for the wanted rows only (:267-272).  A tied head reads the embedding's table.
"""

from __future__ import annotations

import torch

from .. import ops
from .base import Embedding, Head, register
from .spec import TensorSpec


class TokenEmbedding(Embedding):
    """params: vocab, hidden; scale (the rows are multiplied by it, 1 by default); tensor (the name's last part, "weight"
    by default); side_tables: {full tensor name: width}, further tables with a row a token that other parts read by
    name (a part of each layer's own token input, for instance): the embedding lists them, once for the model.
    Tensor <prefix><tensor> (vocab, hidden)."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.vocab = int(params["vocab"])
        self.hidden = int(params["hidden"])
        self.scale = float(params.get("scale", 1.0))
        self.tensor = str(params.get("tensor", "weight"))
        self.side_tables = {str(k): int(v) for k, v in (params.get("side_tables") or {}).items()}
        self.weight = None

    def tensor_specs(self, available):
        return [TensorSpec(self.name(self.tensor), (self.vocab, self.hidden), "table")] + \
               [TensorSpec(name, (self.vocab, width), "table") for name, width in self.side_tables.items()]

    def load(self, tensors):
        self.weight = tensors[self.name(self.tensor)]

    def table(self):
        return self.weight

    def forward(self, step, out):
        ops.embed_gather(self.weight, step.token_ids, out, self.scale)


class LinearHead(Head):
    """params: vocab, hidden, tied (bool); tensor (the name's last part, "weight" by default); logit_scale (the logits are
    multiplied by it, 1 by default) and softcap (c > 0: logits <- c tanh(logits / c), after the scale; None: none).
    Tensor <prefix><tensor> (vocab, hidden) unless tied."""
    graph_safe = True

    def __init__(self, params, prefix, ctx):
        super().__init__(params, prefix, ctx)
        self.vocab = int(params["vocab"])
        self.hidden = int(params["hidden"])
        self.tied = bool(params.get("tied", False))
        self.tensor = str(params.get("tensor", "weight"))
        self.logit_scale = float(params.get("logit_scale", 1.0))
        self.softcap = float(params["softcap"]) if params.get("softcap") else 0.0
        if self.softcap < 0.0:
            raise ValueError("head: a softcap is positive")
        self.weight = None

    def tensor_specs(self, available):
        return [] if self.tied else [TensorSpec(self.name(self.tensor), (self.vocab, self.hidden), "table")]

    def load(self, tensors):
        if not self.tied:
            self.weight = tensors[self.name(self.tensor)]

    def tie(self, table: torch.Tensor) -> None:
        self.weight = table

    def forward(self, step, rows, logits):
        ops.gemm(rows, self.weight, logits)
        if self.logit_scale != 1.0 or self.softcap > 0.0:
            ops.scale_softcap(logits, self.logit_scale, self.softcap)


register("embedding", "token_embedding", TokenEmbedding)
register("head", "linear", LinearHead)
