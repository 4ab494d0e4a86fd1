"""A layer's input from the tokens themselves: every layer reads its own slice of a second
embedding table and lets the residual stream gate it.

    e = table[token][layer * dim : (layer + 1) * dim]
    y = W_proj (gelu_tanh(W_gate x) * e)
    x <- x + y / sqrt(mean(y^2) + eps) * w

x is the residual stream itself (rounded to the activation dtype for the product), the norm an RMS
norm with a plain weight. The table is shared by the layers ([vocab, layers * dim]); the part is told
which columns are its own. The sum into x and the norm are the caller's (the block joins them with what
reads the stream next): ``output`` gives y as float32 rows and ``row_norm`` the norm's parameters.
"""

from __future__ import annotations

from typing import Dict

import torch

from ..config.spec import ConfigError
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Part
from .linear import Linear


class TokenInput(Part):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.dim = int(spec["dim"])
        self.first_column = int(spec["first_column"])
        self.table_columns = int(spec["table_columns"])
        self.vocab = int(spec["vocab_size"])
        self.eps = float(spec["norm_eps"])
        self.table_name = str(spec["table"])
        if self.dim < 1 or self.first_column < 0 or self.first_column + self.dim > self.table_columns:
            raise ConfigError(f"token input: columns {self.first_column}..{self.first_column + self.dim} of a table {self.table_columns} wide")

    def tensors(self) -> Dict[str, TensorDecl]:
        p = self.prefix
        return {self.table_name: TensorDecl((self.vocab, self.table_columns)),
                p + "gate": TensorDecl((self.dim, self.hidden)), p + "proj": TensorDecl((self.hidden, self.dim)),
                p + "norm": TensorDecl((self.hidden,), "vector", "norm")}

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        self.table = tensors[self.table_name]
        self.gate = Linear(tensors[self.prefix + "gate"])
        self.proj = Linear(tensors[self.prefix + "proj"])
        self.weight = tensors[self.prefix + "norm"]

    def row_norm(self):
        return self.weight, self.eps, False

    def gathered_tensors(self):
        """What the part reads by the row (a step's accounting does not count it among the weights it streams)."""
        return (self.table,)

    def output(self, x_rounded: torch.Tensor, ctx) -> torch.Tensor:
        """``x_rounded``: the residual rows in the activation dtype. Returns y, float32 [rows, hidden]."""
        z = self.gate.forward(x_rounded, out_dtype=torch.float32)
        gated = ops.gelu_gate_rows(z, self.table, ctx.token_ids, self.first_column, self.dtype)
        return self.proj.forward(gated, out_dtype=torch.float32)
