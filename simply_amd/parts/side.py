"""A per-layer input from the token itself, added to the residual stream at a block's end:

    g = act(W_gate x) * e,   y = W_proj g,   x <- x + y / sqrt(mean(y^2) + eps) * w

with e the token's row of a side table, columns [column, column + dim) of it (the table is shared by the layers, each
reading its own columns), and x the stream as the feed-forward left it."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import ACTIVATIONS, STREAM_PARTS
from .base import ParamSpec, StreamPart, as_product_weight


@STREAM_PARTS.register("token_side")
class TokenSide(StreamPart):
    def __init__(self, hidden_size: int, dim: int, vocab_size: int, table_width: int, column: int, eps: float,
                 activation: str = "gelu_tanh"):
        self.hidden_size, self.dim, self.vocab_size = int(hidden_size), int(dim), int(vocab_size)
        self.table_width, self.column, self.eps = int(table_width), int(column), float(eps)
        if not 0 <= self.column <= self.table_width - self.dim:
            raise ValueError(f"token_side: columns {self.column}..{self.column + self.dim} of a table {self.table_width} wide")
        self.activation_code = int(ACTIVATIONS.get(activation))
        self.table = self.gate = self.proj = self.norm = None

    def param_specs(self):
        D, d = self.hidden_size, self.dim
        return {"table": ParamSpec((self.vocab_size, self.table_width)), "gate": ParamSpec((d, D)),
                "proj": ParamSpec((D, d)), "norm": ParamSpec((D,), role="vector", init="norm")}

    def load(self, tensors):
        self.table = tensors["table"]
        self.gate, self.proj = as_product_weight(tensors["gate"]), as_product_weight(tensors["proj"])
        self.norm = tensors["norm"].contiguous()

    def forward(self, h, ctx, x=None):
        if x is None:
            x = h if ctx.dtype == torch.float32 else ops.residual_add_norm(None, h, out_dtype=ctx.dtype)
        z = ops.gemm(x, self.gate)
        ops.token_gate_(z, ctx.tokens, self.table, self.column, self.activation_code)
        y = ops.gemm(z, self.proj)
        ops.residual_add_norm(y, h, weight=self.norm, eps=self.eps, plus_one=False)
