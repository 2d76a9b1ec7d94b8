"""RMSNorm with an optional `(1 + scale)` gain (simply/model_lib.py:114-178, LayerNorm with
use_bias=False).  Statistics and the multiplication are in float32."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import NORMS
from .base import Norm, ParamSpec


@NORMS.register("none")
class NoNorm(Norm):
    """No norm: the part behind it reads the residual stream itself, in the activation type.  (The 32-bit path hands
    the stream on as it is: a part never writes into what it is given.)"""

    def forward(self, x, out_dtype):
        if x.dtype == out_dtype:
            return x
        return ops.residual_add_norm(None, x, out_dtype=out_dtype)

    def add_into(self, residual, y, next_norm, out_dtype):
        ops.residual_add_norm(y, residual)
        return next_norm.forward(residual, out_dtype) if next_norm is not None else None


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    #: the fused norm-and-product kernel computes exactly this norm from (scale, eps, scale_plus_one)
    fusable_rms = True
    #: add_into takes a product whose cuts of K are not added up yet (`ops.PartialSums`) in place of y
    adds_partial_sums = True

    def __init__(self, dim: int, eps: float, scale_plus_one: bool = True, mult: float = 1.0):
        self.dim = int(dim)
        self.eps = float(eps)
        self.scale_plus_one = bool(scale_plus_one)
        #: a constant that the norm's result is multiplied by (a residual multiplier of blocks that norm what a part
        #: returns); the kernels that fuse this norm into a product compute the norm without it
        self.mult = float(mult)
        self.fusable_rms = self.mult == 1.0
        self.adds_partial_sums = self.mult == 1.0
        self.scale: torch.Tensor | None = None

    def param_specs(self):
        return {"scale": ParamSpec((self.dim,), role="vector", init="norm")}

    def forward(self, x, out_dtype):
        if self.mult != 1.0:
            raise NotImplementedError("rmsnorm: a norm with a factor is applied through add_into only")
        return ops.rmsnorm(x, self.scale, self.eps, self.scale_plus_one, out_dtype)

    def add_into(self, residual, y, next_norm, out_dtype):
        """residual += self(y) and, fused when the next norm is an RMSNorm too, next_norm(residual)."""
        if self.mult != 1.0 or isinstance(next_norm, NoNorm):
            # one kernel: the sum, and the residual handed on in the activation type where no norm follows
            hand_on = isinstance(next_norm, NoNorm) and out_dtype != torch.float32
            out = ops.residual_add_norm(y, residual, weight=self.scale, eps=self.eps, plus_one=self.scale_plus_one,
                                        mult=self.mult, out_dtype=out_dtype if hand_on else None)
            if next_norm is None:
                return None
            return out if hand_on else next_norm.forward(residual, out_dtype)
        if next_norm is None or isinstance(next_norm, RMSNorm):
            return ops.add_rmsnorm(
                y, residual, post_weight=self.scale, post_eps=self.eps, post_plus_one=self.scale_plus_one,
                next_weight=None if next_norm is None else next_norm.scale,
                next_eps=0.0 if next_norm is None else next_norm.eps,
                next_plus_one=True if next_norm is None else next_norm.scale_plus_one, out_dtype=out_dtype)
        ops.add_rmsnorm(y, residual, post_weight=self.scale, post_eps=self.eps, post_plus_one=self.scale_plus_one)
        return next_norm.forward(residual, out_dtype)
