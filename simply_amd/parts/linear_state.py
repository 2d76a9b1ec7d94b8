"""Recurrent mixers whose state is one matrix per head that decays and takes an outer product per token:

    S_t = diag(a_t) S_(t-1) + c_t k_t v_t^T,      o_t = S_t^T q_t

'gated_linear_attention': a decay per key channel, a_t = sigmoid(z_t)^(1 / tau) with z from a low-rank projection
(two factors and a bias), c = 1; each head's o is divided by its root mean square, multiplied by a weight that the
heads share and by silu(gate x), then projected.

'matrix_memory': the matrix memory with exponential gates.  Per head the logarithm of an input gate,
i = cap tanh((W_i x + b_i) / cap), and of a forget gate, f = log sigmoid(cap tanh((W_f x + b_f) / cap)); with a running
maximum m_t = max(f + m_(t-1), i) that starts at 0, a = exp(f + m_(t-1) - m_t) and c = exp(i - m_t).  A normalizer
n_t = a n_(t-1) + c k_t runs beside S (stored as one more column of it, whose value is always 1), and
o = S^T q / (max(|n . q|, exp(-m)) + 1e-6); each head's o is then divided by its root mean square, multiplied by a
weight (one entry per head and channel) and by sigmoid(gate x), then projected.

Queries are multiplied by key size^(-1/2).  The state (and m) lives in one float32 row of a state slot per request;
gates, decays and the recurrence are 32-bit, q, k, v and the gate come out of one product in the activation type.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import MIXERS
from .base import Mixer, ParamSpec, StateNeed, as_product_weight, project


@MIXERS.register("gated_linear_attention")
class GatedLinearAttention(Mixer):
    #: the mixer's input enters one product only: for a few rows the norm in front of it runs in that product's kernel
    accepts_pending = True

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decay_rank: int, tau: float,
                 norm_eps: float):
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.key_dim, self.value_dim, self.decay_rank = int(key_dim), int(value_dim), int(decay_rank)
        self.tau, self.norm_eps = float(tau), float(norm_eps)
        if self.tau <= 0:
            raise ValueError("gated_linear_attention: tau must be positive")
        self.state_words = self.num_heads * self.key_dim * self.value_dim
        self.in_proj = self.o_proj = self.decay_out = self.decay_bias = self.norm = None

    def param_specs(self):
        D, H, dk, dv, R = self.hidden_size, self.num_heads, self.key_dim, self.value_dim, self.decay_rank
        return {"q_proj": ParamSpec((H * dk, D)), "k_proj": ParamSpec((H * dk, D)), "v_proj": ParamSpec((H * dv, D)),
                "gate_proj": ParamSpec((H * dv, D)), "o_proj": ParamSpec((D, H * dv)),
                "decay_in": ParamSpec((R, D)), "decay_out": ParamSpec((H * dk, R)),
                "decay_bias": ParamSpec((H * dk,), role="vector", init="norm"),
                "norm": ParamSpec((dv,), role="vector", init="norm")}

    def load(self, tensors):
        t = tensors
        # one product for q, k, v, the gate and the decay's first factor
        self.in_proj = as_product_weight(torch.cat([t["q_proj"], t["k_proj"], t["v_proj"], t["gate_proj"],
                                                    t["decay_in"]], dim=0).contiguous())
        self.o_proj = as_product_weight(t["o_proj"])
        self.decay_out, self.decay_bias = as_product_weight(t["decay_out"]), t["decay_bias"].contiguous()
        self.norm = t["norm"].contiguous()

    def cache_need(self):
        return StateNeed((self.state_words,), torch.float32)

    def forward(self, x, ctx, cache):
        if not cache.write:
            raise RuntimeError("gated_linear_attention: a recurrent state cannot be read through another entry's cache")
        H, dk, dv, R = self.num_heads, self.key_dim, self.value_dim, self.decay_rank
        C = H * dk
        g_at = 2 * C + H * dv
        u_at = g_at + H * dv
        proj = project(x, self.in_proj)
        # the decay's second factor is a product of its own, kept in 32-bit; sigmoid(. + bias)^(1 / tau) is computed
        # where the recurrence stages its tiles
        z = ops.gemm(proj[:, u_at:u_at + R], self.decay_out, out_dtype=torch.float32)
        o = ops.linear_state(proj, 0, C, 2 * C, dk ** -0.5, z, False, H, dk, dv, False, cache.state, ctx.seq_meta,
                             ctx.num_seqs, decay_bias=self.decay_bias, tau=self.tau)
        z = ops.gated_heads(o, proj[:, g_at:g_at + H * dv], H, dv, kind=ops.GATE_SILU, weight=self.norm,
                            eps=self.norm_eps, out_dtype=ctx.dtype)
        return ops.gemm(z, self.o_proj)


@MIXERS.register("matrix_memory")
class MatrixMemory(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, gate_cap: float, norm_eps: float):
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        if self.gate_cap <= 0:
            raise ValueError("matrix_memory: the gates' cap must be positive")
        #: the matrices with the normalizer's column, then the running maxima
        self.matrix_words = self.num_heads * self.key_dim * (self.value_dim + 1)
        self.in_proj = self.gates_proj = self.gates_bias = self.o_proj = self.norm = None

    def param_specs(self):
        D, H, dk, dv = self.hidden_size, self.num_heads, self.key_dim, self.value_dim
        return {"q_proj": ParamSpec((H * dk, D)), "k_proj": ParamSpec((H * dk, D)), "v_proj": ParamSpec((H * dv, D)),
                "gate_proj": ParamSpec((H * dv, D)), "o_proj": ParamSpec((D, H * dv)),
                "input_gate": ParamSpec((H, D)), "forget_gate": ParamSpec((H, D)),
                "input_bias": ParamSpec((H,), role="vector", init="norm"),
                "forget_bias": ParamSpec((H,), role="vector", init="norm"),
                "norm": ParamSpec((H * dv,), role="vector", init="norm")}

    def load(self, tensors):
        t = tensors
        self.in_proj = as_product_weight(torch.cat([t["q_proj"], t["k_proj"], t["v_proj"], t["gate_proj"]], dim=0).contiguous())
        # the gates' projections are a product of their own, kept in 32-bit
        self.gates_proj = as_product_weight(torch.cat([t["input_gate"], t["forget_gate"]], dim=0).contiguous())
        self.gates_bias = torch.cat([t["input_bias"], t["forget_bias"].to(t["input_bias"].dtype)]).contiguous()
        self.o_proj = as_product_weight(t["o_proj"])
        self.norm = t["norm"].contiguous()

    def cache_need(self):
        return StateNeed((self.matrix_words + self.num_heads,), torch.float32)

    def forward(self, x, ctx, cache):
        if not cache.write:
            raise RuntimeError("matrix_memory: a recurrent state cannot be read through another entry's cache")
        H, dk, dv = self.num_heads, self.key_dim, self.value_dim
        C = H * dk
        g_at = 2 * C + H * dv
        proj = ops.gemm(x, self.in_proj)
        raw = ops.gemm(x, self.gates_proj, out_dtype=torch.float32)
        maxima = cache.state[:, self.matrix_words:self.matrix_words + H]
        gates = ops.exp_gates(raw, self.gates_bias, self.gate_cap, H, maxima, ctx.seq_meta, ctx.num_seqs)
        o = ops.linear_state(proj, 0, C, 2 * C, dk ** -0.5, gates, True, H, dk, dv, True, cache.state, ctx.seq_meta,
                             ctx.num_seqs)
        z = ops.normalized_readout(o, gates[:, 2 * H:3 * H], proj[:, g_at:g_at + H * dv], self.norm, self.norm_eps, H, dv,
                                   ctx.dtype)
        return ops.gemm(z, self.o_proj)
