"""Recurrent mixer with a matrix memory per head (the mLSTM cell of xLSTM)."""
import dataclasses

import torch

from ..cache.store import StateNeed
from ..config.spec import MatrixMemorySpec
from ..ops import linear as L
from ..ops import matrix_memory as M
from .base import Param, Part, Runtime, add_late, check_bound, register_mixer


class MatrixMemory(Part):
    """Per head a state ``S [dk, dv]``, ``n [dk]`` and a running maximum ``m`` of the log
    gates, float32, zero at a sequence's start, kept in the cache's state slot of the
    sequence and carried from step to step:

        i = cap tanh((w_i x + b_i) / cap)       f = logsigmoid(cap tanh((w_f x + b_f) / cap))
        m' = max(f + m, i)     S' = exp(f + m - m') S + exp(i - m') k v^T     (n likewise, with k)
        o = S'^T q / (max(|n' . q|, exp(-m')) + den_eps),     q = w_q x / sqrt(dk)

    then each head's o over its root mean square, times ``norm``, times sigmoid(w_g x), then
    ``wo``.  The six input projections are one matrix ``w_in`` (rows of q, k, v, g, i, f)
    whose product keeps its float32 accumulators: gates, state and everything between them
    are float32 whatever the engine's type; the rounding to the compute type happens once,
    at the operand of ``wo``."""

    replayable = True
    libraries = ("matrix_memory",)
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream
    takes_prepared = True          # x may be an ops.linear.HalfNormed

    def __init__(self, spec: MatrixMemorySpec, runtime: Runtime):
        if spec.key_dim > M.MAX_KEY_DIM:
            raise ValueError(f"matrix memory: key_dim {spec.key_dim} > {M.MAX_KEY_DIM}")
        self.spec = spec
        self.rt = runtime
        rows = M.RowLayout.fused(spec.n_heads, spec.key_dim, spec.value_dim)
        self.in_rows = rows.width                       # rows of w_in as it is stored
        self.rows = dataclasses.replace(rows, width=(rows.width + 7) // 8 * 8)
        self.w_in = self.wo = self.norm = self.gate_bias = None

    def parameters(self):
        s = self.spec
        return {"w_in": Param((self.in_rows, s.dim)),
                "gate_bias": Param((2 * s.n_heads,), role="vector", init="unit"),
                "norm": Param((s.n_heads * s.value_dim,), role="vector", init="norm"),
                "wo": Param((s.dim, s.n_heads * s.value_dim))}

    def bind(self, tensors):
        check_bound("MatrixMemory", self.parameters(), tensors)
        # zero rows up to a multiple of eight: the products' kernels store whole groups
        self.w_in, self.wo = L.pad_rows(tensors["w_in"], 8), tensors["wo"]
        self.norm = tensors["norm"].to(torch.float32).contiguous()
        self.gate_bias = tensors["gate_bias"].to(torch.float32).contiguous()

    def cache_need(self):
        s = self.spec
        return StateNeed((M.state_size(s.n_heads, s.key_dim, s.value_dim),), "float32")

    def step_flops(self, q_lens, starts) -> float:
        s = self.spec
        n = sum(q_lens)
        cell = 2.0 * 2.0 * s.n_heads * s.key_dim * s.value_dim          # update and read of S
        return n * (2.0 * (self.in_rows + s.n_heads * s.value_dim) * s.dim + cell)

    def forward(self, x, batch, entry, residual):
        s = self.spec
        proj = L.linear(x, self.w_in, out_dtype=torch.float32)
        o = M.cell(proj, self.rows, self.gate_bias, entry.state, batch.q_start, batch.slots,
                   batch.n_seqs, batch.max_q_len, s.n_heads, s.key_dim, s.value_dim,
                   s.key_dim ** -0.5, s.gate_cap or 0.0, s.den_eps)
        y = M.head_norm_gate(o, self.norm, proj, self.rows, s.eps, self.rt.dtype)
        add_late(residual, lambda rows, then_norm, takes_halves: L.linear_into(
            y, self.wo, rows, then_norm, takes_halves))


register_mixer("matrix_memory", MatrixMemory)
