"""Differential attention: two softmax maps per head over the same values, over the paged
cache, with a sliding window that keeps the first keys."""
import math

import torch

from ..cache.store import KVNeed
from ..config.spec import DifferentialAttentionSpec
from ..ops import differential_attention as DA
from ..ops import kernels as K
from ..ops import linear as L
from .base import POSITIONS, Param, Part, Runtime, add_late, check_bound, register_mixer


class DifferentialAttention(Part):
    """Query head h holds two maps ``[q1, q2]`` and reads the two maps ``[k1, k2]`` and the
    values of kv head ``h // (H / G)``.  Both maps are rotated by position, scored against
    the visible keys (``j <= i`` and ``i - j < window`` or ``j < keep_first``) and softmaxed
    on their own; the head's result is ``a1 - lam a2`` with
    ``lam = exp(lq1 . lk1) - exp(lq2 . lk2) + lam_init``, divided by its root mean square
    over the value size, times ``1 - lam_init``, times sigmoid of one gate number per head,
    then ``wo``.  The projections of q, k, v and the gate are one matrix ``w_in`` whose product
    keeps its float32 sums until the rotation has been applied.  Scores, softmax, sums, the
    combination, the norm and the gate are float32."""

    libraries = ("differential_attention",)
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream
    takes_prepared = True          # x may be an ops.linear.HalfNormed

    def __init__(self, spec: DifferentialAttentionSpec, runtime: Runtime):
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError(f"{spec.n_heads} heads do not divide into {spec.n_kv_heads} kv heads")
        self.spec = spec
        self.rt = runtime
        self.position = POSITIONS.build(spec.position, runtime)
        if spec.position.kind == "rope":
            if spec.position.layout != "interleaved" or not hasattr(self.position, "freqs"):
                raise ValueError("differential attention rotates interleaved pairs by a "
                                 "frequency vector (position kind 'rope', layout 'interleaved')")
            self.rotary_dim, self.freqs = spec.position.rotary_dim, self.position.freqs
        elif spec.position.kind == "none":
            self.rotary_dim, self.freqs = 0, None
        else:
            raise ValueError(f"differential attention: position kind '{spec.position.kind}'")
        self.scale = spec.scale if spec.scale is not None else K.default_scale(spec.head_dim)
        self.window = 0 if spec.window is None else int(spec.window)
        s = spec
        self.q_off = 0
        self.k_off = s.n_heads * DA.MAPS * s.head_dim
        self.v_off = self.k_off + s.n_kv_heads * DA.MAPS * s.head_dim
        self.g_off = self.v_off + s.n_kv_heads * s.value_dim
        self.in_rows = self.g_off + (s.n_heads if s.head_gate else 0)
        self.w_in = self.wo = None
        self.lam = None

    def parameters(self):
        s = self.spec
        p = {"w_in": Param((self.in_rows, s.dim)),
             "wo": Param((s.dim, s.n_heads * s.value_dim))}
        for name in ("lq1", "lk1", "lq2", "lk2"):
            p[name] = Param((s.head_dim,), role="vector", init="linear")
        return p

    def bind(self, tensors):
        check_bound("DifferentialAttention", self.parameters(), tensors)
        # zero rows up to a multiple of eight: the products' kernels store whole groups
        self.w_in, self.wo = L.pad_rows(tensors["w_in"], 8), tensors["wo"]
        v = {n: tensors[n].to(torch.float32) for n in ("lq1", "lk1", "lq2", "lk2")}
        # one number for the layer, float32
        lam = (torch.exp((v["lq1"] * v["lk1"]).sum()) - torch.exp((v["lq2"] * v["lk2"]).sum())
               + torch.tensor(self.spec.lam_init, dtype=torch.float32, device=v["lq1"].device))
        self.lam = float(lam)
        if not math.isfinite(self.lam):
            raise ValueError("differential attention: lambda is not finite")

    def cache_need(self):
        s = self.spec
        return KVNeed(s.n_kv_heads, DA.MAPS * s.head_dim, s.window, s.value_dim,
                      s.keep_first if s.window is not None else 0)

    replayable = True

    def step_flops(self, q_lens, starts) -> float:
        s = self.spec
        n = sum(q_lens)
        flops = 2.0 * n * (self.in_rows + s.n_heads * s.value_dim) * s.dim
        for q, start in zip(q_lens, starts):
            keys = q * start + q * (q + 1) / 2.0
            if s.window is not None:
                keys = min(keys, q * float(s.window + s.keep_first))
            flops += 2.0 * DA.MAPS * s.n_heads * (s.head_dim + s.value_dim) * keys
        return flops

    def forward(self, x, batch, entry, residual):
        s = self.spec
        # the projection keeps its float32 sums: q and k are rounded once, after the rotation
        proj = L.linear(x, self.w_in, out_dtype=torch.float32)
        write = entry is not None and entry.writes
        table = batch.table(entry.group_id)
        q, gate = DA.rope_store(proj, self.q_off, self.k_off, self.v_off, self.g_off, self.freqs,
                                batch.tok_seq, batch.tok_pos, table,
                                entry.k_pages if write else None, entry.v_pages if write else None,
                                s.n_heads, s.n_kv_heads, s.head_dim, s.value_dim, self.rotary_dim,
                                self.rt.dtype, with_gate=s.head_gate)

        def finish(rows, then_norm, takes_halves):
            y = DA.attention(q, entry.k_pages, entry.v_pages, gate, batch, table, self.scale,
                             self.window, s.keep_first, self.lam, s.eps, 1.0 - s.lam_init)
            return L.linear_into(y, self.wo, rows, then_norm, takes_halves)

        add_late(residual, finish)


register_mixer("differential_attention", DifferentialAttention)
