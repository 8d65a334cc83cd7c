"""Gated feed-forward (reference model.py:219-227)."""
import math

import torch

from ..config.spec import DenseFeedForwardSpec, GatedFeedForwardSpec
from ..ops import kernels as K
from ..ops import linear as L
from .base import Param, Part, Runtime, add_late, check_bound, register_feed_forward


class GatedFeedForward(Part):
    """``w2( act(w1 x) * (w3 x) )`` without biases, act = silu or the tanh form of gelu.  w1
    and w3 are one matrix ``w13`` (rows of w1, then rows of w3) so that the gate is applied
    where the products end."""

    def __init__(self, spec: GatedFeedForwardSpec, runtime: Runtime):
        if spec.activation not in L.GATE_ACTIVATIONS:
            raise ValueError(f"activation '{spec.activation}': {sorted(L.GATE_ACTIVATIONS)}")
        self.spec = spec
        self.rt = runtime
        self.w13 = self.w2 = None

    def parameters(self):
        s = self.spec
        return {"w13": Param((2 * s.hidden, s.dim)), "w2": Param((s.dim, s.hidden))}

    def bind(self, tensors):
        check_bound("GatedFeedForward", self.parameters(), tensors)
        self.w13, self.w2 = tensors["w13"], tensors["w2"]

    replayable = True
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream
    # x may be an ops.linear.HalfNormed, from one row on (the least number of rows; with the
    # weights streamed past the caches the matrix-core kernel that takes the halves is as fast
    # at one row as the dot-product kernel that does not, and the norm kernel is saved)
    takes_prepared = 1

    def step_flops(self, q_lens, starts) -> float:
        return 2.0 * sum(q_lens) * 3 * self.spec.hidden * self.spec.dim

    def forward(self, x, batch, residual):
        # both products wait until the stream is read next: whether the gate's result stays in
        # the order the second product loads it in depends on the norm that follows
        add_late(residual, lambda rows, then_norm, takes_halves: L.gated_into(
            x, self.w13, self.w2, rows, then_norm, takes_halves, self.spec.activation))


register_feed_forward("gated", GatedFeedForward)


def _softplus(z: float) -> float:
    return max(z, 0.0) + math.log1p(math.exp(-abs(z)))


class DenseFeedForward(Part):
    """``w_down( act(w_up x) )`` without biases and without a gate.  ``activation`` "xielu"
    has two learned numbers p, q (the parameter ``act``): for z > 0 ``softplus(p) z^2 + z/2``,
    for z <= 0 ``(1/2 + softplus(q)) (exp(z) - 1 - z) + z/2``; the two factors are worked out
    once, when the weights are bound.  "silu" and "gelu_tanh" have no parameter."""

    replayable = True
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream

    def __init__(self, spec: DenseFeedForwardSpec, runtime: Runtime):
        if spec.activation not in K.ACTIVATIONS:
            raise ValueError(f"activation '{spec.activation}': {sorted(K.ACTIVATIONS)}")
        self.spec = spec
        self.rt = runtime
        self.w_up = self.w_down = None
        self.a = self.b = 0.0

    def parameters(self):
        s = self.spec
        p = {"w_up": Param((s.hidden, s.dim)), "w_down": Param((s.dim, s.hidden))}
        if s.activation == "xielu":
            p["act"] = Param((2,), role="vector", init="unit")
        return p

    def bind(self, tensors):
        check_bound("DenseFeedForward", self.parameters(), tensors)
        self.w_up, self.w_down = tensors["w_up"], tensors["w_down"]
        if self.spec.activation == "xielu":
            p, q = (float(v) for v in tensors["act"].to(torch.float32).cpu())
            self.a, self.b = _softplus(p), 0.5 + _softplus(q)

    def step_flops(self, q_lens, starts) -> float:
        return 2.0 * sum(q_lens) * 2 * self.spec.hidden * self.spec.dim

    def _inner(self, x):
        h = L.linear(x, self.w_up)
        return K.activate(h, self.spec.activation, self.a, self.b, out=h)

    def forward(self, x, batch, residual):
        add_late(residual, lambda rows, then_norm, takes_halves: L.linear_into(
            self._inner(x), self.w_down, rows, then_norm, takes_halves))

    def forward_rows(self, x, batch):
        """The feed-forward's output alone: the second product's float32 sums."""
        return L.linear(self._inner(x), self.w_down, out_dtype=torch.float32)


register_feed_forward("dense", DenseFeedForward)
