"""Steps on the residual stream that a plan puts before a run (``Run.enter``)."""
import torch

from ..config.spec import InputMixSpec
from ..ops import kernels as K
from ..ops import linear as L
from .base import Param, Part, Runtime, check_bound, register_stream_step


class InputMix(Part):
    """``x <- W [x; x0]``: the stream and the embedded rows of the step's tokens side by side,
    through one matrix ``W [dim, 2 dim]`` (the columns for x first).  The operand is rounded
    to the compute type once; the product's float32 sums are the new stream."""

    replayable = True

    def __init__(self, spec: InputMixSpec, runtime: Runtime):
        self.spec = spec
        self.rt = runtime
        self.weight = None

    def parameters(self):
        return {self.spec.name: Param((self.spec.dim, 2 * self.spec.dim))}

    def bind(self, tensors):
        check_bound("InputMix", self.parameters(), tensors)
        self.weight = tensors[self.spec.name]

    def step_flops(self, q_lens, starts) -> float:
        return 2.0 * sum(q_lens) * 2 * self.spec.dim * self.spec.dim

    def forward(self, residual: torch.Tensor, embedded: torch.Tensor, batch) -> torch.Tensor:
        both = K.concat_rows(residual, embedded, self.rt.dtype)
        return L.linear(both, self.weight, out_dtype=torch.float32)


register_stream_step("input_mix", InputMix)
