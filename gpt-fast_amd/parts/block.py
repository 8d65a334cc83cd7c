"""How norms, mixer, feed-forward and the residual stream are wired in one layer."""
import torch

from ..config.spec import LayerSpec
from ..ops import kernels as K
from .base import FEED_FORWARDS, MIXERS, NORMS, Part, ResidualStream, Runtime, register_block


class PreNormBlock(Part):
    """``h = x + mixer(norm1(x)); out = h + ffn(norm2(h))`` (reference model.py:161-164).
    The residual stream is float32 and updated in place; the sums happen in the
    parts' epilogues.  A spec without a feed-forward gives ``out = h``."""

    def __init__(self, spec: LayerSpec, runtime: Runtime):
        self.spec = spec
        self.mixer_norm = NORMS.build(spec.mixer_norm, runtime)
        self.mixer = MIXERS.build(spec.mixer, runtime)
        self.feed_forward_norm = self.feed_forward = None
        if spec.feed_forward is not None:
            self.feed_forward_norm = NORMS.build(spec.feed_forward_norm, runtime)
            self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, runtime)

    def children(self):
        s = self.spec
        out = {s.mixer_norm_name: self.mixer_norm, s.mixer_name: self.mixer}
        if self.feed_forward is not None:
            out[s.feed_forward_norm_name] = self.feed_forward_norm
            out[s.feed_forward_name] = self.feed_forward
        return out

    def parameters(self):
        out = {}
        for child_name, child in self.children().items():
            for name, p in child.parameters().items():
                out[f"{child_name}.{name}"] = p
        return out

    def bind(self, tensors):
        for child_name, child in self.children().items():
            prefix = child_name + "."
            child.bind({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})

    def cache_need(self):
        return self.mixer.cache_need()

    def step_flops(self, q_lens, starts) -> float:
        """Matrix-product work of one run of this block (parts that do not say count as 0)."""
        return sum(getattr(c, "step_flops", lambda q, s: 0.0)(q_lens, starts)
                   for c in self.children().values())

    def step_fields(self):
        out = []
        for child in self.children().values():
            out += list(getattr(child, "step_fields", lambda: ())())
        return out

    # Reads the stream through ``stream.normed`` so that the kernel which completed it can
    # hand over the norm's rows (parts.base.ResidualStream); parts that do not put off their
    # sum get the plain tensor.
    takes_stream = True

    @property
    def replayable(self):
        return all(getattr(c, "replayable", False) for c in self.children().values())

    @property
    def takes_prepared(self):
        return getattr(self.mixer, "takes_prepared", False)

    @staticmethod
    def _residual_for(part, stream):
        return stream if getattr(part, "defers_sum", False) else stream.tensor

    def forward(self, residual, batch, entry):
        stream = residual if isinstance(residual, ResidualStream) else ResidualStream(residual)
        x = stream.normed(self.mixer_norm, reader=self.mixer)
        self.mixer.forward(x, batch, entry, self._residual_for(self.mixer, stream))
        if self.feed_forward is not None:
            h = stream.normed(self.feed_forward_norm, reader=self.feed_forward)
            self.feed_forward.forward(h, batch, self._residual_for(self.feed_forward, stream))
        if stream is not residual:
            stream.tensor                    # a caller with a plain tensor gets the sums now


# up to this many rows a sandwich block takes a sublayer's result as its last product's float32
# sums (the few-row kernels store them directly); measured on a 4,096-wide stack: 1.51 -> 1.44 ms
# a step at 8 rows, but 2.26 -> 2.82 ms at 64 rows and 12.5 -> 13.6 ms for 2,048 tokens
DIRECT_MAX_ROWS = 16


class SandwichNormBlock(PreNormBlock):
    """``h = x + norm1b(mixer(norm1(x))); out = h + norm2b(ffn(norm2(h)))``: a norm before
    each sublayer and a second one on its result, before that joins the stream.  A sublayer
    that offers ``forward_rows(x, batch[, entry]) -> float32 [N, D]`` hands its result over as
    its last product's float32 sums where that product is one of the library's own kernels
    with a float32 store (few rows, or the float32 engine); else it adds into a float32 tensor
    of its own, which starts at zero (with many bfloat16 rows the vendor library's bfloat16
    result plus the kernel that adds it is faster than its float32 result).  One kernel then norms the result, adds it to the stream and, where the
    block knows which norm reads the stream next (its own feed-forward's), applies that one in
    the same pass."""

    takes_stream = False
    takes_prepared = False

    def __init__(self, spec: LayerSpec, runtime: Runtime):
        super().__init__(spec, runtime)
        if spec.mixer_out_norm is None or (spec.feed_forward is not None
                                           and spec.feed_forward_out_norm is None):
            raise ValueError("a sandwich_norm block needs a norm on each sublayer's result")
        self.rt = runtime
        self.mixer_out_norm = NORMS.build(spec.mixer_out_norm, runtime)
        self.feed_forward_out_norm = None
        if spec.feed_forward is not None:
            self.feed_forward_out_norm = NORMS.build(spec.feed_forward_out_norm, runtime)

    def children(self):
        out = super().children()
        out[self.spec.mixer_out_norm_name] = self.mixer_out_norm
        if self.feed_forward is not None:
            out[self.spec.feed_forward_out_norm_name] = self.feed_forward_out_norm
        return out

    def _join(self, residual, y, out_norm, next_norm):
        """residual += out_norm(y); the rows of ``next_norm`` over the sum, or None."""
        form = getattr(out_norm, "row_and_column_form", None)
        next_form = getattr(next_norm, "row_and_column_form", None)
        if form is None:
            K.add_into(residual, out_norm.forward(y))
            return None if next_norm is None else next_norm.forward(residual)
        weight, eps = form()
        if next_form is None:
            K.normed_add(residual, y, weight, eps)
            return None if next_norm is None else next_norm.forward(residual)
        next_weight, next_eps = next_form()
        return K.normed_add(residual, y, weight, eps, next_weight, next_eps, self.rt.dtype)

    def forward(self, residual, batch, entry):
        if isinstance(residual, ResidualStream):
            residual = residual.tensor
        direct = self.rt.is_float32 or residual.shape[0] <= DIRECT_MAX_ROWS
        x = self.mixer_norm.forward(residual)
        if direct and hasattr(self.mixer, "forward_rows"):
            y = self.mixer.forward_rows(x, batch, entry)
        else:
            y = torch.zeros_like(residual)
            self.mixer.forward(x, batch, entry, y)
        h = self._join(residual, y, self.mixer_out_norm, self.feed_forward_norm)
        if self.feed_forward is not None:
            if direct and hasattr(self.feed_forward, "forward_rows"):
                y = self.feed_forward.forward_rows(h, batch)
            else:
                y = torch.zeros_like(residual)
                self.feed_forward.forward(h, batch, y)
            self._join(residual, y, self.feed_forward_out_norm, None)


register_block("pre_norm", PreNormBlock)
register_block("sandwich_norm", SandwichNormBlock)
