"""Causal attention with grouped key/value heads whose scores are mixed across heads before
the softmax, over the paged cache."""
import torch

from ..cache.store import KVNeed
from ..config.spec import MixedHeadsAttentionSpec
from ..ops import kernels as K
from ..ops import linear as L
from ..ops import scored_attention as SA
from .base import Param, Part, Runtime, add_late, check_bound, register_mixer


class MixedHeadsAttention(Part):
    """q, k, v = split(wqkv x + bqkv); every head of q and k divided by its root mean square;
    for query i, key j <= i and head g: ``s_g = (q_g . k_j) * scale * temperature[g]``, capped
    by ``softcap tanh(s / softcap)``, plus ``distance_bias[row(i - j), g]``; the heads' scores
    are mixed, ``score_h = sum_g talk[h, g] s_g``, softmaxed over j, and weigh the values of kv
    head ``h // (H / G)``; then ``wo`` and its bias.  No position encoding besides the bias.
    The projection keeps its float32 sums until q and k are normed; scores, the mix, the
    softmax and the weighted sums are float32.  The cache holds the normed keys."""

    libraries = ("scored_attention",)
    replayable = True
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream

    def __init__(self, spec: MixedHeadsAttentionSpec, runtime: Runtime):
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError(f"{spec.n_heads} heads do not divide into {spec.n_kv_heads} kv heads")
        self.spec = spec
        self.rt = runtime
        s = spec
        self.in_rows = (s.n_heads + s.n_kv_heads) * s.head_dim + s.n_kv_heads * s.value_dim
        self.wqkv = self.wo = self.bqkv = self.bo = None
        self.temperature = self.talk = self.bias = self.lookup = None
        if s.bias_rows:
            self.lookup = torch.tensor(SA.distance_rows(s.bias_rows, s.bias_max), dtype=torch.int32,
                                       device=runtime.device)

    def parameters(self):
        s = self.spec
        p = {"wqkv": Param((self.in_rows, s.dim)), "wo": Param((s.dim, s.n_heads * s.value_dim))}
        if s.biases:
            p["bqkv"] = Param((self.in_rows,), role="vector", init="around_zero")
            p["bo"] = Param((s.dim,), role="vector", init="around_zero")
        if s.head_temperature:
            p["temperature"] = Param((s.n_heads,), role="vector", init="norm")
        if s.bias_rows:
            p["distance_bias"] = Param((s.bias_rows, s.n_heads), role="vector", init="unit")
        if s.mix_heads:
            p["talk"] = Param((s.n_heads, s.n_heads), role="vector", init="head_mix")
        return p

    def bind(self, tensors):
        check_bound("MixedHeadsAttention", self.parameters(), tensors)
        # zero rows up to a multiple of eight: the products' kernels store whole groups
        self.wqkv, self.wo = L.pad_rows(tensors["wqkv"], 8), tensors["wo"]
        f32 = lambda name: tensors[name].to(torch.float32).contiguous() if name in tensors else None
        self.bqkv, self.bo = f32("bqkv"), f32("bo")
        self.temperature, self.talk, self.bias = f32("temperature"), f32("talk"), f32("distance_bias")

    def cache_need(self):
        s = self.spec
        return KVNeed(s.n_kv_heads, s.head_dim, None, s.value_dim)

    def step_flops(self, q_lens, starts) -> float:
        s = self.spec
        n = sum(q_lens)
        flops = 2.0 * n * (self.in_rows + s.n_heads * s.value_dim) * s.dim
        for q, start in zip(q_lens, starts):
            keys = q * start + q * (q + 1) / 2.0
            per_key = s.n_heads * (s.head_dim + s.value_dim)
            if s.mix_heads:
                per_key += s.n_heads * s.n_heads
            flops += 2.0 * per_key * keys
        return flops

    def _heads(self, x, batch, entry):
        s = self.spec
        proj = L.linear(x, self.wqkv, out_dtype=torch.float32)
        write = entry is not None and entry.writes
        table = batch.table(entry.group_id)
        q = SA.unit_heads_store(proj, self.bqkv, batch.tok_seq, batch.tok_pos, table,
                                entry.k_pages if write else None, entry.v_pages if write else None,
                                s.n_heads, s.n_kv_heads, s.head_dim, s.value_dim, s.qk_norm_eps,
                                self.rt.dtype)
        y = SA.attention(q, entry.k_pages, entry.v_pages, batch.tok_seq, batch.tok_pos, table,
                         s.scale, temperature=self.temperature, softcap=s.softcap or 0.0,
                         bias=self.bias, lookup=self.lookup, talk=self.talk,
                         step=(batch.q_start, batch.start_pos, batch.n_seqs, batch.max_q_len))
        return y.view(q.shape[0], s.n_heads * s.value_dim)

    def forward(self, x, batch, entry, residual):
        y = self._heads(x, batch, entry)

        def finish(rows, then_norm, takes_halves):
            # the bias joins after the product: no norm can ride on the product's kernel
            L.linear_into(y, self.wo, rows, None if self.bo is not None else then_norm, takes_halves)
            if self.bo is not None:
                K.add_bias(rows, self.bo)
            return None

        add_late(residual, finish)

    def forward_rows(self, x, batch, entry):
        """The mixer's output alone: the output projection's float32 sums and its bias."""
        out = L.linear(self._heads(x, batch, entry), self.wo, out_dtype=torch.float32)
        return out if self.bo is None else K.add_bias(out, self.bo)


register_mixer("mixed_heads_attention", MixedHeadsAttention)
