"""The Nizedra decoder as data: its plan and its checkpoint layout.

Plan: the layers ``config.json`` lists, each a block with a norm before and a norm after
each sublayer (``x + norm1b(mixer(norm1(x)))``, ``x + norm2b(ff(norm2(x)))``), the mixer one
of lightning attention (a decayed memory per head), latent attention over a sliding window,
or causal attention whose scores are mixed across heads; the feed-forward dense with the
xIELU activation.  The layers ``loop.start .. loop.stop - 1`` run ``loop.times`` times in a
row with the same weights and a cache entry per run; before the first of them, every time,
the stream becomes ``W [x; x0]`` with the embedded rows x0.

Checkpoint layout: ``embed``, ``loop.in``, ``l<i>.norm1`` ..., ``l<i>.mix.<name>``,
``l<i>.mlp.<name>``, ``final.norm``, ``head``; linear weights [out, in]; biases under the
weight's name with ``.b``.  Projections that read the same input are joined into one matrix
when they are loaded.
"""
import re

import torch

from ..config.nizedra import LatentMixer, LightningMixer, MixedHeadsMixer, NizedraConfig
from ..config.registry import Architecture, register_architecture
from ..config.spec import (DecayedMemorySpec, DenseFeedForwardSpec, InputMixSpec,
                           LatentAttentionSpec, LayerSpec, MixedHeadsAttentionSpec, ModelPlan,
                           NormSpec, PositionSpec, Run)
from ..weights.bindings import Binding, CheckpointLayout, Source

LOOP_INPUT = "loop.in"


def _mixer_spec(c: NizedraConfig, m):
    if isinstance(m, LightningMixer):
        return DecayedMemorySpec(dim=c.width, n_heads=m.heads, key_dim=m.dim, value_dim=m.vdim,
                                 decay=tuple(m.decay), eps=c.norm_eps)
    if isinstance(m, LatentMixer):
        position = (PositionSpec(kind="rope", rotary_dim=m.rot_dims, base=m.rot_base,
                                 layout="interleaved") if m.rot_dims else PositionSpec(kind="none"))
        return LatentAttentionSpec(dim=c.width, n_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim,
                                   value_dim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank,
                                   scale=m.scale, eps=c.norm_eps, position=position, window=m.window)
    assert isinstance(m, MixedHeadsMixer)
    return MixedHeadsAttentionSpec(dim=c.width, n_heads=m.heads, n_kv_heads=m.kv_heads,
                                   head_dim=m.dim, value_dim=m.vdim, scale=m.scale,
                                   softcap=m.softcap, bias_rows=m.bias_rows, bias_max=m.bias_max,
                                   qk_norm_eps=c.norm_eps)


def nizedra_order(c: NizedraConfig):
    """The runs: layers before the loop, the loop's layers ``times`` times (the input mix
    before the first of them each time), the layers behind it."""
    n = len(c.layers)
    if c.loop is None:
        return [Run(i) for i in range(n)]
    enter = InputMixSpec(c.width, LOOP_INPUT)
    order = [Run(i) for i in range(c.loop.start)]
    for _ in range(c.loop.times):
        order += [Run(i, enter=enter if i == c.loop.start else None)
                  for i in range(c.loop.start, c.loop.stop)]
    return order + [Run(i) for i in range(c.loop.stop, n)]


def nizedra_plan(c: NizedraConfig) -> ModelPlan:
    def norm():
        return NormSpec(c.width, c.norm_eps)

    layers = []
    for i, l in enumerate(c.layers):
        has_ff = l.mlp is not None
        layers.append(LayerSpec(
            name=f"l{i}", arrangement="sandwich_norm", mixer=_mixer_spec(c, l.mixer),
            mixer_norm=norm(), mixer_out_norm=norm(),
            feed_forward=DenseFeedForwardSpec(c.width, l.mlp.ff, "xielu") if has_ff else None,
            feed_forward_norm=norm() if has_ff else None,
            feed_forward_out_norm=norm() if has_ff else None,
            mixer_name="mix", mixer_norm_name="norm1", mixer_out_norm_name="norm1b",
            feed_forward_name="mlp", feed_forward_norm_name="norm2",
            feed_forward_out_norm_name="norm2b"))
    plan = ModelPlan(
        dim=c.width, vocab_size=c.vocab, layers=layers, order=nizedra_order(c),
        final_norm=norm(), tie_embeddings=False, max_positions=c.max_positions,
        embedding_name="embed", final_norm_name="final.norm", head_name="head")
    plan.validate()
    return plan


def nizedra_bindings(c: NizedraConfig) -> CheckpointLayout:
    D, V = c.width, c.vocab
    b = [Binding("embed", (Source("embed", (V, D)),))]
    # a loop without a pass (no layer in it, or no time round) never uses its matrix: a
    # checkpoint may still hold it
    looped = c.loop is not None and c.loop.times > 0 and c.loop.stop > c.loop.start
    if looped:
        b.append(Binding(LOOP_INPUT, (Source(LOOP_INPUT, (D, 2 * D)),)))

    def vector(target, name, shape, init="norm"):
        return Binding(target, (Source(name, shape, init),), role="vector")

    for i, l in enumerate(c.layers):
        p = f"l{i}."
        m = l.mixer
        b += [vector(p + "norm1.weight", p + "norm1", (D,)),
              vector(p + "norm1b.weight", p + "norm1b", (D,))]
        if isinstance(m, LightningMixer):
            H, dk, dv = m.heads, m.dim, m.vdim
            b += [
                Binding(p + "mix.w_in",
                        (Source(p + "mix.q", (H * dk, D)), Source(p + "mix.k", (H * dk, D)),
                         Source(p + "mix.v", (H * dv, D)), Source(p + "mix.g", (H * dv, D))),
                        combine=torch.cat),
                vector(p + "mix.norm", p + "mix.norm", (H * dv,)),
                Binding(p + "mix.wo", (Source(p + "mix.o", (D, H * dv)),)),
            ]
        elif isinstance(m, LatentMixer):
            H, d, dr, dv = m.heads, m.dim, m.rot_dim, m.vdim
            b += [
                Binding(p + "mix.w_down",
                        (Source(p + "mix.dq", (m.q_rank, D)), Source(p + "mix.dkv", (m.kv_rank + dr, D))),
                        combine=torch.cat),
                vector(p + "mix.q_norm", p + "mix.dq.norm", (m.q_rank,)),
                vector(p + "mix.kv_norm", p + "mix.dkv.norm", (m.kv_rank,)),
                Binding(p + "mix.w_uq", (Source(p + "mix.uq", (H * (d + dr), m.q_rank)),)),
                Binding(p + "mix.w_uk", (Source(p + "mix.uk", (H * d, m.kv_rank)),)),
                Binding(p + "mix.w_uv", (Source(p + "mix.uv", (H * dv, m.kv_rank)),)),
                Binding(p + "mix.wo", (Source(p + "mix.o", (D, H * dv)),)),
            ]
        else:
            assert isinstance(m, MixedHeadsMixer)
            H, G, d, dv = m.heads, m.kv_heads, m.dim, m.vdim
            b += [
                Binding(p + "mix.wqkv",
                        (Source(p + "mix.q", (H * d, D)), Source(p + "mix.k", (G * d, D)),
                         Source(p + "mix.v", (G * dv, D))), combine=torch.cat),
                Binding(p + "mix.bqkv",
                        (Source(p + "mix.q.b", (H * d,), "around_zero"),
                         Source(p + "mix.k.b", (G * d,), "around_zero"),
                         Source(p + "mix.v.b", (G * dv,), "around_zero")),
                        role="vector", combine=torch.cat),
                vector(p + "mix.distance_bias", p + "mix.rel", (m.bias_rows, H), "unit"),
                vector(p + "mix.talk", p + "mix.talk", (H, H), "head_mix"),
                vector(p + "mix.temperature", p + "mix.temp", (H,), "norm"),
                Binding(p + "mix.wo", (Source(p + "mix.o", (D, H * dv)),)),
                vector(p + "mix.bo", p + "mix.o.b", (D,), "around_zero"),
            ]
        if l.mlp is not None:
            F = l.mlp.ff
            b += [
                vector(p + "norm2.weight", p + "norm2", (D,)),
                vector(p + "norm2b.weight", p + "norm2b", (D,)),
                Binding(p + "mlp.w_up", (Source(p + "mlp.up", (F, D)),)),
                Binding(p + "mlp.w_down", (Source(p + "mlp.down", (D, F)),)),
                vector(p + "mlp.act", p + "mlp.act", (2,), "unit"),
            ]
    b.append(vector("final.norm.weight", "final.norm", (D,)))
    b.append(Binding("head", (Source("head", (V, D)),)))
    unused = (r"^loop\.in$",) if c.loop is not None and not looped else ()
    return CheckpointLayout(tuple(b), ignored=unused)


_REL = re.compile(r"^l(\d+)\.mix\.rel$")


def nizedra_sizes_from_tensors(c: NizedraConfig, shapes: dict) -> NizedraConfig:
    """Sizes that only the checkpoint's tensors give: the rows of each distance table."""
    rows = {}
    for name, shape in shapes.items():
        m = _REL.match(name)
        if m and len(shape) == 2 and int(m.group(1)) < len(c.layers):
            rows[int(m.group(1))] = shape[0]
    return c.with_table_rows(rows) if rows else c


def nizedra_sizes(c: NizedraConfig) -> dict:
    """The sizes that the layers share, flat; per-layer sizes as short strings."""
    letter = {"lightning": "l", "latent_attention": "c", "attention": "a"}
    out = {"n_layer": len(c.layers), "dim": c.width, "vocab_size": c.vocab, "norm_eps": c.norm_eps,
           "layer_kinds": "".join(letter[l.type] for l in c.layers)}
    if c.loop is not None:
        out["loop"] = f"layers {c.loop.start}..{c.loop.stop - 1} x {c.loop.times}"
    for l in c.layers:
        m = l.mixer
        if isinstance(m, LightningMixer) and "lightning" not in out:
            out["lightning"] = f"{m.heads} heads, keys {m.dim}, values {m.vdim}"
        if isinstance(m, LatentMixer) and "latent_attention" not in out:
            out["latent_attention"] = (f"{m.heads} heads of {m.dim}+{m.rot_dim}, values {m.vdim}, "
                                       f"latents {m.q_rank}/{m.kv_rank}, window {m.window}")
        if isinstance(m, MixedHeadsMixer) and "attention" not in out:
            out["attention"] = (f"{m.heads} heads of {m.dim}, {m.kv_heads} kv heads, values {m.vdim}, "
                                f"{m.bias_rows} distance rows")
        if l.mlp is not None and "intermediate_size" not in out:
            out["intermediate_size"] = l.mlp.ff
    return out


NIZEDRA = register_architecture(Architecture(
    names=("Nizedra", "nizedra"),
    read_config=NizedraConfig.from_dict,
    plan=nizedra_plan,
    bindings=nizedra_bindings,
    config_dict=NizedraConfig.to_dict,
    presets=NizedraConfig.from_name,
    describe=nizedra_sizes,
    layer_count_key="layers",
    sizes_from_tensors=nizedra_sizes_from_tensors,
))
