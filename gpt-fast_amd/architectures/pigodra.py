"""The Pigodra decoder as data: its plan and its checkpoint layout.

Plan: the layers ``config.json`` lists, in its order, each a pre-norm block of a mixer -
a matrix memory per head ("mlstm") or differential attention over a sliding window that
keeps the first keys ("attention") - and, where the layer has one, a gated feed-forward with
the tanh form of gelu.  Norm weights are stored around zero (``1 + w``); the embedded rows
are multiplied by a constant.

Checkpoint layout: tensors are named ``l<i>.norm1``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``,
``embed``, ``final.norm``, ``head``; linear weights [out, in].  The projections that read the
same input are joined into one matrix when they are loaded (q, k, v, g, i, f of a matrix
memory; q, k, v, g of an attention; gate and up of a feed-forward).
"""
import torch

from ..config.pigodra import DifferentialMixer, MatrixMemoryMixer, PigodraConfig
from ..config.registry import Architecture, register_architecture
from ..config.spec import (DifferentialAttentionSpec, GatedFeedForwardSpec, LayerSpec,
                           MatrixMemorySpec, ModelPlan, NormSpec, PositionSpec, Run)
from ..weights.bindings import Binding, CheckpointLayout, Source


def _mixer_spec(c: PigodraConfig, m):
    if isinstance(m, MatrixMemoryMixer):
        return MatrixMemorySpec(dim=c.width, n_heads=m.heads, key_dim=m.dim, value_dim=m.vdim,
                                eps=c.norm_eps, gate_cap=m.gate_cap)
    if m.rot_dims:
        scaling = None
        if m.rot_factor is not None:
            scaling = (("rope_type", "linear"), ("factor", m.rot_factor))
        position = PositionSpec(kind="rope", rotary_dim=m.rot_dims, base=m.rot_base,
                                layout="interleaved", scaling=scaling)
    else:
        position = PositionSpec(kind="none")
    return DifferentialAttentionSpec(
        dim=c.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
        position=position, lam_init=m.diff, eps=c.norm_eps, scale=m.scale, window=m.window,
        keep_first=m.keep_first, head_gate=True)


def pigodra_plan(c: PigodraConfig) -> ModelPlan:
    def norm():
        return NormSpec(c.width, c.norm_eps, weight_offset=1.0)

    layers = []
    for i, l in enumerate(c.layers):
        layers.append(LayerSpec(
            name=f"l{i}", arrangement="pre_norm", mixer=_mixer_spec(c, l.mixer), mixer_norm=norm(),
            feed_forward=None if l.mlp is None else GatedFeedForwardSpec(c.width, l.mlp.ff, "gelu_tanh"),
            feed_forward_norm=None if l.mlp is None else norm(),
            mixer_name="mix", mixer_norm_name="norm1", feed_forward_name="mlp",
            feed_forward_norm_name="norm2"))
    plan = ModelPlan(
        dim=c.width, vocab_size=c.vocab, layers=layers, order=[Run(i) for i in range(len(layers))],
        final_norm=norm(), tie_embeddings=False, max_positions=c.max_positions,
        embedding_name="embed", final_norm_name="final.norm", head_name="head",
        embedding_scale=None if c.embedding_scale == 1.0 else c.embedding_scale)
    plan.validate()
    return plan


def pigodra_bindings(c: PigodraConfig) -> CheckpointLayout:
    D, V = c.width, c.vocab
    b = [Binding("embed", (Source("embed", (V, D)),))]
    for i, l in enumerate(c.layers):
        p = f"l{i}."
        m = l.mixer
        b.append(Binding(p + "norm1.weight", (Source(p + "norm1", (D,), "around_zero"),), role="vector"))
        if isinstance(m, MatrixMemoryMixer):
            H, dk, dv = m.heads, m.dim, m.vdim
            b += [
                Binding(p + "mix.w_in",
                        (Source(p + "mix.q", (H * dk, D)), Source(p + "mix.k", (H * dk, D)),
                         Source(p + "mix.v", (H * dv, D)), Source(p + "mix.g", (H * dv, D)),
                         Source(p + "mix.i", (H, D)), Source(p + "mix.f", (H, D))),
                        combine=torch.cat),
                Binding(p + "mix.gate_bias",
                        (Source(p + "mix.i.b", (H,), "unit"), Source(p + "mix.f.b", (H,), "unit")),
                        role="vector", combine=torch.cat),
                Binding(p + "mix.norm", (Source(p + "mix.norm", (H * dv,), "norm"),), role="vector"),
                Binding(p + "mix.wo", (Source(p + "mix.o", (D, H * dv)),)),
            ]
        else:
            assert isinstance(m, DifferentialMixer)
            H, G, d, dv = m.heads, m.kv_heads, m.dim, m.vdim
            b += [
                Binding(p + "mix.w_in",
                        (Source(p + "mix.q", (H * 2 * d, D)), Source(p + "mix.k", (G * 2 * d, D)),
                         Source(p + "mix.v", (G * dv, D)), Source(p + "mix.g", (H, D))),
                        combine=torch.cat),
                Binding(p + "mix.wo", (Source(p + "mix.o", (D, H * dv)),)),
            ]
            for name in ("lq1", "lk1", "lq2", "lk2"):
                b.append(Binding(p + "mix." + name, (Source(p + "mix." + name, (d,), "around_zero"),),
                                 role="vector"))
        if l.mlp is not None:
            F = l.mlp.ff
            b += [
                Binding(p + "norm2.weight", (Source(p + "norm2", (D,), "around_zero"),), role="vector"),
                Binding(p + "mlp.w13", (Source(p + "mlp.gate", (F, D)), Source(p + "mlp.up", (F, D))),
                        combine=torch.cat),
                Binding(p + "mlp.w2", (Source(p + "mlp.down", (D, F)),)),
            ]
    b.append(Binding("final.norm.weight", (Source("final.norm", (D,), "around_zero"),), role="vector"))
    b.append(Binding("head", (Source("head", (V, D)),)))
    return CheckpointLayout(tuple(b))


def pigodra_sizes(c: PigodraConfig) -> dict:
    """The sizes that the layers share, flat; per-layer sizes as short strings."""
    kinds = "".join("m" if l.type == "mlstm" else "a" for l in c.layers)
    out = {"n_layer": len(c.layers), "dim": c.width, "vocab_size": c.vocab, "norm_eps": c.norm_eps,
           "layer_kinds": kinds}
    for l in c.layers:
        m = l.mixer
        if isinstance(m, MatrixMemoryMixer) and "mlstm" not in out:
            out["mlstm"] = f"{m.heads} heads, keys {m.dim}, values {m.vdim}"
        if isinstance(m, DifferentialMixer) and "attention" not in out:
            out["attention"] = (f"{m.heads} heads of 2 x {m.dim}, {m.kv_heads} kv heads, values "
                                f"{m.vdim}, window {m.window}, first {m.keep_first}")
        if l.mlp is not None and "intermediate_size" not in out:
            out["intermediate_size"] = l.mlp.ff
    return out


PIGODRA = register_architecture(Architecture(
    names=("Pigodra", "pigodra"),
    read_config=PigodraConfig.from_dict,
    plan=pigodra_plan,
    bindings=pigodra_bindings,
    config_dict=PigodraConfig.to_dict,
    presets=PigodraConfig.from_name,
    describe=pigodra_sizes,
    layer_count_key="layers",
))
