"""Small Pigodra configurations for the tests, and model folders made from them.

The configurations differ from one another in every size and option: widths that are no
power of two, key and value sizes that differ, head sizes that are and are not multiples of
8, 16 or 32, one kv head for all heads and one per head, windows below and above a cache
page, no window, kept first keys from none to more than a page, rotation of a whole map or
of part of it, with and without a scaling factor, gates with and without a cap, layers with
and without a feed-forward, attention first or last.
"""
import json
import os
import zlib

import torch


def _att(heads, kv, dim, vdim, size, first, rot, base=10000.0, factor=None, scale=None, diff=0.25,
         ff=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "diff": diff,
         "mask": {"size": size, "keep_first": first},
         "rot": {"dims": rot, "base": base}}
    if factor is not None:
        m["rot"]["scaling"] = {"factor": factor}
    if scale is not None:
        m["scale"] = scale
    return {"type": "attention", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _mem(heads, dim, vdim, cap, ff=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim}
    if cap is not None:
        m["gate_cap"] = cap
    return {"type": "mlstm", "mixer": m, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _model(width, vocab, eps, scale, layers):
    return {"architecture": "Pigodra", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": scale}, "layers": layers}


CASES = {
    # attention first; head sizes in multiples of 16; three heads to a kv head; a window of
    # less than a page; rotation of the whole map
    "A": _model(96, 300, 1e-5, 1.7, [
        _att(6, 2, 16, 32, 24, 3, 16, ff=136),
        _mem(3, 16, 32, 8.0, ff=72),
        _att(2, 2, 32, 16, 100, 1, 8, base=5000.0, factor=4.0, scale=0.21, diff=0.45),
        _mem(2, 48, 24, 15.0),
    ]),
    # sizes that are multiples of 4 only; one head; one kv head for all; no kept keys; a
    # window of 7; more kept keys than a page holds; no cap on the gates
    "B": _model(104, 211, 1e-6, 1.0, [
        _mem(1, 24, 40, None),
        _att(4, 1, 24, 24, 7, 0, 8, base=250.0, factor=1.5, scale=0.3, diff=0.1),
        _mem(5, 20, 12, 3.0, ff=52),
        _att(3, 3, 20, 40, 90, 70, 20, ff=88, diff=0.6),
    ]),
    # memory layers only, keys wider than values and the other way round
    "M": _model(64, 97, 1e-5, 0.25, [_mem(2, 64, 16, 10.0), _mem(4, 8, 48, 6.0, ff=40)]),
    # a width and head sizes that are multiples of two only: no kernel's fast form applies
    "O": _model(100, 131, 1e-5, 0.8, [
        _mem(2, 10, 6, 5.0),
        _att(2, 1, 10, 6, 9, 2, 4, ff=36, factor=3.0),
    ]),
    # attention layers only, no window (every earlier key) and no rotation
    "T": _model(72, 150, 1e-6, 2.0, [
        _att(3, 3, 16, 24, None, 0, 0, ff=64),
        _att(4, 2, 8, 16, 33, 2, 4, factor=2.0),
    ]),
}


def write_model(folder, config, seed, dtype="bfloat16", std=0.08, patch=None):
    """A model folder of ``config`` with seeded random weights (the library's random-weights
    mode draws them; ``patch(tensors)`` may change them before they are written)."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.weights.random_init import random_checkpoint
    from gpt_fast_amd.weights.safetensors_io import write_safetensors
    arch = gfa.config.registry.architecture_of(config)
    cfg = arch.read_config(config)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    tensors = random_checkpoint(arch.bindings(cfg), seed, dtype, std=std, norm_std=0.2)
    # the four vectors behind lambda are drawn small: make lambda differ from its constant
    for name in tensors:
        if name.rsplit(".", 1)[-1] in ("lq1", "lk1", "lq2", "lk2"):
            g = torch.Generator().manual_seed(seed * 7919 + zlib.crc32(name.encode()))
            tensors[name] = (torch.randn(tensors[name].shape, generator=g) * 0.3).to(tensors[name].dtype)
    if patch is not None:
        patch(tensors)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def make_folder(tmp, name, seed=0, dtype="bfloat16", patch=None, tag=""):
    folder = os.path.join(str(tmp), f"pigodra_{name}_{dtype}_{seed}{tag}")
    if not os.path.isdir(folder):
        write_model(folder, CASES[name], seed, dtype, patch=patch)
    return folder
