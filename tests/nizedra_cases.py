"""Small Nizedra configurations for the tests, and model folders made from them.

The configurations differ from one another in every size and option: widths that are no
power of two, key and value sizes that differ, head sizes that are and are not multiples of
8 or 16, one kv head for all heads and one per head, windows below and above a cache page and
none, distance tables of few and many rows with a far distance below and above the prompts'
lengths, rotation of the whole rotated part or of some of it, layers with and without a
feed-forward, a loop at the start, in the middle, over everything, of one pass, and none.
"""
import json
import os

import torch


def _ff(ff):
    return None if ff is None else {"kind": "dense", "ff": ff}


def _lightning(heads, dim, vdim, decay, ff=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay},
            "mlp": _ff(ff)}


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, size, rot=None, base=10000.0, scale=None, ff=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
         "kv_rank": kv_rank, "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
         "rot": {"dims": rot_dim if rot is None else rot, "base": base}}
    if size is not None:
        m["mask"] = {"size": size}
    return {"type": "latent_attention", "mixer": m, "mlp": _ff(ff)}


def _attention(heads, kv, dim, vdim, far, cap, rows, scale=None, ff=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "bias_max": far,
         "scale": scale if scale is not None else 4.0 * dim ** -0.5, "bias_rows": rows}
    if cap is not None:
        m["softcap"] = cap
    return {"type": "attention", "mixer": m, "mlp": _ff(ff)}


def _model(width, vocab, eps, layers, loop=None):
    d = {"architecture": "Nizedra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if loop is not None:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


CASES = {
    # a loop in the middle, three passes; a window of less than a page; head sizes in multiples
    # of 8; two kv heads for four heads; a table of 8 rows whose far distance lies inside the prompts
    "A": _model(96, 300, 1e-5, [
        _latent(3, 16, 8, 24, 40, 32, 24, ff=136),
        _lightning(2, 16, 32, [0.9, 0.995], ff=72),
        _attention(4, 2, 16, 16, 50, 10.0, 8, ff=64),
        _lightning(3, 8, 16, [0.5, 0.8, 0.97]),
    ], loop=(1, 3, 3)),
    # sizes that are multiples of 4 only; no loop; one head; a kv head per head; no window; part
    # of the rotated elements turned; no cap; a table of 6 rows
    "B": _model(104, 211, 1e-6, [
        _lightning(1, 24, 40, [0.93]),
        _attention(3, 3, 20, 12, 9, None, 6, scale=0.8),
        _latent(2, 12, 8, 20, 28, 20, None, rot=4, base=250.0, scale=0.3, ff=52),
        _attention(2, 1, 12, 20, 300, 4.0, 7, ff=88),
    ]),
    # the loop is everything, two passes, attention first; a window beyond a page; a table of 32
    # rows with a far distance beyond the prompts; values wider than 128; one kv head for all
    "C": _model(64, 97, 1e-5, [
        _attention(6, 1, 8, 24, 2000, 30.0, 32, ff=40),
        _latent(4, 8, 16, 8, 24, 144, 70, base=500.0),
        _lightning(2, 64, 16, [0.999, 0.6]),
    ], loop=(0, 3, 2)),
    # a width and sizes that are multiples of two only: no kernel's fast form applies; a loop of
    # one pass over the last layers (the input mix still stands before it)
    "O": _model(100, 131, 1e-5, [
        _lightning(2, 10, 6, [0.7, 0.9]),
        _latent(2, 10, 6, 6, 14, 10, 9, rot=2, ff=36),
        _attention(2, 1, 10, 6, 11, 5.0, 5),
    ], loop=(1, 3, 1)),
}


def write_model(folder, config, seed, dtype="bfloat16", std=0.08, patch=None):
    """A model folder of ``config`` with seeded random weights (the library's random-weights
    mode draws them; ``patch(tensors)`` may change them before they are written).  The rows of
    the distance tables are the checkpoint's to say: the written config.json does not name them."""
    import gpt_fast_amd as gfa
    from gpt_fast_amd.weights.random_init import random_checkpoint
    from gpt_fast_amd.weights.safetensors_io import write_safetensors
    arch = gfa.config.registry.architecture_of(config)
    cfg = arch.read_config(config)
    os.makedirs(folder, exist_ok=True)
    stored = json.loads(json.dumps(config))
    for layer in stored["layers"]:
        layer["mixer"].pop("bias_rows", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(stored, f)
    tensors = random_checkpoint(arch.bindings(cfg), seed, dtype, std=std, norm_std=0.2)
    for name in tensors:                      # the activation's two numbers: both signs, not small
        if name.endswith("mlp.act"):
            tensors[name] = torch.tensor([0.7, -1.3]).to(tensors[name].dtype)
    if patch is not None:
        patch(tensors)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def make_folder(tmp, name, seed=0, dtype="bfloat16", patch=None, tag=""):
    folder = os.path.join(str(tmp), f"nizedra_{name}_{dtype}_{seed}{tag}")
    if not os.path.isdir(folder):
        write_model(folder, CASES[name], seed, dtype, patch=patch)
    return folder
