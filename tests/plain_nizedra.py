"""A plain, slow implementation of the Nizedra decoder in float64 on the CPU, one function
per mechanism, written from the design's equations.  It shares no code with the library:
it reads ``config.json`` and the safetensors file by itself and works on whole sequences
with dense masks, full keys and values per head, and a token-by-token recurrence.
"""
import json
import math
import os

import torch

from plain_llama import read_safetensors

F = torch.float64


def load_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {k: v.to(F) for k, v in read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


# --------------------------------------------------------------------------- small pieces
def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def softplus(z):
    return math.log1p(math.exp(z))


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    pos = softplus(float(p)) * z * z + 0.5 * z
    neg = (0.5 + softplus(float(q))) * (torch.expm1(z) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def dense_feed_forward(h, w_up, w_down, act):
    return xielu(h @ w_up.T, act[0], act[1]) @ w_down.T


def rotate_pairs(x, positions, dims, base):
    """x [T, ..., d]: the pair (2i, 2i+1), i < dims / 2, turned by p * base^(-2i/dims)."""
    if not dims:
        return x
    i = torch.arange(dims // 2, dtype=F)
    ang = positions.to(F)[:, None] * (base ** (-2.0 * i / dims))[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    y = x.clone()
    y[..., 0:dims:2] = u * c - v * s
    y[..., 1:dims:2] = v * c + u * s
    return y


def distance_bucket(n, rows, far):
    """Row of the distance table for distance n >= 0: the first rows // 2 rows are exact
    distances, the others logarithmic steps up to ``far``; the last row takes the rest."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


# --------------------------------------------------------------------------- mixers
def softmax_attention(h, w, p, m, eps):
    """Grouped heads with biased projections, unit-norm queries and keys, a temperature per
    head, capped scores, a bias by bucketed distance and scores mixed across heads before
    the softmax; causal."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = unit_rms((h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, d), eps)
    k = unit_rms((h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, d), eps)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, dv)
    rel = w[p + "rel"]                                           # [rows, H]
    rows = rel.shape[0]
    dist = torch.tensor([[distance_bucket(i - j, rows, m["bias_max"]) if j <= i else 0
                          for j in range(T)] for i in range(T)], dtype=torch.long)
    cap = m.get("softcap")
    s = torch.empty(H, T, T, dtype=F)
    for hh in range(H):
        z = (q[:, hh] @ k[:, hh // (H // G)].T) * m["scale"] * w[p + "temp"][hh]
        if cap:
            z = cap * torch.tanh(z / cap)
        s[hh] = z + rel[dist, hh]
    s = torch.einsum("hg,gij->hij", w[p + "talk"], s)
    see = torch.tril(torch.ones(T, T, dtype=torch.bool))
    a = torch.softmax(s.masked_fill(~see, -math.inf), -1)
    o = torch.stack([a[hh] @ v[:, hh // (H // G)] for hh in range(H)], 1)      # [T, H, dv]
    return o.reshape(T, H * dv) @ w[p + "o"].T + w[p + "o.b"]


def decayed_memory_cell(q, k, v, decay, state=None):
    """Token by token: S <- decay_h S + k v^T, o = S^T q.  q, k [T, H, dk], v [T, H, dv]."""
    T, H, dk = k.shape
    dv = v.shape[-1]
    S = torch.zeros(H, dk, dv, dtype=F) if state is None else state
    out = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return out, S


def lightning(h, w, p, m, eps, state=None):
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    silu = torch.nn.functional.silu
    q = silu(h @ w[p + "q"].T).view(T, H, dk)
    k = silu(h @ w[p + "k"].T).view(T, H, dk)
    v = silu(h @ w[p + "v"].T).view(T, H, dv)
    o, state = decayed_memory_cell(q, k, v, torch.tensor(m["decay"], dtype=F), state)
    y = rms_norm(o.reshape(T, H * dv), w[p + "norm"], eps) * torch.sigmoid(h @ w[p + "g"].T)
    return y @ w[p + "o"].T, state


def latent_attention(h, w, p, m, eps):
    """Queries through a normed latent; keys and values expanded per head from one normed
    latent per token, plus one rotated key part that all heads share; sliding window."""
    T = h.shape[0]
    H, d, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {}
    pos = torch.arange(T)
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).view(T, H, d + dr)
    q_flat, q_rot = q[..., :d], rotate_pairs(q[..., d:], pos, rot.get("dims", 0), rot.get("base", 10000.0))
    dkv = h @ w[p + "dkv"].T
    c = rms_norm(dkv[:, :R], w[p + "dkv.norm"], eps)
    k_rot = rotate_pairs(dkv[:, R:], pos, rot.get("dims", 0), rot.get("base", 10000.0))   # [T, dr]
    k_flat = (c @ w[p + "uk"].T).view(T, H, d)
    v = (c @ w[p + "uv"].T).view(T, H, dv)
    size = (m.get("mask") or {}).get("size")
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    see = (j <= i) if size is None else (j <= i) & (i - j < size)
    heads = []
    for hh in range(H):
        s = (q_flat[:, hh] @ k_flat[:, hh].T + q_rot[:, hh] @ k_rot.T) * m["scale"]
        heads.append(torch.softmax(s.masked_fill(~see, -math.inf), -1) @ v[:, hh])
    return torch.cat(heads, -1) @ w[p + "o"].T


MIXERS = {"attention": softmax_attention, "latent_attention": latent_attention}


# --------------------------------------------------------------------------- the model
def run_order(cfg):
    """Layer indices in the order they run: the layers of the loop ``times`` times in a row;
    with each, whether the loop's input product stands before it."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    order = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        order += [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


def forward(w, cfg, tokens, layer_outputs=None):
    """float64 logits [T, vocab] of a whole sequence from its first token."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    x0 = x
    for i, enters in run_order(cfg):
        layer = cfg["layers"][i]
        p = f"l{i}."
        if enters:
            x = torch.cat([x, x0], -1) @ w["loop.in"].T
        h = rms_norm(x, w[p + "norm1"], eps)
        if layer["type"] == "lightning":
            y = lightning(h, w, p + "mix.", layer["mixer"], eps)[0]
        else:
            y = MIXERS[layer["type"]](h, w, p + "mix.", layer["mixer"], eps)
        x = x + rms_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            h = rms_norm(x, w[p + "norm2"], eps)
            y = dense_feed_forward(h, w[p + "mlp.up"], w[p + "mlp.down"], w[p + "mlp.act"])
            x = x + rms_norm(y, w[p + "norm2b"], eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T


def greedy_generate(w, cfg, prompt, max_new_tokens):
    toks = list(prompt)
    for _ in range(max_new_tokens):
        toks.append(int(forward(w, cfg, toks)[-1].argmax()))
    return toks[len(prompt):]
