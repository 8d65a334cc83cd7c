"""A plain, slow implementation of the Pigodra decoder in float64 on the CPU, one function
per mechanism, written from the design's equations.  It shares no code with the library:
it reads ``config.json`` and the safetensors file by itself and works on whole sequences
with dense masks and a token-by-token recurrence.
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
def rms_norm_around_zero(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * (1 + w)"""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + w)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def dense_feed_forward(h, w_gate, w_up, w_down):
    return (gelu_tanh(h @ w_gate.T) * (h @ w_up.T)) @ w_down.T


def rotate_pairs(x, positions, dims, base, factor):
    """x [T, heads, d]: pair (2i, 2i+1), i < dims / 2, turned by p * base^(-2i/dims) / factor."""
    if not dims:
        return x
    i = torch.arange(dims // 2, dtype=F)
    ang = positions.to(F)[:, None] * (base ** (-2.0 * i / dims) / factor)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    y = x.clone()
    y[..., 0:dims:2] = u * c - v * s
    y[..., 1:dims:2] = v * c + u * s
    return y


def visible(T, size, keep_first):
    """[T, T] bool: row i sees column j if j <= i and (i - j < size or j < keep_first)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    near = torch.ones(T, T, dtype=torch.bool) if size is None else (i - j < size)
    return (j <= i) & (near | (j < keep_first))


# --------------------------------------------------------------------------- mixers
def differential_attention(h, w, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, 2 * H, d)
    k = (h @ w[p + "k"].T).view(T, 2 * G, d)
    v = (h @ w[p + "v"].T).view(T, G, dv)
    rot = m.get("rot") or {}
    factor = (rot.get("scaling") or {}).get("factor", 1.0)
    pos = torch.arange(T)
    q = rotate_pairs(q, pos, rot.get("dims", 0), rot.get("base", 10000.0), factor).view(T, H, 2, d)
    k = rotate_pairs(k, pos, rot.get("dims", 0), rot.get("base", 10000.0), factor).view(T, G, 2, d)
    mask = m.get("mask") or {}
    see = visible(T, mask.get("size"), mask.get("keep_first") or 0)
    scale = m["scale"] if m.get("scale") is not None else d ** -0.5
    lam = (torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum())
           - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + m["diff"])
    gate = torch.sigmoid(h @ w[p + "g"].T)                       # [T, H]
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        a = []
        for mp in range(2):
            s = (q[:, hh, mp] @ k[:, g, mp].T) * scale
            a.append(torch.softmax(s.masked_fill(~see, -math.inf), -1) @ v[:, g])
        o = unit_rms(a[0] - lam * a[1], eps) * (1.0 - m["diff"])
        heads.append(o * gate[:, hh:hh + 1])
    return torch.cat(heads, -1) @ w[p + "o"].T


def log_gates(h, w, p, m):
    cap = m.get("gate_cap")

    def capped(z):
        return z if cap is None else cap * torch.tanh(z / cap)
    i = capped(h @ w[p + "i"].T + w[p + "i.b"])
    f = torch.nn.functional.logsigmoid(capped(h @ w[p + "f"].T + w[p + "f.b"]))
    return i, f


def matrix_memory_cell(q, k, v, ig, fg, state=None):
    """Token by token.  q, k [T, H, dk], v [T, H, dv], log gates [T, H]; state (S, n, m) or
    None for a sequence's start.  Returns o [T, H, dv] and the state after the last token."""
    T, H, dk = k.shape
    dv = v.shape[-1]
    if state is None:
        state = (torch.zeros(H, dk, dv, dtype=F), torch.zeros(H, dk, dtype=F), torch.zeros(H, dtype=F))
    S, n, m = state
    out = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        m_new = torch.maximum(fg[t] + m, ig[t])
        a, b = torch.exp(fg[t] + m - m_new), torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        m = m_new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = torch.einsum("hkv,hk->hv", S, q[t]) / den[:, None]
    return out, (S, n, m)


def matrix_memory_all_pairs(q, k, v, ig, fg):
    """The same cell for a whole sequence from its start, without a carried state: with
    F_t the running sum of the log forget gates, m_t = max(F_t, max_{s<=t} F_t - F_s + i_s)
    and the weight of token s at t is exp(F_t - F_s + i_s - m_t)."""
    T, H, dk = k.shape
    Fc = torch.cumsum(fg, 0)                                      # [T, H]
    logw = Fc[:, None, :] - Fc[None, :, :] + ig[None, :, :]       # [t, s, H]
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))[:, :, None]
    logw = logw.masked_fill(~causal, -math.inf)
    m = torch.maximum(Fc, logw.max(1).values)                     # the start's m = 0 decays by F_t
    wts = torch.exp(logw - m[:, None, :])                         # [t, s, H]
    scores = torch.einsum("thk,shk->tsh", q, k) * wts
    num = torch.einsum("tsh,shv->thv", scores, v)
    den = torch.maximum(scores.sum(1).abs(), torch.exp(-m)) + 1e-6
    return num / den[:, :, None]


def matrix_memory(h, w, p, m, eps, state=None):
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, dk)
    v = (h @ w[p + "v"].T).view(T, H, dv)
    ig, fg = log_gates(h, w, p, m)
    o, state = matrix_memory_cell(q, k, v, ig, fg, state)
    y = unit_rms(o, eps).reshape(T, H * dv) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return y @ w[p + "o"].T, state


# --------------------------------------------------------------------------- the model
def forward(w, cfg, tokens, layer_outputs=None):
    """float64 logits [T, vocab] of a whole sequence from its first token."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(list(tokens), dtype=torch.long)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_norm_around_zero(x, w[p + "norm1"], eps)
        if layer["type"] == "mlstm":
            x = x + matrix_memory(h, w, p + "mix.", layer["mixer"], eps)[0]
        elif layer["type"] == "attention":
            x = x + differential_attention(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            h = rms_norm_around_zero(x, w[p + "norm2"], eps)
            x = x + dense_feed_forward(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"])
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return rms_norm_around_zero(x, w["final.norm"], eps) @ w["head"].T


def greedy_generate(w, cfg, prompt, max_new_tokens):
    toks = list(prompt)
    for _ in range(max_new_tokens):
        toks.append(int(forward(w, cfg, toks)[-1].argmax()))
    return toks[len(prompt):]
