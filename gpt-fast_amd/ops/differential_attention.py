"""Python faces of the differential-attention kernels of csrc/differential_attention.hip:
shape checks on the host, then the launch."""
import ctypes

import torch

from .kernels import PAGE
from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i, _f = ctypes.c_int, ctypes.c_float
MAPS = 2


def _is_bf16(t):
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise KernelError(f"activation dtype {t.dtype}: float32 or bfloat16 only")


def _check_pages(k_pages, v_pages, G, dim, vdim, dtype):
    for name, p, tail in (("k_pages", k_pages, (G, PAGE, MAPS * dim)),
                          ("v_pages", v_pages, (G, vdim, PAGE))):
        if p is None:
            continue
        if p.dim() != 4 or tuple(p.shape[1:]) != tail:
            raise KernelError(f"{name} must be [n_pages, {tail[0]}, {tail[1]}, {tail[2]}], "
                              f"is {tuple(p.shape)}")
        if p.dtype != dtype or not p.is_contiguous():
            raise KernelError(f"{name} must be contiguous {dtype}")


def _check_maps(n, tok_seq, tok_pos, table):
    for name, t in (("tok_seq", tok_seq), ("tok_pos", tok_pos), ("table", table)):
        if t.dtype != torch.int32:
            raise KernelError(f"{name} must be int32")
    if tok_seq.numel() < n or tok_pos.numel() < n:
        raise KernelError("token maps are shorter than the batch")


def rope_store(proj, q_off, k_off, v_off, freqs, tok_seq, tok_pos, table, k_pages, v_pages,
               n_heads, n_kv_heads, dim, vdim, rotary_dim):
    """Rotate the first ``rotary_dim`` elements (pairs 2i, 2i+1) of every map of q and k of
    proj [N, width] by position; q to a new [N, H, 2, dim]; k and v into the pages (skipped
    if they are None)."""
    require_device(proj, freqs, tok_seq, tok_pos, table, k_pages, v_pages)
    require_contiguous(proj=proj, freqs=freqs, tok_seq=tok_seq, tok_pos=tok_pos, table=table)
    n, width = proj.shape
    if (q_off + n_heads * MAPS * dim > width or k_off + n_kv_heads * MAPS * dim > width
            or v_off + n_kv_heads * vdim > width):
        raise KernelError("rope_store: q, k, v do not fit the rows")
    if rotary_dim % 2 or not 0 <= rotary_dim <= dim:
        raise KernelError(f"rope_store: rotary_dim {rotary_dim} must be even and at most {dim}")
    if rotary_dim and (freqs is None or freqs.dtype != torch.float32 or freqs.numel() != rotary_dim // 2):
        raise KernelError(f"rope_store: float32 frequencies for rotary_dim {rotary_dim}")
    _check_maps(n, tok_seq, tok_pos, table)
    if (k_pages is None) != (v_pages is None):
        raise KernelError("rope_store: give both k_pages and v_pages, or neither")
    _check_pages(k_pages, v_pages, n_kv_heads, dim, vdim, proj.dtype)
    q_out = torch.empty((n, n_heads, MAPS, dim), dtype=proj.dtype, device=proj.device)
    check(library("differential_attention").gfa_da_rope_store(
        ptr(proj), _i(width), _i(q_off), _i(k_off), _i(v_off), ptr(q_out), ptr(k_pages),
        ptr(v_pages), ptr(freqs), ptr(tok_seq), ptr(tok_pos), ptr(table), _i(table.shape[1]),
        _i(n), _i(n_heads), _i(n_kv_heads), _i(dim), _i(vdim), _i(rotary_dim), _i(_is_bf16(proj)),
        stream_handle()), "da_rope_store")
    return q_out


def attention_generic(q, k_pages, v_pages, gate, tok_seq, tok_pos, table, scale, window,
                      keep_first, lam, eps, out_scale):
    """q [N, H, 2, dim]; gate None or a view [N, H] (unit stride along H) of the heads' gate
    pre-activations.  Returns [N, H * vdim]."""
    require_device(q, k_pages, v_pages, gate, tok_seq, tok_pos, table)
    require_contiguous(q=q, tok_seq=tok_seq, tok_pos=tok_pos, table=table)
    n, H, maps, dim = q.shape
    G, vdim = k_pages.shape[1], v_pages.shape[2]
    if maps != MAPS or H % G:
        raise KernelError(f"differential attention: q {tuple(q.shape)} against {G} kv heads")
    if vdim > 512:
        raise KernelError(f"differential attention: value_dim {vdim} > 512 is not supported")
    _check_pages(k_pages, v_pages, G, dim, vdim, q.dtype)
    _check_maps(n, tok_seq, tok_pos, table)
    gate_stride = 0
    if gate is not None:
        if gate.shape != (n, H) or gate.dtype != q.dtype or (H > 1 and gate.stride(1) != 1):
            raise KernelError("differential attention: gate must be [N, H] of q's type")
        gate_stride = gate.stride(0)
    out = torch.empty((n, H * vdim), dtype=q.dtype, device=q.device)
    check(library("differential_attention").gfa_da_attention_generic(
        ptr(q), ptr(k_pages), ptr(v_pages), ptr(gate), _i(gate_stride), ptr(tok_seq), ptr(tok_pos),
        ptr(table), _i(table.shape[1]), ptr(out), _i(n), _i(H), _i(G), _i(dim), _i(vdim),
        _f(scale), _i(window or 0), _i(keep_first), _f(lam), _f(eps), _f(out_scale),
        _i(_is_bf16(q)), stream_handle()), "da_attention_generic")
    return out


def attention(q, k_pages, v_pages, gate, batch, table, scale, window, keep_first, lam, eps,
              out_scale):
    """Which kernel runs a step's differential attention: the plain one, for every shape."""
    return attention_generic(q, k_pages, v_pages, gate, batch.tok_seq, batch.tok_pos, table,
                             scale, window, keep_first, lam, eps, out_scale)
