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


def rope_store(proj, q_off, k_off, v_off, g_off, freqs, tok_seq, tok_pos, table, k_pages, v_pages,
               n_heads, n_kv_heads, dim, vdim, rotary_dim, out_dtype, with_gate=True):
    """Rotate the first ``rotary_dim`` elements (pairs 2i, 2i+1) of every map of q and k of
    proj (float32 [N, width], the projection's unrounded sums) by position; q to a new
    [N, H, 2, dim] of ``out_dtype``; k and v into the pages of that type (skipped if they are
    None); the heads' gate numbers at ``g_off`` to a new float32 [N, H] (None without a gate).
    Returns (q, gate)."""
    require_device(proj, freqs, tok_seq, tok_pos, table, k_pages, v_pages)
    require_contiguous(proj=proj, freqs=freqs, tok_seq=tok_seq, tok_pos=tok_pos, table=table)
    if proj.dtype != torch.float32 or proj.dim() != 2:
        raise KernelError("rope_store: the projection's rows must be float32 [N, width]")
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise KernelError(f"rope_store: output type {out_dtype}")
    n, width = proj.shape
    if (q_off + n_heads * MAPS * dim > width or k_off + n_kv_heads * MAPS * dim > width
            or v_off + n_kv_heads * vdim > width or (with_gate and g_off + n_heads > width)):
        raise KernelError("rope_store: q, k, v and the gates do not fit the rows")
    if rotary_dim % 2 or not 0 <= rotary_dim <= dim:
        raise KernelError(f"rope_store: rotary_dim {rotary_dim} must be even and at most {dim}")
    if rotary_dim and (freqs is None or freqs.dtype != torch.float32 or freqs.numel() != rotary_dim // 2):
        raise KernelError(f"rope_store: float32 frequencies for rotary_dim {rotary_dim}")
    _check_maps(n, tok_seq, tok_pos, table)
    if (k_pages is None) != (v_pages is None):
        raise KernelError("rope_store: give both k_pages and v_pages, or neither")
    _check_pages(k_pages, v_pages, n_kv_heads, dim, vdim, out_dtype)
    q_out = torch.empty((n, n_heads, MAPS, dim), dtype=out_dtype, device=proj.device)
    gate = torch.empty((n, n_heads), dtype=torch.float32, device=proj.device) if with_gate else None
    check(library("differential_attention").gfa_da_rope_store(
        ptr(proj), _i(width), _i(q_off), _i(k_off), _i(v_off), _i(g_off), ptr(q_out), ptr(k_pages),
        ptr(v_pages), ptr(gate), ptr(freqs), ptr(tok_seq), ptr(tok_pos), ptr(table),
        _i(table.shape[1]), _i(n), _i(n_heads), _i(n_kv_heads), _i(dim), _i(vdim), _i(rotary_dim),
        _i(int(out_dtype == torch.bfloat16)), stream_handle()), "da_rope_store")
    return q_out, gate


def attention_generic(q, k_pages, v_pages, gate, tok_seq, tok_pos, table, scale, window,
                      keep_first, lam, eps, out_scale):
    """q [N, H, 2, dim]; gate None or float32 [N, H] (unit stride along H), the heads' gate
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
        if gate.shape != (n, H) or gate.dtype != torch.float32 or (H > 1 and gate.stride(1) != 1):
            raise KernelError("differential attention: gate must be float32 [N, H]")
        gate_stride = gate.stride(0)
    out = torch.empty((n, H * vdim), dtype=q.dtype, device=q.device)
    check(library("differential_attention").gfa_da_attention_generic(
        ptr(q), ptr(k_pages), ptr(v_pages), ptr(gate), _i(gate_stride), ptr(tok_seq), ptr(tok_pos),
        ptr(table), _i(table.shape[1]), ptr(out), _i(n), _i(H), _i(G), _i(dim), _i(vdim),
        _f(scale), _i(window or 0), _i(keep_first), _f(lam), _f(eps), _f(out_scale),
        _i(_is_bf16(q)), stream_handle()), "da_attention_generic")
    return out


MFMA_MAX_DIM, MFMA_MAX_VDIM = 128, 256
SPLIT_MAX_WAVES = 8
LDS_BYTES = 64 * 1024


def mfma_takes(q, k_pages, v_pages) -> bool:
    """The matrix-core kernel's shapes: bfloat16, head sizes in eights up to 128, value sizes
    in sixteens up to 256."""
    dim, vdim = q.shape[3], v_pages.shape[2]
    return (q.dtype == torch.bfloat16 and dim % 8 == 0 and dim <= MFMA_MAX_DIM
            and vdim % 16 == 0 and vdim <= MFMA_MAX_VDIM)


def split_waves_for(heads_per_group: int, vdim: int) -> int:
    """Waves that share one sequence's keys in a step of one token per sequence: as many as
    their partial results fit the workgroup's shared memory, at most eight; 0: not available."""
    if heads_per_group > 16:
        return 0
    per_wave = (64 + MAPS * vdim * heads_per_group) * 4
    return min(SPLIT_MAX_WAVES, LDS_BYTES // per_wave)


def attention_mfma(q, k_pages, v_pages, gate, q_start, start_pos, table, n_seqs, max_q_len,
                   scale, window, keep_first, lam, eps, out_scale, single_tokens=False):
    """As :func:`attention_generic`, on the matrix cores; sequences are given by ``q_start``
    [n_seqs + 1] (first row of each) and ``start_pos`` [n_seqs] (tokens cached before the
    step).  ``single_tokens``: every sequence brings one token, and the waves of a workgroup
    share its keys."""
    require_device(q, k_pages, v_pages, gate, q_start, start_pos, table)
    require_contiguous(q=q, q_start=q_start, start_pos=start_pos, table=table)
    n, H, maps, dim = q.shape
    G, vdim = k_pages.shape[1], v_pages.shape[2]
    if maps != MAPS or H % G or not mfma_takes(q, k_pages, v_pages):
        raise KernelError(f"differential attention on the matrix cores: q {tuple(q.shape)}, "
                          f"values of {vdim}, {G} kv heads")
    _check_pages(k_pages, v_pages, G, dim, vdim, q.dtype)
    for name, t in (("q_start", q_start), ("start_pos", start_pos), ("table", table)):
        if t.dtype != torch.int32:
            raise KernelError(f"{name} must be int32")
    if q_start.numel() < n_seqs + 1 or start_pos.numel() < n_seqs or table.shape[0] < n_seqs:
        raise KernelError("differential attention: the step's description is shorter than the batch")
    gate_stride = 0
    if gate is not None:
        if gate.shape != (n, H) or gate.dtype != torch.float32 or (H > 1 and gate.stride(1) != 1):
            raise KernelError("differential attention: gate must be float32 [N, H]")
        gate_stride = gate.stride(0)
    waves = 0
    if single_tokens:
        waves = split_waves_for(H // G, vdim)
        if n != n_seqs or max_q_len != 1 or waves < 1:
            raise KernelError("differential attention: single_tokens needs one row per sequence")
    out = torch.empty((n, H * vdim), dtype=q.dtype, device=q.device)
    check(library("differential_attention").gfa_da_attention_mfma(
        ptr(q), ptr(k_pages), ptr(v_pages), ptr(gate), _i(gate_stride), ptr(q_start), ptr(start_pos),
        ptr(table), _i(table.shape[1]), ptr(out), _i(n_seqs), _i(max_q_len * (H // G)), _i(H), _i(G),
        _i(dim), _i(vdim), _f(scale), _i(window or 0), _i(keep_first), _f(lam), _f(eps),
        _f(out_scale), _i(waves), stream_handle()), "da_attention_mfma")
    return out


def attention(q, k_pages, v_pages, gate, batch, table, scale, window, keep_first, lam, eps,
              out_scale):
    """Which kernel runs a step's differential attention.  float32 engine, and shapes the
    matrix-core kernel refuses: the plain kernel.  bfloat16: the matrix-core kernel, with the
    waves of a workgroup sharing a sequence's keys when every sequence brings one token."""
    if mfma_takes(q, k_pages, v_pages):
        H, G, vdim = q.shape[1], k_pages.shape[1], v_pages.shape[2]
        single = bool(batch.is_decode) and split_waves_for(H // G, vdim) >= 1
        return attention_mfma(q, k_pages, v_pages, gate, batch.q_start, batch.start_pos, table,
                              batch.n_seqs, batch.max_q_len, scale, window, keep_first, lam, eps,
                              out_scale, single_tokens=single)
    return attention_generic(q, k_pages, v_pages, gate, batch.tok_seq, batch.tok_pos, table,
                             scale, window, keep_first, lam, eps, out_scale)
