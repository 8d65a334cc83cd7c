"""Python faces of the matrix-memory (mLSTM cell) kernels of csrc/matrix_memory.hip: shape
checks on the host, then the launch."""
import ctypes
from dataclasses import dataclass

import torch

from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i, _f, _sz = ctypes.c_int, ctypes.c_float, ctypes.c_size_t

MAX_KEY_DIM = 512            # rows of S a workgroup's threads hold in registers


@dataclass(frozen=True)
class RowLayout:
    """Where a token's q, k, v, output gate and the two log-gate pre-activations lie in a row
    of the fused projection (column offsets, in elements)."""
    width: int
    q: int
    k: int
    v: int
    g: int
    i: int
    f: int

    @staticmethod
    def fused(n_heads: int, key_dim: int, value_dim: int) -> "RowLayout":
        """Rows of q, k, v, g, i, f one after the other."""
        q = 0
        k = q + n_heads * key_dim
        v = k + n_heads * key_dim
        g = v + n_heads * value_dim
        i = g + n_heads * value_dim
        f = i + n_heads
        return RowLayout(f + n_heads, q, k, v, g, i, f)


def state_size(n_heads: int, key_dim: int, value_dim: int) -> int:
    """float32 elements of one sequence's state: S [H, dk, dv], n [H, dk], m [H]."""
    return n_heads * (key_dim * value_dim + key_dim + 1)


CHUNK_MAX_KEY_DIM = 128      # the chunked kernel keeps a chunk's q and k in shared memory
CHUNKS_FROM_TOKENS = 16      # runs shorter than this go token by token


def cell(proj, layout, gate_bias, state, q_start, slots, n_seqs, max_q_len, n_heads, key_dim,
         value_dim, q_scale, gate_cap, den_eps) -> torch.Tensor:
    """Which kernel runs the cell: token by token for short runs (single-token steps), a
    chunk of tokens at a time where some sequence brings many."""
    chunked = max_q_len >= CHUNKS_FROM_TOKENS and key_dim <= CHUNK_MAX_KEY_DIM
    return scan(proj, layout, gate_bias, state, q_start, slots, n_seqs, n_heads, key_dim,
                value_dim, q_scale, gate_cap, den_eps, chunked=chunked)


def scan(proj: torch.Tensor, layout: RowLayout, gate_bias: torch.Tensor, state: torch.Tensor,
         q_start: torch.Tensor, slots: torch.Tensor, n_seqs: int, n_heads: int, key_dim: int,
         value_dim: int, q_scale: float, gate_cap: float, den_eps: float,
         chunked: bool = False, chunk: int = 0) -> torch.Tensor:
    """The cell over every sequence's new tokens in order; ``state`` [slots, state_size] is
    read and left updated.  proj float32 [N, layout.width]; returns o float32 [N, H, dv].
    ``chunked``: the kernel that takes ``chunk`` = 32 or 64 tokens at a time (key_dim up to
    128; 0: 64 where the device's shared memory holds them, else 32)."""
    require_device(proj, gate_bias, state, q_start, slots)
    require_contiguous(proj=proj, gate_bias=gate_bias, state=state, q_start=q_start, slots=slots)
    for name, t in (("proj", proj), ("gate_bias", gate_bias), ("state", state)):
        if t.dtype != torch.float32:
            raise KernelError(f"matrix memory: {name} must be float32, is {t.dtype}")
    for name, t in (("q_start", q_start), ("slots", slots)):
        if t.dtype != torch.int32:
            raise KernelError(f"matrix memory: {name} must be int32")
    if proj.dim() != 2 or proj.shape[1] != layout.width:
        raise KernelError(f"matrix memory: rows are {tuple(proj.shape)}, expected [N, {layout.width}]")
    if max(layout.q, layout.k) + n_heads * key_dim > layout.width or \
            layout.v + n_heads * value_dim > layout.width or max(layout.i, layout.f) + n_heads > layout.width:
        raise KernelError("matrix memory: the row layout does not fit the row width")
    if gate_bias.numel() != 2 * n_heads:
        raise KernelError("matrix memory: gate_bias holds the input gates' biases, then the forget gates'")
    if state.dim() != 2 or state.shape[1] != state_size(n_heads, key_dim, value_dim):
        raise KernelError(f"matrix memory: state is {tuple(state.shape)}, expected "
                          f"[slots, {state_size(n_heads, key_dim, value_dim)}]")
    if q_start.numel() < n_seqs + 1 or slots.numel() < n_seqs:
        raise KernelError("matrix memory: q_start / slots are shorter than the batch")
    if key_dim > MAX_KEY_DIM:
        raise KernelError(f"matrix memory: key_dim {key_dim} > {MAX_KEY_DIM} is not supported")
    out = torch.empty((proj.shape[0], n_heads, value_dim), dtype=torch.float32, device=proj.device)
    if chunked and key_dim > CHUNK_MAX_KEY_DIM:
        raise KernelError(f"matrix memory: the chunked kernel takes key_dim up to {CHUNK_MAX_KEY_DIM}")
    args = (ptr(proj), ptr(gate_bias), ptr(state), _sz(state.stride(0)), ptr(q_start), ptr(slots),
            ptr(out), _i(n_seqs), _i(n_heads), _i(key_dim), _i(value_dim), _i(layout.width),
            _i(layout.q), _i(layout.k), _i(layout.v), _i(layout.i), _i(layout.f), _f(q_scale),
            _f(gate_cap or 0.0), _f(den_eps))
    if chunked:
        check(library("matrix_memory").gfa_matrix_memory_chunks(*args, _i(chunk), stream_handle()),
              "matrix_memory_chunks")
    else:
        check(library("matrix_memory").gfa_matrix_memory_scan(*args, stream_handle()),
              "matrix_memory_scan")
    return out


def long_chunks_available(key_dim: int) -> bool:
    """Chunks of 64 tokens fit a workgroup's shared memory on the current device."""
    return bool(library("matrix_memory").gfa_matrix_memory_long_chunks(_i(key_dim)))


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, proj: torch.Tensor, layout: RowLayout,
                   eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """y[t, h, :] = o[t, h, :] / rms(o[t, h, :]) * weight[h, :] * sigmoid(gate[t, h, :]) in
    ``out_dtype``; o float32 [N, H, dv], the gate's pre-activations in proj at ``layout.g``."""
    require_device(o, weight, proj)
    require_contiguous(o=o, weight=weight, proj=proj)
    n, H, dv = o.shape
    if weight.numel() != H * dv or weight.dtype != torch.float32 or o.dtype != torch.float32:
        raise KernelError("head_norm_gate: o and weight must be float32, weight of H * dv elements")
    if proj.dtype != torch.float32 or proj.shape != (n, layout.width) or layout.g + H * dv > layout.width:
        raise KernelError("head_norm_gate: the projection's rows do not fit")
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise KernelError(f"head_norm_gate: output type {out_dtype}")
    y = torch.empty((n, H * dv), dtype=out_dtype, device=o.device)
    check(library("matrix_memory").gfa_head_norm_gate(
        ptr(o), ptr(weight), ptr(proj), _i(layout.width), _i(layout.g), ptr(y),
        _i(int(out_dtype == torch.bfloat16)), _i(n), _i(H), _i(dv), _f(eps), stream_handle()),
        "head_norm_gate")
    return y
