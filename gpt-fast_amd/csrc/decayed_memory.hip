// Linear attention with a fixed decay per head (lightning attention): per sequence and head a
// float state S [dk, dv], zero at the sequence's start and kept in the cache's state slots:
//     q = silu(q'), k = silu(k'), v = silu(v')        (q', k', v': the projection's float sums)
//     S' = decay_h S + k v^T          o = S'^T q
// Everything here is float arithmetic.  One slot's state: S [H][dk][dv].
//
// Two kernels: token by token (single-token steps and short runs), and a chunk of tokens at a
// time (prompts).  Inside a chunk that starts from S0, with a = decay_h and tokens t = 0, 1, ...:
//     o_t = a^(t+1) S0^T q_t + sum_{s<=t} a^(t-s) (k_s . q_t) v_s
//     S_L = a^L S0 + sum_s a^(L-1-s) k_s v_s^T
// which is the recurrence written out; every power of a has a non-negative exponent.
#include "common.h"

#define DM_THREADS 256
#define DM_COLS 32                      // columns of S (elements of v) per workgroup
#define DM_GROUPS (DM_THREADS / DM_COLS)

struct DMShape {
    int H, dk, dv;
    int row_width;                      // floats per row of proj
    int q_off, k_off, v_off;            // column offsets in a row of proj
};

__device__ __forceinline__ float dm_silu(float z) { return z / (1.f + expf(-z)); }

// Token by token.  grid (dv / DM_COLS, H, sequences).  Thread (c, g) = (tid % 32, tid / 32)
// holds rows g, g + 8, ... of column c of S in registers.
template <int RPT>
__global__ __launch_bounds__(DM_THREADS) void decayed_memory_scan_kernel(
        const float* __restrict__ proj, const float* __restrict__ decay, float* __restrict__ state,
        size_t slot_stride, const int* __restrict__ q_start, const int* __restrict__ slots,
        float* __restrict__ out, DMShape s) {
    __shared__ float qs[RPT * DM_GROUPS], ks[RPT * DM_GROUPS];
    __shared__ float red[DM_GROUPS][DM_COLS];
    const int tid = threadIdx.x, c = tid % DM_COLS, g = tid / DM_COLS;
    const int col = blockIdx.x * DM_COLS + c;
    const int h = blockIdx.y, b = blockIdx.z;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    float* const S = state + (size_t)slots[b] * slot_stride + (size_t)h * s.dk * s.dv;
    const bool col_ok = col < s.dv;
    const float a = decay[h];

    float Sreg[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = g + r * DM_GROUPS;
        Sreg[r] = (col_ok && row < s.dk) ? S[(size_t)row * s.dv + col] : 0.f;
    }
    for (int t = t0; t < t1; ++t) {
        const float* row = proj + (size_t)t * s.row_width;
        for (int e = tid; e < RPT * DM_GROUPS; e += DM_THREADS) {
            qs[e] = e < s.dk ? dm_silu(row[s.q_off + h * s.dk + e]) : 0.f;
            ks[e] = e < s.dk ? dm_silu(row[s.k_off + h * s.dk + e]) : 0.f;
        }
        const float v = col_ok ? dm_silu(row[s.v_off + h * s.dv + col]) : 0.f;
        __syncthreads();
        float part = 0.f;
#pragma unroll
        for (int r = 0; r < RPT; ++r) {
            const int e = g + r * DM_GROUPS;
            Sreg[r] = fmaf(a, Sreg[r], ks[e] * v);
            part = fmaf(Sreg[r], qs[e], part);
        }
        red[g][c] = part;
        __syncthreads();
        if (g == 0 && col_ok) {
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < DM_GROUPS; ++r) o += red[r][c];
            out[(size_t)t * s.H * s.dv + (size_t)h * s.dv + col] = o;
        }
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = g + r * DM_GROUPS;
        if (col_ok && row < s.dk) S[(size_t)row * s.dv + col] = Sreg[r];
    }
}

extern "C" int gfa_decayed_memory_scan(const float* proj, const float* decay, float* state,
                                       size_t slot_stride, const int* q_start, const int* slots,
                                       float* out, int n_seqs, int H, int dk, int dv, int row_width,
                                       int q_off, int k_off, int v_off, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (dk > 64 * DM_GROUPS || H > 65535 || n_seqs > 65535) return (int)hipErrorInvalidValue;
    DMShape s{H, dk, dv, row_width, q_off, k_off, v_off};
    dim3 grid((dv + DM_COLS - 1) / DM_COLS, H, n_seqs);
    const int rpt = (dk + DM_GROUPS - 1) / DM_GROUPS;
#define DM_LAUNCH(R) decayed_memory_scan_kernel<R><<<grid, DM_THREADS, 0, stream>>>( \
        proj, decay, state, slot_stride, q_start, slots, out, s)
    if (rpt <= 4) DM_LAUNCH(4);
    else if (rpt <= 8) DM_LAUNCH(8);
    else if (rpt <= 16) DM_LAUNCH(16);
    else if (rpt <= 32) DM_LAUNCH(32);
    else DM_LAUNCH(64);
#undef DM_LAUNCH
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The heads' results side by side, normed as one row, times a weight per element, times sigmoid
// of the gate projection; rounded once, to the type of the output projection's operand.
//     y[t, :] = o[t, :] * rsqrt(mean(o[t, :]^2) + eps) * weight[:] * sigmoid(gate[t, :])
// The gate's pre-activations lie in proj at column g_off.  One workgroup per token.
template <typename T>
__global__ __launch_bounds__(256) void row_norm_gate_kernel(
        const float* __restrict__ o, const float* __restrict__ weight, const float* __restrict__ proj,
        int row_width, int g_off, T* __restrict__ y, int width, float eps) {
    __shared__ float scratch[16];
    const size_t t = blockIdx.x;
    const float* src = o + t * width;
    float ss = 0.f;
    for (int d = threadIdx.x; d < width; d += 256) ss = fmaf(src[d], src[d], ss);
    const float r = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
    const float* gate = proj + t * row_width + g_off;
    for (int d = threadIdx.x; d < width; d += 256)
        store_from_float(y + t * width + d, src[d] * r * weight[d] / (1.f + expf(-gate[d])));
}

extern "C" int gfa_row_norm_gate(const float* o, const float* weight, const float* proj,
                                 int row_width, int g_off, void* y, int y_bf16, int n_tokens,
                                 int width, float eps, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (y_bf16)
        row_norm_gate_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(o, weight, proj, row_width, g_off,
                                                                  (bf16_t*)y, width, eps);
    else
        row_norm_gate_kernel<float><<<n_tokens, 256, 0, stream>>>(o, weight, proj, row_width, g_off,
                                                                 (float*)y, width, eps);
    return GFA_LAUNCH_RESULT();
}
