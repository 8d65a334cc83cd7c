// Recurrent mixer with a matrix memory per head (the mLSTM cell): plain kernels.
//
// Per sequence and head the state is S [dk, dv], n [dk] and a running maximum m of the log
// gates, all float and kept in the cache's state slots:
//     i = cap tanh((ipre + ib) / cap)          f = logsigmoid(cap tanh((fpre + fb) / cap))
//     m' = max(f + m, i)     a = exp(f + m - m')     b = exp(i - m')
//     S' = a S + b k v^T     n' = a n + b k
//     o = S'^T q / (max(|n' . q|, exp(-m')) + den_eps)
// Everything here is float arithmetic: the rows of q, k, v and the gates' pre-activations
// arrive as float (the projection's float accumulators, unrounded).
//
// One slot's state: S [H][dk][dv], then n [H][dk], then m [H].
#include "common.h"

#define MM_THREADS 256
#define MM_COLS 32                      // columns of S (elements of v) per workgroup
#define MM_GROUPS (MM_THREADS / MM_COLS)

struct MMShape {
    int H, dk, dv;
    int row_width;                      // floats per row of proj
    int q_off, k_off, v_off, i_off, f_off;   // column offsets in a row of proj
    float q_scale, cap, den_eps;
};

__device__ __forceinline__ float mm_cap(float x, float cap) {
    return cap > 0.f ? cap * tanhf(x / cap) : x;
}
__device__ __forceinline__ float mm_logsigmoid(float x) {
    // log(1 / (1 + exp(-x))), stable on both sides
    return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}

// Token by token.  grid (dv / MM_COLS, H, sequences).  Thread (c, g) = (tid % 32, tid / 32)
// holds rows g, g + 8, ... of column c of S in registers; every workgroup of a head keeps n
// and m for itself (the same arithmetic in each), the first one stores them.
template <int RPT>
__global__ __launch_bounds__(MM_THREADS) void matrix_memory_scan_kernel(
        const float* __restrict__ proj, const float* __restrict__ gate_bias,   // [2H]: i then f
        float* __restrict__ state, size_t slot_stride, const int* __restrict__ q_start,
        const int* __restrict__ slots, float* __restrict__ out, MMShape s) {
    __shared__ float qs[RPT * MM_GROUPS], ks[RPT * MM_GROUPS];
    __shared__ float red[MM_GROUPS][MM_COLS];
    __shared__ float scratch[16];
    const int tid = threadIdx.x, c = tid % MM_COLS, g = tid / MM_COLS;
    const int col = blockIdx.x * MM_COLS + c;
    const int h = blockIdx.y, b = blockIdx.z;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    float* const base = state + (size_t)slots[b] * slot_stride;
    float* const S = base + (size_t)h * s.dk * s.dv;
    float* const nvec = base + (size_t)s.H * s.dk * s.dv + (size_t)h * s.dk;
    float* const mptr = base + (size_t)s.H * s.dk * (s.dv + 1) + h;
    const bool col_ok = col < s.dv;

    float Sreg[RPT];
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = g + r * MM_GROUPS;
        Sreg[r] = (col_ok && row < s.dk) ? S[(size_t)row * s.dv + col] : 0.f;
    }
    // n: element tid + j * 256 of the head's n lives in thread tid
    constexpr int NPT = (RPT * MM_GROUPS + MM_THREADS - 1) / MM_THREADS;
    float nreg[NPT];
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
        const int e = tid + j * MM_THREADS;
        nreg[j] = e < s.dk ? nvec[e] : 0.f;
    }
    float m = *mptr;
    const float ib = gate_bias[h], fb = gate_bias[s.H + h];

    for (int t = t0; t < t1; ++t) {
        const float* row = proj + (size_t)t * s.row_width;
        for (int e = tid; e < RPT * MM_GROUPS; e += MM_THREADS) {
            qs[e] = e < s.dk ? row[s.q_off + h * s.dk + e] * s.q_scale : 0.f;
            ks[e] = e < s.dk ? row[s.k_off + h * s.dk + e] : 0.f;
        }
        const float v = col_ok ? row[s.v_off + h * s.dv + col] : 0.f;
        const float ig = mm_cap(row[s.i_off + h] + ib, s.cap);
        const float fg = mm_logsigmoid(mm_cap(row[s.f_off + h] + fb, s.cap));
        const float m_new = fmaxf(fg + m, ig);
        const float a = expf(fg + m - m_new), bb = expf(ig - m_new);
        __syncthreads();
        float part = 0.f;
        const float bv = bb * v;
#pragma unroll
        for (int r = 0; r < RPT; ++r) {
            const int e = g + r * MM_GROUPS;
            Sreg[r] = fmaf(a, Sreg[r], bv * ks[e]);
            part = fmaf(Sreg[r], qs[e], part);
        }
        red[g][c] = part;
        float nq = 0.f;
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const int e = tid + j * MM_THREADS;
            if (e < RPT * MM_GROUPS) {
                nreg[j] = fmaf(a, nreg[j], bb * ks[e]);
                nq = fmaf(nreg[j], qs[e], nq);
            }
        }
        nq = block_sum(nq, scratch);                 // its barriers publish red as well
        if (g == 0 && col_ok) {
            float o = 0.f;
#pragma unroll
            for (int r = 0; r < MM_GROUPS; ++r) o += red[r][c];
            const float den = fmaxf(fabsf(nq), expf(-m_new)) + s.den_eps;
            out[(size_t)t * s.H * s.dv + (size_t)h * s.dv + col] = o / den;
        }
        m = m_new;
        __syncthreads();
    }
#pragma unroll
    for (int r = 0; r < RPT; ++r) {
        const int row = g + r * MM_GROUPS;
        if (col_ok && row < s.dk) S[(size_t)row * s.dv + col] = Sreg[r];
    }
    if (blockIdx.x == 0) {
#pragma unroll
        for (int j = 0; j < NPT; ++j) {
            const int e = tid + j * MM_THREADS;
            if (e < s.dk) nvec[e] = nreg[j];
        }
        if (tid == 0) *mptr = m;
    }
}

extern "C" int gfa_matrix_memory_scan(const float* proj, const float* gate_bias, float* state,
                                      size_t slot_stride, const int* q_start, const int* slots,
                                      float* out, int n_seqs, int H, int dk, int dv, int row_width,
                                      int q_off, int k_off, int v_off, int i_off, int f_off,
                                      float q_scale, float cap, float den_eps, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (dk > 64 * MM_GROUPS || H > 65535 || n_seqs > 65535) return (int)hipErrorInvalidValue;
    MMShape s{H, dk, dv, row_width, q_off, k_off, v_off, i_off, f_off, q_scale, cap, den_eps};
    dim3 grid((dv + MM_COLS - 1) / MM_COLS, H, n_seqs);
    const int rpt = (dk + MM_GROUPS - 1) / MM_GROUPS;
#define MM_LAUNCH(R) matrix_memory_scan_kernel<R><<<grid, MM_THREADS, 0, stream>>>( \
        proj, gate_bias, state, slot_stride, q_start, slots, out, s)
    if (rpt <= 4) MM_LAUNCH(4);
    else if (rpt <= 8) MM_LAUNCH(8);
    else if (rpt <= 16) MM_LAUNCH(16);
    else if (rpt <= 32) MM_LAUNCH(32);
    else MM_LAUNCH(64);
#undef MM_LAUNCH
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// What follows the cell: each head's o is divided by its root mean square (eps inside the
// root), times a weight per element, times sigmoid of the gate projection; rounded once, to
// the type of the output projection's operand.  One wave per (token, head).
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(
        const float* __restrict__ o, const float* __restrict__ weight, const float* __restrict__ proj,
        int row_width, int g_off, T* __restrict__ y, int n_tokens, int H, int dv, float eps) {
    const int lane = threadIdx.x & 63;
    const long long unit = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= (long long)n_tokens * H) return;
    const int t = (int)(unit / H), h = (int)(unit % H);
    const float* src = o + ((size_t)t * H + h) * dv;
    float ss = 0.f;
    for (int d = lane; d < dv; d += 64) ss = fmaf(src[d], src[d], ss);
    ss = wave_sum(ss);
    const float r = rsqrtf(ss / (float)dv + eps);
    const float* gate = proj + (size_t)t * row_width + g_off + h * dv;
    T* dst = y + ((size_t)t * H + h) * dv;
    for (int d = lane; d < dv; d += 64) {
        const float gv = 1.f / (1.f + expf(-gate[d]));
        store_from_float(dst + d, src[d] * r * weight[h * dv + d] * gv);
    }
}

extern "C" int gfa_head_norm_gate(const float* o, const float* weight, const float* proj,
                                  int row_width, int g_off, void* y, int y_bf16, int n_tokens,
                                  int H, int dv, float eps, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    const long long units = (long long)n_tokens * H;
    const unsigned blocks = (unsigned)((units + 3) / 4);
    if (y_bf16)
        head_norm_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(o, weight, proj, row_width, g_off,
                                                                 (bf16_t*)y, n_tokens, H, dv, eps);
    else
        head_norm_gate_kernel<float><<<blocks, 256, 0, stream>>>(o, weight, proj, row_width, g_off,
                                                                (float*)y, n_tokens, H, dv, eps);
    return GFA_LAUNCH_RESULT();
}
