// Recurrent mixer with a matrix memory per head (the mLSTM cell): a kernel that goes token by
// token (single-token steps), one that takes a chunk of tokens at a time (prompts), and the
// head norm and gate that follow the cell.
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
// The same cell for runs of many tokens, a chunk of MC_L (32 or 64) tokens at a time instead
// of token by token.  Inside a chunk that starts from (S0, n0, m0), with F_t the running sum of the log
// forget gates from the chunk's start, g_s = i_s - F_s and M_t = max(m0, max_{s<=t} g_s):
//     m_t = F_t + M_t
//     S_t^T q_t = exp(m0 - M_t) S0^T q_t + sum_{s<=t} exp(g_s - M_t) (k_s . q_t) v_s
//     n_t . q_t = exp(m0 - M_t) n0 . q_t + sum_{s<=t} exp(g_s - M_t) (k_s . q_t)
// and the state after the chunk's last token L is
//     S_L = exp(m0 - M_L) S0 + sum_s exp(g_s - M_L) k_s v_s^T        (n_L likewise)
// which is the recurrence written out; every exponent is <= 0.  All float.
// grid (dv / MC_COLS, H, sequences), eight threads per token of a chunk; q, k, v of the chunk, the weighted scores
// and the workgroup's columns of S are in shared memory.
#define MC_COLS 32

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float mc_floatx4_t;

// rows of q and k in shared memory: dk filled up to a multiple of 16 (the matrix cores' tiles)
// plus four floats, so that the sixteen rows a load touches lie in different banks
__host__ __device__ inline int mc_padded(int dk) { return (dk + 15) / 16 * 16; }
__host__ __device__ inline int mc_row_stride(int dk) { return mc_padded(dk) + 4; }

template <int MC_L>
__global__ __launch_bounds__(MC_L * 8) void matrix_memory_chunk_kernel(
        const float* __restrict__ proj, const float* __restrict__ gate_bias,
        float* __restrict__ state, size_t slot_stride, const int* __restrict__ q_start,
        const int* __restrict__ slots, float* __restrict__ out, MMShape s) {
    extern __shared__ __attribute__((aligned(16))) float mc_lds[];
    constexpr int NT = MC_L * 8;                 // threads: eight per token of a chunk
    constexpr int NWV = NT / 64;                 // waves
    constexpr int MC_PS = MC_L + 1;
    const int KS = mc_row_stride(s.dk);
    const int dkp = mc_padded(s.dk);
    float* Qs = mc_lds;                          // [MC_L][KS]
    float* Ks = Qs + MC_L * KS;                  // [MC_L][KS]
    float* Vs = Ks + MC_L * KS;                  // [MC_L][MC_COLS]
    float* Ps = Vs + MC_L * MC_COLS;             // [MC_L][MC_PS]
    float* Ss = Ps + MC_L * MC_PS;               // [dkp][MC_COLS]
    float* ns = Ss + dkp * MC_COLS;              // [dkp]
    float* gs = ns + dkp;                        // [MC_L] g_s
    float* Ms = gs + MC_L;                       // [MC_L] M_t
    float* mt = Ms + MC_L;                       // [MC_L] m_t
    float* ws = mt + MC_L;                       // [MC_L] exp(g_s - M of the chunk's last token)
    float* nqs = ws + MC_L;                      // [MC_L] n_t . q_t
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col0 = blockIdx.x * MC_COLS;
    const int h = blockIdx.y, b = blockIdx.z;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    float* const base = state + (size_t)slots[b] * slot_stride;
    float* const S = base + (size_t)h * s.dk * s.dv;
    float* const nvec = base + (size_t)s.H * s.dk * s.dv + (size_t)h * s.dk;
    float* const mptr = base + (size_t)s.H * s.dk * (s.dv + 1) + h;
    const float ib = gate_bias[h], fb = gate_bias[s.H + h];

    for (int e = tid; e < dkp * MC_COLS; e += NT) {
        const int d = e / MC_COLS, c = e % MC_COLS;
        Ss[e] = (d < s.dk && col0 + c < s.dv) ? S[(size_t)d * s.dv + col0 + c] : 0.f;
    }
    for (int d = tid; d < dkp; d += NT) ns[d] = d < s.dk ? nvec[d] : 0.f;
    for (int e = tid; e < 2 * MC_L * KS; e += NT) Qs[e] = 0.f;      // q and k: the filling stays zero
    float m_prev = *mptr;

    // The rows of a chunk come from memory a chunk ahead: they are asked for before the chunk
    // in hand is worked on and put into shared memory when it is done.  Rows whose q, k and v
    // start at multiples of four floats travel as float4, four of q and k and one of v per
    // thread (dk <= 128); other shapes element by element, without the look-ahead.
    const int kq4 = s.dk / 4;
    const bool vec = s.dk % 4 == 0 && s.dv % 4 == 0 && s.row_width % 4 == 0 && s.q_off % 4 == 0
                     && s.k_off % 4 == 0 && s.v_off % 4 == 0;
    float4 rq[4], rk[4], rv;
    float ri = 0.f, rf = 0.f;
    auto fetch = [&](int c0) {
        const int Lc = t1 - c0 < MC_L ? t1 - c0 : MC_L;
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = tid + NT * i, t = e / kq4, d4 = e - t * kq4;
            rq[i] = rk[i] = zero;
            if (t < Lc) {
                const float* row = proj + (size_t)(c0 + t) * s.row_width + h * s.dk + d4 * 4;
                rq[i] = *(const float4*)(row + s.q_off);
                rk[i] = *(const float4*)(row + s.k_off);
            }
        }
        {
            const int t = tid >> 3, c4 = (tid & 7) * 4;
            rv = zero;
            if (t < Lc && col0 + c4 < s.dv)
                rv = *(const float4*)(proj + (size_t)(c0 + t) * s.row_width + s.v_off + h * s.dv + col0 + c4);
        }
        if (wave == 0 && lane < Lc) {
            const float* row = proj + (size_t)(c0 + lane) * s.row_width;
            ri = row[s.i_off + h];
            rf = row[s.f_off + h];
        }
    };
    if (vec && t0 < t1) fetch(t0);

    for (int c0 = t0; c0 < t1; c0 += MC_L) {
        const int Lc = t1 - c0 < MC_L ? t1 - c0 : MC_L;
        __syncthreads();                         // the chunk before is done with Qs .. Ss
        float ipre = 0.f, fpre = 0.f;
        if (vec) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int e = tid + NT * i, t = e / kq4, d4 = e - t * kq4;
                if (t < MC_L) {
                    float4 x = rq[i];
                    x.x *= s.q_scale; x.y *= s.q_scale; x.z *= s.q_scale; x.w *= s.q_scale;
                    *(float4*)(Qs + t * KS + d4 * 4) = x;
                    *(float4*)(Ks + t * KS + d4 * 4) = rk[i];
                }
            }
            *(float4*)(Vs + (tid >> 3) * MC_COLS + (tid & 7) * 4) = rv;
            ipre = ri;
            fpre = rf;
            if (c0 + MC_L < t1) fetch(c0 + MC_L);
        } else {
            // q (scaled), k, v of the chunk; rows beyond its end and columns beyond dk are zero
            for (int e = tid; e < MC_L * KS; e += NT) {
                const int t = e / KS, d = e - t * KS;
                const bool ok = t < Lc && d < s.dk;
                const float* row = proj + (size_t)(c0 + t) * s.row_width;
                Qs[e] = ok ? row[s.q_off + h * s.dk + d] * s.q_scale : 0.f;
                Ks[e] = ok ? row[s.k_off + h * s.dk + d] : 0.f;
            }
            for (int e = tid; e < MC_L * MC_COLS; e += NT) {
                const int t = e / MC_COLS, c = e % MC_COLS;
                Vs[e] = (t < Lc && col0 + c < s.dv)
                    ? proj[(size_t)(c0 + t) * s.row_width + s.v_off + h * s.dv + col0 + c] : 0.f;
            }
            if (wave == 0 && lane < Lc) {
                const float* row = proj + (size_t)(c0 + lane) * s.row_width;
                ipre = row[s.i_off + h];
                fpre = row[s.f_off + h];
            }
        }
        if (wave == 0) {
            // the gates of the chunk: running sum of f, running maximum of g, one token per lane
            const int t = lane;
            float ig = -INFINITY, fg = 0.f;
            if (t < Lc) {
                ig = mm_cap(ipre + ib, s.cap);
                fg = mm_logsigmoid(mm_cap(fpre + fb, s.cap));
            }
            float F = fg;
#pragma unroll
            for (int o = 1; o < MC_L; o <<= 1) {
                const float up = __shfl_up(F, o, GFA_WAVE);
                if (lane >= o) F += up;
            }
            const float g = ig - F;
            float M = fmaxf(g, m_prev);
#pragma unroll
            for (int o = 1; o < MC_L; o <<= 1) {
                const float up = __shfl_up(M, o, GFA_WAVE);
                if (lane >= o) M = fmaxf(M, up);
            }
            const float M_last = __shfl(M, Lc - 1, GFA_WAVE);
            if (t < MC_L) {
                gs[t] = g;
                Ms[t] = M;
                mt[t] = F + M;
                ws[t] = expf(g - M_last);
            }
        }
        __syncthreads();
        // The products run on the matrix cores in float (v_mfma_f32_16x16x4_f32: lane l
        // supplies A[l % 16][l / 16] and B[l / 16][l % 16] and holds C[4 (l / 16) .. +3][l % 16]),
        // a 16 x 16 tile of the result per wave and loop.
        const int li = lane & 15, lg = lane >> 4;
        // scores of the chunk, weighted: P[t][s] = (q_t . k_s) exp(g_s - M_t) for s <= t
        // (the 16 x 16 tiles on and below the diagonal, handed out over the waves)
        for (int idx = wave; idx < (MC_L / 16) * (MC_L / 16 + 1) / 2; idx += NWV) {
            int ti = 0;
            while ((ti + 1) * (ti + 2) / 2 <= idx) ++ti;
            const int si = idx - ti * (ti + 1) / 2;
            mc_floatx4_t acc = {0.f, 0.f, 0.f, 0.f};
            const float* qa = Qs + (ti * 16 + li) * KS + lg;
            const float* kb = Ks + (si * 16 + li) * KS + lg;
#pragma unroll 4
            for (int d0 = 0; d0 < dkp; d0 += 4)
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[d0], kb[d0], acc, 0, 0, 0);
            const int ss = si * 16 + li;
            const float g = gs[ss];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = ti * 16 + lg * 4 + r;
                Ps[t * MC_PS + ss] = ss <= t ? acc[r] * expf(g - Ms[t]) : 0.f;   // g of a missing token is -inf
            }
        }
        __syncthreads();
        // n_t . q_t: eight threads per token
        {
            const int t = tid >> 3, j = tid & 7;
            const float* qr = Qs + t * KS;
            const float* pr = Ps + t * MC_PS;
            float nq0 = 0.f, nq1 = 0.f;
            for (int d = j; d < s.dk; d += 8) nq0 = fmaf(qr[d], ns[d], nq0);
            for (int ss = j; ss <= t; ss += 8) nq1 += pr[ss];
            float nq = expf(m_prev - Ms[t]) * nq0 + nq1;
            nq += __shfl_xor(nq, 1, GFA_WAVE);
            nq += __shfl_xor(nq, 2, GFA_WAVE);
            nq += __shfl_xor(nq, 4, GFA_WAVE);
            if (j == 0) nqs[t] = nq;
        }
        // o_t for the workgroup's columns: exp(m0 - M_t) (Q S0) + P V
        mc_floatx4_t num;
        const int oti = wave >> 1, oci = wave & 1;
        {
            num = mc_floatx4_t{0.f, 0.f, 0.f, 0.f};
            const float* qa = Qs + (oti * 16 + li) * KS + lg;
            const float* sb = Ss + lg * MC_COLS + oci * 16 + li;
#pragma unroll 4
            for (int d0 = 0; d0 < dkp; d0 += 4)
                num = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[d0], sb[d0 * MC_COLS], num, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) num[r] *= expf(m_prev - Ms[oti * 16 + lg * 4 + r]);
            const float* pa = Ps + (oti * 16 + li) * MC_PS + lg;
            const float* vb = Vs + lg * MC_COLS + oci * 16 + li;
#pragma unroll 4
            for (int s0 = 0; s0 < (oti + 1) * 16; s0 += 4)
                num = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[s0], vb[s0 * MC_COLS], num, 0, 0, 0);
        }
        __syncthreads();                         // nqs is written; Ss has been read by every wave
        {
            const int c = col0 + oci * 16 + li;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int t = oti * 16 + lg * 4 + r;
                if (t < Lc && c < s.dv) {
                    const float den = fmaxf(fabsf(nqs[t]), expf(-mt[t])) + s.den_eps;
                    out[(size_t)(c0 + t) * s.H * s.dv + (size_t)h * s.dv + c] = num[r] / den;
                }
            }
        }
        // the state after the chunk's last token: S = decay S + (w K)^T V, a wave's tiles of 16
        // rows of S by 16 columns in turn
        {
            const float decay = expf(m_prev - Ms[Lc - 1]);
            for (int tile = wave; tile < (dkp / 16) * 2; tile += NWV) {
                const int di = tile >> 1, ci = tile & 1;
                float* sc = Ss + (di * 16 + lg * 4) * MC_COLS + ci * 16 + li;
                mc_floatx4_t acc;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[r] = decay * sc[r * MC_COLS];
                const float* ka = Ks + lg * KS + di * 16 + li;
                const float* vb = Vs + lg * MC_COLS + ci * 16 + li;
#pragma unroll
                for (int s0 = 0; s0 < MC_L; s0 += 4)
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(ws[s0 + lg] * ka[s0 * KS], vb[s0 * MC_COLS],
                                                              acc, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 4; ++r) sc[r * MC_COLS] = acc[r];
            }
            for (int d = tid; d < s.dk; d += NT) {
                float a = decay * ns[d];
                for (int ss = 0; ss < Lc; ++ss) a = fmaf(ws[ss], Ks[ss * KS + d], a);
                ns[d] = a;
            }
            m_prev = mt[Lc - 1];
        }
    }
    __syncthreads();
    for (int e = tid; e < s.dk * MC_COLS; e += NT) {
        const int d = e / MC_COLS, c = e % MC_COLS;
        if (col0 + c < s.dv) S[(size_t)d * s.dv + col0 + c] = Ss[e];
    }
    if (blockIdx.x == 0) {
        for (int d = tid; d < s.dk; d += NT) nvec[d] = ns[d];
        if (tid == 0) *mptr = m_prev;
    }
}

static int mc_lds_bytes(int dk, int L) {
    const int dkp = mc_padded(dk);
    return (int)sizeof(float) * (2 * L * mc_row_stride(dk) + L * MC_COLS + L * (L + 1)
                                 + dkp * MC_COLS + dkp + 5 * L);
}

static int mc_lds_limit() {
    static int limit = -1;
    if (limit < 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess)
            v = 64 * 1024;
        limit = v;
    }
    return limit;
}

// 1 if chunks of 64 tokens fit a workgroup's shared memory on this device for this key size
extern "C" int gfa_matrix_memory_long_chunks(int dk) {
    return dk <= 128 && mc_lds_bytes(dk, 64) <= mc_lds_limit() ? 1 : 0;
}

// Chunks of 64 tokens (512 threads) where the device lets a workgroup have the shared memory
// for them (109 KB at dk = 128), else chunks of 32 (256 threads, at most 60 KB): a longer
// chunk spreads the chain of barriers, the gates' scans and the state's products over twice
// the tokens.
extern "C" int gfa_matrix_memory_chunks(const float* proj, const float* gate_bias, float* state,
                                        size_t slot_stride, const int* q_start, const int* slots,
                                        float* out, int n_seqs, int H, int dk, int dv, int row_width,
                                        int q_off, int k_off, int v_off, int i_off, int f_off,
                                        float q_scale, float cap, float den_eps, int chunk,
                                        hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (dk > 128 || H > 65535 || n_seqs > 65535 || (chunk != 0 && chunk != 32 && chunk != 64))
        return (int)hipErrorInvalidValue;
    const int lds_limit = mc_lds_limit();
    MMShape s{H, dk, dv, row_width, q_off, k_off, v_off, i_off, f_off, q_scale, cap, den_eps};
    dim3 grid((dv + MC_COLS - 1) / MC_COLS, H, n_seqs);
    const int big = mc_lds_bytes(dk, 64);
    if (chunk == 64 && big > lds_limit) return (int)hipErrorInvalidValue;
    if (chunk != 32 && big <= lds_limit) {
        static bool allowed = false;
        if (!allowed) {
            const hipError_t e = hipFuncSetAttribute((const void*)matrix_memory_chunk_kernel<64>,
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (e != hipSuccess) return (int)e;
            allowed = true;
        }
        matrix_memory_chunk_kernel<64><<<grid, 512, big, stream>>>(proj, gate_bias, state, slot_stride,
                                                                  q_start, slots, out, s);
        return GFA_LAUNCH_RESULT();
    }
    const int small = mc_lds_bytes(dk, 32);
    if (small > 64 * 1024) return (int)hipErrorInvalidValue;
    matrix_memory_chunk_kernel<32><<<grid, 256, small, stream>>>(proj, gate_bias, state, slot_stride,
                                                                q_start, slots, out, s);
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
