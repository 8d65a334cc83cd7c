// Differential attention over the paged cache: the rotation and cache write, a plain
// attention kernel (float32 and any size), and one on the matrix cores (bfloat16).
//
// A head holds MAPS = 2 softmax maps over the same values.  Query rows lie head by head as
// [map 1, map 2], each map `dim` wide; so do key rows per kv head; values are `vdim` wide.
// A head's result is a1 - lam a2, divided by its root mean square over vdim (eps inside the
// root), times out_scale, times sigmoid(gate) if a gate per head is given.  Position i sees
// key j if j <= i and (i - j < window or j < keep_first); window 0: every earlier key.
//
// Cache: the region of (page, kv head) in the key pool holds PAGE * 2 dim elements, map 1's
// keys first, then map 2's, each in the order of common.h's key_offset for head size dim;
// the value pool's region holds PAGE * vdim elements in the order of value_offset for vdim.
#include "common.h"

#define DA_MAPS 2

// --------------------------------------------------------------------------------------
// Rotation of q and k and the cache write.  proj [N, row_width], float (the projection's
// accumulators, unrounded), holds per token q [H][2][dim] at q_off, k [G][2][dim] at k_off,
// v [G][vdim] at v_off and, if gate_out is given, one gate number per head at g_off.  Pairs
// (2i, 2i+1) of the first `rot` elements of every map are rotated by pos * freqs[i], angle,
// cos and sin in float; the rest passes through.  q goes to q_out [N, H, 2, dim], k and v
// into the pages, each rounded once to T; the gates are copied to gate_out [N, H], float.
template <typename T>
__global__ __launch_bounds__(256) void da_rope_store_kernel(
        const float* __restrict__ proj, int row_width, int q_off, int k_off, int v_off, int g_off,
        T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
        float* __restrict__ gate_out, const float* __restrict__ freqs,
        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
        const int* __restrict__ table, int table_stride, int H, int G, int dim, int vdim, int rot) {
    extern __shared__ float cs[];                          // [rot / 2][2]
    // blockIdx.y walks the token's elements in groups of 256; each workgroup works out the
    // token's cos and sin for itself
    const int n = blockIdx.x;
    const int pos = tok_pos[n];
    for (int i = threadIdx.x; i < rot / 2; i += 256)
        sincosf((float)pos * freqs[i], &cs[2 * i + 1], &cs[2 * i]);
    __syncthreads();
    const float* row = proj + (size_t)n * row_width;
    int page = 0;
    if (k_pages) page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int off = pos % GFA_PAGE;
    const int q_elems = H * DA_MAPS * dim, k_elems = G * DA_MAPS * dim, v_elems = G * vdim;
    const int e = blockIdx.y * 256 + threadIdx.x;
    if (e < q_elems + k_elems) {
        const bool is_q = e < q_elems;
        const int ee = is_q ? e : e - q_elems;
        const int mh = ee / dim, d = ee - mh * dim;    // mh = head * 2 + map
        const float* src = row + (is_q ? q_off : k_off) + (size_t)mh * dim;
        float val;
        if (d < rot) {
            const int i = d >> 1;
            const float u = src[2 * i], w = src[2 * i + 1];
            const float c = cs[2 * i], s = cs[2 * i + 1];
            val = (d & 1) ? w * c + u * s : u * c - w * s;
        } else {
            val = src[d];
        }
        if (is_q) {
            store_from_float(q_out + (size_t)n * q_elems + ee, val);
        } else if (k_pages) {
            const int g = mh / DA_MAPS, map = mh % DA_MAPS;
            T* dst = k_pages + cache_region(page, g, G, DA_MAPS * dim) + (size_t)map * GFA_PAGE * dim;
            store_from_float(dst + key_offset(off, d, dim), val);
        }
    } else if (e < q_elems + k_elems + v_elems) {
        if (v_pages) {
            const int ev = e - q_elems - k_elems;
            const int g = ev / vdim, d = ev - g * vdim;
            store_from_float(v_pages + cache_region(page, g, G, vdim) + value_offset(d, off, vdim),
                             row[v_off + ev]);
        }
    } else if (gate_out && e < q_elems + k_elems + v_elems + H) {
        const int h = e - q_elems - k_elems - v_elems;
        gate_out[(size_t)n * H + h] = row[g_off + h];
    }
}

extern "C" int gfa_da_rope_store(const float* proj, int row_width, int q_off, int k_off, int v_off,
                                 int g_off, void* q_out, void* k_pages, void* v_pages,
                                 float* gate_out, const float* freqs, const int* tok_seq,
                                 const int* tok_pos, const int* table, int table_stride,
                                 int n_tokens, int H, int G, int dim, int vdim, int rot,
                                 int out_bf16, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    const size_t shmem = (size_t)(rot > 0 ? rot : 2) * sizeof(float);
    const int elems = (H + G) * DA_MAPS * dim + G * vdim + H;
    if ((elems + 255) / 256 > 65535) return (int)hipErrorInvalidValue;
    const dim3 grid(n_tokens, (elems + 255) / 256);
    if (out_bf16)
        da_rope_store_kernel<bf16_t><<<grid, 256, shmem, stream>>>(
            proj, row_width, q_off, k_off, v_off, g_off, (bf16_t*)q_out, (bf16_t*)k_pages,
            (bf16_t*)v_pages, gate_out, freqs, tok_seq, tok_pos, table, table_stride, H, G, dim,
            vdim, rot);
    else
        da_rope_store_kernel<float><<<grid, 256, shmem, stream>>>(
            proj, row_width, q_off, k_off, v_off, g_off, (float*)q_out, (float*)k_pages,
            (float*)v_pages, gate_out, freqs, tok_seq, tok_pos, table, table_stride, H, G, dim,
            vdim, rot);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// Attention of each new token, both maps, and what follows them.  One workgroup of 128
// threads per (token, head); visible keys in chunks of 128 (the kept first keys, then the
// window), one key per thread for the two scores, one output element per thread for the
// values.  Scores, softmax, sums, the combination and the norm are float.
#define DA_THREADS 128
#define DA_MAX_PER_THREAD 4            // vdim <= 512
template <typename T>
__global__ __launch_bounds__(DA_THREADS) void da_attention_generic_kernel(
        const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
        const float* __restrict__ gate, int gate_stride, const int* __restrict__ tok_seq,
        const int* __restrict__ tok_pos, const int* __restrict__ table, int table_stride,
        T* __restrict__ out, int H, int G, int dim, int vdim, float scale, int window,
        int keep_first, float lam, float eps, float out_scale) {
    extern __shared__ float shared[];
    float* qs = shared;                               // [2][dim]
    float* sc = shared + DA_MAPS * dim;               // [2][DA_THREADS]
    float* scratch = sc + DA_MAPS * DA_THREADS;       // [16]
    const int n = blockIdx.x, h = blockIdx.y;
    const int g = h / (H / G);
    const int pos = tok_pos[n];
    const int* pages = table + (size_t)tok_seq[n] * table_stride;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int n_first = keep_first < lo ? keep_first : lo;     // kept keys before the window
    const int total = n_first + (pos - lo + 1);
    const T* qrow = q + ((size_t)n * H + h) * DA_MAPS * dim;
    for (int d = threadIdx.x; d < DA_MAPS * dim; d += DA_THREADS) qs[d] = load_as_float(qrow + d);
    __syncthreads();

    float m[DA_MAPS], l[DA_MAPS], acc[DA_MAPS][DA_MAX_PER_THREAD];
#pragma unroll
    for (int a = 0; a < DA_MAPS; ++a) {
        m[a] = -INFINITY;
        l[a] = 0.f;
#pragma unroll
        for (int i = 0; i < DA_MAX_PER_THREAD; ++i) acc[a][i] = 0.f;
    }
    auto key_of = [&](int x) { return x < n_first ? x : lo + (x - n_first); };

    for (int base = 0; base < total; base += DA_THREADS) {
        const int x = base + threadIdx.x;
        float s[DA_MAPS] = {-INFINITY, -INFINITY};
        if (x < total) {
            const int j = key_of(x);
            const T* kr = k_pages + cache_region(pages[j / GFA_PAGE], g, G, DA_MAPS * dim);
#pragma unroll
            for (int a = 0; a < DA_MAPS; ++a) {
                const T* km = kr + (size_t)a * GFA_PAGE * dim;
                float dot = 0.f;
                for (int d = 0; d < dim; ++d)
                    dot = fmaf(qs[a * dim + d], load_as_float(km + key_offset(j % GFA_PAGE, d, dim)), dot);
                s[a] = dot * scale;
            }
        }
        float alpha[DA_MAPS];
#pragma unroll
        for (int a = 0; a < DA_MAPS; ++a) {
            const float m_new = fmaxf(m[a], block_max(s[a], scratch));
            alpha[a] = expf(m[a] - m_new);            // 0 on the first chunk (m = -inf)
            const float p = (x < total) ? expf(s[a] - m_new) : 0.f;
            sc[a * DA_THREADS + threadIdx.x] = p;
            l[a] = l[a] * alpha[a] + block_sum(p, scratch);   // its barriers publish sc
            m[a] = m_new;
        }
        const int count = (total - base < DA_THREADS) ? total - base : DA_THREADS;
#pragma unroll
        for (int i = 0; i < DA_MAX_PER_THREAD; ++i) {
            const int d = threadIdx.x + i * DA_THREADS;
            if (d < vdim) {
                float a0 = acc[0][i] * alpha[0], a1 = acc[1][i] * alpha[1];
                for (int jj = 0; jj < count; ++jj) {
                    const int key = key_of(base + jj);
                    const float v = load_as_float(v_pages + cache_region(pages[key / GFA_PAGE], g, G, vdim)
                                                  + value_offset(d, key % GFA_PAGE, vdim));
                    a0 = fmaf(sc[jj], v, a0);
                    a1 = fmaf(sc[DA_THREADS + jj], v, a1);
                }
                acc[0][i] = a0;
                acc[1][i] = a1;
            }
        }
        __syncthreads();
    }
    // a1 - lam a2, the head's norm, the gate
    float o[DA_MAX_PER_THREAD], ss = 0.f;
#pragma unroll
    for (int i = 0; i < DA_MAX_PER_THREAD; ++i) {
        const int d = threadIdx.x + i * DA_THREADS;
        o[i] = d < vdim ? acc[0][i] / l[0] - lam * (acc[1][i] / l[1]) : 0.f;
        ss = fmaf(o[i], o[i], ss);
    }
    ss = block_sum(ss, scratch);
    float f = rsqrtf(ss / (float)vdim + eps) * out_scale;
    if (gate) f *= 1.f / (1.f + expf(-gate[(size_t)n * gate_stride + h]));
    T* orow = out + ((size_t)n * H + h) * vdim;
#pragma unroll
    for (int i = 0; i < DA_MAX_PER_THREAD; ++i) {
        const int d = threadIdx.x + i * DA_THREADS;
        if (d < vdim) store_from_float(orow + d, o[i] * f);
    }
}

extern "C" int gfa_da_attention_generic(const void* q, const void* k_pages, const void* v_pages,
                                        const float* gate, int gate_stride, const int* tok_seq,
                                        const int* tok_pos, const int* table, int table_stride,
                                        void* out, int n_tokens, int H, int G, int dim, int vdim,
                                        float scale, int window, int keep_first, float lam,
                                        float eps, float out_scale, int is_bf16,
                                        hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (vdim > DA_THREADS * DA_MAX_PER_THREAD || H > 65535) return (int)hipErrorInvalidValue;
    dim3 grid(n_tokens, H);
    const size_t shmem = (size_t)(DA_MAPS * dim + DA_MAPS * DA_THREADS + 16) * sizeof(float);
    if (is_bf16)
        da_attention_generic_kernel<bf16_t><<<grid, DA_THREADS, shmem, stream>>>(
            (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, gate,
            gate_stride, tok_seq, tok_pos, table, table_stride, (bf16_t*)out, H, G, dim, vdim,
            scale, window, keep_first, lam, eps, out_scale);
    else
        da_attention_generic_kernel<float><<<grid, DA_THREADS, shmem, stream>>>(
            (const float*)q, (const float*)k_pages, (const float*)v_pages, gate,
            gate_stride, tok_seq, tok_pos, table, table_stride, (float*)out, H, G, dim, vdim,
            scale, window, keep_first, lam, eps, out_scale);
    return GFA_LAUNCH_RESULT();
}

// --------------------------------------------------------------------------------------
// The same on the matrix cores, bfloat16, for head sizes in eights up to 128 and value sizes
// in sixteens up to 256 (the cache orders of common.h that those sizes have).
//
// A wavefront owns 16 rows of one sequence and kv head; a row is a (token, query head of the
// kv head's group) pair, heads fastest.  It walks the visible keys in blocks of 32 - the
// blocks of the kept first keys, then those of the window - with a running maximum and sum
// per row and map, all float.  Both products are formed transposed, so that every operand is
// read in the order the cache has and the weights never leave their registers:
//   S^T = K Q^T   A = 16 keys x 32 dims of a key page, B = Q^T from registers;
//   O^T = V^T P^T A = 16 dims x 32 keys of a value page, B = the eight weights a lane holds.
// v_mfma_f32_16x16x32_bf16: lane l supplies row (A) / column (B) l % 16, k = 8 (l / 16) .. +7,
// and receives rows 4 (l / 16) .. +3 of column l % 16; with the key order of common.h those
// rows of the two 16-key tiles are the lane's keys 8 (l / 16) .. +7 of the block.
// Head sizes that are no multiple of 32 and value sizes below the template's are filled up:
// the query's registers are zero there and the loads are pointed at valid elements.
//
// SPLIT (one token per sequence, a group of at most 16 heads): the waves of a workgroup share
// the blocks of one tile of rows and the first wave adds their partial results in wave order.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 da_bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float da_floatx4_t;
union DAFrag {
    uint4 u;
    bf16_t e[8];
    da_bf16x8_t v;
};

__device__ __forceinline__ float da_max_lane_groups(float v) {
    v = fmaxf(v, __shfl_xor(v, 16, GFA_WAVE));
    return fmaxf(v, __shfl_xor(v, 32, GFA_WAVE));
}
__device__ __forceinline__ float da_sum_lane_groups(float v) {
    v += __shfl_xor(v, 16, GFA_WAVE);
    return v + __shfl_xor(v, 32, GFA_WAVE);
}

template <int DK, int DVT, bool SPLIT>
__global__ __launch_bounds__(SPLIT ? 512 : 256) void da_attention_mfma_kernel(
        const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
        const bf16_t* __restrict__ v_pages, const float* __restrict__ gate, int gate_stride,
        const int* __restrict__ q_start, const int* __restrict__ start_pos,
        const int* __restrict__ table, int table_stride, bf16_t* __restrict__ out, int H, int G,
        int dim, int vdim, float scale_log2, int window, int keep_first, float lam, float eps,
        float out_scale) {
    extern __shared__ float da_lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nw = blockDim.x >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int g = blockIdx.y, seq = blockIdx.z;
    const int Rg = H / G;
    const int q0 = q_start[seq];
    const int rows_total = (q_start[seq + 1] - q0) * Rg;
    const int row0 = SPLIT ? 0 : (blockIdx.x * nw + wave) * 16;
    if (!SPLIT && row0 >= rows_total) return;          // no barrier follows without SPLIT
    const int spos = start_pos[seq];
    const int* pages = table + (size_t)seq * table_stride;
    const bool row_ok = row0 + li < rows_total;
    const int row = row_ok ? row0 + li : rows_total - 1;
    const int tok = row / Rg, head = g * Rg + row % Rg;
    const int pos = spos + tok;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

    DAFrag qf[DA_MAPS][DK];
    const bf16_t* qrow = q + ((size_t)(q0 + tok) * H + head) * DA_MAPS * dim;
#pragma unroll
    for (int a = 0; a < DA_MAPS; ++a)
#pragma unroll
        for (int kk = 0; kk < DK; ++kk) {
            const int d = kk * 32 + lg * 8;
            qf[a][kk].u = d < dim ? *(const uint4*)(qrow + a * dim + d) : make_uint4(0, 0, 0, 0);
        }

    // blocks of 32 keys that some row of this wave sees
    const int last_row = row0 + 15 < rows_total ? row0 + 15 : rows_total - 1;
    const int p_min = spos + row0 / Rg, p_max = spos + last_row / Rg;
    const int win_lo = (window > 0 && p_min - window + 1 > 0) ? p_min - window + 1 : 0;
    const int n_first = keep_first < win_lo ? keep_first : win_lo;
    const int a_end = (n_first + 31) / 32;
    const int b_begin = win_lo / 32 > a_end ? win_lo / 32 : a_end;
    const int n_blocks = a_end + (p_max / 32 + 1 - b_begin);
    const int vtiles = vdim / 16;

    da_floatx4_t o[DA_MAPS][DVT];
    float m[DA_MAPS], l[DA_MAPS];
#pragma unroll
    for (int a = 0; a < DA_MAPS; ++a) {
        m[a] = -INFINITY;
        l[a] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DVT; ++dt) o[a][dt] = da_floatx4_t{0.f, 0.f, 0.f, 0.f};
    }

    for (int it = SPLIT ? wave : 0; it < n_blocks; it += SPLIT ? nw : 1) {
        const int bi = it < a_end ? it : b_begin + (it - a_end);
        const int page = pages[bi >> 1];
        const bf16_t* kb = k_pages + cache_region(page, g, G, DA_MAPS * dim) + (size_t)(bi & 1) * 32 * dim;
        const bf16_t* vb = v_pages + cache_region(page, g, G, vdim) + (size_t)(bi & 1) * 512;
        // slots beyond the newest key this wave reads may hold no data yet: their weight is
        // zero, and so must their value be (whatever bits lie there)
        uint4 keep;
        {
            const int key0 = bi * 32 + lg * 8;
            auto two = [&](int e) {
                return (key0 + e <= p_max ? 0xffffu : 0u) | (key0 + e + 1 <= p_max ? 0xffff0000u : 0u);
            };
            keep = make_uint4(two(0), two(2), two(4), two(6));
        }
        DAFrag pf[DA_MAPS];
        float alpha[DA_MAPS];
#pragma unroll
        for (int a = 0; a < DA_MAPS; ++a) {
            da_floatx4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < DK; ++kk) {
                const int chunk = kk * 4 + lg;
                const int c = chunk * 8 < dim ? chunk : 0;
                const bf16_t* src = kb + (size_t)a * GFA_PAGE * dim + c * 256 + li * 8;
                DAFrag k0, k1;
                k0.u = *(const uint4*)src;
                k1.u = *(const uint4*)(src + 128);
                s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0.v, qf[a][kk].v, s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1.v, qf[a][kk].v, s1, 0, 0, 0);
            }
            float sv[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
            float mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int j = bi * 32 + lg * 8 + e;
                const bool see = j <= pos && (j >= lo || j < keep_first);
                sv[e] = see ? sv[e] * scale_log2 : -INFINITY;
                mx = fmaxf(mx, sv[e]);
            }
            mx = da_max_lane_groups(mx);
            const float m_new = fmaxf(m[a], mx);
            const float m_use = m_new == -INFINITY ? 0.f : m_new;
            alpha[a] = exp2f(m[a] - m_use);
            float ps = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float p = exp2f(sv[e] - m_use);
                ps += p;
                pf[a].e[e] = float_to_bf16(p);
            }
            l[a] = l[a] * alpha[a] + ps;
            m[a] = m_new;
        }
#pragma unroll
        for (int dt = 0; dt < DVT; ++dt) {
            const int dtc = dt < vtiles ? dt : vtiles - 1;
            DAFrag vf;
            vf.u = *(const uint4*)(vb + (size_t)dtc * 1024 + lg * 128 + li * 8);
            vf.u.x &= keep.x;
            vf.u.y &= keep.y;
            vf.u.z &= keep.z;
            vf.u.w &= keep.w;
#pragma unroll
            for (int a = 0; a < DA_MAPS; ++a) {
                o[a][dt] *= alpha[a];
                o[a][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf[a].v, o[a][dt], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int a = 0; a < DA_MAPS; ++a) l[a] = da_sum_lane_groups(l[a]);

    if (SPLIT) {
        // per wave: m and l of 16 rows and two maps, then O [map][dim][row < rows_total]
        const int per_wave = 64 + DA_MAPS * vdim * rows_total;
        float* mine = da_lds + (size_t)wave * per_wave;
        if (lg == 0) {
#pragma unroll
            for (int a = 0; a < DA_MAPS; ++a) {
                mine[a * 32 + li] = m[a];
                mine[a * 32 + 16 + li] = l[a];
            }
        }
        if (row_ok) {
#pragma unroll
            for (int a = 0; a < DA_MAPS; ++a)
#pragma unroll
                for (int dt = 0; dt < DVT; ++dt)
                    if (dt < vtiles)
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            mine[64 + ((size_t)a * vdim + dt * 16 + lg * 4 + j) * rows_total + li] = o[a][dt][j];
        }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int a = 0; a < DA_MAPS; ++a) {
            float M = -INFINITY;
            for (int w = 0; w < nw; ++w) M = fmaxf(M, da_lds[(size_t)w * per_wave + a * 32 + li]);
            float L = 0.f;
#pragma unroll
            for (int dt = 0; dt < DVT; ++dt) o[a][dt] = da_floatx4_t{0.f, 0.f, 0.f, 0.f};
            for (int w = 0; w < nw; ++w) {
                const float* theirs = da_lds + (size_t)w * per_wave;
                const float mw = theirs[a * 32 + li];
                const float f = mw == -INFINITY ? 0.f : exp2f(mw - M);
                L += theirs[a * 32 + 16 + li] * f;
                if (row_ok) {
#pragma unroll
                    for (int dt = 0; dt < DVT; ++dt)
                        if (dt < vtiles)
#pragma unroll
                            for (int j = 0; j < 4; ++j)
                                o[a][dt][j] += f * theirs[64 + ((size_t)a * vdim + dt * 16 + lg * 4 + j) * rows_total + li];
                }
            }
            l[a] = L;
        }
    }

    // a1 - lam a2, the head's norm, the gate
    const float inv0 = 1.f / l[0], inv1 = lam / l[1];
    float ss = 0.f;
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt)
        if (dt < vtiles)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float v = o[0][dt][j] * inv0 - o[1][dt][j] * inv1;
                o[0][dt][j] = v;
                ss = fmaf(v, v, ss);
            }
    ss = da_sum_lane_groups(ss);
    float f = rsqrtf(ss / (float)vdim + eps) * out_scale;
    if (gate) f *= 1.f / (1.f + expf(-gate[(size_t)(q0 + tok) * gate_stride + head]));
    if (!row_ok) return;
    bf16_t* orow = out + ((size_t)(q0 + tok) * H + head) * vdim;
#pragma unroll
    for (int dt = 0; dt < DVT; ++dt)
        if (dt < vtiles) {
            union { uint2 u; bf16_t e[4]; } w;
#pragma unroll
            for (int j = 0; j < 4; ++j) w.e[j] = float_to_bf16(o[0][dt][j] * f);
            *(uint2*)(orow + dt * 16 + lg * 4) = w.u;
        }
}

// rows_max: the most rows (tokens times heads of a group) any sequence of the step brings.
// split_waves > 0: one token per sequence, that many waves share a tile's blocks.
extern "C" int gfa_da_attention_mfma(const void* q, const void* k_pages, const void* v_pages,
                                     const float* gate, int gate_stride, const int* q_start,
                                     const int* start_pos, const int* table, int table_stride,
                                     void* out, int n_seqs, int rows_max, int H, int G, int dim,
                                     int vdim, float scale, int window, int keep_first, float lam,
                                     float eps, float out_scale, int split_waves,
                                     hipStream_t stream) {
    if (n_seqs <= 0 || rows_max <= 0) return 0;
    if (dim % 8 || dim > 128 || vdim % 16 || vdim > 256 || n_seqs > 65535 || G > 65535 || H % G)
        return (int)hipErrorInvalidValue;
    const int Rg = H / G;
    if (split_waves > 0 && (Rg > 16 || rows_max != Rg || split_waves > 8)) return (int)hipErrorInvalidValue;
    const float scale_log2 = scale * 1.4426950408889634f;
    const int dk = dim <= 32 ? 1 : dim <= 64 ? 2 : 4, dvt = vdim <= 64 ? 4 : vdim <= 128 ? 8 : 16;
    const dim3 grid(split_waves > 0 ? 1 : (rows_max + 63) / 64, G, n_seqs);
    const int threads = split_waves > 0 ? split_waves * 64 : 256;
    const size_t shmem = split_waves > 0 ? (size_t)split_waves * (64 + DA_MAPS * vdim * Rg) * sizeof(float) : 0;
    if (shmem > 64 * 1024) return (int)hipErrorInvalidValue;
#define DA_LAUNCH(K_, V_, S_) da_attention_mfma_kernel<K_, V_, S_><<<grid, threads, shmem, stream>>>( \
        (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, gate, \
        gate_stride, q_start, start_pos, table, table_stride, (bf16_t*)out, H, G, dim, vdim, \
        scale_log2, window, keep_first, lam, eps, out_scale)
#define DA_PICK_V(K_, S_) do { if (dvt == 4) DA_LAUNCH(K_, 4, S_); else if (dvt == 8) DA_LAUNCH(K_, 8, S_); \
        else DA_LAUNCH(K_, 16, S_); } while (0)
#define DA_PICK(S_) do { if (dk == 1) DA_PICK_V(1, S_); else if (dk == 2) DA_PICK_V(2, S_); \
        else DA_PICK_V(4, S_); } while (0)
    if (split_waves > 0) DA_PICK(true);
    else DA_PICK(false);
#undef DA_PICK
#undef DA_PICK_V
#undef DA_LAUNCH
    return GFA_LAUNCH_RESULT();
}
