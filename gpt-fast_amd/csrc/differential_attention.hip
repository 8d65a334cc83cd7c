// Differential attention over the paged cache: plain kernels.
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
// Rotation of q and k and the cache write.  proj [N, row_width] holds per token
// q [H][2][dim] at q_off, k [G][2][dim] at k_off, v [G][vdim] at v_off.  Pairs (2i, 2i+1) of
// the first `rot` elements of every map are rotated by pos * freqs[i], angle, cos and sin in
// float; the rest passes through.  q goes to q_out [N, H, 2, dim].
template <typename T>
__global__ __launch_bounds__(256) void da_rope_store_kernel(
        const T* __restrict__ proj, int row_width, int q_off, int k_off, int v_off,
        T* __restrict__ q_out, T* __restrict__ k_pages, T* __restrict__ v_pages,
        const float* __restrict__ freqs, const int* __restrict__ tok_seq,
        const int* __restrict__ tok_pos, const int* __restrict__ table, int table_stride, int H,
        int G, int dim, int vdim, int rot) {
    extern __shared__ float cs[];                          // [rot / 2][2]
    const int n = blockIdx.x;
    const int pos = tok_pos[n];
    for (int i = threadIdx.x; i < rot / 2; i += 256)
        sincosf((float)pos * freqs[i], &cs[2 * i + 1], &cs[2 * i]);
    __syncthreads();
    const T* row = proj + (size_t)n * row_width;
    int page = 0;
    if (k_pages) page = table[(size_t)tok_seq[n] * table_stride + pos / GFA_PAGE];
    const int off = pos % GFA_PAGE;
    const int q_elems = H * DA_MAPS * dim, k_elems = G * DA_MAPS * dim, v_elems = G * vdim;
    for (int e = threadIdx.x; e < q_elems + k_elems + v_elems; e += 256) {
        if (e < q_elems + k_elems) {
            const bool is_q = e < q_elems;
            const int ee = is_q ? e : e - q_elems;
            const int mh = ee / dim, d = ee - mh * dim;    // mh = head * 2 + map
            const T* src = row + (is_q ? q_off : k_off) + (size_t)mh * dim;
            float val;
            if (d < rot) {
                const int i = d >> 1;
                const float u = load_as_float(src + 2 * i), w = load_as_float(src + 2 * i + 1);
                const float c = cs[2 * i], s = cs[2 * i + 1];
                val = (d & 1) ? w * c + u * s : u * c - w * s;
            } else {
                val = load_as_float(src + d);
            }
            if (is_q) {
                store_from_float(q_out + (size_t)n * q_elems + ee, val);
            } else if (k_pages) {
                const int g = mh / DA_MAPS, map = mh % DA_MAPS;
                T* dst = k_pages + cache_region(page, g, G, DA_MAPS * dim) + (size_t)map * GFA_PAGE * dim;
                store_from_float(dst + key_offset(off, d, dim), val);
            }
        } else if (v_pages) {
            const int ev = e - q_elems - k_elems;
            const int g = ev / vdim, d = ev - g * vdim;
            v_pages[cache_region(page, g, G, vdim) + value_offset(d, off, vdim)] = row[v_off + ev];
        }
    }
}

extern "C" int gfa_da_rope_store(const void* proj, int row_width, int q_off, int k_off, int v_off,
                                 void* q_out, void* k_pages, void* v_pages, const float* freqs,
                                 const int* tok_seq, const int* tok_pos, const int* table,
                                 int table_stride, int n_tokens, int H, int G, int dim, int vdim,
                                 int rot, int is_bf16, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    const size_t shmem = (size_t)(rot > 0 ? rot : 2) * sizeof(float);
    if (is_bf16)
        da_rope_store_kernel<bf16_t><<<n_tokens, 256, shmem, stream>>>(
            (const bf16_t*)proj, row_width, q_off, k_off, v_off, (bf16_t*)q_out, (bf16_t*)k_pages,
            (bf16_t*)v_pages, freqs, tok_seq, tok_pos, table, table_stride, H, G, dim, vdim, rot);
    else
        da_rope_store_kernel<float><<<n_tokens, 256, shmem, stream>>>(
            (const float*)proj, row_width, q_off, k_off, v_off, (float*)q_out, (float*)k_pages,
            (float*)v_pages, freqs, tok_seq, tok_pos, table, table_stride, H, G, dim, vdim, rot);
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
        const T* __restrict__ gate, int gate_stride, const int* __restrict__ tok_seq,
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
    if (gate) f *= 1.f / (1.f + expf(-load_as_float(gate + (size_t)n * gate_stride + h)));
    T* orow = out + ((size_t)n * H + h) * vdim;
#pragma unroll
    for (int i = 0; i < DA_MAX_PER_THREAD; ++i) {
        const int d = threadIdx.x + i * DA_THREADS;
        if (d < vdim) store_from_float(orow + d, o[i] * f);
    }
}

extern "C" int gfa_da_attention_generic(const void* q, const void* k_pages, const void* v_pages,
                                        const void* gate, int gate_stride, const int* tok_seq,
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
            (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, (const bf16_t*)gate,
            gate_stride, tok_seq, tok_pos, table, table_stride, (bf16_t*)out, H, G, dim, vdim,
            scale, window, keep_first, lam, eps, out_scale);
    else
        da_attention_generic_kernel<float><<<grid, DA_THREADS, shmem, stream>>>(
            (const float*)q, (const float*)k_pages, (const float*)v_pages, (const float*)gate,
            gate_stride, tok_seq, tok_pos, table, table_stride, (float*)out, H, G, dim, vdim,
            scale, window, keep_first, lam, eps, out_scale);
    return GFA_LAUNCH_RESULT();
}
