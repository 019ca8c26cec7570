// Differential attention over the paged cache: every head has two score maps over one set of values,
//
//   a_m = softmax_j(scale * q_m . k_(m,j)) V,  m = 1, 2         (causal; keys j <= the query's position)
//   o   = a_1 - lambda * a_2;   out = o / sqrt(mean(o^2) + eps) * gain
//
// with per-map RMS norms of q and k (one weight vector each for all heads and maps) and no rotation.  Query head h
// reads key/value head h / (heads / kv_heads).  Keys are kept as [pages, 2 * kv_heads, 64, dim] (head g's maps are
// rows 2g and 2g + 1), values transposed as [pages, kv_heads, vdim, 64]: the layout of the other attention kernels,
// with a key size and a value size of their own.
//
// This file: the pass that norms q and k and writes the step's keys and values to their pages, and the exact
// kernel (32-bit arithmetic, any sizes), which serves the float32 mode and single tokens.
#include "common.h"

constexpr int DIFF_WAVES = 4;
constexpr int DIFF_MAX_VDIM = 512;
constexpr int DIFF_MAX_DIM = 512;
constexpr int DIFF_ACC = DIFF_MAX_VDIM / WAVE;

// One block per token.  A wave takes a row (one map of one head) at a time: sum of squares over the row, then
// q goes to q_out and k to its page.  The values are copied to their page by all threads.
template <typename T>
__global__ __launch_bounds__(256) void diff_qkv_store_kernel(
    const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ tok_slot, const int* __restrict__ positions,
    const float* __restrict__ q_w, const float* __restrict__ k_w, float eps, int heads, int kv_heads, int dim, int vdim,
    int write_cache) {
    const size_t t = blockIdx.x;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    const int q_rows = 2 * heads, k_rows = 2 * kv_heads;
    const size_t stride = (size_t)(q_rows + k_rows) * dim + (size_t)kv_heads * vdim;
    const T* row = qkv + t * stride;
    const int pos = positions[t];
    const int page = write_cache ? block_table[(size_t)tok_slot[t] * max_pages + pos / PAGE_TOKENS] : 0;
    const int at = pos % PAGE_TOKENS;
    for (int r = wave; r < q_rows + k_rows; r += n_waves) {
        const bool is_q = r < q_rows;
        if (!is_q && !write_cache) continue;
        const T* src = row + (size_t)r * dim;
        float ss = 0.f;
        for (int d = lane; d < dim; d += WAVE) { const float v = to_float(src[d]); ss += v * v; }
        ss = wave_sum(ss);
        const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
        const float* w = is_q ? q_w : k_w;
        T* dst = is_q ? q_out + (t * q_rows + r) * dim
                      : k_cache + (((size_t)page * k_rows + (r - q_rows)) * PAGE_TOKENS + at) * dim;
        for (int d = lane; d < dim; d += WAVE) dst[d] = from_float<T>((to_float(src[d]) * inv) * w[d]);
    }
    if (write_cache) {
        const T* vs = row + (size_t)(q_rows + k_rows) * dim;
        for (int i = threadIdx.x; i < kv_heads * vdim; i += blockDim.x)
            v_cache[((size_t)page * kv_heads * vdim + i) * PAGE_TOKENS + at] = vs[i];
    }
}

PALM_API int palm_diff_qkv_store(hipStream_t stream, const void* qkv, int dtype, void* q_out, void* k_cache, void* v_cache,
                                 const int* block_table, int max_pages, const int* tok_slot, const int* positions,
                                 const float* q_w, const float* k_w, float eps, int n_tokens, int heads, int kv_heads, int dim,
                                 int vdim, int write_cache) {
    PALM_CHECK(n_tokens >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "diff_qkv_store: tokens=%d heads=%d kv=%d dim=%d vdim=%d",
               n_tokens, heads, kv_heads, dim, vdim);
    PALM_CHECK(!write_cache || (k_cache && v_cache && block_table && tok_slot && max_pages > 0), "diff_qkv_store: writing needs cache, pages and slots");
    if (n_tokens == 0) return 0;
    PALM_DTYPE_SWITCH(dtype, T,
        diff_qkv_store_kernel<T><<<n_tokens, 256, 0, stream>>>((const T*)qkv, (T*)q_out, (T*)k_cache, (T*)v_cache, block_table,
                                                              max_pages, tok_slot, positions, q_w, k_w, eps, heads, kv_heads, dim,
                                                              vdim, write_cache));
    PALM_LAUNCHED();
    return 0;
}

// ---- the exact kernel ---------------------------------------------------------------------------------
// One block of four waves per (query, head, slice of the key range).  A wave takes every fourth page of the slice;
// in a page each lane scores one key for both maps (the key's row is read in pieces of 16 bytes where the key size
// allows), the wave keeps a running (max, sum, output) for each map, and the four waves' partial results are
// merged at the end.  With one slice the block then combines the maps and norms the head's output; with more (a
// decode step: few queries over long ranges) it leaves its partial result in a workspace for the merging kernel.
template <typename T> struct Pieces;
template <> struct Pieces<float> {
    static constexpr int N = 4;
    static __device__ inline void load(const float* p, float (&v)[4]) {
        const float4 t = *reinterpret_cast<const float4*>(p);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    }
};
template <> struct Pieces<bf16_t> {
    static constexpr int N = 8;
    static __device__ inline void load(const bf16_t* p, float (&v)[8]) {
        const uint4 t = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(w[i] << 16); v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
    }
};

template <typename T>
__device__ inline float dot_with_row(const float* __restrict__ q_s, const T* __restrict__ row, int dim) {
    constexpr int N = Pieces<T>::N;
    float dot = 0.f;
    if (dim % N == 0) {
        for (int d = 0; d < dim; d += N) {
            float v[N];
            Pieces<T>::load(row + d, v);
#pragma unroll
            for (int e = 0; e < N; ++e) dot = fmaf(q_s[d + e], v[e], dot);
        }
    } else {
        for (int d = 0; d < dim; ++d) dot = fmaf(q_s[d], to_float(row[d]), dot);
    }
    return dot;
}

// the per-slice record in the workspace: [2 maps][max, sum, output[vdim]]
__device__ inline size_t diff_record(int vdim) { return 2 * ((size_t)vdim + 2); }

template <typename T>
__global__ __launch_bounds__(DIFF_WAVES * WAVE) void attention_diff_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, const int* __restrict__ seq_new, const int* __restrict__ cu_new,
    int heads, int kv_heads, int dim, int vdim, float scale, float lambda, float gain, float eps, int n_slices,
    float* __restrict__ work, T* __restrict__ out) {
    extern __shared__ float smem[];
    float* q_s = smem;                                   // [2][dim]
    float* acc_s = smem + 2 * dim;                       // [2][DIFF_WAVES][vdim]
    __shared__ float m_s[2][DIFF_WAVES], l_s[2][DIFF_WAVES];
    __shared__ float scratch[16];

    const int qi = blockIdx.x / n_slices, slice = blockIdx.x % n_slices, h = blockIdx.y, b = blockIdx.z;
    if (qi >= seq_new[b]) return;
    const size_t t = (size_t)cu_new[b] + qi;
    const int pos = seq_start[b] + qi;
    const int g = h / (heads / kv_heads);
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;
    const int n_pages = pos / PAGE_TOKENS + 1;
    const int per_slice = (n_pages + n_slices - 1) / n_slices;
    const int pg_lo = slice * per_slice, pg_hi = min(n_pages, pg_lo + per_slice);

    const T* qp = q + (t * heads + h) * 2 * dim;
    for (int d = threadIdx.x; d < 2 * dim; d += blockDim.x) q_s[d] = to_float(qp[d]);
    __syncthreads();

    float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
    float acc[2][DIFF_ACC];
#pragma unroll
    for (int i = 0; i < DIFF_ACC; ++i) acc[0][i] = acc[1][i] = 0.f;

    for (int pg = pg_lo + wave; pg < pg_hi; pg += DIFF_WAVES) {
        const int page = pages[pg];
        const T* vp = v_cache + ((size_t)page * kv_heads + g) * vdim * PAGE_TOKENS;
        const int j = pg * PAGE_TOKENS + lane;
        float p[2];
#pragma unroll
        for (int mp = 0; mp < 2; ++mp) {
            float s = -INFINITY;
            if (j <= pos) {
                const T* kr = k_cache + (((size_t)page * 2 * kv_heads + 2 * g + mp) * PAGE_TOKENS + lane) * dim;
                s = dot_with_row<T>(q_s + mp * dim, kr, dim) * scale;
            }
            const float m_new = fmaxf(m[mp], wave_max(s));     // finite: the page's first key is visible
            const float alpha = expf(m[mp] - m_new);           // m = -inf at the wave's first page: exp(-inf) = 0
            p[mp] = expf(s - m_new);                           // an invisible key: exp(-inf) = 0
            l[mp] = l[mp] * alpha + wave_sum(p[mp]);
            m[mp] = m_new;
#pragma unroll
            for (int i = 0; i < DIFF_ACC; ++i) acc[mp][i] *= alpha;
        }
        // lane d (and d + 64, ..) owns a value dimension: its row of the transposed page holds the 64 keys in a run
        constexpr int N = Pieces<T>::N;
        for (int j0 = 0; j0 < PAGE_TOKENS; j0 += N) {
            float p0[N], p1[N];
#pragma unroll
            for (int e = 0; e < N; ++e) { p0[e] = __shfl(p[0], j0 + e, WAVE); p1[e] = __shfl(p[1], j0 + e, WAVE); }
#pragma unroll
            for (int i = 0; i < DIFF_ACC; ++i) {
                if (i * WAVE < vdim) {                        // the same for all lanes; a lane beyond vdim reads the last row
                    const int d = min(lane + i * WAVE, vdim - 1);
                    float v[N];
                    Pieces<T>::load(vp + (size_t)d * PAGE_TOKENS + j0, v);
#pragma unroll
                    for (int e = 0; e < N; ++e) {             // keys beyond the query have weight zero
                        acc[0][i] = fmaf(p0[e], v[e], acc[0][i]);
                        acc[1][i] = fmaf(p1[e], v[e], acc[1][i]);
                    }
                }
            }
        }
    }
    if (lane == 0) { m_s[0][wave] = m[0]; l_s[0][wave] = l[0]; m_s[1][wave] = m[1]; l_s[1][wave] = l[1]; }
#pragma unroll
    for (int i = 0; i < DIFF_ACC; ++i) {
        const int d = lane + i * WAVE;
        if (d < vdim) {
            acc_s[(0 * DIFF_WAVES + wave) * vdim + d] = acc[0][i];
            acc_s[(1 * DIFF_WAVES + wave) * vdim + d] = acc[1][i];
        }
    }
    __syncthreads();
    float f[2][DIFF_WAVES], m_all[2], l_all[2];
#pragma unroll
    for (int mp = 0; mp < 2; ++mp) {
        m_all[mp] = -INFINITY;
        for (int w = 0; w < DIFF_WAVES; ++w) m_all[mp] = fmaxf(m_all[mp], m_s[mp][w]);
        l_all[mp] = 0.f;
        for (int w = 0; w < DIFF_WAVES; ++w) {
            f[mp][w] = m_s[mp][w] == -INFINITY ? 0.f : expf(m_s[mp][w] - m_all[mp]);      // a wave (or a slice) without pages
            l_all[mp] += l_s[mp][w] * f[mp][w];
        }
    }
    if (n_slices > 1) {
        float* rec = work + ((t * heads + h) * n_slices + slice) * diff_record(vdim);
        for (int mp = 0; mp < 2; ++mp) {
            float* r = rec + mp * ((size_t)vdim + 2);
            if (threadIdx.x == 0) { r[0] = m_all[mp]; r[1] = l_all[mp]; }
            for (int d = threadIdx.x; d < vdim; d += blockDim.x) {
                float a = 0.f;
                for (int w = 0; w < DIFF_WAVES; ++w) a = fmaf(acc_s[(mp * DIFF_WAVES + w) * vdim + d], f[mp][w], a);
                r[2 + d] = a;
            }
        }
        return;
    }
    // every thread owns the dimensions d = thread, thread + 256: at most two for a value size of 512
    float o[2] = {0.f, 0.f};
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int d = threadIdx.x + i * DIFF_WAVES * WAVE;
        if (d < vdim) {
            float a0 = 0.f, a1 = 0.f;
            for (int w = 0; w < DIFF_WAVES; ++w) {
                a0 = fmaf(acc_s[(0 * DIFF_WAVES + w) * vdim + d], f[0][w], a0);
                a1 = fmaf(acc_s[(1 * DIFF_WAVES + w) * vdim + d], f[1][w], a1);
            }
            o[i] = a0 / l_all[0] - lambda * (a1 / l_all[1]);
            ss += o[i] * o[i];
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
    T* op = out + (t * heads + h) * vdim;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int d = threadIdx.x + i * DIFF_WAVES * WAVE;
        if (d < vdim) op[d] = from_float<T>((o[i] * inv) * gain);
    }
}

// The slices' partial results of one (query, head) merged, the maps combined, the head's output normed.
template <typename T>
__global__ __launch_bounds__(DIFF_WAVES * WAVE) void attention_diff_merge_kernel(
    const float* __restrict__ work, int n_slices, int vdim, float lambda, float gain, float eps, T* __restrict__ out) {
    __shared__ float scratch[16];
    const size_t th = blockIdx.x;                         // token * heads + head
    const float* rec = work + th * n_slices * diff_record(vdim);
    float top[2] = {-INFINITY, -INFINITY}, sum[2] = {0.f, 0.f};
    for (int mp = 0; mp < 2; ++mp) {
        for (int s = 0; s < n_slices; ++s) top[mp] = fmaxf(top[mp], rec[s * diff_record(vdim) + mp * ((size_t)vdim + 2)]);
        for (int s = 0; s < n_slices; ++s) {
            const float* r = rec + s * diff_record(vdim) + mp * ((size_t)vdim + 2);
            sum[mp] += r[0] == -INFINITY ? 0.f : r[1] * expf(r[0] - top[mp]);
        }
    }
    float o[2] = {0.f, 0.f};
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int d = threadIdx.x + i * DIFF_WAVES * WAVE;
        if (d < vdim) {
            float a[2] = {0.f, 0.f};
            for (int mp = 0; mp < 2; ++mp)
                for (int s = 0; s < n_slices; ++s) {
                    const float* r = rec + s * diff_record(vdim) + mp * ((size_t)vdim + 2);
                    if (r[0] != -INFINITY) a[mp] = fmaf(r[2 + d], expf(r[0] - top[mp]), a[mp]);
                }
            o[i] = a[0] / sum[0] - lambda * (a[1] / sum[1]);
            ss += o[i] * o[i];
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int d = threadIdx.x + i * DIFF_WAVES * WAVE;
        if (d < vdim) out[th * vdim + d] = from_float<T>((o[i] * inv) * gain);
    }
}

// n_slices > 1: every sequence brings one query (a decode step), and `work` holds n_tokens * heads * n_slices *
// 2 * (vdim + 2) floats; nothing in it has to be cleared.
PALM_API int palm_attention_diff(hipStream_t stream, const void* q, int dtype, const void* k_cache, const void* v_cache,
                                 const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                 const int* seq_new, const int* cu_new, int n_seqs, int max_new, int heads, int kv_heads, int dim,
                                 int vdim, float scale, float lambda, float gain, float eps, void* out, int n_slices, float* work,
                                 int n_tokens) {
    PALM_CHECK(n_seqs >= 0 && max_new >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0,
               "attention_diff: seqs=%d max_new=%d heads=%d kv=%d dim=%d vdim=%d", n_seqs, max_new, heads, kv_heads, dim, vdim);
    PALM_CHECK(heads % kv_heads == 0, "attention_diff: %d heads are not a multiple of %d kv heads", heads, kv_heads);
    PALM_CHECK(dim <= DIFF_MAX_DIM && vdim <= DIFF_MAX_VDIM, "attention_diff: key size %d / value size %d exceed %d / %d", dim, vdim,
               DIFF_MAX_DIM, DIFF_MAX_VDIM);
    PALM_CHECK(max_pages > 0, "attention_diff: max_pages %d", max_pages);
    PALM_CHECK(n_slices >= 1 && (n_slices == 1 || (work && max_new == 1 && n_tokens == n_seqs)),
               "attention_diff: %d slices need a workspace and one query a sequence", n_slices);
    if (n_seqs == 0 || max_new == 0) return 0;
    PALM_CHECK(heads <= 65535 && n_seqs <= 65535, "attention_diff: %d heads / %d sequences are more than one launch takes", heads, n_seqs);
    dim3 grid((unsigned)max_new * n_slices, heads, n_seqs);
    const size_t lds = sizeof(float) * (2 * (size_t)dim + 2 * (size_t)DIFF_WAVES * vdim);
    PALM_DTYPE_SWITCH(dtype, T, {
        attention_diff_kernel<T><<<grid, DIFF_WAVES * WAVE, lds, stream>>>(
            (const T*)q, (const T*)k_cache, (const T*)v_cache, block_table, max_pages, seq_slot, seq_start, seq_new, cu_new,
            heads, kv_heads, dim, vdim, scale, lambda, gain, eps, n_slices, work, (T*)out);
        if (n_slices > 1)
            attention_diff_merge_kernel<T><<<(unsigned)n_tokens * heads, DIFF_WAVES * WAVE, 0, stream>>>(work, n_slices, vdim, lambda, gain,
                                                                                                       eps, (T*)out);
    });
    PALM_LAUNCHED();
    return 0;
}
