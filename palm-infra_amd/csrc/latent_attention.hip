// Attention whose keys and values are made from one compressed row per position.
//
// For every position the cache keeps a row [c | r]: c the normed latent (kv_rank values), r one rotated key part
// (rot_dim values) shared by all heads.  Head h's key is [U_k,h c | r] and its value U_v,h c, so with
//
//   a_h = U_k,h^T q_plain,h          (the query taken through the key matrix once: kv_rank values)
//
// a score is (a_h . c_j + q_rot,h . r_j) * scale and the head's output U_v,h (sum_j p_j c_j): keys and values are never
// expanded, all heads read the same rows.  Scores, softmax and sums are 32-bit.
//
//   latent_prep        the joined down projection's rows -> the normed query latent; the normed latent and the
//                      rotated key part into the position's cache row (and, where the caller keeps one for the prompt
//                      kernel of latent_attention_mfma.hip, the latent into a bfloat16 copy with the positions innermost)
//   latent_query       q rows -> [a_h | rotated q_rot,h] per head, 32-bit
//   latent_attention   softmax over the visible rows (causal, optional window), o_lat,h = sum_j p_j c_j, 32-bit
//   latent_output      head h: sigmoid(gate_h) * U_v,h o_lat,h
#include "common.h"

constexpr int LAT_THREADS = 256;

__device__ inline float lat_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

// Eight neighbouring values of a row as floats: one 16-byte read of bfloat16, two of float32.
__device__ inline void lat_load8(const bf16_t* p, float (&v)[8]) {
    const uint4 t = *reinterpret_cast<const uint4*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    v[4] = __uint_as_float(t.z << 16); v[5] = __uint_as_float(t.z & 0xffff0000u);
    v[6] = __uint_as_float(t.w << 16); v[7] = __uint_as_float(t.w & 0xffff0000u);
}
__device__ inline void lat_load8(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// One block per token.  down: [n, stride] holding the query latent at 0 (q_rank), the key/value latent at kv_off
// (kv_rank) and the key part to rotate behind it (rot_dim).  rows_cache: [pages, PAGE_TOKENS, kv_rank + rot_dim].
template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void latent_prep_kernel(
    const T* __restrict__ down, int stride, int q_rank, int kv_off, int kv_rank, int rot_dim, const float* __restrict__ q_norm_w,
    const float* __restrict__ kv_norm_w, float eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ tok_slot, const int* __restrict__ block_table, int max_pages,
    T* __restrict__ rows_cache, int write_cache, T* __restrict__ cq, bf16_t* __restrict__ rows_t,
    const int* __restrict__ block_table_t) {
    __shared__ float scratch[16];
    const size_t row = blockIdx.x;
    const T* dr = down + row * stride;
    float ss = 0.f;
    for (int d = threadIdx.x; d < q_rank; d += LAT_THREADS) {
        const float v = to_float(dr[d]);
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, scratch);
    const float qi = 1.0f / sqrtf(ss / (float)q_rank + eps);
    for (int d = threadIdx.x; d < q_rank; d += LAT_THREADS) cq[row * q_rank + d] = from_float<T>((to_float(dr[d]) * qi) * q_norm_w[d]);
    if (!write_cache) return;
    float sk = 0.f;
    for (int d = threadIdx.x; d < kv_rank; d += LAT_THREADS) {
        const float v = to_float(dr[kv_off + d]);
        sk = fmaf(v, v, sk);
    }
    sk = block_sum(sk, scratch);
    const float ki = 1.0f / sqrtf(sk / (float)kv_rank + eps);
    const int pos = positions[row];
    const int page = block_table[(size_t)tok_slot[row] * max_pages + pos / PAGE_TOKENS];
    T* cr = rows_cache + ((size_t)page * PAGE_TOKENS + pos % PAGE_TOKENS) * (kv_rank + rot_dim);
    for (int d = threadIdx.x; d < kv_rank; d += LAT_THREADS) cr[d] = from_float<T>((to_float(dr[kv_off + d]) * ki) * kv_norm_w[d]);
    if (rows_t) {                                   // the latent once more, positions innermost: [pages, kv_rank, PAGE_TOKENS]
        const int page_t = block_table_t[(size_t)tok_slot[row] * max_pages + pos / PAGE_TOKENS];
        bf16_t* ct = rows_t + (size_t)page_t * kv_rank * PAGE_TOKENS + pos % PAGE_TOKENS;
        for (int d = threadIdx.x; d < kv_rank; d += LAT_THREADS)
            ct[(size_t)d * PAGE_TOKENS] = f32_to_bf16((to_float(dr[kv_off + d]) * ki) * kv_norm_w[d]);
    }
    const int half = rot_dim / 2;
    for (int i = threadIdx.x; i < half; i += LAT_THREADS) {
        const float c = cos_t[row * half + i], s = sin_t[row * half + i];
        const float a = to_float(dr[kv_off + kv_rank + i]), b = to_float(dr[kv_off + kv_rank + half + i]);
        cr[kv_rank + i] = from_float<T>(a * c - b * s);
        cr[kv_rank + half + i] = from_float<T>(b * c + a * s);
    }
}

// One block per (tile of LQ_TILE tokens, head, run of LQ_COLS latent columns).  q: [n, heads * (dim + rot_dim)], a head's
// plain part first.  uk: [heads * dim, kv_rank].  qa: float32 [n, heads, kv_rank + rot_dim].  A thread owns a column of
// the key matrix and walks down it (neighbouring threads read neighbouring values); the first run's block also rotates.
constexpr int LQ_TILE = 8;
constexpr int LQ_COLS = 64;
constexpr int LQ_MAX_DIM = 512;

template <typename T, typename TW>
__global__ __launch_bounds__(LQ_COLS) void latent_query_kernel(
    const T* __restrict__ q, const TW* __restrict__ uk, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    int n_tokens, int heads, int dim, int rot_dim, int kv_rank, float* __restrict__ qa) {
    __shared__ float q_s[LQ_TILE][LQ_MAX_DIM];
    const int t0 = blockIdx.x * LQ_TILE, h = blockIdx.y;
    const int tt = min(LQ_TILE, n_tokens - t0);
    const int hd = dim + rot_dim, dk = kv_rank + rot_dim, half = rot_dim / 2;
    for (int idx = threadIdx.x; idx < LQ_TILE * dim; idx += LQ_COLS) {
        const int ti = idx / dim, d = idx % dim;
        q_s[ti][d] = ti < tt ? to_float(q[((size_t)(t0 + ti) * heads + h) * hd + d]) : 0.f;
    }
    if (blockIdx.z == 0) {
        for (int idx = threadIdx.x; idx < tt * half; idx += LQ_COLS) {
            const int ti = idx / half, i = idx % half;
            const size_t row = t0 + ti;
            const T* qr = q + (row * heads + h) * hd + dim;
            const float c = cos_t[row * half + i], s = sin_t[row * half + i];
            const float a = to_float(qr[i]), b = to_float(qr[half + i]);
            float* o = qa + (row * heads + h) * dk + kv_rank;
            o[i] = a * c - b * s;
            o[half + i] = b * c + a * s;
        }
    }
    __syncthreads();
    const TW* w = uk + (size_t)h * dim * kv_rank;
    const int r = blockIdx.z * LQ_COLS + threadIdx.x;
    if (r >= kv_rank) return;
    float acc[LQ_TILE];
#pragma unroll
    for (int ti = 0; ti < LQ_TILE; ++ti) acc[ti] = 0.f;
#pragma unroll 4
    for (int d = 0; d < dim; ++d) {
        const float wv = to_float(w[(size_t)d * kv_rank + r]);
#pragma unroll
        for (int ti = 0; ti < LQ_TILE; ++ti) acc[ti] = fmaf(q_s[ti][d], wv, acc[ti]);
    }
#pragma unroll
    for (int ti = 0; ti < LQ_TILE; ++ti)
        if (ti < tt) qa[((size_t)(t0 + ti) * heads + h) * dk + r] = acc[ti];
}

// One block of LA_WAVES waves per (query, group of HG heads).  A wave takes every LA_WAVES-th page of the key range;
// inside a page each lane scores one row against the group's HG queries (the row is read once for all of them), the
// wave keeps a running (max, sum, output) per head with the output's kv_rank values spread over the lanes, and the
// waves' partial results are merged at the end in a fixed order.
constexpr int LA_WAVES = 8;
constexpr int LA_MAX_RANK = 1024;                 // kv_rank: what a lane accumulates, 64 values apart
constexpr int LA_ACC = LA_MAX_RANK / WAVE;
constexpr int LA_MAX_DK = 1280;                   // kv_rank + rot_dim

template <typename T, int HG, int ACC>
__global__ __launch_bounds__(LA_WAVES * WAVE) void latent_attention_kernel(
    const float* __restrict__ qa, const T* __restrict__ rows_cache, const int* __restrict__ block_table, int max_pages,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_start, const int* __restrict__ seq_new,
    const int* __restrict__ cu_new, int heads, int kv_rank, int rot_dim, float scale, int window, float* __restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int dk = kv_rank + rot_dim;
    float* q_s = lds;                                  // [HG][dk]
    float* acc_s = lds + HG * dk;                      // [HG][kv_rank]
    __shared__ float m_s[LA_WAVES][HG], l_s[LA_WAVES][HG];

    const int qi = blockIdx.x, h0 = blockIdx.y * HG, b = blockIdx.z;
    if (qi >= seq_new[b]) return;
    const int t = cu_new[b] + qi;
    const int pos = seq_start[b] + qi;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;
    const int hg = min(HG, heads - h0);

    for (int idx = threadIdx.x; idx < HG * dk; idx += blockDim.x) {
        const int g = idx / dk, d = idx % dk;
        q_s[idx] = g < hg ? qa[((size_t)t * heads + h0 + g) * dk + d] : 0.f;
    }
    for (int idx = threadIdx.x; idx < HG * kv_rank; idx += blockDim.x) acc_s[idx] = 0.f;
    __syncthreads();

    float m[HG], l[HG], acc[HG][ACC];
#pragma unroll
    for (int g = 0; g < HG; ++g) {
        m[g] = -INFINITY;
        l[g] = 0.f;
#pragma unroll
        for (int i = 0; i < ACC; ++i) acc[g][i] = 0.f;
    }
    for (int pg = lo / PAGE_TOKENS + wave; pg <= pos / PAGE_TOKENS; pg += LA_WAVES) {
        const T* pp = rows_cache + (size_t)pages[pg] * PAGE_TOKENS * dk;
        const int j = pg * PAGE_TOKENS + lane;
        const bool seen = j >= lo && j <= pos;
        const T* kr = pp + (size_t)lane * dk;
        float s[HG];
#pragma unroll
        for (int g = 0; g < HG; ++g) s[g] = 0.f;
        if (dk % 8 == 0) {                          // rows start on 16 bytes: eight values a read, the queries four a read
            for (int d = 0; d < dk; d += 8) {
                float kd[8];
                lat_load8(kr + d, kd);
#pragma unroll
                for (int g = 0; g < HG; ++g) {
                    const float4 qa0 = *reinterpret_cast<const float4*>(q_s + g * dk + d);
                    const float4 qa1 = *reinterpret_cast<const float4*>(q_s + g * dk + d + 4);
                    s[g] = fmaf(qa0.x, kd[0], s[g]); s[g] = fmaf(qa0.y, kd[1], s[g]);
                    s[g] = fmaf(qa0.z, kd[2], s[g]); s[g] = fmaf(qa0.w, kd[3], s[g]);
                    s[g] = fmaf(qa1.x, kd[4], s[g]); s[g] = fmaf(qa1.y, kd[5], s[g]);
                    s[g] = fmaf(qa1.z, kd[6], s[g]); s[g] = fmaf(qa1.w, kd[7], s[g]);
                }
            }
        } else {
            for (int d = 0; d < dk; ++d) {
                const float kd = to_float(kr[d]);
#pragma unroll
                for (int g = 0; g < HG; ++g) s[g] = fmaf(q_s[g * dk + d], kd, s[g]);
            }
        }
        float p[HG];
#pragma unroll
        for (int g = 0; g < HG; ++g) {
            const float sg = seen ? s[g] * scale : -INFINITY;           // (a row of a page handed out uncleared may hold anything)
            const float m_new = fmaxf(m[g], wave_max(sg));
            const float alpha = expf(m[g] - m_new);                     // m = -inf at the first page: exp(-inf) = 0
            p[g] = expf(sg - m_new);                                    // an invisible row: exp(-inf) = 0
            l[g] = l[g] * alpha + wave_sum(p[g]);
            m[g] = m_new;
#pragma unroll
            for (int i = 0; i < ACC; ++i) acc[g][i] *= alpha;
        }
        const int j_first = max(lo, pg * PAGE_TOKENS) - pg * PAGE_TOKENS;
        const int j_last = min(pos, pg * PAGE_TOKENS + PAGE_TOKENS - 1) - pg * PAGE_TOKENS;
        for (int jj = j_first; jj <= j_last; ++jj) {
            const T* vr = pp + (size_t)jj * dk;
            float c[ACC];
#pragma unroll
            for (int i = 0; i < ACC; ++i) c[i] = to_float(vr[min(lane + i * WAVE, kv_rank - 1)]);
#pragma unroll
            for (int g = 0; g < HG; ++g) {
                const float pj = __shfl(p[g], jj, WAVE);                // jj is the same in every lane
#pragma unroll
                for (int i = 0; i < ACC; ++i) acc[g][i] = fmaf(pj, c[i], acc[g][i]);
            }
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int g = 0; g < HG; ++g) { m_s[wave][g] = m[g]; l_s[wave][g] = l[g]; }
    }
    __syncthreads();
    float f[HG], l_all[HG];
#pragma unroll
    for (int g = 0; g < HG; ++g) {
        float m_all = -INFINITY;
        for (int w = 0; w < LA_WAVES; ++w) m_all = fmaxf(m_all, m_s[w][g]);
        float sum = 0.f;
        for (int w = 0; w < LA_WAVES; ++w) sum += l_s[w][g] * expf(m_s[w][g] - m_all);      // a wave without pages: l = 0
        l_all[g] = sum;
        f[g] = expf(m[g] - m_all);                                                          // m = -inf: 0 (m_all is finite: the
    }                                                                                       // query sees at least itself)
    for (int w = 0; w < LA_WAVES; ++w) {            // the waves add their parts one after the other: a fixed order
        if (wave == w) {
#pragma unroll
            for (int g = 0; g < HG; ++g)
#pragma unroll
                for (int i = 0; i < ACC; ++i) {
                    const int d = lane + i * WAVE;
                    if (d < kv_rank) acc_s[g * kv_rank + d] += acc[g][i] * f[g];
                }
        }
        __syncthreads();
    }
    for (int idx = threadIdx.x; idx < hg * kv_rank; idx += blockDim.x) {
        const int g = idx / kv_rank, d = idx % kv_rank;
        float lg = 0.f;
#pragma unroll
        for (int k = 0; k < HG; ++k) lg = k == g ? l_all[k] : lg;
        out[((size_t)t * heads + h0 + g) * kv_rank + d] = acc_s[idx] / lg;
    }
}

// One block per (tile of LO_TILE tokens, head, group of `rows` output rows):
// out[t, h, j] = sigmoid(gate[t, h]) * sum_r uv[h * vdim + j, r] * o_lat[t, h, r].  A wave takes a row j at a time.  A
// step of few tokens cuts a head's rows into groups of 16 so that blocks enough run; a prompt's blocks take all rows of a
// head (the tile's sums are brought into LDS once).
constexpr int LO_TILE = 8;
constexpr int LO_FEW_ROWS = 16;

template <typename T, typename TW>
__global__ __launch_bounds__(LAT_THREADS) void latent_output_kernel(
    const float* __restrict__ o_lat, const TW* __restrict__ uv, const T* __restrict__ gate, int gate_stride, int n_tokens,
    int heads, int kv_rank, int vdim, int rows, T* __restrict__ out) {
    extern __shared__ float lds[];                    // [LO_TILE][kv_rank]
    const int t0 = blockIdx.x * LO_TILE, h = blockIdx.y, j0 = blockIdx.z * rows;
    const int tt = min(LO_TILE, n_tokens - t0);
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = LAT_THREADS / WAVE;
    for (int idx = threadIdx.x; idx < LO_TILE * kv_rank; idx += LAT_THREADS) {
        const int ti = idx / kv_rank, r = idx % kv_rank;
        lds[idx] = ti < tt ? o_lat[((size_t)(t0 + ti) * heads + h) * kv_rank + r] : 0.f;
    }
    __syncthreads();
    for (int j = j0 + wave; j < min(vdim, j0 + rows); j += n_waves) {
        const TW* wr = uv + ((size_t)h * vdim + j) * kv_rank;
        float acc[LO_TILE];
#pragma unroll
        for (int ti = 0; ti < LO_TILE; ++ti) acc[ti] = 0.f;
        if (kv_rank % 8 == 0 && kv_rank >= WAVE * 8) {            // (a shorter row: a value a lane keeps all lanes busy)
            for (int r = lane * 8; r < kv_rank; r += WAVE * 8) {
                float wv[8];
                lat_load8(wr + r, wv);
#pragma unroll
                for (int ti = 0; ti < LO_TILE; ++ti)
#pragma unroll
                    for (int i = 0; i < 8; ++i) acc[ti] = fmaf(lds[ti * kv_rank + r + i], wv[i], acc[ti]);
            }
        } else {
            for (int r = lane; r < kv_rank; r += WAVE) {
                const float wv = to_float(wr[r]);
#pragma unroll
                for (int ti = 0; ti < LO_TILE; ++ti) acc[ti] = fmaf(lds[ti * kv_rank + r], wv, acc[ti]);
            }
        }
#pragma unroll
        for (int ti = 0; ti < LO_TILE; ++ti) {
            const float total = wave_sum(acc[ti]);
            if (lane == 0 && ti < tt) {
                const size_t row = t0 + ti;
                const float g = gate ? lat_sigmoid(to_float(gate[row * gate_stride + h])) : 1.0f;
                out[(row * heads + h) * vdim + j] = from_float<T>(total * g);
            }
        }
    }
}

PALM_API int palm_latent_prep(hipStream_t stream, const void* down, int dtype, int stride, int q_rank, int kv_off, int kv_rank,
                              int rot_dim, const float* q_norm_w, const float* kv_norm_w, float eps, const float* cos_t,
                              const float* sin_t, const int* positions, const int* tok_slot, const int* block_table, int max_pages,
                              void* rows_cache, int write_cache, void* cq, int n_tokens, void* rows_t, const int* block_table_t) {
    PALM_CHECK(n_tokens >= 0 && q_rank > 0 && kv_rank > 0 && rot_dim >= 0 && rot_dim % 2 == 0, "latent_prep: n=%d q_rank=%d kv_rank=%d rot_dim=%d",
               n_tokens, q_rank, kv_rank, rot_dim);
    PALM_CHECK(stride >= kv_off + kv_rank + rot_dim && kv_off >= q_rank, "latent_prep: rows of %d do not hold %d + %d + %d", stride, q_rank,
               kv_rank, rot_dim);
    PALM_CHECK(rot_dim == 0 || (cos_t && sin_t), "latent_prep: a rotation needs its cos and sin rows");
    PALM_CHECK(max_pages > 0, "latent_prep: max_pages %d", max_pages);
    PALM_CHECK(!rows_t || block_table_t, "latent_prep: the transposed copy needs its page table");
    if (n_tokens == 0) return 0;
    PALM_DTYPE_SWITCH(dtype, T,
        latent_prep_kernel<T><<<n_tokens, LAT_THREADS, 0, stream>>>((const T*)down, stride, q_rank, kv_off, kv_rank, rot_dim, q_norm_w,
                                                                   kv_norm_w, eps, cos_t, sin_t, positions, tok_slot, block_table,
                                                                   max_pages, (T*)rows_cache, write_cache, (T*)cq, (bf16_t*)rows_t,
                                                                   block_table_t));
    PALM_LAUNCHED();
    return 0;
}

PALM_API int palm_latent_query(hipStream_t stream, const void* q, int dtype, const void* uk, int w_dtype, const float* cos_t,
                               const float* sin_t, int n_tokens, int heads, int dim, int rot_dim, int kv_rank, float* qa) {
    PALM_CHECK(n_tokens >= 0 && heads > 0 && dim > 0 && kv_rank > 0 && rot_dim >= 0 && rot_dim % 2 == 0,
               "latent_query: n=%d heads=%d dim=%d rot_dim=%d kv_rank=%d", n_tokens, heads, dim, rot_dim, kv_rank);
    PALM_CHECK(dim <= LQ_MAX_DIM, "latent_query: an unrotated key size of %d exceeds %d", dim, LQ_MAX_DIM);
    PALM_CHECK(rot_dim == 0 || (cos_t && sin_t), "latent_query: a rotation needs its cos and sin rows");
    PALM_CHECK(heads <= 65535, "latent_query: %d heads are more than one launch takes", heads);
    if (n_tokens == 0) return 0;
    dim3 grid((n_tokens + LQ_TILE - 1) / LQ_TILE, heads, (kv_rank + LQ_COLS - 1) / LQ_COLS);
    PALM_DTYPE_SWITCH(dtype, T, {
        PALM_DTYPE_SWITCH(w_dtype, TW, {
            latent_query_kernel<T, TW><<<grid, LQ_COLS, 0, stream>>>((const T*)q, (const TW*)uk, cos_t, sin_t, n_tokens, heads, dim,
                                                                        rot_dim, kv_rank, qa);
        });
    });
    PALM_LAUNCHED();
    return 0;
}

PALM_API int palm_latent_attention(hipStream_t stream, const float* qa, const void* rows_cache, int dtype, const int* block_table,
                                   int max_pages, const int* seq_slot, const int* seq_start, const int* seq_new, const int* cu_new,
                                   int n_seqs, int max_new, int heads, int kv_rank, int rot_dim, float scale, int window, float* out) {
    PALM_CHECK(n_seqs >= 0 && max_new >= 0 && heads > 0 && kv_rank > 0 && rot_dim >= 0, "latent_attention: seqs=%d max_new=%d heads=%d kv_rank=%d rot_dim=%d",
               n_seqs, max_new, heads, kv_rank, rot_dim);
    PALM_CHECK(kv_rank <= LA_MAX_RANK && kv_rank + rot_dim <= LA_MAX_DK, "latent_attention: a latent of %d + %d exceeds %d + %d", kv_rank, rot_dim,
               LA_MAX_RANK, LA_MAX_DK - LA_MAX_RANK);
    PALM_CHECK(window >= 0 && max_pages > 0, "latent_attention: window %d, max_pages %d", window, max_pages);
    if (n_seqs == 0 || max_new == 0) return 0;
    PALM_CHECK(n_seqs <= 65535 && heads <= 65535, "latent_attention: %d sequences / %d heads are more than one launch takes", n_seqs, heads);
    const int acc = (kv_rank + WAVE - 1) / WAVE;
    // heads a block: as many as a lane's registers take beside the outputs (acc values a head)
    const int hg = acc <= 2 ? 4 : acc <= 8 ? 2 : 1;
    dim3 grid(max_new, (heads + hg - 1) / hg, n_seqs);
    const size_t lds = (size_t)hg * (2 * kv_rank + rot_dim) * sizeof(float);
#define LA_CASE(HGV, ACCV) latent_attention_kernel<T, HGV, ACCV><<<grid, LA_WAVES * WAVE, lds, stream>>>( \
        qa, (const T*)rows_cache, block_table, max_pages, seq_slot, seq_start, seq_new, cu_new, heads, kv_rank, rot_dim, scale, window, out)
    PALM_DTYPE_SWITCH(dtype, T, {
        if (acc <= 1) LA_CASE(4, 1);
        else if (acc <= 2) LA_CASE(4, 2);
        else if (acc <= 4) LA_CASE(2, 4);
        else if (acc <= 8) LA_CASE(2, 8);
        else LA_CASE(1, 16);
    });
#undef LA_CASE
    PALM_LAUNCHED();
    return 0;
}

PALM_API int palm_latent_output(hipStream_t stream, const float* o_lat, const void* uv, int w_dtype, const void* gate, int gate_stride,
                                int dtype, int n_tokens, int heads, int kv_rank, int vdim, void* out) {
    PALM_CHECK(n_tokens >= 0 && heads > 0 && kv_rank > 0 && vdim > 0, "latent_output: n=%d heads=%d kv_rank=%d vdim=%d", n_tokens, heads,
               kv_rank, vdim);
    PALM_CHECK(kv_rank <= 1536, "latent_output: a latent of %d exceeds 1536", kv_rank);
    PALM_CHECK(heads <= 65535 && vdim <= 65535 * LO_FEW_ROWS, "latent_output: %d heads of %d are more than one launch takes", heads, vdim);
    if (n_tokens == 0) return 0;
    const int rows = n_tokens <= 64 ? LO_FEW_ROWS : vdim;
    dim3 grid((n_tokens + LO_TILE - 1) / LO_TILE, heads, (vdim + rows - 1) / rows);
    const size_t lds = (size_t)LO_TILE * kv_rank * sizeof(float);
    PALM_DTYPE_SWITCH(dtype, T, {
        PALM_DTYPE_SWITCH(w_dtype, TW, {
            latent_output_kernel<T, TW><<<grid, LAT_THREADS, lds, stream>>>(o_lat, (const TW*)uv, (const T*)gate, gate_stride, n_tokens, heads,
                                                                           kv_rank, vdim, rows, (T*)out);
        });
    });
    PALM_LAUNCHED();
    return 0;
}
