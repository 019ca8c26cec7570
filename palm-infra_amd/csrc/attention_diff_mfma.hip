// Differential attention for prompts on the matrix cores, bfloat16, compiled for one padded key size and one padded
// value size (PALM_DIFF_KK: key size / 32 rounded up; PALM_DIFF_VT: value size / 16 rounded up).
//
// A wave owns 16 queries of one head and both of the head's score maps; a block is four waves, 64 consecutive
// queries.  For every page of 64 keys the wave computes the transposed scores S^T = K Q^T (keys down, queries
// across), so that a lane's four results of a tile are four keys of ONE query: the softmax statistics of a query
// then live in the lanes of its column, and the weights are already laid out as the B operand of the second product
// O^T += V^T P^T, whose A operand reads runs of keys from the transposed value pages.  Scores leave the matrix cores
// as 32-bit sums; maximum, exponentials (base 2: the scores are scaled by scale * log2 e), sums, the combination
// a1 - lambda a2 and the unit norm are 32-bit; the
// weights are rounded to bfloat16 for the second product, whose sums are 32-bit again.
//
// Layouts as in attention_diff.hip: K [pages, 2 kv_heads, 64, dim], V [pages, kv_heads, vdim, 64].
#include "mfma.h"

#ifndef PALM_DIFF_KK
#error "compile with -DPALM_DIFF_KK=<ceil(key size / 32)> -DPALM_DIFF_VT=<ceil(value size / 16)>"
#endif

PALM_DEFINE_LAST_ERROR()

constexpr int KK = PALM_DIFF_KK;
constexpr int VT = PALM_DIFF_VT;
constexpr int DM_WAVES = 4;
constexpr int DM_QUERIES = 16 * DM_WAVES;

PALM_API int palm_attention_diff_mfma_sizes(int which) { return which == 0 ? KK * 32 : VT * 16; }

__device__ inline bf16x8 load_row8(const bf16_t* row, int col, int dim) {
    // eight values of a row from column `col`; columns beyond `dim` are zero (dim is a multiple of eight).  The read
    // itself is unconditional (of the row's last eight values where the column lies beyond it): no branch around it
    const bf16x8 v = load_bf16x8(row + min(col, dim - 8));
    return col < dim ? v : zero_bf16x8();
}

__global__ __launch_bounds__(DM_WAVES * WAVE) void attention_diff_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int* __restrict__ block_table, int max_pages, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_start, const int* __restrict__ seq_new, const int* __restrict__ cu_new,
    int heads, int kv_heads, int dim, int vdim, float scale, float lambda, float gain, float eps, bf16_t* __restrict__ out) {
    const int h = blockIdx.y, b = blockIdx.z;
    const int n_new = seq_new[b];
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int q0 = blockIdx.x * DM_QUERIES + wave * 16;           // the wave's first query among the sequence's new tokens
    if (q0 >= n_new) return;
    const int r = lane % 16, g = lane / 16;
    const int qi = min(q0 + r, n_new - 1);                        // a column beyond the run repeats the last query and stores nothing
    const bool live = q0 + r < n_new;
    const int start = seq_start[b];
    const int qpos = start + qi;
    const int last_pos = start + min(q0 + 15, n_new - 1), first_pos = start + q0;
    const float scale2 = scale * 1.4426950408889634f;
    const int kvh = h / (heads / kv_heads);
    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;

    // the queries, as the B operand: column r, eight values of group g for each step of 32 over the key size
    bf16x8 qf[2][KK];
    {
        const bf16_t* qr = q + (((size_t)cu_new[b] + qi) * heads + h) * 2 * dim;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) qf[m][kk] = load_row8(qr + m * dim, kk * 32 + g * 8, dim);
    }
    f32x4 acc[2][VT];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) acc[m][vt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mx[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};

    for (int pg = 0; pg <= last_pos / PAGE_TOKENS; ++pg) {
        const int page = pages[pg];
        bf16x8 pf[2][2];                                           // the weights as B operands: [map][32 keys]
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            const bf16_t* kp = k_cache + ((size_t)page * 2 * kv_heads + 2 * kvh + m) * PAGE_TOKENS * dim;
            f32x4 s[4];
#pragma unroll
            for (int n = 0; n < 4; ++n) {
                s[n] = f32x4{0.f, 0.f, 0.f, 0.f};
                const bf16_t* kr = kp + (size_t)(16 * n + r) * dim;
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) s[n] = mfma_16x16x32(load_row8(kr, kk * 32 + g * 8, dim), qf[m][kk], s[n]);
            }
            // lane (r, g) holds the keys 16 n + 4 g + i of query r
            // scores in units of log2: a weight is then one exp2 away
            float top = -INFINITY;
            if (pg * PAGE_TOKENS + PAGE_TOKENS - 1 > first_pos) {      // the page reaches beyond some query of the wave
#pragma unroll
                for (int n = 0; n < 4; ++n)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int j = pg * PAGE_TOKENS + 16 * n + 4 * g + i;
                        s[n][i] = j <= qpos ? s[n][i] * scale2 : -INFINITY;
                        top = fmaxf(top, s[n][i]);
                    }
            } else {
#pragma unroll
                for (int n = 0; n < 4; ++n)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s[n][i] *= scale2;
                        top = fmaxf(top, s[n][i]);
                    }
            }
            top = fmaxf(top, __shfl_xor(top, 16, WAVE));
            top = fmaxf(top, __shfl_xor(top, 32, WAVE));
            const float m_new = fmaxf(mx[m], top);                 // finite from the first page on: key 0 is visible to all
            const float alpha = exp2f(mx[m] - m_new);
            mx[m] = m_new;
            float sum = 0.f;
#pragma unroll
            for (int n = 0; n < 4; ++n)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[n][i] = exp2f(s[n][i] - m_new);
                    sum += s[n][i];
                }
            l[m] = l[m] * alpha + sum;                             // this lane's part; the groups are added at the end
#pragma unroll
            for (int vt = 0; vt < VT; ++vt)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[m][vt][i] *= alpha;
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    pf[m][half][i] = (__bf16)s[2 * half][i];
                    pf[m][half][4 + i] = (__bf16)s[2 * half + 1][i];
                }
        }
        // O^T += V^T P^T: row r of a value tile, the same eight keys of group g as the weights hold
        const bf16_t* vp = v_cache + ((size_t)page * kv_heads + kvh) * vdim * PAGE_TOKENS;
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            const int vd = 16 * vt + r;
            const bf16_t* vr = vp + (size_t)min(vd, vdim - 1) * PAGE_TOKENS;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const uint2 lo = *reinterpret_cast<const uint2*>(vr + 32 * half + 4 * g);       // row min(vd, vdim - 1): always there
                const uint2 hi = *reinterpret_cast<const uint2*>(vr + 32 * half + 16 + 4 * g);
                const uint4 both = make_uint4(lo.x, lo.y, hi.x, hi.y);
                const bf16x8 vf = vd < vdim ? __builtin_bit_cast(bf16x8, both) : zero_bf16x8();
                acc[0][vt] = mfma_16x16x32(vf, pf[0][half], acc[0][vt]);
                acc[1][vt] = mfma_16x16x32(vf, pf[1][half], acc[1][vt]);
            }
        }
    }
    // lane (r, g) holds value dimensions 16 vt + 4 g + i of query r
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        l[m] += __shfl_xor(l[m], 16, WAVE);
        l[m] += __shfl_xor(l[m], 32, WAVE);
    }
    const float f0 = 1.0f / l[0], f1 = lambda / l[1];
    float ss = 0.f;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float o = acc[0][vt][i] * f0 - acc[1][vt][i] * f1;
            acc[0][vt][i] = o;
            if (16 * vt + 4 * g + i < vdim) ss += o * o;
        }
    ss += __shfl_xor(ss, 16, WAVE);
    ss += __shfl_xor(ss, 32, WAVE);
    const float inv = gain / sqrtf(ss / (float)vdim + eps);
    if (!live) return;
    bf16_t* op = out + (((size_t)cu_new[b] + qi) * heads + h) * vdim;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt) {
        const int vd = 16 * vt + 4 * g;
        if (vd < vdim) {                                            // vdim is a multiple of four
            uint2 w;
            w.x = (uint32_t)f32_to_bf16(acc[0][vt][0] * inv).bits | ((uint32_t)f32_to_bf16(acc[0][vt][1] * inv).bits << 16);
            w.y = (uint32_t)f32_to_bf16(acc[0][vt][2] * inv).bits | ((uint32_t)f32_to_bf16(acc[0][vt][3] * inv).bits << 16);
            *reinterpret_cast<uint2*>(op + vd) = w;
        }
    }
}

PALM_API int palm_attention_diff_mfma(hipStream_t stream, const void* q, const void* k_cache, const void* v_cache,
                                      const int* block_table, int max_pages, const int* seq_slot, const int* seq_start,
                                      const int* seq_new, const int* cu_new, int n_seqs, int max_new, int heads, int kv_heads,
                                      int dim, int vdim, float scale, float lambda, float gain, float eps, void* out) {
    PALM_CHECK(n_seqs >= 0 && max_new >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0,
               "attention_diff_mfma: seqs=%d max_new=%d heads=%d kv=%d dim=%d vdim=%d", n_seqs, max_new, heads, kv_heads, dim, vdim);
    PALM_CHECK(heads % kv_heads == 0, "attention_diff_mfma: %d heads are not a multiple of %d kv heads", heads, kv_heads);
    PALM_CHECK(dim % 8 == 0 && dim <= KK * 32 && dim > (KK - 1) * 32, "attention_diff_mfma: built for key sizes %d..%d in steps of 8, not %d",
               (KK - 1) * 32 + 8, KK * 32, dim);
    PALM_CHECK(vdim % 4 == 0 && vdim <= VT * 16 && vdim > (VT - 1) * 16, "attention_diff_mfma: built for value sizes %d..%d in steps of 4, not %d",
               (VT - 1) * 16 + 4, VT * 16, vdim);
    PALM_CHECK(max_pages > 0, "attention_diff_mfma: max_pages %d", max_pages);
    if (n_seqs == 0 || max_new == 0) return 0;
    PALM_CHECK(heads <= 65535 && n_seqs <= 65535, "attention_diff_mfma: %d heads / %d sequences are more than one launch takes", heads, n_seqs);
    dim3 grid((max_new + DM_QUERIES - 1) / DM_QUERIES, heads, n_seqs);
    attention_diff_mfma_kernel<<<grid, DM_WAVES * WAVE, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, max_pages, seq_slot, seq_start, seq_new,
        cu_new, heads, kv_heads, dim, vdim, scale, lambda, gain, eps, (bf16_t*)out);
    PALM_LAUNCHED();
    return 0;
}
