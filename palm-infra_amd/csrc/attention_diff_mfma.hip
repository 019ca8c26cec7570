// Differential attention for prompts on the matrix cores, bfloat16, compiled for one padded key size and one padded
// value size (PALM_DIFF_KK: key size / 32 rounded up; PALM_DIFF_VT: value size / 16 rounded up).
//
// A wave owns one or two tiles of 16 queries of one head and both of the head's score maps; a block is four waves,
// 64 or 128 consecutive queries (a block of one wave: 16 or 32).  For every page of 64 keys the wave computes the transposed scores S^T = K Q^T (keys down, queries
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
constexpr int DM_WAVES = 1;          // waves of a block: they share nothing, and single waves spread evenly over the SIMDs
// tiles of 16 queries a wave: with two, every key and value fragment that the wave reads feeds twice the products
// (what bounds the kernel is bringing the pages to the matrix cores); the output tiles of two maps and two query tiles
// fit a lane's registers up to a value size of 128
#ifndef PALM_DIFF_QT
#define PALM_DIFF_QT 1
#endif
constexpr int QT = PALM_DIFF_QT;
constexpr bool V_AHEAD = VT * QT <= 8;                 // whether a page's value fragments are all read at its top (registers allowing)
constexpr int DM_QUERIES = 16 * QT * DM_WAVES;

PALM_API int palm_attention_diff_mfma_sizes(int which) { return which == 0 ? KK * 32 : which == 1 ? VT * 16 : QT; }

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
    // the wave's first query among the sequence's new tokens; the blocks of late queries, which have the most keys before
    // them, are handed out first, so that the short ones fill in at the end
    const int q0 = (gridDim.x - 1 - blockIdx.x) * DM_QUERIES + wave * 16 * QT;
    if (q0 >= n_new) return;
    const int r = lane % 16, g = lane / 16;
    const int start = seq_start[b];
    int qi[QT], qpos[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        qi[t] = min(q0 + 16 * t + r, n_new - 1);                  // a column beyond the run repeats the last query and stores nothing
        qpos[t] = start + qi[t];
    }
    const int last_pos = start + min(q0 + 16 * QT - 1, n_new - 1), first_pos = start + q0;
    const float scale2 = scale * 1.4426950408889634f;
    const int kvh = h / (heads / kv_heads);
    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;

    // the queries, as the B operand: column r, eight values of group g for each step of 32 over the key size
    bf16x8 qf[QT][2][KK];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        const bf16_t* qr = q + (((size_t)cu_new[b] + qi[t]) * heads + h) * 2 * dim;
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) qf[t][m][kk] = load_row8(qr + m * dim, kk * 32 + g * 8, dim);
    }
    f32x4 acc[QT][2][VT];
#pragma unroll
    for (int t = 0; t < QT; ++t)
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int vt = 0; vt < VT; ++vt) acc[t][m][vt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mx[QT][2], l[QT][2];
#pragma unroll
    for (int t = 0; t < QT; ++t) { mx[t][0] = mx[t][1] = -INFINITY; l[t][0] = l[t][1] = 0.f; }

    // The key fragments of a page are read one page ahead and the value fragments at the top of their page: both are
    // under way while the matrix cores and the softmax work on what came before.
    bf16x8 kf[2][4][KK];
    auto read_keys = [&](int pg) {
        const int page = pages[pg];
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            const bf16_t* kp = k_cache + ((size_t)page * 2 * kv_heads + 2 * kvh + m) * PAGE_TOKENS * dim;
#pragma unroll
            for (int n = 0; n < 4; ++n)
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) kf[m][n][kk] = load_row8(kp + (size_t)(16 * n + r) * dim, kk * 32 + g * 8, dim);
        }
    };
    const int last_page = last_pos / PAGE_TOKENS;
    read_keys(0);
    for (int pg = 0; pg <= last_page; ++pg) {
        const int page = pages[pg];
        bf16x8 kc[2][4][KK];
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int n = 0; n < 4; ++n)
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) kc[m][n][kk] = kf[m][n][kk];
        read_keys(min(pg + 1, last_page));
        const bf16_t* vp = v_cache + ((size_t)page * kv_heads + kvh) * vdim * PAGE_TOKENS;
        auto read_values = [&](int vt, int half) {
            const int vd = 16 * vt + r;
            const bf16_t* vr = vp + (size_t)min(vd, vdim - 1) * PAGE_TOKENS;    // row min(vd, vdim - 1): always there
            const uint2 lo = *reinterpret_cast<const uint2*>(vr + 32 * half + 4 * g);
            const uint2 hi = *reinterpret_cast<const uint2*>(vr + 32 * half + 16 + 4 * g);
            const uint4 both = make_uint4(lo.x, lo.y, hi.x, hi.y);
            return vd < vdim ? __builtin_bit_cast(bf16x8, both) : zero_bf16x8();
        };
        bf16x8 vf[V_AHEAD ? VT : 1][2];
        if constexpr (V_AHEAD) {
#pragma unroll
            for (int vt = 0; vt < VT; ++vt) { vf[vt][0] = read_values(vt, 0); vf[vt][1] = read_values(vt, 1); }
        }
        const bool edge = pg * PAGE_TOKENS + PAGE_TOKENS - 1 > first_pos;      // the page reaches beyond some query of the wave
        bf16x8 pf[QT][2][2];                                       // the weights as B operands: [query tile][map][32 keys]
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            f32x4 s[QT][4];
#pragma unroll
            for (int n = 0; n < 4; ++n) {
#pragma unroll
                for (int t = 0; t < QT; ++t) s[t][n] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < KK; ++kk)
#pragma unroll
                    for (int t = 0; t < QT; ++t) s[t][n] = mfma_16x16x32(kc[m][n][kk], qf[t][m][kk], s[t][n]);
            }
            // lane (r, g) holds the keys 16 n + 4 g + i of query r; scores in units of log2: a weight is one exp2 away
#pragma unroll
            for (int t = 0; t < QT; ++t) {
                float top = -INFINITY;
                if (edge) {
#pragma unroll
                    for (int n = 0; n < 4; ++n)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int j = pg * PAGE_TOKENS + 16 * n + 4 * g + i;
                            s[t][n][i] = j <= qpos[t] ? s[t][n][i] * scale2 : -INFINITY;
                            top = fmaxf(top, s[t][n][i]);
                        }
                } else {
#pragma unroll
                    for (int n = 0; n < 4; ++n)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            s[t][n][i] *= scale2;
                            top = fmaxf(top, s[t][n][i]);
                        }
                }
                top = fmaxf(top, __shfl_xor(top, 16, WAVE));
                top = fmaxf(top, __shfl_xor(top, 32, WAVE));
                const float m_new = fmaxf(mx[t][m], top);          // finite from the first page on: key 0 is visible to all
                const float alpha = exp2f(mx[t][m] - m_new);
                mx[t][m] = m_new;
                float sum = 0.f;
#pragma unroll
                for (int n = 0; n < 4; ++n)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s[t][n][i] = exp2f(s[t][n][i] - m_new);
                        sum += s[t][n][i];
                    }
                l[t][m] = l[t][m] * alpha + sum;                   // this lane's part; the groups are added at the end
#pragma unroll
                for (int vt = 0; vt < VT; ++vt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[t][m][vt][i] *= alpha;
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        pf[t][m][half][i] = (__bf16)s[t][2 * half][i];
                        pf[t][m][half][4 + i] = (__bf16)s[t][2 * half + 1][i];
                    }
            }
        }
        // O^T += V^T P^T: row r of a value tile, the same eight keys of group g as the weights hold
#pragma unroll
        for (int vt = 0; vt < VT; ++vt)
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const bf16x8 v8 = V_AHEAD ? vf[V_AHEAD ? vt : 0][half] : read_values(vt, half);
#pragma unroll
                for (int t = 0; t < QT; ++t) {
                    acc[t][0][vt] = mfma_16x16x32(v8, pf[t][0][half], acc[t][0][vt]);
                    acc[t][1][vt] = mfma_16x16x32(v8, pf[t][1][half], acc[t][1][vt]);
                }
            }
    }
    // lane (r, g) holds value dimensions 16 vt + 4 g + i of query r
#pragma unroll
    for (int t = 0; t < QT; ++t) {
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            l[t][m] += __shfl_xor(l[t][m], 16, WAVE);
            l[t][m] += __shfl_xor(l[t][m], 32, WAVE);
        }
        const float f0 = 1.0f / l[t][0], f1 = lambda / l[t][1];
        float ss = 0.f;
#pragma unroll
        for (int vt = 0; vt < VT; ++vt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float o = acc[t][0][vt][i] * f0 - acc[t][1][vt][i] * f1;
                acc[t][0][vt][i] = o;
                if (16 * vt + 4 * g + i < vdim) ss += o * o;
            }
        ss += __shfl_xor(ss, 16, WAVE);
        ss += __shfl_xor(ss, 32, WAVE);
        const float inv = gain / sqrtf(ss / (float)vdim + eps);
        if (q0 + 16 * t + r >= n_new) continue;
        bf16_t* op = out + (((size_t)cu_new[b] + qi[t]) * heads + h) * vdim;
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            const int vd = 16 * vt + 4 * g;
            if (vd < vdim) {                                        // vdim is a multiple of four
                uint2 w;
                w.x = (uint32_t)f32_to_bf16(acc[t][0][vt][0] * inv).bits | ((uint32_t)f32_to_bf16(acc[t][0][vt][1] * inv).bits << 16);
                w.y = (uint32_t)f32_to_bf16(acc[t][0][vt][2] * inv).bits | ((uint32_t)f32_to_bf16(acc[t][0][vt][3] * inv).bits << 16);
                *reinterpret_cast<uint2*>(op + vd) = w;
            }
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
