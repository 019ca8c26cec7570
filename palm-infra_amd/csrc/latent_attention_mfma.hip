// Attention over one compressed row per position, for prompts, on the matrix cores, bfloat16; compiled for one padded
// row size and one padded latent size (PALM_LAT_KK: (kv_rank + rot_dim) / 32 rounded up; PALM_LAT_VT: kv_rank / 16
// rounded up).
//
// All heads read the same rows, so a wave owns a tile of 16 queries of HT heads and every fragment of a page that it reads
// feeds HT products.  For every page of 64 keys the wave computes the transposed scores S^T = K Q^T (keys down, queries
// across), so that a lane's four results of a tile are four keys of ONE query: the softmax statistics of a query then live
// in the lanes of its column, and the weights are already laid out as the B operand of the second product O^T += C^T P^T,
// whose A operand reads runs of keys from a transposed copy of the latents.  Scores leave the matrix cores as 32-bit sums;
// maximum, exponentials (base 2: the scores are scaled by scale * log2 e) and sums are 32-bit; the weights are rounded to
// bfloat16 for the second product, whose sums are 32-bit again.
//
// rows [pages, 64, kv_rank + rot_dim]: the keys; rows_t [pages, kv_rank, 64]: the latents once more, positions innermost.
// The two have page tables of their own.  q: float32 [n, heads, kv_rank + rot_dim]; out: float32 [n, heads, kv_rank], or,
// with the value matrices uv [heads * vdim, kv_rank] (and the heads' gates before their sigmoid), out_rows bfloat16
// [n, heads * vdim]: head h's sums through U_v,h times sigmoid(gate_h), made from the registers that hold the sums.
#include "mfma.h"

#ifndef PALM_LAT_KK
#error "compile with -DPALM_LAT_KK=<ceil((kv_rank + rot_dim) / 32)> -DPALM_LAT_VT=<ceil(kv_rank / 16)>"
#endif

PALM_DEFINE_LAST_ERROR()

constexpr int KK = PALM_LAT_KK;
constexpr int VT = PALM_LAT_VT;
// heads a wave: as many as a lane's registers take (a head's output tile is 4 VT values a lane, its queries 4 KK)
constexpr int HT = VT <= 8 ? 4 : VT <= 16 ? 2 : 1;

PALM_API int palm_latent_attention_mfma_sizes(int which) { return which == 0 ? KK * 32 : which == 1 ? VT * 16 : HT; }

__device__ inline bf16x8 load_row8(const bf16_t* row, int col, int dim) {
    // eight values of a row from column `col`; columns beyond `dim` are zero (dim is a multiple of eight).  The read
    // itself is unconditional (of the row's last eight values where the column lies beyond it): no branch around it
    const bf16x8 v = load_bf16x8(row + min(col, dim - 8));
    return col < dim ? v : zero_bf16x8();
}

__device__ inline bf16x8 query8(const float* row, int col, int dim) {
    const float* p = row + min(col, dim - 8);
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    bf16x8 v;
    v[0] = (__bf16)a.x; v[1] = (__bf16)a.y; v[2] = (__bf16)a.z; v[3] = (__bf16)a.w;
    v[4] = (__bf16)b.x; v[5] = (__bf16)b.y; v[6] = (__bf16)b.z; v[7] = (__bf16)b.w;
    return col < dim ? v : zero_bf16x8();
}

__global__ __launch_bounds__(WAVE) void latent_attention_mfma_kernel(
    const float* __restrict__ q, const bf16_t* __restrict__ rows, const bf16_t* __restrict__ rows_t,
    const int* __restrict__ block_table, const int* __restrict__ block_table_t, int max_pages,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_start, const int* __restrict__ seq_new,
    const int* __restrict__ cu_new, int heads, int kv_rank, int rot_dim, float scale, int window, float* __restrict__ out,
    const bf16_t* __restrict__ uv, const bf16_t* __restrict__ gate, int gate_stride, int vdim, bf16_t* __restrict__ out_rows) {
    const int h0 = blockIdx.y * HT, b = blockIdx.z;
    const int n_new = seq_new[b];
    const int lane = threadIdx.x;
    // the blocks of late queries, which have the most keys before them, are handed out first
    const int q0 = (gridDim.x - 1 - blockIdx.x) * 16;
    if (q0 >= n_new) return;
    const int r = lane % 16, g = lane / 16;
    const int start = seq_start[b];
    const int dk = kv_rank + rot_dim;
    const int qi = min(q0 + r, n_new - 1);                        // a column beyond the run repeats the last query and stores nothing
    const int qpos = start + qi;
    const int qlo = window > 0 ? max(0, qpos - window + 1) : 0;
    const int last_pos = start + min(q0 + 15, n_new - 1), first_pos = start + q0;
    const int seq_last = start + n_new - 1;                       // rows beyond it belong to nobody
    const float scale2 = scale * 1.4426950408889634f;
    const int* pages = block_table + (size_t)seq_slot[b] * max_pages;
    const int* pages_t = block_table_t + (size_t)seq_slot[b] * max_pages;

    // the queries, as the B operand: column r, eight values of group g for each step of 32 over the row
    bf16x8 qf[HT][KK];
#pragma unroll
    for (int t = 0; t < HT; ++t) {
        const float* qr = q + (((size_t)cu_new[b] + qi) * heads + min(h0 + t, heads - 1)) * dk;
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) qf[t][kk] = query8(qr, kk * 32 + g * 8, dk);
    }
    f32x4 acc[HT][VT];
#pragma unroll
    for (int t = 0; t < HT; ++t)
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) acc[t][vt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mx[HT], l[HT];
#pragma unroll
    for (int t = 0; t < HT; ++t) { mx[t] = -INFINITY; l[t] = 0.f; }

    const int first_page = (window > 0 ? max(0, first_pos - window + 1) : 0) / PAGE_TOKENS;
    const int last_page = last_pos / PAGE_TOKENS;
    for (int pg = first_page; pg <= last_page; ++pg) {
        const bf16_t* kp = rows + (size_t)pages[pg] * PAGE_TOKENS * dk;
        const bf16_t* vp = rows_t + (size_t)pages_t[pg] * kv_rank * PAGE_TOKENS;
        f32x4 s[HT][4];
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            bf16x8 kf[KK];
#pragma unroll
            for (int kk = 0; kk < KK; ++kk) kf[kk] = load_row8(kp + (size_t)(16 * n + r) * dk, kk * 32 + g * 8, dk);
#pragma unroll
            for (int t = 0; t < HT; ++t) {
                s[t][n] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < KK; ++kk) s[t][n] = mfma_16x16x32(kf[kk], qf[t][kk], s[t][n]);
            }
        }
        // lane (r, g) holds the keys 16 n + 4 g + i of query r; scores in units of log2: a weight is one exp2 away
        bf16x8 pf[HT][2];                                          // the weights as B operands: [head][32 keys]
#pragma unroll
        for (int t = 0; t < HT; ++t) {
            float top = -INFINITY;
#pragma unroll
            for (int n = 0; n < 4; ++n)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int j = pg * PAGE_TOKENS + 16 * n + 4 * g + i;
                    s[t][n][i] = (j <= qpos && j >= qlo) ? s[t][n][i] * scale2 : -INFINITY;     // (a row that belongs to nobody may hold anything)
                    top = fmaxf(top, s[t][n][i]);
                }
            top = fmaxf(top, __shfl_xor(top, 16, WAVE));
            top = fmaxf(top, __shfl_xor(top, 32, WAVE));
            const float m_new = fmaxf(mx[t], top);
            const float m_ref = m_new == -INFINITY ? 0.f : m_new;   // a page of which this query sees nothing yet
            const float alpha = exp2f(mx[t] - m_ref);
            mx[t] = m_new;
            float sum = 0.f;
#pragma unroll
            for (int n = 0; n < 4; ++n)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[t][n][i] = exp2f(s[t][n][i] - m_ref);
                    sum += s[t][n][i];
                }
            l[t] = l[t] * alpha + sum;                             // this lane's part; the groups are added at the end
#pragma unroll
            for (int vt = 0; vt < VT; ++vt)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[t][vt][i] *= alpha;
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    pf[t][half][i] = (__bf16)s[t][2 * half][i];
                    pf[t][half][4 + i] = (__bf16)s[t][2 * half + 1][i];
                }
        }
        // O^T += C^T P^T: row r of a latent tile, the same eight keys of group g as the weights hold.  On the page that
        // holds the sequence's last row the latents of the positions beyond it are taken as zero: their weights are zero,
        // but pages are handed out uncleared and zero times a stale NaN is NaN.
        const int beyond = seq_last - pg * PAGE_TOKENS;            // positions of the page above this belong to nobody
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            const int vd = 16 * vt + r;
            const bf16_t* vr = vp + (size_t)min(vd, kv_rank - 1) * PAGE_TOKENS;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const uint2 lo = *reinterpret_cast<const uint2*>(vr + 32 * half + 4 * g);
                const uint2 hi = *reinterpret_cast<const uint2*>(vr + 32 * half + 16 + 4 * g);
                uint32_t w[4] = {lo.x, lo.y, hi.x, hi.y};
                if (beyond < PAGE_TOKENS - 1) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int j = 32 * half + (e < 4 ? 0 : 16) + 4 * g + (e % 4);
                        if (j > beyond) w[e / 2] &= (e % 2) ? 0x0000ffffu : 0xffff0000u;
                    }
                }
                const bf16x8 v8 = vd < kv_rank ? __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3])) : zero_bf16x8();
#pragma unroll
                for (int t = 0; t < HT; ++t) acc[t][vt] = mfma_16x16x32(v8, pf[t][half], acc[t][vt]);
            }
        }
    }
    // lane (r, g) holds latent dimensions 16 vt + 4 g + i of query r
#pragma unroll
    for (int t = 0; t < HT; ++t) {
        l[t] += __shfl_xor(l[t], 16, WAVE);
        l[t] += __shfl_xor(l[t], 32, WAVE);
    }
    if (uv) {
        // The value matrix in the same kernel: out^T [vdim, 16 queries] = U_v,h [vdim, kv_rank] (O^T / l).  The sums a lane
        // holds (latent dimensions 16 vt + 4 g + i of query r) are, two tiles at a time, the B operand of a step over 32
        // latent dimensions; the A operand takes the same dimensions of a row of U_v,h.  Then the head's gate.
        constexpr int VP = (VT + 1) / 2;
#pragma unroll
        for (int t = 0; t < HT; ++t) {
            const int h = min(h0 + t, heads - 1);
            const float f = 1.0f / l[t];
            bf16x8 of[VP];
#pragma unroll
            for (int m = 0; m < VP; ++m)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    of[m][i] = (__bf16)(acc[t][2 * m][i] * f);
                    of[m][4 + i] = (__bf16)(2 * m + 1 < VT ? acc[t][min(2 * m + 1, VT - 1)][i] * f : 0.f);
                }
            const float gt = gate ? 1.0f / (1.0f + expf(-to_float(gate[((size_t)cu_new[b] + qi) * gate_stride + h]))) : 1.0f;
            for (int j0 = 0; j0 < vdim; j0 += 16) {
                const bf16_t* wr = uv + ((size_t)h * vdim + min(j0 + r, vdim - 1)) * kv_rank;
                f32x4 o = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int m = 0; m < VP; ++m) {
                    const int k0 = 32 * m + 4 * g, k1 = 32 * m + 16 + 4 * g;          // four dimensions each, inside the latent or beyond it
                    const uint2 lo = *reinterpret_cast<const uint2*>(wr + min(k0, kv_rank - 4));
                    const uint2 hi = *reinterpret_cast<const uint2*>(wr + min(k1, kv_rank - 4));
                    const uint4 both = make_uint4(k0 < kv_rank ? lo.x : 0u, k0 < kv_rank ? lo.y : 0u, k1 < kv_rank ? hi.x : 0u, k1 < kv_rank ? hi.y : 0u);
                    o = mfma_16x16x32(__builtin_bit_cast(bf16x8, both), of[m], o);
                }
                // lane (r, g) holds output dimensions j0 + 4 g + i of query r
                const int j = j0 + 4 * g;
                if (q0 + r < n_new && h0 + t < heads && j < vdim) {                   // vdim is a multiple of four
                    uint2 w;
                    w.x = (uint32_t)f32_to_bf16(o[0] * gt).bits | ((uint32_t)f32_to_bf16(o[1] * gt).bits << 16);
                    w.y = (uint32_t)f32_to_bf16(o[2] * gt).bits | ((uint32_t)f32_to_bf16(o[3] * gt).bits << 16);
                    *reinterpret_cast<uint2*>(out_rows + (((size_t)cu_new[b] + qi) * heads + h0 + t) * vdim + j) = w;
                }
            }
        }
        return;
    }
    if (q0 + r >= n_new) return;
#pragma unroll
    for (int t = 0; t < HT; ++t) {
        if (h0 + t >= heads) continue;
        const float f = 1.0f / l[t];
        float* op = out + (((size_t)cu_new[b] + qi) * heads + h0 + t) * kv_rank;
#pragma unroll
        for (int vt = 0; vt < VT; ++vt) {
            const int vd = 16 * vt + 4 * g;
            if (vd < kv_rank)                                      // kv_rank is a multiple of four
                *reinterpret_cast<float4*>(op + vd) = make_float4(acc[t][vt][0] * f, acc[t][vt][1] * f, acc[t][vt][2] * f, acc[t][vt][3] * f);
        }
    }
}

PALM_API int palm_latent_attention_mfma(hipStream_t stream, const float* q, const void* rows, const void* rows_t,
                                        const int* block_table, const int* block_table_t, int max_pages, const int* seq_slot,
                                        const int* seq_start, const int* seq_new, const int* cu_new, int n_seqs, int max_new,
                                        int heads, int kv_rank, int rot_dim, float scale, int window, float* out, const void* uv,
                                        const void* gate, int gate_stride, int vdim, void* out_rows) {
    PALM_CHECK(n_seqs >= 0 && max_new >= 0 && heads > 0 && kv_rank > 0 && rot_dim >= 0, "latent_attention_mfma: seqs=%d max_new=%d heads=%d "
               "kv_rank=%d rot_dim=%d", n_seqs, max_new, heads, kv_rank, rot_dim);
    const int dk = kv_rank + rot_dim;
    PALM_CHECK(dk % 8 == 0 && dk <= KK * 32 && dk > (KK - 1) * 32, "latent_attention_mfma: built for rows of %d..%d in steps of 8, not %d",
               (KK - 1) * 32 + 8, KK * 32, dk);
    PALM_CHECK(kv_rank % 8 == 0 && kv_rank <= VT * 16 && kv_rank > (VT - 1) * 16, "latent_attention_mfma: built for latents of %d..%d in "
               "steps of 8, not %d", (VT - 1) * 16 + 8, VT * 16, kv_rank);
    PALM_CHECK(window >= 0 && max_pages > 0, "latent_attention_mfma: window %d, max_pages %d", window, max_pages);
    PALM_CHECK(uv ? (out_rows && vdim > 0 && vdim % 4 == 0) : out != nullptr, "latent_attention_mfma: either room for the latent sums, or the "
               "value matrix with room for rows of a value size that is a multiple of four (%d)", vdim);
    if (n_seqs == 0 || max_new == 0) return 0;
    PALM_CHECK(heads <= 65535 * HT && n_seqs <= 65535, "latent_attention_mfma: %d heads / %d sequences are more than one launch takes", heads, n_seqs);
    dim3 grid((max_new + 15) / 16, (heads + HT - 1) / HT, n_seqs);
    latent_attention_mfma_kernel<<<grid, WAVE, 0, stream>>>(q, (const bf16_t*)rows, (const bf16_t*)rows_t, block_table, block_table_t,
                                                           max_pages, seq_slot, seq_start, seq_new, cu_new, heads, kv_rank, rot_dim, scale,
                                                           window, out, (const bf16_t*)uv, (const bf16_t*)gate, gate_stride, vdim,
                                                           (bf16_t*)out_rows);
    PALM_LAUNCHED();
    return 0;
}
