// The gated delta rule with one decay per key channel.
//
// Per sequence and head, S [dim, vdim] in 32-bit, kept between steps; for every token, in this order:
//
//   S <- diag(g_t) S                     g_t[d] = exp(-exp(A_h) * softplus(a_t[h, d] + bias[h, d])): one decay per row of S
//   u_t = beta_t (v_t - S^T k_t)         beta_t = sigmoid(b_t[h]): how much of the error is written
//   S <- S + k_t u_t^T
//   o_t = S^T q_t                        (reads the token's own write)
//   out_t = o_t / sqrt(mean_v(o_t^2) + eps) * w * sigmoid(gate_t)           (w [vdim], shared by the heads)
//
// q and k are unit vectors per head, x / sqrt(sum(x^2) + unit_eps), q also times q_scale; head h reads q/k head
// h / (heads / kv_heads).  Decays, gates, unit vectors, state and sums are 32-bit whatever the run's type.
//
// A first pass makes the unit vectors, decays and write strengths of all the step's tokens (32-bit rows, padded to
// the key size that the main kernel is compiled for; the padding's q and k are zero and its decay one, so the main
// kernel's loops need no test).  Then one block per (head, sequence), one thread per value dimension v: the columns
// of S do not depend on each other, so the thread keeps column v in registers and walks over the sequence's new tokens.
// A token's q, k and g are the same for every thread of the block: each wave reads the rows once, one value a lane,
// and hands value d to all its lanes as a scalar operand.  A prompt and a single token run the same code, so a
// prompt leaves the state that its tokens one by one leave.
//
// A long run of new tokens would keep only (heads x sequences) blocks busy, one token after the other.  A token's step is
// linear in S: S_t = A_t S_(t-1) + beta_t k_t v_t^T with A_t = (I - beta_t k_t k_t^T) diag(g_t), so such a run is cut into
// chunks of `chunk` tokens and done in three launches:
//   1. every chunk alone: from a zero state with its values (its own sum L_c, [dim, vdim]), and from the identity with
//      values of zero (the product P_c of its A_t, [dim, dim]: the same walk over dim more columns)       (all chunks at once)
//   2. the chunks' starting states, one after the other: S_(c+1) = P_c S_c + L_c, S_0 the kept state      (small products)
//   3. every chunk from its starting state, now with outputs                                             (all chunks at once)
// The arithmetic of a token is the same in all three; only the order of the 32-bit sums over the past differs.
#include "common.h"

constexpr int DELTA_TILE = 8;

__device__ inline float delta_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ inline float delta_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

// One wave per (token, head).  prep[row][head][0 = q, 1 = k, 2 = g][pad];  beta[row][head].
template <typename T>
__global__ __launch_bounds__(WAVE) void delta_prep_kernel(const T* __restrict__ u, int u_stride, int q_off, int k_off,
                                                          const T* __restrict__ b, int b_stride,
                                                          const float* __restrict__ a, int a_stride,
                                                          const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                                          float q_scale, float unit_eps, int heads, int kv_heads, int dim, int pad,
                                                          float* __restrict__ prep, float* __restrict__ beta) {
    const size_t row = blockIdx.x;
    const int h = blockIdx.y, lane = threadIdx.x;
    const int kh = h / (heads / kv_heads);
    const T* qr = u + row * u_stride + q_off + kh * dim;
    const T* kr = u + row * u_stride + k_off + kh * dim;
    float qq = 0.f, kk = 0.f;
    for (int d = lane; d < dim; d += WAVE) {
        const float qv = to_float(qr[d]), kv = to_float(kr[d]);
        qq = fmaf(qv, qv, qq);
        kk = fmaf(kv, kv, kk);
    }
    const float qi = q_scale / sqrtf(wave_sum(qq) + unit_eps), ki = 1.0f / sqrtf(wave_sum(kk) + unit_eps);
    const float rate = -expf(a_log[h]);
    float* o = prep + ((row * heads + h) * 3) * pad;
    for (int d = lane; d < pad; d += WAVE) {
        const bool in = d < dim;
        o[d] = in ? to_float(qr[d]) * qi : 0.f;
        o[pad + d] = in ? to_float(kr[d]) * ki : 0.f;
        o[2 * pad + d] = in ? expf(rate * delta_softplus(a[row * a_stride + h * dim + d] + dt_bias[h * dim + d])) : 1.f;
    }
    if (lane == 0) beta[row * heads + h] = delta_sigmoid(to_float(b[row * b_stride + h]));
}

enum DeltaMode : int { DELTA_WHOLE = 0, DELTA_LOCAL = 1, DELTA_FROM_STARTS = 2 };

// ext: [sequence x chunk][head][dim][vdim + dim]: a chunk's own sum beside the product of its steps (mode LOCAL writes
// it: blockIdx.z = 0 the value columns, 1 the dim columns that start as the identity).  starts: [sequence x chunk][head]
// [dim][vdim]: the states the chunks start from (mode FROM_STARTS reads them).
template <typename T, int DMAX, int MAXT>
__global__ __launch_bounds__(MAXT) void delta_rule_kernel(int mode, int chunk, int max_chunks, float* __restrict__ ext,
                                                          const float* __restrict__ starts,
                                                          const T* __restrict__ u, int u_stride, int v_off,
                                                          const float* __restrict__ prep, const float* __restrict__ beta,
                                                          const float* __restrict__ gate, int gate_stride,
                                                          const float* __restrict__ norm_w, float eps,
                                                          float* __restrict__ state, const int* __restrict__ seq_slot,
                                                          const int* __restrict__ seq_new, const int* __restrict__ cu_new,
                                                          int heads, int dim, int vdim, T* __restrict__ out) {
    __shared__ float red[DELTA_TILE][16];
    __shared__ float o_s[DELTA_TILE][MAXT];
    constexpr int QREGS = (DMAX + WAVE - 1) / WAVE;
    const int h = blockIdx.x, b = blockIdx.y / max_chunks, c = blockIdx.y % max_chunks;
    const bool steps_part = blockIdx.z == 1;                     // the columns that become the product of the chunk's steps
    const int v = threadIdx.x;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    const int seq_tokens = seq_new[b];
    if (seq_tokens <= 0 || (mode != DELTA_WHOLE && c * chunk >= seq_tokens)) return;
    const int n_new = mode == DELTA_WHOLE ? seq_tokens : min(chunk, seq_tokens - c * chunk);
    const int row0 = cu_new[b] + (mode == DELTA_WHOLE ? 0 : c * chunk);
    const int cols = steps_part ? dim : vdim;
    const bool mine = v < cols;
    const int vc = min(v, vdim - 1);

    // unconditional reads of rows and a column that exist; what does not belong is set to zero after
    float S[DMAX];
    if (mode == DELTA_LOCAL) {
#pragma unroll
        for (int d = 0; d < DMAX; ++d) S[d] = (steps_part && mine && d == v) ? 1.f : 0.f;
    } else {
        const float* sp = mode == DELTA_WHOLE ? state + (((size_t)seq_slot[b] * heads + h) * dim) * vdim + vc
                                              : starts + ((((size_t)b * max_chunks + c) * heads + h) * dim) * vdim + vc;
#pragma unroll
        for (int d = 0; d < DMAX; ++d) {
            const float s0 = sp[(size_t)min(d, dim - 1) * vdim];
            S[d] = (!mine || d >= dim) ? 0.f : s0;
        }
    }

    auto read_token = [&](int t, float& vv, float& bt, float (&qv)[QREGS], float (&kv)[QREGS], float (&gv)[QREGS]) {
        const size_t row = (size_t)(row0 + t);
        vv = to_float(u[row * u_stride + v_off + h * vdim + vc]);
        bt = beta[row * heads + h];
        const float* __restrict__ pr = prep + ((row * heads + h) * 3) * DMAX;
#pragma unroll
        for (int c = 0; c < QREGS; ++c) {
            const int at = min(c * WAVE + lane, DMAX - 1);             // (a key size of 32: the upper lanes repeat)
            qv[c] = pr[at];
            kv[c] = pr[DMAX + at];
            gv[c] = pr[2 * DMAX + at];
        }
    };
    float vv, bt, qv[QREGS], kv[QREGS], gv[QREGS];
    read_token(0, vv, bt, qv, kv, gv);
    for (int t0 = 0; t0 < n_new; t0 += DELTA_TILE) {
        const int tt = min(DELTA_TILE, n_new - t0);
        for (int ti = 0; ti < tt; ++ti) {                        // not unrolled: the body is 2 DMAX steps long already
            float vn, bn, qn[QREGS], kn[QREGS], gn[QREGS];
            read_token(min(t0 + ti + 1, n_new - 1), vn, bn, qn, kn, gn);
            if (!mine || steps_part) vv = 0.f;
            // four partial sums each: the multiply-adds of a sum over d then wait for every fourth one before them only
            float pr[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int d = 0; d < DMAX; ++d) {
                const float gd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, gv[d / WAVE]), d % WAVE));
                const float kd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, kv[d / WAVE]), d % WAVE));
                S[d] *= gd;
                pr[d % 4] = fmaf(S[d], kd, pr[d % 4]);
            }
            const float uu = bt * (vv - ((pr[0] + pr[1]) + (pr[2] + pr[3])));
            float ac[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int d = 0; d < DMAX; ++d) {
                const float qd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, qv[d / WAVE]), d % WAVE));
                const float kd = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, kv[d / WAVE]), d % WAVE));
                S[d] = fmaf(kd, uu, S[d]);
                ac[d % 4] = fmaf(S[d], qd, ac[d % 4]);
            }
            const float acc = (ac[0] + ac[1]) + (ac[2] + ac[3]);
            if (mode != DELTA_LOCAL) {
                o_s[ti][v] = acc;
                const float ss = wave_sum(acc * acc);
                if (lane == 0) red[ti][wave] = ss;
            }
            vv = vn;
            bt = bn;
#pragma unroll
            for (int c = 0; c < QREGS; ++c) { qv[c] = qn[c]; kv[c] = kn[c]; gv[c] = gn[c]; }
        }
        if (mode == DELTA_LOCAL) continue;
        __syncthreads();
        for (int ti = 0; ti < tt; ++ti) {
            float total = 0.f;
            for (int w = 0; w < n_waves; ++w) total += red[ti][w];
            const float inv = 1.0f / sqrtf(total / (float)vdim + eps);
            const size_t row = (size_t)(row0 + t0 + ti);
            const float gt = gate[row * gate_stride + h * vdim + vc];
            if (mine) out[row * ((size_t)heads * vdim) + h * vdim + v] = from_float<T>((o_s[ti][v] * inv) * norm_w[vc] * delta_sigmoid(gt));
        }
        __syncthreads();
    }
    if (mine && mode == DELTA_WHOLE) {
        float* sp = state + (((size_t)seq_slot[b] * heads + h) * dim) * vdim + v;
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
            if (d < dim) sp[(size_t)d * vdim] = S[d];
    }
    if (mine && mode == DELTA_LOCAL) {
        const int ev = vdim + dim;
        float* ep = ext + ((((size_t)b * max_chunks + c) * heads + h) * dim) * ev + (steps_part ? vdim : 0) + v;
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
            if (d < dim) ep[(size_t)d * ev] = S[d];
    }
}

// Step 2 above.  One block per (head, sequence, tile of DS_COLS value columns): the tile of S lies in LDS.  For every chunk
// the block first hands the chunk its starting state, then makes S <- P_c S + L_c: a thread owns one column of the tile and
// every 32nd row of the result (a quarter of a wave a column run, 8 waves x 4 quarters = 32 row groups), reads its rows of
// P_c four values at a time and S from LDS.
constexpr int DS_WAVES = 8;
constexpr int DS_COLS = 16;
constexpr int DS_GROUPS = DS_WAVES * (WAVE / DS_COLS);          // 32 row groups
constexpr int DS_MAX_ROWS = 256 / DS_GROUPS;                    // rows a thread owns at most (dim up to 256)

__global__ __launch_bounds__(DS_WAVES * WAVE) void delta_starts_kernel(const float* __restrict__ ext, float* __restrict__ starts,
                                                                       float* __restrict__ state, const int* __restrict__ seq_slot,
                                                                       const int* __restrict__ seq_new, int chunk, int max_chunks,
                                                                       int heads, int dim, int vdim) {
    extern __shared__ __attribute__((aligned(16))) float s_s[];         // [dim][DS_COLS]
    const int h = blockIdx.x, b = blockIdx.y, v0 = blockIdx.z * DS_COLS;
    const int col = threadIdx.x % DS_COLS, group = threadIdx.x / DS_COLS;
    const int n_new = seq_new[b];
    if (n_new <= 0) return;
    const int v = v0 + col;
    const bool mine = v < vdim;
    const int vc = min(v, vdim - 1), ev = vdim + dim;
    float* st = state + (((size_t)seq_slot[b] * heads + h) * dim) * vdim;
    for (int d = group; d < dim; d += DS_GROUPS) s_s[d * DS_COLS + col] = mine ? st[(size_t)d * vdim + vc] : 0.f;
    __syncthreads();
    for (int c = 0; c * chunk < n_new; ++c) {
        const size_t at = (((size_t)b * max_chunks + c) * heads + h) * dim;
        const float* ep = ext + at * ev;
        float* sc = starts + at * vdim;
        float fresh[DS_MAX_ROWS];
#pragma unroll
        for (int i = 0; i < DS_MAX_ROWS; ++i) {
            const int d = group + i * DS_GROUPS;
            const int dc = min(d, dim - 1);
            const float* pr = ep + (size_t)dc * ev + vdim;              // row d of P_c (16-byte reads where the rows allow them)
            float acc = ep[(size_t)dc * ev + vc];                       // L_c
            if (d < dim) {
                if (ev % 4 == 0 && vdim % 4 == 0 && dim % 4 == 0) {
                    for (int e = 0; e < dim; e += 4) {
                        const float4 p = *reinterpret_cast<const float4*>(pr + e);
                        acc = fmaf(p.x, s_s[e * DS_COLS + col], acc);
                        acc = fmaf(p.y, s_s[(e + 1) * DS_COLS + col], acc);
                        acc = fmaf(p.z, s_s[(e + 2) * DS_COLS + col], acc);
                        acc = fmaf(p.w, s_s[(e + 3) * DS_COLS + col], acc);
                    }
                } else {
                    for (int e = 0; e < dim; ++e) acc = fmaf(pr[e], s_s[e * DS_COLS + col], acc);
                }
            }
            fresh[i] = acc;
        }
        // the chunk starts from the state as it was
        for (int d = group; d < dim; d += DS_GROUPS)
            if (mine) sc[(size_t)d * vdim + v] = s_s[d * DS_COLS + col];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < DS_MAX_ROWS; ++i) {
            const int d = group + i * DS_GROUPS;
            if (d < dim) s_s[d * DS_COLS + col] = fresh[i];
        }
        __syncthreads();
    }
    for (int d = group; d < dim; d += DS_GROUPS)
        if (mine) st[(size_t)d * vdim + v] = s_s[d * DS_COLS + col];
}

PALM_API int palm_delta_pad(int dim) { return dim <= 32 ? 32 : dim <= 64 ? 64 : dim <= 128 ? 128 : 256; }

// u: the convolution's output [n, u_stride] holding q at q_off (kv_heads * dim), k at k_off, v at v_off (heads * vdim);
// b: the write strengths before the sigmoid, [n, b_stride] of the same type, one a head; a: float32 [n, a_stride], the
// decays' rows before bias and softplus (heads * dim); gate: float32 [n, gate_stride], the output gate before the
// sigmoid (heads * vdim).  prep: room for n * heads * 3 * palm_delta_pad(dim) floats, beta_buf: n * heads floats.
// chunk == 0: every sequence's run in one block per head.  Else, with max_chunks = ceil(max_new / chunk): ext holds
// n_seqs * max_chunks * heads * dim * (vdim + dim) floats and starts n_seqs * max_chunks * heads * dim * vdim.
PALM_API int palm_delta_rule(hipStream_t stream, const void* u, int dtype, int u_stride, int q_off, int k_off, int v_off,
                             const void* b, int b_stride, const float* a, int a_stride, const float* gate, int gate_stride,
                             const float* a_log, const float* dt_bias, const float* norm_w, float q_scale, float unit_eps,
                             float eps, float* state, const int* seq_slot, const int* seq_new, const int* cu_new, int n_seqs,
                             int heads, int kv_heads, int dim, int vdim, void* out, int n_tokens, float* prep, float* beta_buf,
                             int max_new, int chunk, float* ext, float* starts) {
    PALM_CHECK(n_seqs >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "delta_rule: seqs=%d heads=%d kv=%d dim=%d vdim=%d",
               n_seqs, heads, kv_heads, dim, vdim);
    PALM_CHECK(heads % kv_heads == 0, "delta_rule: %d heads are not a multiple of %d q/k heads", heads, kv_heads);
    PALM_CHECK(dim <= 256, "delta_rule: a key size of %d exceeds 256", dim);
    PALM_CHECK(vdim <= 1024, "delta_rule: a value size of %d exceeds 1024", vdim);
    PALM_CHECK(n_tokens >= 0 && (n_tokens == 0 || (prep && beta_buf)), "delta_rule: the prepared rows need their room");
    PALM_CHECK(chunk >= 0 && (chunk == 0 || (ext && starts && max_new > 0)), "delta_rule: chunks of %d tokens need room for their sums, "
               "products and starting states", chunk);
    if (n_seqs == 0 || n_tokens == 0) return 0;
    const int max_chunks = chunk > 0 ? (max_new + chunk - 1) / chunk : 1;
    PALM_CHECK(heads <= 65535 && (long long)n_seqs * max_chunks <= 65535, "delta_rule: %d heads / %d sequences x %d chunks are more than one "
               "launch takes", heads, n_seqs, max_chunks);
    const int pad = palm_delta_pad(dim);
    const int threads = (vdim + WAVE - 1) / WAVE * WAVE;
    const int local_threads = (max(vdim, dim) + WAVE - 1) / WAVE * WAVE;
    dim3 grid(heads, n_seqs * max_chunks);
#define DELTA_LAUNCH(D, GRID, THREADS, MODE) { if ((THREADS) <= 256) delta_rule_kernel<T, D, 256><<<GRID, THREADS, 0, stream>>>(MODE, chunk, max_chunks, \
            ext, starts, (const T*)u, u_stride, v_off, prep, beta_buf, gate, gate_stride, norm_w, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out); \
        else delta_rule_kernel<T, D, 1024><<<GRID, THREADS, 0, stream>>>(MODE, chunk, max_chunks, \
            ext, starts, (const T*)u, u_stride, v_off, prep, beta_buf, gate, gate_stride, norm_w, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out); }
#define DELTA_CASE(GRID, THREADS, MODE) { if (dim <= 32) DELTA_LAUNCH(32, GRID, THREADS, MODE) else if (dim <= 64) DELTA_LAUNCH(64, GRID, THREADS, MODE) \
        else if (dim <= 128) DELTA_LAUNCH(128, GRID, THREADS, MODE) else DELTA_LAUNCH(256, GRID, THREADS, MODE) }
    PALM_DTYPE_SWITCH(dtype, T, {
        delta_prep_kernel<T><<<dim3(n_tokens, heads), WAVE, 0, stream>>>((const T*)u, u_stride, q_off, k_off, (const T*)b, b_stride, a,
                                                                        a_stride, a_log, dt_bias, q_scale, unit_eps, heads, kv_heads,
                                                                        dim, pad, prep, beta_buf);
        if (chunk == 0) {
            DELTA_CASE(grid, threads, DELTA_WHOLE)
        } else {
            DELTA_CASE(dim3(heads, n_seqs * max_chunks, 2), local_threads, DELTA_LOCAL)
            delta_starts_kernel<<<dim3(heads, n_seqs, (vdim + DS_COLS - 1) / DS_COLS), DS_WAVES * WAVE, (size_t)dim * DS_COLS * sizeof(float), stream>>>(
                ext, starts, state, seq_slot, seq_new, chunk, max_chunks, heads, dim, vdim);
            DELTA_CASE(grid, threads, DELTA_FROM_STARTS)
        }
    });
#undef DELTA_CASE
#undef DELTA_LAUNCH
    PALM_LAUNCHED();
    return 0;
}
