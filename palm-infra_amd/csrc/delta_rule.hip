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

template <typename T, int DMAX, int MAXT>
__global__ __launch_bounds__(MAXT) void delta_rule_kernel(const T* __restrict__ u, int u_stride, int v_off,
                                                          const float* __restrict__ prep, const float* __restrict__ beta,
                                                          const float* __restrict__ gate, int gate_stride,
                                                          const float* __restrict__ norm_w, float eps,
                                                          float* __restrict__ state, const int* __restrict__ seq_slot,
                                                          const int* __restrict__ seq_new, const int* __restrict__ cu_new,
                                                          int heads, int dim, int vdim, T* __restrict__ out) {
    __shared__ float red[DELTA_TILE][16];
    __shared__ float o_s[DELTA_TILE][MAXT];
    constexpr int QREGS = (DMAX + WAVE - 1) / WAVE;
    const int h = blockIdx.x, b = blockIdx.y;
    const int v = threadIdx.x;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    const int n_new = seq_new[b];
    if (n_new <= 0) return;
    const int row0 = cu_new[b];
    const bool mine = v < vdim;
    const int vc = min(v, vdim - 1);
    float* sp = state + (((size_t)seq_slot[b] * heads + h) * dim) * vdim + vc;

    // unconditional reads of rows and a column that exist; what does not belong is set to zero after
    float S[DMAX];
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
        const float s0 = sp[(size_t)min(d, dim - 1) * vdim];
        S[d] = (!mine || d >= dim) ? 0.f : s0;
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
            if (!mine) vv = 0.f;
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
            o_s[ti][v] = acc;
            const float ss = wave_sum(acc * acc);
            if (lane == 0) red[ti][wave] = ss;
            vv = vn;
            bt = bn;
#pragma unroll
            for (int c = 0; c < QREGS; ++c) { qv[c] = qn[c]; kv[c] = kn[c]; gv[c] = gn[c]; }
        }
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
    if (mine) {
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
            if (d < dim) sp[(size_t)d * vdim] = S[d];
    }
}

PALM_API int palm_delta_pad(int dim) { return dim <= 32 ? 32 : dim <= 64 ? 64 : dim <= 128 ? 128 : 256; }

// u: the convolution's output [n, u_stride] holding q at q_off (kv_heads * dim), k at k_off, v at v_off (heads * vdim);
// b: the write strengths before the sigmoid, [n, b_stride] of the same type, one a head; a: float32 [n, a_stride], the
// decays' rows before bias and softplus (heads * dim); gate: float32 [n, gate_stride], the output gate before the
// sigmoid (heads * vdim).  prep: room for n * heads * 3 * palm_delta_pad(dim) floats, beta_buf: n * heads floats.
PALM_API int palm_delta_rule(hipStream_t stream, const void* u, int dtype, int u_stride, int q_off, int k_off, int v_off,
                             const void* b, int b_stride, const float* a, int a_stride, const float* gate, int gate_stride,
                             const float* a_log, const float* dt_bias, const float* norm_w, float q_scale, float unit_eps,
                             float eps, float* state, const int* seq_slot, const int* seq_new, const int* cu_new, int n_seqs,
                             int heads, int kv_heads, int dim, int vdim, void* out, int n_tokens, float* prep, float* beta_buf) {
    PALM_CHECK(n_seqs >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, "delta_rule: seqs=%d heads=%d kv=%d dim=%d vdim=%d",
               n_seqs, heads, kv_heads, dim, vdim);
    PALM_CHECK(heads % kv_heads == 0, "delta_rule: %d heads are not a multiple of %d q/k heads", heads, kv_heads);
    PALM_CHECK(dim <= 256, "delta_rule: a key size of %d exceeds 256", dim);
    PALM_CHECK(vdim <= 1024, "delta_rule: a value size of %d exceeds 1024", vdim);
    PALM_CHECK(n_tokens >= 0 && (n_tokens == 0 || (prep && beta_buf)), "delta_rule: the prepared rows need their room");
    if (n_seqs == 0 || n_tokens == 0) return 0;
    PALM_CHECK(heads <= 65535 && n_seqs <= 65535, "delta_rule: %d heads / %d sequences are more than one launch takes", heads, n_seqs);
    const int threads = (vdim + WAVE - 1) / WAVE * WAVE;
    const int pad = palm_delta_pad(dim);
    dim3 grid(heads, n_seqs);
#define DELTA_CASE(D) { if (threads <= 256) delta_rule_kernel<T, D, 256><<<grid, threads, 0, stream>>>((const T*)u, u_stride, v_off, prep, \
            beta_buf, gate, gate_stride, norm_w, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out); \
        else delta_rule_kernel<T, D, 1024><<<grid, threads, 0, stream>>>((const T*)u, u_stride, v_off, prep, \
            beta_buf, gate, gate_stride, norm_w, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out); }
    PALM_DTYPE_SWITCH(dtype, T, {
        delta_prep_kernel<T><<<dim3(n_tokens, heads), WAVE, 0, stream>>>((const T*)u, u_stride, q_off, k_off, (const T*)b, b_stride, a,
                                                                        a_stride, a_log, dt_bias, q_scale, unit_eps, heads, kv_heads,
                                                                        dim, pad, prep, beta_buf);
        if (dim <= 32) DELTA_CASE(32)
        else if (dim <= 64) DELTA_CASE(64)
        else if (dim <= 128) DELTA_CASE(128)
        else DELTA_CASE(256)
    });
#undef DELTA_CASE
    PALM_LAUNCHED();
    return 0;
}
