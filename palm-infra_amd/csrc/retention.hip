// Retention: linear attention with one fixed decay per head, no softmax and no denominator.
//
//   S_t = g_h S_(t-1) + k_t v_t^T        S: [dim, vdim] per sequence and head, 32-bit, kept between steps
//   o_t = S_t^T q_t
//   out_t = o_t / sqrt(mean_v(o_t^2) + eps) * silu(gate_t)         (the unit norm is per head)
//
// q and k are rotated first (pairs (i, i + rot/2) of the first `rot` dimensions, cos/sin rows of the tokens'
// positions) and k is multiplied by k_scale after the rotation; rotated values, state and sums are 32-bit.
//
// One block per (head, sequence), one thread per value dimension v: the thread keeps column v of S in
// registers and walks over the sequence's new tokens, a tile of them at a time: the block rotates the tile's
// q and k into LDS, every thread then does its column's updates and dot products for the tile's tokens, and the
// per-token sums of squares over v are reduced for the whole tile at once.  A prompt and a single token run
// the same code, so a prompt leaves the state that its tokens one by one leave.
#include "common.h"

constexpr int RET_TILE = 8;

template <typename T, int DMAX>
__global__ void retention_kernel(const T* __restrict__ qkvg, int row_stride, int q_off, int k_off, int v_off, int g_off,
                                 const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot,
                                 const float* __restrict__ decay, float k_scale, float eps,
                                 float* __restrict__ state, const int* __restrict__ seq_slot,
                                 const int* __restrict__ seq_new, const int* __restrict__ cu_new,
                                 int heads, int dim, int vdim, T* __restrict__ out) {
    __shared__ float q_s[RET_TILE][DMAX], k_s[RET_TILE][DMAX];
    __shared__ float red[RET_TILE][16];
    const int h = blockIdx.x, b = blockIdx.y;
    const int v = threadIdx.x;
    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE, n_waves = blockDim.x / WAVE;
    const int n_new = seq_new[b], row0 = cu_new[b];
    const bool mine = v < vdim;
    const float g = decay[h];
    const int half = rot / 2;
    float* sp = state + (((size_t)seq_slot[b] * heads + h) * dim) * vdim + v;

    float S[DMAX];
#pragma unroll
    for (int d = 0; d < DMAX; ++d) S[d] = (mine && d < dim) ? sp[(size_t)d * vdim] : 0.f;

    for (int t0 = 0; t0 < n_new; t0 += RET_TILE) {
        const int tt = min(RET_TILE, n_new - t0);
        for (int idx = threadIdx.x; idx < tt * dim; idx += blockDim.x) {
            const int ti = idx / dim, d = idx % dim;
            const size_t row = (size_t)(row0 + t0 + ti);
            const T* qr = qkvg + row * row_stride + q_off + h * dim;
            const T* kr = qkvg + row * row_stride + k_off + h * dim;
            float qv = to_float(qr[d]), kv = to_float(kr[d]);
            if (d < rot) {
                const int i = d < half ? d : d - half;
                const float c = cos_t[row * half + i], s = sin_t[row * half + i];
                const int partner = d < half ? d + half : d - half;
                const float qp = to_float(qr[partner]), kp = to_float(kr[partner]);
                // the pair (u, w) becomes (u c - w s, w c + u s)
                qv = d < half ? qv * c - qp * s : qv * c + qp * s;
                kv = d < half ? kv * c - kp * s : kv * c + kp * s;
            }
            q_s[ti][d] = qv;
            k_s[ti][d] = kv * k_scale;
        }
        __syncthreads();
        float o[RET_TILE];
#pragma unroll
        for (int ti = 0; ti < RET_TILE; ++ti) {
            o[ti] = 0.f;
            if (ti < tt) {
                const size_t row = (size_t)(row0 + t0 + ti);
                const float vv = mine ? to_float(qkvg[row * row_stride + v_off + h * vdim + v]) : 0.f;
                float acc = 0.f;
#pragma unroll
                for (int d = 0; d < DMAX; ++d) {
                    if (d < dim) {
                        S[d] = fmaf(g, S[d], k_s[ti][d] * vv);
                        acc = fmaf(S[d], q_s[ti][d], acc);
                    }
                }
                o[ti] = acc;
            }
            const float ss = wave_sum(o[ti] * o[ti]);
            if (lane == 0) red[ti][wave] = ss;
        }
        __syncthreads();
#pragma unroll
        for (int ti = 0; ti < RET_TILE; ++ti) {
            if (ti < tt && mine) {
                float total = 0.f;
                for (int w = 0; w < n_waves; ++w) total += red[ti][w];
                const float inv = 1.0f / sqrtf(total / (float)vdim + eps);
                const size_t row = (size_t)(row0 + t0 + ti);
                const float gate = to_float(qkvg[row * row_stride + g_off + h * vdim + v]);
                out[row * ((size_t)heads * vdim) + h * vdim + v] = from_float<T>(o[ti] * inv * (gate / (1.0f + expf(-gate))));
            }
        }
        __syncthreads();
    }
    if (mine && n_new > 0) {
#pragma unroll
        for (int d = 0; d < DMAX; ++d)
            if (d < dim) sp[(size_t)d * vdim] = S[d];
    }
}

template <typename T>
static int retention_launch(hipStream_t stream, dim3 grid, int threads, const T* qkvg, int row_stride, int q_off, int k_off,
                            int v_off, int g_off, const float* cos_t, const float* sin_t, int rot, const float* decay,
                            float k_scale, float eps, float* state, const int* seq_slot, const int* seq_new,
                            const int* cu_new, int heads, int dim, int vdim, T* out) {
#define RET_CASE(D) retention_kernel<T, D><<<grid, threads, 0, stream>>>(qkvg, row_stride, q_off, k_off, v_off, g_off, cos_t, \
        sin_t, rot, decay, k_scale, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, out)
    if (dim <= 16) RET_CASE(16);
    else if (dim <= 32) RET_CASE(32);
    else if (dim <= 64) RET_CASE(64);
    else if (dim <= 128) RET_CASE(128);
    else RET_CASE(256);
#undef RET_CASE
    return 0;
}

PALM_API int palm_retention(hipStream_t stream, const void* qkvg, int dtype, int row_stride, int q_off, int k_off, int v_off,
                            int g_off, const float* cos_t, const float* sin_t, int rot, const float* decay, float k_scale,
                            float eps, float* state, const int* seq_slot, const int* seq_new, const int* cu_new, int n_seqs,
                            int heads, int dim, int vdim, void* out) {
    PALM_CHECK(n_seqs >= 0 && heads > 0 && dim > 0 && vdim > 0, "retention: seqs=%d heads=%d dim=%d vdim=%d", n_seqs, heads, dim, vdim);
    PALM_CHECK(dim <= 256, "retention: a key size of %d exceeds 256", dim);
    PALM_CHECK(vdim <= 1024, "retention: a value size of %d exceeds 1024", vdim);
    PALM_CHECK(rot >= 0 && rot <= dim && rot % 2 == 0, "retention: %d rotated dimensions of %d", rot, dim);
    PALM_CHECK(rot == 0 || (cos_t && sin_t), "retention: a rotation needs its cos and sin rows");
    PALM_CHECK(heads <= 65535 && n_seqs <= 65535, "retention: %d heads / %d sequences are more than one launch takes", heads, n_seqs);
    if (n_seqs == 0) return 0;
    const int threads = (vdim + WAVE - 1) / WAVE * WAVE;
    dim3 grid(heads, n_seqs);
    PALM_DTYPE_SWITCH(dtype, T,
        retention_launch<T>(stream, grid, threads, (const T*)qkvg, row_stride, q_off, k_off, v_off, g_off, cos_t, sin_t, rot,
                            decay, k_scale, eps, state, seq_slot, seq_new, cu_new, heads, dim, vdim, (T*)out));
    PALM_LAUNCHED();
    return 0;
}
