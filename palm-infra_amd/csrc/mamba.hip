// The selective scan of a Mamba layer and the short causal convolution in front of it.
//
//   conv     u_t[c] = silu(bias[c] + sum_j w[c][j] x_(t - (taps-1) + j)[c]),  j = 0 .. taps-1 (the last column is the current
//            token's); inputs before the sequence's start are zero; the last taps-1 inputs are kept per sequence.
//   scan     dt_t[c] = softplus(dtl_t[c] + dt_bias[c]);   A[c][n] = -exp(A_log[c][n])
//            S_t[c][n] = exp(dt_t[c] A[c][n]) S_(t-1)[c][n] + dt_t[c] u_t[c] B_t[n]
//            y_t[c] = (sum_n S_t[c][n] C_t[n] + D[c] u_t[c]) * silu(z_t[c])
//
// S is 32-bit and kept per sequence; step sizes, decays, exponentials and the sums are 32-bit.  Both kernels walk
// over a sequence's new tokens whatever their number: a prompt leaves what its tokens one by one leave.
#include "common.h"

constexpr int CONV_MAX_TAPS = 16;

__device__ inline float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ inline float softplus_dt(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// One thread per (token of a sequence, channel): grid (channel blocks, longest run of new tokens, sequences).
template <typename T>
__global__ void causal_conv_kernel(const T* __restrict__ x, int x_stride, const float* __restrict__ w,
                                   const float* __restrict__ bias, const float* __restrict__ conv_state,
                                   const int* __restrict__ seq_slot, const int* __restrict__ seq_new,
                                   const int* __restrict__ cu_new, int channels, int taps, T* __restrict__ out) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, ti = blockIdx.y, b = blockIdx.z;
    if (c >= channels || ti >= seq_new[b]) return;
    const size_t row0 = (size_t)cu_new[b];
    const float* st = conv_state + (size_t)seq_slot[b] * (taps - 1) * channels;      // [taps-1, channels], oldest first
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int at = ti - (taps - 1) + j;                 // index among the step's tokens; negative: from the state
        const float v = at >= 0 ? to_float(x[(row0 + at) * x_stride + c]) : st[(size_t)(taps - 1 + at) * channels + c];
        acc = fmaf(w[(size_t)c * taps + j], v, acc);
    }
    out[(row0 + ti) * channels + c] = from_float<T>(silu_f(acc));
}

// After the convolution has read the old state: the last taps-1 inputs of each sequence, old ones moved up.
template <typename T>
__global__ void conv_state_kernel(const T* __restrict__ x, int x_stride, float* __restrict__ conv_state,
                                  const int* __restrict__ seq_slot, const int* __restrict__ seq_new,
                                  const int* __restrict__ cu_new, int channels, int taps) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    if (c >= channels) return;
    const int n_new = seq_new[b];
    if (n_new <= 0) return;
    const size_t row0 = (size_t)cu_new[b];
    float* st = conv_state + (size_t)seq_slot[b] * (taps - 1) * channels;
    float keep[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
        if (j < taps - 1) {
            const int at = n_new - (taps - 1) + j;
            keep[j] = at >= 0 ? to_float(x[(row0 + at) * x_stride + c]) : st[(size_t)(taps - 1 + at) * channels + c];
        }
    }
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j)
        if (j < taps - 1) st[(size_t)j * channels + c] = keep[j];
}

PALM_API int palm_causal_conv(hipStream_t stream, const void* x, int dtype, int x_stride, const float* w, const float* bias,
                              float* conv_state, const int* seq_slot, const int* seq_new, const int* cu_new, int n_seqs,
                              int max_new, int channels, int taps, void* out) {
    PALM_CHECK(n_seqs >= 0 && max_new >= 0 && channels > 0, "causal_conv: seqs=%d max_new=%d channels=%d", n_seqs, max_new, channels);
    PALM_CHECK(taps >= 1 && taps <= CONV_MAX_TAPS, "causal_conv: %d taps (1 to %d)", taps, CONV_MAX_TAPS);
    PALM_CHECK(n_seqs <= 65535 && max_new <= 65535, "causal_conv: %d sequences / %d tokens are more than one launch takes", n_seqs, max_new);
    if (n_seqs == 0 || max_new == 0) return 0;
    const int threads = 256, cb = (channels + threads - 1) / threads;
    PALM_DTYPE_SWITCH(dtype, T, {
        causal_conv_kernel<T><<<dim3(cb, max_new, n_seqs), threads, 0, stream>>>(
            (const T*)x, x_stride, w, bias, conv_state, seq_slot, seq_new, cu_new, channels, taps, (T*)out);
        if (taps > 1)
            conv_state_kernel<T><<<dim3(cb, n_seqs), threads, 0, stream>>>((const T*)x, x_stride, conv_state, seq_slot, seq_new,
                                                                          cu_new, channels, taps);
    });
    PALM_LAUNCHED();
    return 0;
}

// ---- the scan ---------------------------------------------------------------------------------------
// A channel's row of S is spread over a group of G lanes (G a power of two, at most 64, chosen from the state
// size): lane j of the group holds states j, j + G, ..; a block of four waves serves 256 / G channels.  The block
// walks over a sequence's new tokens a tile at a time, in three phases with a barrier between them:
//   in     all threads bring the tile's inputs into LDS with reads that follow the memory's rows: B_t and C_t (the
//          same for all channels), and for the block's channels u_t and the step size softplus(dtl_t + bias),
//          computed once for each (token, channel)
//   scan   for every token a lane updates its states from LDS and the group adds up its part of y with shuffles;
//          nothing but the multiply-add on S waits for the token before it, so the exponentials of a tile overlap
//   out    all threads add the skip term, gate with silu(z_t) and store the tile's outputs row by row
constexpr int SCAN_TILE = 16;

// Sum over groups of G consecutive lanes (G a power of two), every lane gets its group's sum.  Within a row of 16
// lanes the partners come through the data-parallel lane crossbar of the vector unit (one instruction a step: quads
// swap, halves of 8 and rows of 16 mirror: any pairing of disjoint partial sums does); only steps across rows go
// through the permute unit.
template <int CTRL> __device__ inline float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
template <int G> __device__ inline float group_sum(float y) {
    if constexpr (G >= 2) y += dpp_move<0xB1>(y);            // quad_perm [1, 0, 3, 2]
    if constexpr (G >= 4) y += dpp_move<0x4E>(y);            // quad_perm [2, 3, 0, 1]
    if constexpr (G >= 8) y += dpp_move<0x141>(y);           // row_half_mirror
    if constexpr (G >= 16) y += dpp_move<0x140>(y);          // row_mirror
    if constexpr (G >= 32) y += __shfl_xor(y, 16, WAVE);
    if constexpr (G >= 64) y += __shfl_xor(y, 32, WAVE);
    return y;
}
constexpr int SCAN_WAVES = 4;
constexpr int SCAN_THREADS = SCAN_WAVES * WAVE;

template <typename T, int G, int PER>
__global__ __launch_bounds__(SCAN_THREADS) void selective_scan_kernel(
    const T* __restrict__ u, const T* __restrict__ z, int z_stride, const T* __restrict__ bc, int bc_stride, int b_off, int c_off,
    const float* __restrict__ dtl, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const float* __restrict__ d_skip, float* __restrict__ state, const int* __restrict__ seq_slot,
    const int* __restrict__ seq_new, const int* __restrict__ cu_new, int channels, int n_state, T* __restrict__ out) {
    constexpr int CH = SCAN_THREADS / G;               // channels of a block
    constexpr int NP = G * PER;                        // the state size, padded
    __shared__ float b_s[SCAN_TILE][NP], c_s[SCAN_TILE][NP];
    __shared__ float dt_s[SCAN_TILE][CH], u_s[SCAN_TILE][CH], y_s[SCAN_TILE][CH];
    const int j = threadIdx.x % G, ch = threadIdx.x / G;
    const int c0 = blockIdx.x * CH, b = blockIdx.y;
    const int c = c0 + ch;
    const bool mine = c < channels;
    const int cc = mine ? c : channels - 1;
    const int n_new = seq_new[b];
    const size_t row0 = (size_t)cu_new[b];
    float* sp = state + ((size_t)seq_slot[b] * channels + cc) * n_state;
    float S[PER], A[PER];
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int n = j + k * G;
        S[k] = n < n_state ? sp[n] : 0.f;
        A[k] = n < n_state ? -expf(a_log[(size_t)cc * n_state + n]) : 0.f;
    }
    for (int t0 = 0; t0 < n_new; t0 += SCAN_TILE) {
        const int tt = min(SCAN_TILE, n_new - t0);
        for (int idx = threadIdx.x; idx < tt * NP; idx += SCAN_THREADS) {
            const int ti = idx / NP, n = idx % NP;
            const T* r = bc + (row0 + t0 + ti) * bc_stride;
            b_s[ti][n] = n < n_state ? to_float(r[b_off + n]) : 0.f;
            c_s[ti][n] = n < n_state ? to_float(r[c_off + n]) : 0.f;
        }
        for (int idx = threadIdx.x; idx < tt * CH; idx += SCAN_THREADS) {
            const int ti = idx / CH, k = idx % CH;
            const int ck = min(c0 + k, channels - 1);
            const size_t row = row0 + t0 + ti;
            dt_s[ti][k] = softplus_dt(dtl[row * channels + ck] + dt_bias[ck]);
            u_s[ti][k] = to_float(u[row * channels + ck]);
        }
        __syncthreads();
#define SCAN_TOKEN(ti) { \
            const float dt = dt_s[ti][ch]; \
            const float du = dt * u_s[ti][ch]; \
            float y = 0.f; \
            _Pragma("unroll") for (int k = 0; k < PER; ++k) { \
                const int n = j + k * G; \
                S[k] = fmaf(expf(dt * A[k]), S[k], du * b_s[ti][n]);        /* beyond the state size A, B and C are zero */ \
                y = fmaf(S[k], c_s[ti][n], y); \
            } \
            y = group_sum<G>(y); \
            if (j == 0) y_s[ti][ch] = y; }
        if (tt == SCAN_TILE) {                                  // a whole tile: no test between its tokens
#pragma unroll
            for (int ti = 0; ti < SCAN_TILE; ++ti) SCAN_TOKEN(ti)
        } else {
#pragma unroll
            for (int ti = 0; ti < SCAN_TILE; ++ti)
                if (ti < tt) SCAN_TOKEN(ti)
        }
#undef SCAN_TOKEN
        __syncthreads();
        for (int idx = threadIdx.x; idx < tt * CH; idx += SCAN_THREADS) {
            const int ti = idx / CH, k = idx % CH;
            if (c0 + k < channels) {
                const size_t row = row0 + t0 + ti;
                const float y = fmaf(d_skip[c0 + k], u_s[ti][k], y_s[ti][k]);
                out[row * channels + c0 + k] = from_float<T>(y * silu_f(to_float(z[row * z_stride + c0 + k])));
            }
        }
        __syncthreads();
    }
    if (mine && n_new > 0) {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int n = j + k * G;
            if (n < n_state) sp[n] = S[k];
        }
    }
}

PALM_API int palm_selective_scan(hipStream_t stream, const void* u, const void* z, int z_stride, const void* bc, int bc_stride,
                                 int b_off, int c_off, int dtype, const float* dtl, const float* dt_bias, const float* a_log,
                                 const float* d_skip, float* state, const int* seq_slot, const int* seq_new, const int* cu_new,
                                 int n_seqs, int channels, int n_state, void* out) {
    PALM_CHECK(n_seqs >= 0 && channels > 0 && n_state > 0, "selective_scan: seqs=%d channels=%d state=%d", n_seqs, channels, n_state);
    PALM_CHECK(n_state <= 256, "selective_scan: a state of %d per channel exceeds 256", n_state);
    PALM_CHECK(n_seqs <= 65535, "selective_scan: %d sequences are more than one launch takes", n_seqs);
    if (n_seqs == 0) return 0;
#define SCAN_CASE(G, PER) { \
        const int per_block = SCAN_THREADS / G; \
        dim3 grid((channels + per_block - 1) / per_block, n_seqs); \
        selective_scan_kernel<T, G, PER><<<grid, SCAN_THREADS, 0, stream>>>((const T*)u, (const T*)z, z_stride, \
            (const T*)bc, bc_stride, b_off, c_off, dtl, dt_bias, a_log, d_skip, state, seq_slot, seq_new, cu_new, channels, n_state, (T*)out); }
    PALM_DTYPE_SWITCH(dtype, T, {
        if (n_state <= 4) SCAN_CASE(4, 1)
        else if (n_state <= 8) SCAN_CASE(8, 1)
        else if (n_state <= 16) SCAN_CASE(16, 1)
        else if (n_state <= 32) SCAN_CASE(32, 1)
        else if (n_state <= 64) SCAN_CASE(64, 1)
        else if (n_state <= 128) SCAN_CASE(64, 2)
        else SCAN_CASE(64, 4)
    });
#undef SCAN_CASE
    PALM_LAUNCHED();
    return 0;
}
