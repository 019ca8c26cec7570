// The residual stream of blocks that norm a branch on both sides and scale what they add:
//
//   add_normed_scaled   x[r] += gain * (y[r] / sqrt(mean(y[r]^2) + eps) * w)             (all in 32-bit)
//                       then, if the next reader's norm is given:  out[r] = x[r] / sqrt(mean(x[r]^2) + eps2) * w2
//   softcap             z <- cap * tanh(z / cap), in place, 32-bit
//
// One block per row; a row's values stay in registers between the passes where the row is at most
// ADDN_KEEP * 256 wide, and are read again from the stream beyond.
#include "common.h"

constexpr int ADDN_THREADS = 256;
constexpr int ADDN_KEEP = 16;

template <typename TD, typename TO>
__global__ __launch_bounds__(ADDN_THREADS) void add_normed_scaled_kernel(
    float* __restrict__ x, const TD* __restrict__ delta, const float* __restrict__ w, float eps, float gain, int width,
    const float* __restrict__ next_w, float next_eps, TO* __restrict__ out) {
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    float* xr = x + r * width;
    const TD* dr = delta + r * width;
    const bool keep = width <= ADDN_KEEP * ADDN_THREADS;
    float held[ADDN_KEEP];
    float ss = 0.f;
    if (keep) {
#pragma unroll
        for (int i = 0; i < ADDN_KEEP; ++i) {
            const int d = i * ADDN_THREADS + threadIdx.x;
            held[i] = d < width ? to_float(dr[d]) : 0.f;
            ss += held[i] * held[i];
        }
    } else {
        for (int d = threadIdx.x; d < width; d += ADDN_THREADS) {
            const float v = to_float(dr[d]);
            ss += v * v;
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    float ss2 = 0.f;
    if (keep) {
#pragma unroll
        for (int i = 0; i < ADDN_KEEP; ++i) {
            const int d = i * ADDN_THREADS + threadIdx.x;
            if (d < width) {
                const float v = fmaf(gain, (held[i] * inv) * w[d], xr[d]);
                xr[d] = v;
                held[i] = v;
                ss2 += v * v;
            }
        }
    } else {
        for (int d = threadIdx.x; d < width; d += ADDN_THREADS) {
            const float v = fmaf(gain, (to_float(dr[d]) * inv) * w[d], xr[d]);
            xr[d] = v;
            ss2 += v * v;
        }
    }
    if (!out) return;
    ss2 = block_sum(ss2, scratch);
    const float inv2 = 1.0f / sqrtf(ss2 / (float)width + next_eps);
    if (keep) {
#pragma unroll
        for (int i = 0; i < ADDN_KEEP; ++i) {
            const int d = i * ADDN_THREADS + threadIdx.x;
            if (d < width) out[r * width + d] = from_float<TO>((held[i] * inv2) * next_w[d]);
        }
    } else {
        for (int d = threadIdx.x; d < width; d += ADDN_THREADS)            // a thread reads back what it wrote itself
            out[r * width + d] = from_float<TO>((xr[d] * inv2) * next_w[d]);
    }
}

// delta: [n, width] of delta_dtype; out (may be null, then next_w is not read): [n, width] of out_dtype.
PALM_API int palm_add_normed_scaled(hipStream_t stream, float* x, const void* delta, int delta_dtype, const float* w, float eps,
                                    float gain, int n, int width, const float* next_w, float next_eps, void* out, int out_dtype) {
    PALM_CHECK(n >= 0 && width > 0, "add_normed_scaled: n=%d width=%d", n, width);
    PALM_CHECK(x && delta && w, "add_normed_scaled: the stream, the branch's rows and the norm's weight are needed");
    PALM_CHECK(!out || next_w, "add_normed_scaled: rows for the next reader need that reader's norm weight");
    if (n == 0) return 0;
    PALM_DTYPE_SWITCH(delta_dtype, TD, {
        PALM_DTYPE_SWITCH(out_dtype, TO, {
            add_normed_scaled_kernel<TD, TO><<<n, ADDN_THREADS, 0, stream>>>(x, (const TD*)delta, w, eps, gain, width, next_w,
                                                                            next_eps, (TO*)out);
        });
    });
    PALM_LAUNCHED();
    return 0;
}

__global__ void softcap_kernel(float* __restrict__ z, float cap, long long count) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) z[i] = cap * tanhf(z[i] / cap);
}

PALM_API int palm_softcap(hipStream_t stream, float* z, float cap, long long count) {
    PALM_CHECK(count >= 0 && cap > 0.f, "softcap: count=%lld cap=%g", count, (double)cap);
    if (count == 0) return 0;
    softcap_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(z, cap, count);
    PALM_LAUNCHED();
    return 0;
}
