// The residual stream of blocks that norm a branch's output instead of its input, and what such blocks need
// beside it: a weighted average over the results of all layers so far, and the xIELU activation.
//
//   add_normed   x[r] += y[r] / sqrt(mean(y[r]^2) + eps) * w      (statistics, product and sum in 32-bit)
//                then, if the layer averages over depth: results[J][r] = x[r];  x[r] = sum_j c[j] results[j][r], j = 0..J
//                then, if asked for, x[r] once more in the activation type for the branch that reads it next
//   xielu        z > 0: softplus(p) z^2 + z/2;   z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2
#include "common.h"

PALM_DEFINE_LAST_ERROR()

// One block per row.  The order of the norm's product is (y * r) * w, as in the norm that reads the stream.
template <typename TD, typename TO>
__global__ __launch_bounds__(256) void add_normed_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                                                         const float* __restrict__ w, float eps, int width,
                                                         float* __restrict__ results, const float* __restrict__ mix, int planes,
                                                         size_t plane_stride, TO* __restrict__ out) {
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    float* xr = x + r * width;
    const TD* dr = delta + r * width;
    float ss = 0.f;
    for (int d = threadIdx.x; d < width; d += blockDim.x) {
        const float v = to_float(dr[d]);
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    for (int d = threadIdx.x; d < width; d += blockDim.x) {
        float v = xr[d] + (to_float(dr[d]) * inv) * w[d];
        if (results) {
            float* rr = results + r * width + d;
            rr[(size_t)(planes - 1) * plane_stride] = v;
            float m = 0.f;
            for (int j = 0; j < planes - 1; ++j) m = fmaf(mix[j], rr[(size_t)j * plane_stride], m);
            v = fmaf(mix[planes - 1], v, m);
        }
        xr[d] = v;
        if (out) out[r * width + d] = from_float<TO>(v);
    }
}

PALM_API int palm_add_normed(hipStream_t stream, float* x, const void* delta, int delta_dtype, const float* w, float eps,
                             int n_rows, int width, float* results, const float* mix, int planes, long long plane_stride,
                             void* out, int out_dtype) {
    PALM_CHECK(n_rows >= 0 && width > 0, "add_normed: rows=%d width=%d", n_rows, width);
    PALM_CHECK((results == nullptr) == (mix == nullptr), "add_normed: results and their weights come together");
    PALM_CHECK(results == nullptr || (planes >= 1 && plane_stride >= (long long)n_rows * width),
               "add_normed: %d planes, %lld apart, for %d rows of %d", planes, plane_stride, n_rows, width);
    if (n_rows == 0) return 0;
    PALM_DTYPE_SWITCH(delta_dtype, TD,
        PALM_DTYPE_SWITCH(out_dtype, TO,
            add_normed_kernel<TD, TO><<<n_rows, 256, 0, stream>>>(x, (const TD*)delta, w, eps, width, results, mix, planes,
                                                                  (size_t)plane_stride, (TO*)out)));
    PALM_LAUNCHED();
    return 0;
}

// ---- xIELU ------------------------------------------------------------------------------------------
__device__ inline float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename T>
__global__ void xielu_kernel(const T* __restrict__ in, T* __restrict__ out, const float* __restrict__ pq, long long n) {
    const float a_pos = softplus_f(pq[0]), a_neg = 0.5f + softplus_f(pq[1]);
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        const float z = to_float(in[i]);
        const float y = z > 0.f ? fmaf(a_pos * z, z, 0.5f * z) : fmaf(a_neg, expm1f(z) - z, 0.5f * z);
        out[i] = from_float<T>(y);
    }
}

PALM_API int palm_xielu(hipStream_t stream, const void* in, void* out, int dtype, const float* pq, long long n) {
    PALM_CHECK(n >= 0, "xielu: %lld elements", n);
    if (n == 0) return 0;
    const int blocks = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
    PALM_DTYPE_SWITCH(dtype, T, xielu_kernel<T><<<blocks, 256, 0, stream>>>((const T*)in, (T*)out, pq, n));
    PALM_LAUNCHED();
    return 0;
}
