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

// The same for widths that are a multiple of four: a thread owns groups of four neighbouring values, reads each plane's
// four at once, and a block has threads enough that a row of some thousand values is one or two groups a thread: all
// reads of a row are under way together (a decode step's rows are few, and the kernel's time is the latency of its reads).
constexpr int ADD_NORMED_GROUPS = 4;                   // groups of four a thread holds at most (rows up to 16,384 wide)

__device__ inline void load4f(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ inline void load4f(const bf16_t* p, float (&v)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ inline void store4f(float* p, const float (&v)[4]) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
__device__ inline void store4f(bf16_t* p, const float (&v)[4]) {
    uint2 t;
    t.x = (uint32_t)f32_to_bf16(v[0]).bits | ((uint32_t)f32_to_bf16(v[1]).bits << 16);
    t.y = (uint32_t)f32_to_bf16(v[2]).bits | ((uint32_t)f32_to_bf16(v[3]).bits << 16);
    *reinterpret_cast<uint2*>(p) = t;
}

template <typename TD, typename TO>
__global__ __launch_bounds__(1024) void add_normed_wide_kernel(float* __restrict__ x, const TD* __restrict__ delta,
                                                               const float* __restrict__ w, float eps, int width,
                                                               float* __restrict__ results, const float* __restrict__ mix, int planes,
                                                               size_t plane_stride, TO* __restrict__ out) {
    __shared__ float scratch[16];
    const size_t r = blockIdx.x;
    float y[ADD_NORMED_GROUPS][4], xv[ADD_NORMED_GROUPS][4], wv[ADD_NORMED_GROUPS][4], m[ADD_NORMED_GROUPS][4];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ADD_NORMED_GROUPS; ++it) {
        const int d = (it * blockDim.x + threadIdx.x) * 4;
        const int at = d < width ? d : 0;               // a thread beyond the row reads its start and adds nothing
        load4f(delta + r * width + at, y[it]);
        load4f(x + r * width + at, xv[it]);
        load4f(w + at, wv[it]);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            m[it][e] = 0.f;
            if (d < width) ss += y[it][e] * y[it][e];
        }
    }
    if (results) {
        for (int j = 0; j < planes - 1; ++j) {          // the planes below the layer's own, one after the other
            const float c = mix[j];
#pragma unroll
            for (int it = 0; it < ADD_NORMED_GROUPS; ++it) {
                const int d = (it * blockDim.x + threadIdx.x) * 4;
                float p[4];
                load4f(results + (size_t)j * plane_stride + r * width + (d < width ? d : 0), p);
#pragma unroll
                for (int e = 0; e < 4; ++e) m[it][e] = fmaf(c, p[e], m[it][e]);
            }
        }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    const float last = results ? mix[planes - 1] : 0.f;
#pragma unroll
    for (int it = 0; it < ADD_NORMED_GROUPS; ++it) {
        const int d = (it * blockDim.x + threadIdx.x) * 4;
        if (d >= width) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = xv[it][e] + (y[it][e] * inv) * wv[it][e];
        if (results) {
            store4f(results + (size_t)(planes - 1) * plane_stride + r * width + d, v);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = fmaf(last, v[e], m[it][e]);
        }
        store4f(x + r * width + d, v);
        if (out) store4f(out + r * width + d, v);
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
    // groups of four a thread: as many threads as the row has groups, up to 1024
    const int groups = width / 4, threads = groups >= 1024 ? 1024 : (groups + WAVE - 1) / WAVE * WAVE;
    const bool wide = width % 4 == 0 && groups > 0 && (groups + threads - 1) / threads <= ADD_NORMED_GROUPS;
    PALM_DTYPE_SWITCH(delta_dtype, TD,
        PALM_DTYPE_SWITCH(out_dtype, TO, {
            if (wide)
                add_normed_wide_kernel<TD, TO><<<n_rows, threads, 0, stream>>>(x, (const TD*)delta, w, eps, width, results, mix, planes,
                                                                              (size_t)plane_stride, (TO*)out);
            else
                add_normed_kernel<TD, TO><<<n_rows, 256, 0, stream>>>(x, (const TD*)delta, w, eps, width, results, mix, planes,
                                                                      (size_t)plane_stride, (TO*)out);
        }));
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
