// The residual update of a layer whose norm comes after the sum, and small element-wise kernels.
//
// pulse_scale_add_rmsnorm, for each row:
//     v = alpha * h + ls * (d1 + d2)          (ls, d1, d2 optional; ls one factor a column)
//     h = v / sqrt(mean(v^2) + eps) * w       float32, in place
//     copy = h rounded to the activations' type (optional)
// pulse_activation: y = act(x) element by element (1: relu squared, 2: gelu with tanh, 3: silu).
// pulse_softcap: x <- cap * tanh(x / cap) in place on float32.
// pulse_round_rows: a float32 matrix once more in the activations' type.
#include "common.h"

#include <math.h>

namespace {

template <typename T1, typename T2, typename TW, typename TY>
__global__ void scale_add_rmsnorm_kernel(float* __restrict__ h, const T1* __restrict__ d1, const T2* __restrict__ d2,
                                         const TW* __restrict__ ls, const TW* __restrict__ w, TY* __restrict__ copy,
                                         int hidden, float alpha, float eps) {
    extern __shared__ float row_s[];
    __shared__ float scratch[16];
    const int64_t r = blockIdx.x;
    float* hrow = h + r * hidden;
    float ss = 0.f;
#pragma unroll 4
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        float v = alpha * hrow[i];
        float d = 0.f;
        if (d1) d += to_f32<T1>(d1[r * hidden + i]);
        if (d2) d += to_f32<T2>(d2[r * hidden + i]);
        if (ls) d *= to_f32<TW>(ls[i]);
        v += d;
        row_s[i] = v;
        ss = fmaf(v, v, ss);
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(hidden) + eps);
#pragma unroll 4
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float y = row_s[i] * inv * to_f32<TW>(w[i]);
        hrow[i] = y;
        if (copy) copy[r * hidden + i] = from_f32<TY>(y);
    }
}

template <typename T>
__global__ void activation_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n, int act) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float z = to_f32<T>(x[i]);
    float r;
    if (act == 1) { const float p = fmaxf(z, 0.f); r = p * p; }
    else if (act == 2) r = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    else r = z / (1.0f + expf(-z));
    y[i] = from_f32<T>(r);
}

__global__ void softcap_kernel(float* __restrict__ x, int64_t n, float cap) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

template <typename TY>
__global__ void round_rows_kernel(const float* __restrict__ x, TY* __restrict__ y, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) y[i] = from_f32<TY>(x[i]);
}

}  // namespace

extern "C" int pulse_scale_add_rmsnorm(float* h, const void* d1, int d1_dtype, const void* d2, int d2_dtype,
                                       const void* ls, const void* w, int w_dtype, void* copy, int copy_dtype, int rows,
                                       int hidden, float alpha, float eps, hipStream_t stream) {
    PULSE_REQUIRE(rows >= 0 && hidden > 0 && h && w, "scale_add_rmsnorm: bad arguments");
    PULSE_REQUIRE(pulse_dtype_ok(d1_dtype) && pulse_dtype_ok(d2_dtype) && pulse_dtype_ok(w_dtype) &&
                  pulse_dtype_ok(copy_dtype), "scale_add_rmsnorm: bad dtype tag");
    PULSE_REQUIRE(d1 || !d2, "scale_add_rmsnorm: a second update without a first");
    const size_t lds = sizeof(float) * static_cast<size_t>(hidden);
    PULSE_REQUIRE(lds <= 60 * 1024, "scale_add_rmsnorm: rows of %d values do not fit the workgroup's memory", hidden);
    if (rows == 0) return 0;
    const int threads = hidden >= 2048 || (rows <= 64 && hidden >= 1024) ? 1024 : 256;
    PULSE_DISPATCH_DTYPE(d1_dtype, T1, PULSE_DISPATCH_DTYPE(d2_dtype, T2, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        PULSE_DISPATCH_DTYPE(copy_dtype, TY,
            hipLaunchKernelGGL((scale_add_rmsnorm_kernel<T1, T2, TW, TY>), dim3(rows), dim3(threads), lds, stream, h,
                               static_cast<const T1*>(d1), static_cast<const T2*>(d2), static_cast<const TW*>(ls),
                               static_cast<const TW*>(w), static_cast<TY*>(copy), hidden, alpha, eps)))));
    PULSE_LAUNCH_CHECK("scale_add_rmsnorm");
    return 0;
}

extern "C" int pulse_activation(const void* x, void* y, int dtype, int64_t n, int act, hipStream_t stream) {
    PULSE_REQUIRE(n >= 0 && x && y && pulse_dtype_ok(dtype) && act >= 1 && act <= 3, "activation: bad arguments");
    if (n == 0) return 0;
    const int64_t blocks = (n + 255) / 256;
    PULSE_REQUIRE(blocks < (1ll << 31), "activation: too many elements");
    PULSE_DISPATCH_DTYPE(dtype, T, hipLaunchKernelGGL(activation_kernel<T>, dim3(static_cast<unsigned>(blocks)), dim3(256),
                                                      0, stream, static_cast<const T*>(x), static_cast<T*>(y), n, act));
    PULSE_LAUNCH_CHECK("activation");
    return 0;
}

extern "C" int pulse_softcap(float* x, int64_t n, float cap, hipStream_t stream) {
    PULSE_REQUIRE(n >= 0 && x && cap > 0.f, "softcap: bad arguments");
    if (n == 0) return 0;
    const int64_t blocks = (n + 255) / 256;
    PULSE_REQUIRE(blocks < (1ll << 31), "softcap: too many elements");
    hipLaunchKernelGGL(softcap_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, x, n, cap);
    PULSE_LAUNCH_CHECK("softcap");
    return 0;
}

extern "C" int pulse_round_rows(const float* x, void* y, int y_dtype, int64_t n, hipStream_t stream) {
    PULSE_REQUIRE(n >= 0 && x && y && pulse_dtype_ok(y_dtype), "round_rows: bad arguments");
    if (n == 0) return 0;
    const int64_t blocks = (n + 255) / 256;
    PULSE_REQUIRE(blocks < (1ll << 31), "round_rows: too many elements");
    PULSE_DISPATCH_DTYPE(y_dtype, TY, hipLaunchKernelGGL(round_rows_kernel<TY>, dim3(static_cast<unsigned>(blocks)),
                                                         dim3(256), 0, stream, x, static_cast<TY*>(y), n));
    PULSE_LAUNCH_CHECK("round_rows");
    return 0;
}

// ---------------------------------------------------------------- xIELU
// y = a z^2 + z / 2 for z > 0, else b (exp(z) - 1 - z) + z / 2, with a = softplus(p), b = 1/2 + softplus(q) and the two
// learned numbers p, q read on the device.
namespace {

__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

template <typename T, typename TP>
__global__ void xielu_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n, const TP* __restrict__ pq) {
    __shared__ float ab[2];   // the two factors, formed once a workgroup
    if (threadIdx.x == 0) {
        ab[0] = softplus_f(to_f32<TP>(pq[0]));
        ab[1] = 0.5f + softplus_f(to_f32<TP>(pq[1]));
    }
    __syncthreads();
    const float a = ab[0], b = ab[1];
    const int64_t first = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t i = first + u;
        if (i < n) {
            const float z = to_f32<T>(x[i]);
            y[i] = from_f32<T>(z > 0.f ? fmaf(a * z, z, 0.5f * z) : fmaf(b, expm1f(z) - z, 0.5f * z));
        }
    }
}

}  // namespace

extern "C" int pulse_xielu(const void* x, void* y, int dtype, int64_t n, const void* pq, int pq_dtype, hipStream_t stream) {
    PULSE_REQUIRE(n >= 0 && x && y && pq && pulse_dtype_ok(dtype) && pulse_dtype_ok(pq_dtype), "xielu: bad arguments");
    if (n == 0) return 0;
    const int64_t blocks = (n + 1023) / 1024;   // four neighbouring elements a thread
    PULSE_REQUIRE(blocks < (1ll << 31), "xielu: too many elements");
    PULSE_DISPATCH_DTYPE(dtype, T, PULSE_DISPATCH_DTYPE(pq_dtype, TP,
        hipLaunchKernelGGL((xielu_kernel<T, TP>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                           static_cast<const T*>(x), static_cast<T*>(y), n, static_cast<const TP*>(pq))));
    PULSE_LAUNCH_CHECK("xielu");
    return 0;
}
