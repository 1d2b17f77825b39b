// Mixing the heads' attention weights ("talking heads"), done behind the attention kernel.
//
// With weights a_g(i, j) of query head g and a mixing matrix T [heads, heads], head h uses
// sum_g T[h, g] a_g(i, j) on the values of its own kv head c(h).  The weighted sum over keys is linear in the weights:
//
//     out_h(i) = sum_j (sum_g T[h, g] a_g(i, j)) v_c(h)(j) = sum_g T[h, g] (sum_j a_g(i, j) v_c(h)(j))
//
// so the attention kernel leaves, for every query head g, its weights applied to the values of every kv head
// (x [T, heads, kv_heads, d] float32), and this kernel forms the sums over g.  Everything is float32; the result is
// rounded once.
#include "common.h"

namespace {

template <typename TM, typename TY>
__global__ void head_mix_kernel(const float* __restrict__ x, const TM* __restrict__ mix, TY* __restrict__ y,
                                int64_t y_stride, int heads, int kv_heads, int d, int dv, int out_d, float scale) {
    // a workgroup a (token, head): that head's row of the mixing matrix in LDS
    extern __shared__ float m_s[];   // [heads]
    const int t = blockIdx.x, h = blockIdx.y;
    for (int i = threadIdx.x; i < heads; i += blockDim.x) m_s[i] = to_f32<TM>(mix[h * heads + i]);
    __syncthreads();
    const int group = heads / kv_heads;
    const float* col0 = x + static_cast<int64_t>(t) * heads * kv_heads * d + static_cast<int64_t>(h / group) * d;
    TY* dst = y + static_cast<int64_t>(t) * y_stride + static_cast<int64_t>(h) * out_d;
    for (int e = threadIdx.x; e < out_d; e += blockDim.x) {
        float sum = 0.f;
        if (e < dv) {
            const float* col = col0 + e;
#pragma unroll 4
            for (int g = 0; g < heads; ++g) sum = fmaf(m_s[g], col[static_cast<int64_t>(g) * kv_heads * d], sum);
        }
        dst[e] = from_f32<TY>(sum * scale);
    }
}

}  // namespace

// x [tokens, heads, kv_heads, d] float32; mix [heads, heads] (row h: the factors of head h's sum); y [tokens, y_stride]
// receives heads x out_d values a token: channels 0 .. dv - 1 of the sums times `scale`, zeros up to out_d.
extern "C" int pulse_head_mix(const float* x, const void* mix, int mix_dtype, void* y, int64_t y_stride, int y_dtype,
                              int tokens, int heads, int kv_heads, int d, int dv, int out_d, float scale,
                              hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && d > 0, "head_mix: bad sizes");
    PULSE_REQUIRE(dv > 0 && dv <= d && out_d >= dv && y_stride >= static_cast<int64_t>(heads) * out_d,
                  "head_mix: bad widths (dv %d, d %d, out %d)", dv, d, out_d);
    PULSE_REQUIRE(heads < 65536, "head_mix: too many heads (%d)", heads);
    PULSE_REQUIRE(x && mix && y && pulse_dtype_ok(mix_dtype) && pulse_dtype_ok(y_dtype), "head_mix: bad arguments");
    if (tokens == 0) return 0;
    const size_t lds = sizeof(float) * heads;
    const int threads = out_d >= 256 ? 256 : (out_d + 63) / 64 * 64;
    PULSE_DISPATCH_DTYPE(mix_dtype, TM, PULSE_DISPATCH_DTYPE(y_dtype, TY,
        hipLaunchKernelGGL((head_mix_kernel<TM, TY>), dim3(tokens, heads), dim3(threads), lds, stream, x, static_cast<const TM*>(mix),
                           static_cast<TY*>(y), y_stride, heads, kv_heads, d, dv, out_d, scale)));
    PULSE_LAUNCH_CHECK("head_mix");
    return 0;
}
