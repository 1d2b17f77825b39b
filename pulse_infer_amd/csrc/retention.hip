// What a linear-attention mixer with a rotation needs around its state walk (the walk itself: lightning.hip).
//
// pulse_rotate_qk_rows: from the projection output of a step (q and k of heads x d channels, v of heads x dv) to the
// float32 rows the walk reads: the first `rot` channels of every head of q and k turned by the token's position (pairs
// (i, i + rot / 2) or (2i, 2i + 1)), k times `k_scale` after the turn, v as it is.  Everything behind the projection
// is float32, so nothing that enters the recurrence is rounded again.
//
// pulse_group_norm_gate: every group of n neighbouring values of a row (a head) divided by its own root mean square,
// optionally times a weight, times act(gate) (sigmoid or silu), times a factor; one rounding.
#include "common.h"

#include <math.h>

namespace {

template <typename TX>
__global__ void rotate_qk_rows_kernel(const TX* __restrict__ x, int64_t x_stride, int q0, int k0, int v0,
                                      float* __restrict__ y, int heads, int d, int dv, const float* __restrict__ cos_t,
                                      const float* __restrict__ sin_t, int rot, int pairing, float k_scale) {
    const int t = blockIdx.x;
    const TX* row = x + static_cast<int64_t>(t) * x_stride;
    const int hd = heads * d, hv = heads * dv;
    float* dst = y + static_cast<int64_t>(t) * (2 * hd + hv);
    const int half = rot / 2;
    for (int i = threadIdx.x; i < 2 * hd; i += blockDim.x) {
        const int which = i / hd, j = i % hd, e = j % d;   // which: 0 q, 1 k
        const TX* src = row + (which ? k0 : q0) + (j - e);
        float v = to_f32<TX>(src[e]);
        if (e < rot) {
            int pair, freq;
            bool first;
            if (pairing == 1) { first = e < half; pair = first ? e + half : e - half; freq = first ? e : e - half; }
            else { first = (e & 1) == 0; pair = e ^ 1; freq = e >> 1; }
            const float c = cos_t[static_cast<int64_t>(t) * half + freq], s = sin_t[static_cast<int64_t>(t) * half + freq];
            const float o = to_f32<TX>(src[pair]);
            v = first ? v * c - o * s : v * c + o * s;
        }
        dst[i] = which ? v * k_scale : v;
    }
    for (int i = threadIdx.x; i < hv; i += blockDim.x) dst[2 * hd + i] = to_f32<TX>(row[v0 + i]);
}

template <typename TX, typename TW>
__global__ void group_norm_gate_kernel(const float* __restrict__ o, int64_t o_stride, const TW* __restrict__ w,
                                       const TX* __restrict__ gate, int64_t gate_stride, TX* __restrict__ y,
                                       int64_t y_stride, int groups, int n, float eps, float scale, int gate_act) {
    // one wavefront a (token, group)
    const int t = blockIdx.x, g = blockIdx.y * (blockDim.x / PULSE_WAVE) + threadIdx.x / PULSE_WAVE;
    if (g >= groups) return;
    const int lane = threadIdx.x % PULSE_WAVE;
    const float* row = o + static_cast<int64_t>(t) * o_stride + static_cast<int64_t>(g) * n;
    float ss = 0.f;
    for (int i = lane; i < n; i += PULSE_WAVE) ss = fmaf(row[i], row[i], ss);
    ss = wave_sum(ss);
    const float inv = scale / sqrtf(ss / static_cast<float>(n) + eps);
    const TX* gr = gate ? gate + static_cast<int64_t>(t) * gate_stride + static_cast<int64_t>(g) * n : nullptr;
    TX* dst = y + static_cast<int64_t>(t) * y_stride + static_cast<int64_t>(g) * n;
    for (int i = lane; i < n; i += PULSE_WAVE) {
        float v = row[i] * inv;
        if (w) v *= to_f32<TW>(w[static_cast<int64_t>(g) * n + i]);
        if (gr) {
            const float z = to_f32<TX>(gr[i]);
            const float sg = 1.0f / (1.0f + expf(-z));
            v *= gate_act == 1 ? z * sg : sg;
        }
        dst[i] = from_f32<TX>(v);
    }
}

}  // namespace

// x [tokens, x_stride] holds q, k (heads x d) and v (heads x dv) from columns q0, k0, v0; y [tokens, 2 heads d + heads dv]
// float32 receives q, k, v side by side.  cos / sin [tokens, rot / 2] float32 (null with rot 0: no turn).
// pairing 0: (2i, 2i + 1); 1: (i, i + rot / 2).
extern "C" int pulse_rotate_qk_rows(const void* x, int64_t x_stride, int x_dtype, int q0, int k0, int v0, float* y,
                                    int tokens, int heads, int d, int dv, const float* cos_t, const float* sin_t, int rot,
                                    int pairing, float k_scale, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && heads > 0 && d > 0 && dv > 0 && x && y && pulse_dtype_ok(x_dtype), "rotate_qk_rows: bad arguments");
    PULSE_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= d && (rot == 0 || (cos_t && sin_t)) && (pairing == 0 || pairing == 1),
                  "rotate_qk_rows: bad rotation (%d of %d channels)", rot, d);
    PULSE_REQUIRE(q0 >= 0 && k0 >= 0 && v0 >= 0 && x_stride >= static_cast<int64_t>(q0) + heads * d &&
                  x_stride >= static_cast<int64_t>(k0) + heads * d && x_stride >= static_cast<int64_t>(v0) + heads * dv,
                  "rotate_qk_rows: the rows are too short");
    if (tokens == 0) return 0;
    PULSE_DISPATCH_DTYPE(x_dtype, TX,
        hipLaunchKernelGGL(rotate_qk_rows_kernel<TX>, dim3(tokens), dim3(256), 0, stream, static_cast<const TX*>(x), x_stride,
                           q0, k0, v0, y, heads, d, dv, cos_t, sin_t, rot, pairing, k_scale));
    PULSE_LAUNCH_CHECK("rotate_qk_rows");
    return 0;
}

// y[t, g n + i] = scale * o[t, g n + i] / sqrt(mean_i(o[t, g n + .]^2) + eps) * w[g n + i] * act(gate[t, g n + i]);
// w and gate may be null; gate_act 0: sigmoid, 1: silu.
extern "C" int pulse_group_norm_gate(const float* o, int64_t o_stride, const void* w, int w_dtype, const void* gate,
                                     int64_t gate_stride, void* y, int64_t y_stride, int x_dtype, int tokens, int groups,
                                     int n, float eps, float scale, int gate_act, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && groups > 0 && n > 0 && o && y, "group_norm_gate: bad arguments");
    PULSE_REQUIRE(pulse_dtype_ok(w_dtype) && pulse_dtype_ok(x_dtype) && (gate_act == 0 || gate_act == 1),
                  "group_norm_gate: bad dtype tag or gate");
    const int64_t width = static_cast<int64_t>(groups) * n;
    PULSE_REQUIRE(o_stride >= width && y_stride >= width && (!gate || gate_stride >= width), "group_norm_gate: rows are too short");
    PULSE_REQUIRE(groups < 65536, "group_norm_gate: too many groups");
    if (tokens == 0) return 0;
    const int waves = 4;
    const dim3 grid(tokens, (groups + waves - 1) / waves);
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((group_norm_gate_kernel<TX, TW>), grid, dim3(waves * PULSE_WAVE), 0, stream, o,
                           o_stride, static_cast<const TW*>(w), static_cast<const TX*>(gate), gate_stride,
                           static_cast<TX*>(y), y_stride, groups, n, eps, scale, gate_act)));
    PULSE_LAUNCH_CHECK("group_norm_gate");
    return 0;
}
