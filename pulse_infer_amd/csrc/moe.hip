// A routed feed-forward (mixture of experts) for few tokens at a time.
//
// pulse_moe_route, a wavefront a token: scores s = softmax(z) over all router outputs in float32; the `top`
// outputs with the largest s + correction are chosen (the lowest index among equals); their weights are their
// scores s divided by the sum of the chosen scores (+ 1e-20).  idx [T, top] and weight [T, top] come out in the
// order of choice.
//
// Experts e < E are gated feed-forwards, down_e(silu(gate_e x) * (up_e x)), with weights stacked over the experts;
// outputs e >= E are identity experts, whose result is x itself.
//
// pulse_moe_gate_up, a workgroup per (token, choice) and 64 rows of the expert's inner width: every wavefront takes
// rows in turn, its lanes share the dot products out, act[(t, k), j] = silu(g_j) * u_j.
// pulse_moe_down, a workgroup per token and 64 output columns: out[t, c] = sum_k weight_k * (down row c . act row
// (t, k)) or weight_k * x[t, c] for an identity expert, added up in the order of choice, in float32.
// A token's result depends on its own row alone, whatever else the step holds.
//
// Variations, as arguments: `score_fn` 1 takes s = sigmoid(z) instead of the softmax; `renorm` 0 leaves the chosen
// scores as they are.  `in_weight` (gate/up kernels): the expert is fed weight * x, i.e. both products are multiplied
// by the pair's weight before the activation (the products are linear), and the down kernels are then handed no
// weight.  `act_kind` 1 is the clamped form g' = min(g, limit), u' = clamp(u, -limit, limit),
// act = g' * sigmoid(1.702 g') * (u' + 1).
#include "common.h"

#include <math.h>

namespace {

constexpr int ROUTE_PER_LANE = 16;   // router outputs <= 64 * 16

// One wavefront routes one token: `row` holds its n router logits (in global memory or in LDS).
template <typename TW>
__device__ __forceinline__ void route_row(const float* row, const TW* __restrict__ correction, int* __restrict__ idx,
                                          float* __restrict__ weight, int n, int top, int t, int lane,
                                          int score_fn, int renorm) {
    float s[ROUTE_PER_LANE], c[ROUTE_PER_LANE];
    float m = -INFINITY;
#pragma unroll
    for (int r = 0; r < ROUTE_PER_LANE; ++r) {
        const int j = lane + r * PULSE_WAVE;
        s[r] = j < n ? row[j] : -INFINITY;
        m = fmaxf(m, s[r]);
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < ROUTE_PER_LANE; ++r) {
        const int j = lane + r * PULSE_WAVE;
        if (score_fn == 1) s[r] = j < n ? 1.0f / (1.0f + expf(-s[r])) : 0.f;
        else s[r] = j < n ? expf(s[r] - m) : 0.f;
        sum += s[r];
    }
    sum = score_fn == 1 ? 1.f : wave_sum(sum);
#pragma unroll
    for (int r = 0; r < ROUTE_PER_LANE; ++r) {
        const int j = lane + r * PULSE_WAVE;
        s[r] = s[r] / sum;
        c[r] = j < n ? s[r] + (correction ? to_f32<TW>(correction[j]) : 0.f) : -INFINITY;
    }
    float total = 0.f;
    float mine = 0.f;   // lane k keeps the score of choice k (top <= 64)
    int mine_idx = 0;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int best_j = 0x7fffffff;
#pragma unroll
        for (int r = 0; r < ROUTE_PER_LANE; ++r) {
            const int j = lane + r * PULSE_WAVE;
            if (c[r] > best || (c[r] == best && j < best_j && c[r] > -INFINITY)) { best = c[r]; best_j = j; }
        }
#pragma unroll
        for (int off = PULSE_WAVE / 2; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, PULSE_WAVE);
            const int oj = __shfl_xor(best_j, off, PULSE_WAVE);
            if (ob > best || (ob == best && oj < best_j)) { best = ob; best_j = oj; }
        }
        // the owner of best_j gives its score and retires the output
        float sc = 0.f;
#pragma unroll
        for (int r = 0; r < ROUTE_PER_LANE; ++r) {
            const int j = lane + r * PULSE_WAVE;
            if (j == best_j) { sc = s[r]; c[r] = -INFINITY; }
        }
        sc = wave_sum(sc);
        total += sc;
        if (lane == k) { mine = sc; mine_idx = best_j; }
    }
    if (lane < top) {
        idx[static_cast<int64_t>(t) * top + lane] = mine_idx;
        weight[static_cast<int64_t>(t) * top + lane] = renorm ? mine / (total + 1e-20f) : mine;
    }
}

template <typename TW>
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ z, const TW* __restrict__ correction,
                                                       int* __restrict__ idx, float* __restrict__ weight, int n, int top,
                                                       int score_fn, int renorm) {
    route_row<TW>(z + static_cast<int64_t>(blockIdx.x) * n, correction, idx, weight, n, top, blockIdx.x, threadIdx.x,
                  score_fn, renorm);
}

// The router's product and the routing in one: a workgroup a token holds the token's row in LDS, its wavefronts
// take the router's outputs in turn (float32 multiply-adds over the hidden size, lanes sharing a dot product out),
// and the first wavefront routes.
template <typename TX, typename TW>
__global__ __launch_bounds__(1024) void moe_router_kernel(const TX* __restrict__ x, const TW* __restrict__ w,
                                                         const TW* __restrict__ correction, int* __restrict__ idx,
                                                         float* __restrict__ weight, int hidden, int n, int top,
                                                         int score_fn, int renorm) {
    extern __shared__ float x_s[];          // [hidden] then [n]
    float* z_s = x_s + hidden;
    const int t = blockIdx.x;
#pragma unroll 4
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) x_s[i] = to_f32<TX>(x[static_cast<int64_t>(t) * hidden + i]);
    __syncthreads();
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE, waves = blockDim.x / PULSE_WAVE;
    const bool wide = sizeof(TW) == 2 && hidden % 8 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
    for (int o = wave; o < n; o += waves) {
        const TW* wrow = w + static_cast<int64_t>(o) * hidden;
        float sum = 0.f;
        if (wide) {   // 16 bytes of a bfloat16 row a lane and step
#pragma unroll 4
            for (int i = lane * 8; i < hidden; i += PULSE_WAVE * 8) {
                const pulse_i32x4 raw = *reinterpret_cast<const pulse_i32x4*>(wrow + i);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t two = static_cast<uint32_t>(raw[u]);
                    sum = fmaf(__uint_as_float(two << 16), x_s[i + 2 * u], sum);
                    sum = fmaf(__uint_as_float(two & 0xffff0000u), x_s[i + 2 * u + 1], sum);
                }
            }
        } else {
#pragma unroll 4
            for (int i = lane; i < hidden; i += PULSE_WAVE) sum = fmaf(to_f32<TW>(wrow[i]), x_s[i], sum);
        }
        sum = wave_sum(sum);
        if (lane == 0) z_s[o] = sum;
    }
    __syncthreads();
    if (wave == 0) route_row<TW>(z_s, correction, idx, weight, n, top, t, lane, score_fn, renorm);
}

template <typename TX, typename TW>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const TX* __restrict__ x, const TW* __restrict__ wg,
                                                          const TW* __restrict__ wu, const int* __restrict__ idx,
                                                          TX* __restrict__ act, int hidden, int ff, int experts,
                                                          int top, const float* __restrict__ in_weight, int act_kind,
                                                          float limit) {
    extern __shared__ float x_s[];
    const int a = blockIdx.x;
    const int e = idx[a];
    if (e < 0 || e >= experts) return;   // an identity expert has no inner activations
    const int t = a / top;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) x_s[i] = to_f32<TX>(x[static_cast<int64_t>(t) * hidden + i]);
    __syncthreads();
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
    const int j_end = min(ff, static_cast<int>(blockIdx.y + 1) * 64);
    for (int j = blockIdx.y * 64 + wave; j < j_end; j += 4) {
        const TW* g = wg + (static_cast<int64_t>(e) * ff + j) * hidden;
        const TW* u = wu + (static_cast<int64_t>(e) * ff + j) * hidden;
        float sg = 0.f, su = 0.f;
        for (int i = lane; i < hidden; i += PULSE_WAVE) {
            sg = fmaf(to_f32<TW>(g[i]), x_s[i], sg);
            su = fmaf(to_f32<TW>(u[i]), x_s[i], su);
        }
        sg = wave_sum(sg);
        su = wave_sum(su);
        if (in_weight) { sg *= in_weight[a]; su *= in_weight[a]; }
        float v;
        if (act_kind == 1) {
            const float g = fminf(sg, limit), u = fminf(fmaxf(su, -limit), limit);
            v = g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
        } else {
            v = sg / (1.0f + expf(-sg)) * su;
        }
        if (lane == 0) act[static_cast<int64_t>(a) * ff + j] = from_f32<TX>(v);
    }
}

template <typename TX, typename TW>
__global__ __launch_bounds__(256) void moe_down_kernel(const TX* __restrict__ x, const TX* __restrict__ act,
                                                       const TW* __restrict__ wd, const int* __restrict__ idx,
                                                       const float* __restrict__ weight, float* __restrict__ out,
                                                       int hidden, int ff, int experts, int top) {
    extern __shared__ float a_s[];   // [top][ff]: the token's inner activations
    const int t = blockIdx.x;
    for (int k = 0; k < top; ++k) {
        const int e = idx[static_cast<int64_t>(t) * top + k];
        if (e < 0 || e >= experts) continue;
        for (int i = threadIdx.x; i < ff; i += blockDim.x)
            a_s[k * ff + i] = to_f32<TX>(act[(static_cast<int64_t>(t) * top + k) * ff + i]);
    }
    __syncthreads();
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
    const int c_end = min(hidden, static_cast<int>(blockIdx.y + 1) * 64);
    for (int c = blockIdx.y * 64 + wave; c < c_end; c += 4) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const int e = idx[static_cast<int64_t>(t) * top + k];
            const float wk = weight ? weight[static_cast<int64_t>(t) * top + k] : 1.f;
            if (e >= experts) {
                acc = fmaf(wk, to_f32<TX>(x[static_cast<int64_t>(t) * hidden + c]), acc);
                continue;
            }
            if (e < 0) continue;
            const TW* drow = wd + (static_cast<int64_t>(e) * hidden + c) * ff;
            float s = 0.f;
            for (int i = lane; i < ff; i += PULSE_WAVE) s = fmaf(to_f32<TW>(drow[i]), a_s[k * ff + i], s);
            acc = fmaf(wk, wave_sum(s), acc);
        }
        if (lane == 0) out[static_cast<int64_t>(t) * hidden + c] = acc;
    }
}

}  // namespace

extern "C" int pulse_moe_route(const float* z, const void* correction, int c_dtype, int* idx, float* weight, int tokens,
                               int n, int top, int score_fn, int renorm, hipStream_t stream) {
    PULSE_REQUIRE(score_fn == 0 || score_fn == 1, "moe_route: unknown score function %d", score_fn);
    PULSE_REQUIRE(tokens >= 0 && n > 0 && top > 0 && top <= n && z && idx && weight, "moe_route: bad arguments");
    PULSE_REQUIRE(n <= PULSE_WAVE * ROUTE_PER_LANE && top <= PULSE_WAVE,
                  "moe_route: at most %d router outputs and %d choices", PULSE_WAVE * ROUTE_PER_LANE, PULSE_WAVE);
    PULSE_REQUIRE(pulse_dtype_ok(c_dtype), "moe_route: bad dtype tag");
    if (tokens == 0) return 0;
    PULSE_DISPATCH_DTYPE(c_dtype, TW, hipLaunchKernelGGL(moe_route_kernel<TW>, dim3(tokens), dim3(64), 0, stream, z,
                                                         static_cast<const TW*>(correction), idx, weight, n, top,
                                                         score_fn, renorm));
    PULSE_LAUNCH_CHECK("moe_route");
    return 0;
}

extern "C" int pulse_moe_router(const void* x, int x_dtype, const void* w, const void* correction, int w_dtype, int* idx,
                                float* weight, int tokens, int hidden, int n, int top, int score_fn, int renorm,
                                hipStream_t stream) {
    PULSE_REQUIRE(score_fn == 0 || score_fn == 1, "moe_router: unknown score function %d", score_fn);
    PULSE_REQUIRE(tokens >= 0 && hidden > 0 && n > 0 && top > 0 && top <= n && x && w && idx && weight,
                  "moe_router: bad arguments");
    PULSE_REQUIRE(n <= PULSE_WAVE * ROUTE_PER_LANE && top <= PULSE_WAVE,
                  "moe_router: at most %d router outputs and %d choices", PULSE_WAVE * ROUTE_PER_LANE, PULSE_WAVE);
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype), "moe_router: bad dtype tag");
    const size_t lds = sizeof(float) * (static_cast<size_t>(hidden) + n);
    PULSE_REQUIRE(lds <= 60 * 1024, "moe_router: rows of %d values do not fit the workgroup's memory", hidden);
    if (tokens == 0) return 0;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((moe_router_kernel<TX, TW>), dim3(tokens), dim3(tokens <= 256 ? 1024 : 256), lds, stream,
                           static_cast<const TX*>(x),
                           static_cast<const TW*>(w), static_cast<const TW*>(correction), idx, weight, hidden, n, top,
                           score_fn, renorm)));
    PULSE_LAUNCH_CHECK("moe_router");
    return 0;
}

extern "C" int pulse_moe_gate_up(const void* x, int x_dtype, const void* wg, const void* wu, int w_dtype, const int* idx,
                                 void* act, int tokens, int hidden, int ff, int experts, int top, const float* in_weight,
                                 int act_kind, float limit, hipStream_t stream) {
    PULSE_REQUIRE(act_kind == 0 || act_kind == 1, "moe_gate_up: unknown activation %d", act_kind);
    PULSE_REQUIRE(tokens >= 0 && hidden > 0 && ff > 0 && experts >= 0 && top > 0 && x && idx && act,
                  "moe_gate_up: bad arguments");
    PULSE_REQUIRE(experts == 0 || (wg && wu), "moe_gate_up: the experts' weights are missing");
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype), "moe_gate_up: bad dtype tag");
    PULSE_REQUIRE(sizeof(float) * static_cast<size_t>(hidden) <= 60 * 1024, "moe_gate_up: rows of %d values are too long", hidden);
    PULSE_REQUIRE((ff + 63) / 64 < 65536, "moe_gate_up: an inner width of %d is too large", ff);
    if (tokens == 0 || experts == 0) return 0;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((moe_gate_up_kernel<TX, TW>), dim3(tokens * top, (ff + 63) / 64), dim3(256),
                           sizeof(float) * hidden, stream, static_cast<const TX*>(x), static_cast<const TW*>(wg),
                           static_cast<const TW*>(wu), idx, static_cast<TX*>(act), hidden, ff, experts, top, in_weight,
                           act_kind, limit)));
    PULSE_LAUNCH_CHECK("moe_gate_up");
    return 0;
}

extern "C" int pulse_moe_down(const void* x, const void* act, int x_dtype, const void* wd, int w_dtype, const int* idx,
                              const float* weight, float* out, int tokens, int hidden, int ff, int experts, int top,
                              hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && hidden > 0 && ff > 0 && experts >= 0 && top > 0 && x && act && idx && out,
                  "moe_down: bad arguments");
    PULSE_REQUIRE(experts == 0 || wd, "moe_down: the experts' weights are missing");
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype), "moe_down: bad dtype tag");
    const size_t lds = sizeof(float) * static_cast<size_t>(top) * ff;
    PULSE_REQUIRE(lds <= 60 * 1024, "moe_down: %d choices of %d inner values do not fit the workgroup's memory", top, ff);
    PULSE_REQUIRE((hidden + 63) / 64 < 65536, "moe_down: a width of %d is too large", hidden);
    if (tokens == 0) return 0;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((moe_down_kernel<TX, TW>), dim3(tokens, (hidden + 63) / 64), dim3(256), lds, stream,
                           static_cast<const TX*>(x), static_cast<const TX*>(act), static_cast<const TW*>(wd), idx,
                           weight, out, hidden, ff, experts, top)));
    PULSE_LAUNCH_CHECK("moe_down");
    return 0;
}

// ------------------------------------------------------- a gate of one number a token
// acc[t, :] += sigmoid(w . x[t]) * y[t, :]: an always-on expert's result y enters the float32 sum of the routed ones
// times a gate of its own, one number a token, whose logit is a product with the expert's input (float32 inside).
namespace {

template <typename TX, typename TW>
__global__ void token_gate_add_kernel(const TX* __restrict__ x, const TW* __restrict__ w, const TX* __restrict__ y,
                                      float* __restrict__ acc, int hidden) {
    __shared__ float scratch[16];
    const int64_t t = blockIdx.x;
    const TX* xr = x + t * hidden;
    float dot = 0.f;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) dot = fmaf(to_f32<TX>(xr[i]), to_f32<TW>(w[i]), dot);
    dot = block_sum(dot, scratch);
    const float g = 1.0f / (1.0f + expf(-dot));
    const TX* yr = y + t * hidden;
    float* ar = acc + t * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) ar[i] = fmaf(g, to_f32<TX>(yr[i]), ar[i]);
}

}  // namespace

extern "C" int pulse_token_gate_add(const void* x, const void* w, int w_dtype, const void* y, int x_dtype, float* acc,
                                    int tokens, int hidden, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && hidden > 0 && x && w && y && acc && pulse_dtype_ok(w_dtype) && pulse_dtype_ok(x_dtype),
                  "token_gate_add: bad arguments");
    if (tokens == 0) return 0;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((token_gate_add_kernel<TX, TW>), dim3(tokens), dim3(256), 0, stream, static_cast<const TX*>(x),
                           static_cast<const TW*>(w), static_cast<const TX*>(y), acc, hidden)));
    PULSE_LAUNCH_CHECK("token_gate_add");
    return 0;
}
