// Attention over one latent row a token ("latent attention"), around the paged attention kernels.
//
// A token stores c (`rank` values: the first rows of the down projection, divided by their root mean square and
// multiplied by a weight) and one turned key part (`rot` values) shared by all heads.  Head h's key is
// [W_uk,h c | turned part] and its value W_uv,h c.  Scores and weighted sums are linear in c, so the kernels work in the
// latent space: the query of head h becomes [W_uk,h^T q_plain,h | q_turned,h], the stored "key" of the one kv head is
// [c | turned part], its "value" is c, and head h's result W_uv,h (sum_j a_h(j) c_j) is expanded afterwards.
//
// pulse_latent_rows:   c and the turned key part into the pages; the queries' turned parts into their places.
// pulse_latent_absorb: q_abs[t, h, :] = W_uk,h^T q_plain[t, h]        (float32 sums, one rounding)
// pulse_latent_expand: y[t, h, :] = (W_uv,h o[t, h, :rank]) * sigmoid(gate[t, h, :])
// pulse_heads_product: both of these products for bfloat16 weights on the matrix cores: y[t, h, m] = sum_k
//                      w[h, m, k] x[t, h, k] (w_uk transposed once at load, w_uv as it is), 16 tokens a workgroup
#include "common.h"

#include <math.h>

namespace {

struct LatentArgs {
    int heads, d, rot, rank, stored;   // stored: channels of a stored key / value row (>= rank + rot)
    int64_t x_stride, q_stride;
    int q0, c0;                        // first columns of the queries and of the down projection in a row of x
    int page_size, num_pages, bt_width;
    int pairing, write;
    float eps;
};

// One workgroup a token.
template <typename TX, typename TW, typename TC>
__global__ void latent_rows_kernel(const TX* __restrict__ x, TX* __restrict__ q, const TW* __restrict__ w,
                                   const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                   TC* __restrict__ kcache, TC* __restrict__ vcache, const int* __restrict__ positions,
                                   const int* __restrict__ token_entry, const int* __restrict__ block_table, LatentArgs a) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const TX* row = x + static_cast<int64_t>(t) * a.x_stride;
    const int half = a.rot / 2;
    const float* ct = cos_t + static_cast<int64_t>(t) * half;
    const float* st = sin_t + static_cast<int64_t>(t) * half;
    auto turned = [&](const TX* src, int e) -> float {
        int pair, freq;
        bool first;
        if (a.pairing == 1) { first = e < half; pair = first ? e + half : e - half; freq = first ? e : e - half; }
        else { first = (e & 1) == 0; pair = e ^ 1; freq = e >> 1; }
        const float v = to_f32<TX>(src[e]), o = to_f32<TX>(src[pair]);
        return first ? v * ct[freq] - o * st[freq] : v * ct[freq] + o * st[freq];
    };
    // the queries' turned parts: q[t, h, rank + e]
    TX* qrow = q + static_cast<int64_t>(t) * a.q_stride;
    const int width = a.rank + a.rot;
    for (int i = threadIdx.x; i < a.heads * a.rot; i += blockDim.x) {
        const int h = i / a.rot, e = i % a.rot;
        qrow[static_cast<int64_t>(h) * a.stored + a.rank + e] =
            from_f32<TX>(turned(row + a.q0 + static_cast<int64_t>(h) * (a.d + a.rot) + a.d, e));
    }
    for (int i = threadIdx.x; i < a.heads * (a.stored - width); i += blockDim.x) {
        const int h = i / (a.stored - width), e = i % (a.stored - width);
        qrow[static_cast<int64_t>(h) * a.stored + width + e] = from_f32<TX>(0.f);
    }
    if (!a.write) return;
    const TX* down = row + a.c0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < a.rank; i += blockDim.x) { const float v = to_f32<TX>(down[i]); ss = fmaf(v, v, ss); }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(a.rank) + a.eps);
    const int pos = positions[t];
    const int pi = pos / a.page_size;
    const int page = pi < a.bt_width ? block_table[static_cast<int64_t>(token_entry[t]) * a.bt_width + pi] : -1;
    if (page < 0 || page >= a.num_pages) return;   // the host has checked the tables; a stale entry is not written through
    const int slot = pos % a.page_size;
    TC* krow = kcache + (static_cast<int64_t>(page) * a.page_size + slot) * a.stored;
    TC* vrow = vcache + static_cast<int64_t>(page) * a.stored * a.page_size + slot;
    for (int i = threadIdx.x; i < a.stored; i += blockDim.x) {
        float k = 0.f, v = 0.f;
        if (i < a.rank) k = v = to_f32<TX>(down[i]) * inv * to_f32<TW>(w[i]);
        else if (i < width) k = turned(down + a.rank, i - a.rank);
        krow[i] = from_f32<TC>(k);
        vrow[static_cast<int64_t>(i) * a.page_size] = from_f32<TC>(v);
    }
}

// q_abs[t, h, r] = sum_e q[t, h, e] * W_uk[h * d + e, r]; one workgroup a (token, head), a thread a latent channel.
template <typename TX, typename TW>
__global__ void latent_absorb_kernel(const TX* __restrict__ x, int64_t x_stride, int q0, int q_head, const TW* __restrict__ w,
                                     TX* __restrict__ q, int64_t q_stride, int stored, int d, int rank) {
    extern __shared__ float q_s[];
    const int t = blockIdx.x, h = blockIdx.y;
    const TX* src = x + static_cast<int64_t>(t) * x_stride + q0 + static_cast<int64_t>(h) * q_head;
    for (int e = threadIdx.x; e < d; e += blockDim.x) q_s[e] = to_f32<TX>(src[e]);
    __syncthreads();
    const TW* wh = w + static_cast<int64_t>(h) * d * rank;
    TX* dst = q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(h) * stored;
    for (int r = threadIdx.x; r < rank; r += blockDim.x) {
        float sum = 0.f;
        for (int e = 0; e < d; ++e) sum = fmaf(q_s[e], to_f32<TW>(wh[static_cast<int64_t>(e) * rank + r]), sum);
        dst[r] = from_f32<TX>(sum);
    }
}

// y[t, h, e] = (sum_r W_uv[h * dv + e, r] * o[t, h, r]) * sigmoid(gate[t, h * dv + e]); a wavefront an output channel.
template <typename TO, typename TX, typename TW>
__global__ void latent_expand_kernel(const TO* __restrict__ o, int64_t o_stride, int stored, const TW* __restrict__ w,
                                     const TX* __restrict__ gate, int64_t gate_stride, TX* __restrict__ y,
                                     int64_t y_stride, int dv, int rank, float scale) {
    extern __shared__ float o_s[];
    const int t = blockIdx.x, h = blockIdx.y;
    const TO* src = o + static_cast<int64_t>(t) * o_stride + static_cast<int64_t>(h) * stored;
    for (int r = threadIdx.x; r < rank; r += blockDim.x) o_s[r] = to_f32<TO>(src[r]);
    __syncthreads();
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE, waves = blockDim.x / PULSE_WAVE;
    for (int e = wave; e < dv; e += waves) {
        const TW* wr = w + (static_cast<int64_t>(h) * dv + e) * rank;
        float sum = 0.f;
        for (int r = lane; r < rank; r += PULSE_WAVE) sum = fmaf(to_f32<TW>(wr[r]), o_s[r], sum);
        sum = wave_sum(sum);
        if (lane == 0) {
            float v = sum * scale;
            if (gate) v *= 1.0f / (1.0f + expf(-to_f32<TX>(gate[static_cast<int64_t>(t) * gate_stride + static_cast<int64_t>(h) * dv + e])));
            y[static_cast<int64_t>(t) * y_stride + static_cast<int64_t>(h) * dv + e] = from_f32<TX>(v);
        }
    }
}


// ------------------------------------------------------------------ a product a head, on the matrix cores
typedef __attribute__((ext_vector_type(8))) __bf16 hp_bf16x8;
typedef __attribute__((ext_vector_type(4))) float hp_f32x4;

template <typename T> __device__ __forceinline__ hp_bf16x8 load8(const T* p);
template <> __device__ __forceinline__ hp_bf16x8 load8<bf16_t>(const bf16_t* p) { return *reinterpret_cast<const hp_bf16x8*>(p); }
template <> __device__ __forceinline__ hp_bf16x8 load8<float>(const float* p) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    hp_bf16x8 out;
    out[0] = static_cast<__bf16>(a.x); out[1] = static_cast<__bf16>(a.y); out[2] = static_cast<__bf16>(a.z); out[3] = static_cast<__bf16>(a.w);
    out[4] = static_cast<__bf16>(b.x); out[5] = static_cast<__bf16>(b.y); out[6] = static_cast<__bf16>(b.z); out[7] = static_cast<__bf16>(b.w);
    return out;
}

// A workgroup takes 16 tokens of one head; a wavefront a tile of 16 output channels at a time.  W rows are the matrix
// cores' row operand (m = output channel), the tokens' rows of x the column operand, so a lane ends up with four
// neighbouring channels of its token: one 8-byte store.
template <typename TX>
__global__ __launch_bounds__(256) void heads_product_kernel(const TX* __restrict__ x, int64_t x_stride, int x_head,
                                                            const bf16_t* __restrict__ w, const bf16_t* __restrict__ gate,
                                                            int64_t gate_stride, bf16_t* __restrict__ y, int64_t y_stride,
                                                            int y_head, int tokens, int m_out, int k_in, float scale) {
    const int t0 = blockIdx.x * 16, h = blockIdx.y;
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int tok = min(t0 + r, tokens - 1);
    const TX* xrow = x + static_cast<int64_t>(tok) * x_stride + static_cast<int64_t>(h) * x_head;
    const hp_bf16x8 zero = __builtin_bit_cast(hp_bf16x8, make_uint4(0u, 0u, 0u, 0u));
    for (int m0 = wave * 16; m0 < m_out; m0 += 64) {
        const int m = m0 + r;
        const bf16_t* wrow = m < m_out ? w + (static_cast<int64_t>(h) * m_out + m) * k_in : nullptr;
        hp_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int k0 = 0; k0 < k_in; k0 += 32) {
            const int k = k0 + 8 * g;
            const bool in = k < k_in;
            const hp_bf16x8 wa = (in && wrow) ? *reinterpret_cast<const hp_bf16x8*>(wrow + k) : zero;
            const hp_bf16x8 xb = in ? load8<TX>(xrow + k) : zero;
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa, xb, acc, 0, 0, 0);
        }
        // lane: token r, channels m0 + 4 g + i
        if (t0 + r < tokens) {
            const int c0 = m0 + 4 * g;
            bf16_t* dst = y + static_cast<int64_t>(t0 + r) * y_stride + static_cast<int64_t>(h) * y_head + c0;
            const bf16_t* gr = gate ? gate + static_cast<int64_t>(t0 + r) * gate_stride + static_cast<int64_t>(h) * m_out + c0 : nullptr;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (c0 + i < m_out) {
                    float v = acc[i] * scale;
                    if (gr) v *= 1.0f / (1.0f + expf(-bf16_to_f32(gr[i])));
                    dst[i] = f32_to_bf16(v);
                }
            }
        }
    }
}

}  // namespace

// x [tokens, x_stride]: the projection output; queries from column q0 (heads x (d + rot), the turned part last), the
// down projection from column c0 (rank + rot).  q [tokens, q_stride] receives, for head h at h * stored, the turned
// part at rank .. rank + rot and zeros behind it (the first rank channels are pulse_latent_absorb's).  With `write`
// the token's c and turned key part go to kcache [pages, 1, page, stored] and c to vcache [pages, 1, stored, page].
extern "C" int pulse_latent_rows(const void* x, int64_t x_stride, int x_dtype, int q0, int c0, void* q, int64_t q_stride,
                                 const void* norm_w, int w_dtype, const float* cos_t, const float* sin_t, int pairing,
                                 void* kcache, void* vcache, int c_dtype, const int* positions, const int* token_entry,
                                 const int* block_table, int bt_width, int tokens, int heads, int d, int rot, int rank,
                                 int stored, int page_size, int num_pages, float eps, int write, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && heads > 0 && d >= 0 && rank > 0 && rot > 0 && rot % 2 == 0, "latent_rows: bad sizes");
    PULSE_REQUIRE(stored >= rank + rot && q_stride >= static_cast<int64_t>(heads) * stored, "latent_rows: stored rows too narrow");
    PULSE_REQUIRE(x && q && norm_w && cos_t && sin_t && kcache && vcache && positions && token_entry && block_table,
                  "latent_rows: null pointer");
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype) && pulse_dtype_ok(c_dtype), "latent_rows: bad dtype tag");
    PULSE_REQUIRE(q0 >= 0 && c0 >= 0 && x_stride >= static_cast<int64_t>(q0) + static_cast<int64_t>(heads) * (d + rot) &&
                  x_stride >= static_cast<int64_t>(c0) + rank + rot, "latent_rows: the rows are too short");
    PULSE_REQUIRE(page_size > 0 && num_pages > 0 && bt_width > 0 && (pairing == 0 || pairing == 1), "latent_rows: bad cache geometry");
    if (tokens == 0) return 0;
    LatentArgs a;
    a.heads = heads; a.d = d; a.rot = rot; a.rank = rank; a.stored = stored; a.x_stride = x_stride; a.q_stride = q_stride;
    a.q0 = q0; a.c0 = c0; a.page_size = page_size; a.num_pages = num_pages; a.bt_width = bt_width; a.pairing = pairing;
    a.write = write; a.eps = eps;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW, PULSE_DISPATCH_DTYPE(c_dtype, TC,
        hipLaunchKernelGGL((latent_rows_kernel<TX, TW, TC>), dim3(tokens), dim3(256), 0, stream, static_cast<const TX*>(x),
                           static_cast<TX*>(q), static_cast<const TW*>(norm_w), cos_t, sin_t, static_cast<TC*>(kcache),
                           static_cast<TC*>(vcache), positions, token_entry, block_table, a))));
    PULSE_LAUNCH_CHECK("latent_rows");
    return 0;
}

// w_uk [heads * d, rank]; q_head: columns a head takes in x (d + rot).
extern "C" int pulse_latent_absorb(const void* x, int64_t x_stride, int x_dtype, int q0, int q_head, const void* w_uk,
                                   int w_dtype, void* q, int64_t q_stride, int stored, int tokens, int heads, int d,
                                   int rank, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && heads > 0 && d > 0 && rank > 0 && q_head >= d && stored >= rank, "latent_absorb: bad sizes");
    PULSE_REQUIRE(heads < 65536 && x && w_uk && q && pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype), "latent_absorb: bad arguments");
    PULSE_REQUIRE(q_stride >= static_cast<int64_t>(heads) * stored && x_stride >= static_cast<int64_t>(q0) + static_cast<int64_t>(heads) * q_head,
                  "latent_absorb: the rows are too short");
    if (tokens == 0) return 0;
    const int threads = rank >= 256 ? 256 : (rank + 63) / 64 * 64;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((latent_absorb_kernel<TX, TW>), dim3(tokens, heads), dim3(threads), sizeof(float) * d, stream,
                           static_cast<const TX*>(x), x_stride, q0, q_head, static_cast<const TW*>(w_uk),
                           static_cast<TX*>(q), q_stride, stored, d, rank)));
    PULSE_LAUNCH_CHECK("latent_absorb");
    return 0;
}

// o [tokens, o_stride] (float32 or the activations' type): head h's weighted latent row at h * stored; w_uv
// [heads * dv, rank]; gate [tokens, gate_stride] holds heads * dv logits a token (null: no gate).
extern "C" int pulse_latent_expand(const void* o, int64_t o_stride, int o_dtype, int stored, const void* w_uv, int w_dtype,
                                   const void* gate, int64_t gate_stride, void* y, int64_t y_stride, int x_dtype,
                                   int tokens, int heads, int dv, int rank, float scale, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && heads > 0 && dv > 0 && rank > 0 && stored >= rank, "latent_expand: bad sizes");
    PULSE_REQUIRE(heads < 65536 && o && w_uv && y && pulse_dtype_ok(o_dtype) && pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype),
                  "latent_expand: bad arguments");
    PULSE_REQUIRE(o_stride >= static_cast<int64_t>(heads) * stored && y_stride >= static_cast<int64_t>(heads) * dv &&
                  (!gate || gate_stride >= static_cast<int64_t>(heads) * dv), "latent_expand: the rows are too short");
    PULSE_REQUIRE(rank * sizeof(float) <= 60 * 1024, "latent_expand: a latent row of %d values does not fit", rank);
    if (tokens == 0) return 0;
    PULSE_DISPATCH_DTYPE(o_dtype, TO, PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((latent_expand_kernel<TO, TX, TW>), dim3(tokens, heads), dim3(256), sizeof(float) * rank, stream,
                           static_cast<const TO*>(o), o_stride, stored, static_cast<const TW*>(w_uv),
                           static_cast<const TX*>(gate), gate_stride, static_cast<TX*>(y), y_stride, dv, rank, scale))));
    PULSE_LAUNCH_CHECK("latent_expand");
    return 0;
}

// y[t, h * y_head + m] = scale * (sum_k w[h, m, k] * x[t, h * x_head + k]) * sigmoid(gate[t, h * m_out + m]) for bfloat16
// w [heads, m_out, k_in] and y, x bfloat16 or float32 (rounded to bfloat16 as it is read); k_in a multiple of 8, rows
// of x and w 16-byte aligned.  gate may be null.
extern "C" int pulse_heads_product(const void* x, int64_t x_stride, int x_head, int x_dtype, const void* w, const void* gate,
                                   int64_t gate_stride, void* y, int64_t y_stride, int y_head, int tokens, int heads,
                                   int m_out, int k_in, float scale, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && heads > 0 && heads < 65536 && m_out > 0 && k_in > 0 && k_in % 8 == 0, "heads_product: bad sizes");
    PULSE_REQUIRE(x && w && y && pulse_dtype_ok(x_dtype), "heads_product: bad arguments");
    const int xb = x_dtype == PULSE_F32 ? 4 : 2;
    PULSE_REQUIRE(x_head >= k_in && x_stride >= static_cast<int64_t>(heads - 1) * x_head + k_in &&
                  y_head >= m_out && y_stride >= static_cast<int64_t>(heads - 1) * y_head + m_out &&
                  (!gate || gate_stride >= static_cast<int64_t>(heads) * m_out), "heads_product: the rows are too short");
    PULSE_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && (x_stride * xb) % 16 == 0 && (static_cast<int64_t>(x_head) * xb) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(w) % 16 == 0, "heads_product: operands must be 16-byte aligned");
    if (tokens == 0) return 0;
    const dim3 grid((tokens + 15) / 16, heads);
    PULSE_DISPATCH_DTYPE(x_dtype, TX,
        hipLaunchKernelGGL(heads_product_kernel<TX>, grid, dim3(256), 0, stream, static_cast<const TX*>(x), x_stride, x_head,
                           static_cast<const bf16_t*>(w), static_cast<const bf16_t*>(gate), gate_stride,
                           static_cast<bf16_t*>(y), y_stride, y_head, tokens, m_out, k_in, scale));
    PULSE_LAUNCH_CHECK("heads_product");
    return 0;
}
