// Preparation of attention inputs whose query/key norm runs over a token's whole
// projection, whose projections have biases, and whose keys and values may differ
// in width.
//
// A row of the projection output holds q [nq, d], k [nkv, d] and v [nkv, dv].  For a token:
//   q += bq, k += bk, v += bv                                  (biases optional)
//   q <- q / sqrt(mean over all nq*d values of q^2 + eps) * wq  (one norm over the row; wq [nq*d]; optional)
//   k likewise with wk [nkv*d]
//   or (norm 2) every head of q and of k divided by the root mean square of its own d values, without weights;
//   a rotation keeps a head's sum of squares, so this is the same before or after it
//   q, k <- rotated at the token's position on the first rotary_dim channels of every head
//           (pairing 0: channels 2i, 2i+1; pairing 1: channels i, i + rotary_dim/2)
//   v <- v * value_scale
// q goes to q_out [T, nq*D], k and v to the token's slot of its page, each head filled
// with zeros up to D channels (D >= d, dv): the attention kernels then see heads of one
// width D, the zero channels add nothing to a score, and the value channels beyond dv
// come out as zeros.  Everything is float32 until the one rounding of the store.
// One workgroup a token, or several that each redo the token's sums of squares and share its channels out (few
// tokens: a decoding step).
#include "common.h"

#include <math.h>

namespace {

struct PrepArgs {
    int nq, nkv, d, dv, D;
    int64_t x_stride, q_stride;
    int norm;           // 0: none, 1: over the whole projection, 2: every head by itself, no weights
    float eps;
    int rotary_dim, pairing;
    int page_size, num_pages, bt_width;
    int write_kv;
    float value_scale;
};

template <typename TX, typename TW, typename TC>
__global__ __launch_bounds__(256) void qkv_rows_kernel(const TX* __restrict__ x, const TW* __restrict__ bq,
                                                       const TW* __restrict__ bk, const TW* __restrict__ bv,
                                                       const TW* __restrict__ wq, const TW* __restrict__ wk,
                                                       const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                       TX* __restrict__ q_out, TC* __restrict__ kcache,
                                                       TC* __restrict__ vcache, const int* __restrict__ positions,
                                                       const int* __restrict__ token_entry,
                                                       const int* __restrict__ block_table, PrepArgs a) {
    extern __shared__ float row_s[];   // [nq*d + nkv*d]: q and k of the token, biased
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const int tid = threadIdx.x;
    const int nqd = a.nq * a.d, nkd = a.nkv * a.d, nvd = a.nkv * a.dv;
    const TX* row = x + static_cast<int64_t>(t) * a.x_stride;
    float sq = 0.f, sk = 0.f;
#pragma unroll 4
    for (int i = tid; i < nqd; i += blockDim.x) {
        float v = to_f32<TX>(row[i]);
        if (bq) v += to_f32<TW>(bq[i]);
        row_s[i] = v;
        sq = fmaf(v, v, sq);
    }
    if (a.write_kv) {
#pragma unroll 4
        for (int i = tid; i < nkd; i += blockDim.x) {
            float v = to_f32<TX>(row[nqd + i]);
            if (bk) v += to_f32<TW>(bk[i]);
            row_s[nqd + i] = v;
            sk = fmaf(v, v, sk);
        }
    }
    float inv_q = 1.f, inv_k = 1.f;
    float* inv_s = row_s + nqd + nkd;   // [nq + nkv], norm 2 only
    if (a.norm == 1) {
        inv_q = 1.0f / sqrtf(block_sum(sq, scratch) / static_cast<float>(nqd) + a.eps);
        if (a.write_kv) inv_k = 1.0f / sqrtf(block_sum(sk, scratch) / static_cast<float>(nkd) + a.eps);
    } else if (a.norm == 2) {
        __syncthreads();
        const int lane = tid % PULSE_WAVE, wave = tid / PULSE_WAVE, waves = blockDim.x / PULSE_WAVE;
        const int heads = a.nq + (a.write_kv ? a.nkv : 0);
        for (int hh = wave; hh < heads; hh += waves) {
            float ss = 0.f;
            for (int c = lane; c < a.d; c += PULSE_WAVE) ss = fmaf(row_s[hh * a.d + c], row_s[hh * a.d + c], ss);
            ss = wave_sum(ss);
            if (lane == 0) inv_s[hh] = 1.0f / sqrtf(ss / static_cast<float>(a.d) + a.eps);
        }
        __syncthreads();
    } else {
        __syncthreads();
    }
    const int half = a.rotary_dim / 2;
    const float* cs = cos_t ? cos_t + static_cast<int64_t>(t) * half : nullptr;
    const float* sn = sin_t ? sin_t + static_cast<int64_t>(t) * half : nullptr;
    // a value of q or k, normed and rotated: element c of head hd of the vector that starts at row_s + base
    auto prepared = [&](int base, int hd, int c, float inv, const TW* w) -> float {
        const int at = base + hd * a.d + c;
        if (a.norm == 2) inv = inv_s[base / a.d + hd];
        float u = row_s[at] * inv;
        if (w) u *= to_f32<TW>(w[at - base]);
        if (cs && c < a.rotary_dim) {
            int partner, i;
            bool first;
            if (a.pairing == 0) { i = c / 2; first = (c % 2) == 0; partner = first ? c + 1 : c - 1; }
            else { i = c % half; first = c < half; partner = first ? c + half : c - half; }
            const int pat = base + hd * a.d + partner;
            float p = row_s[pat] * inv;
            if (w) p *= to_f32<TW>(w[pat - base]);
            // (u, p) -> first: u cos - p sin; second: u cos + p sin   (u the element itself, p its partner)
            u = first ? u * cs[i] - p * sn[i] : u * cs[i] + p * sn[i];
        }
        return u;
    };
    TX* qrow = q_out + static_cast<int64_t>(t) * a.q_stride;
    const int first = blockIdx.y * blockDim.x + tid, stride = blockDim.x * gridDim.y;
#pragma unroll 4
    for (int idx = first; idx < a.nq * a.D; idx += stride) {
        const int hd = idx / a.D, c = idx % a.D;
        qrow[idx] = from_f32<TX>(c < a.d ? prepared(0, hd, c, inv_q, wq) : 0.f);
    }
    if (!a.write_kv) return;
    const int pos = positions[t];
    const int pi = pos / a.page_size;
    const int page = pi < a.bt_width ? block_table[static_cast<int64_t>(token_entry[t]) * a.bt_width + pi] : -1;
    if (page < 0 || page >= a.num_pages) return;   // no page: the step's host checks make this unreachable
    const int slot = pos % a.page_size;
#pragma unroll 2
    for (int idx = first; idx < a.nkv * a.D; idx += stride) {
        const int g = idx / a.D, c = idx % a.D;
        const int64_t pg = static_cast<int64_t>(page) * a.nkv + g;
        kcache[(pg * a.page_size + slot) * a.D + c] = from_f32<TC>(c < a.d ? prepared(nqd, g, c, inv_k, wk) : 0.f);
    }
    (void)nvd;
    (void)bv;
    (void)vcache;
}

// The values go to their pages from a kernel of their own: a page holds a channel's slots side by side, so a
// workgroup takes 16 consecutive tokens and one key/value head, a token a lane of every group of 16 lanes: the 16
// lanes of a group then fill neighbouring slots of one channel (32 contiguous bytes in bfloat16) where a token at a
// time would write two-byte pieces a whole page row apart.
template <typename TX, typename TW, typename TC>
__global__ __launch_bounds__(256) void v_rows_kernel(const TX* __restrict__ x, const TW* __restrict__ bv,
                                                     TC* __restrict__ vcache, const int* __restrict__ positions,
                                                     const int* __restrict__ token_entry,
                                                     const int* __restrict__ block_table, int tokens, PrepArgs a) {
    const int tt = threadIdx.x % 16, cc = threadIdx.x / 16;
    const int t = blockIdx.x * 16 + tt, g = blockIdx.y;
    if (t >= tokens) return;
    const int pos = positions[t];
    const int pi = pos / a.page_size;
    const int page = pi < a.bt_width ? block_table[static_cast<int64_t>(token_entry[t]) * a.bt_width + pi] : -1;
    if (page < 0 || page >= a.num_pages) return;
    const int slot = pos % a.page_size;
    const TX* src = x + static_cast<int64_t>(t) * a.x_stride + a.nq * a.d + a.nkv * a.d + g * a.dv;
    TC* dst = vcache + (static_cast<int64_t>(page) * a.nkv + g) * a.D * a.page_size + slot;
    for (int c = cc; c < a.D; c += 16) {
        float v = 0.f;
        if (c < a.dv) {
            v = to_f32<TX>(src[c]);
            if (bv) v += to_f32<TW>(bv[g * a.dv + c]);
            v *= a.value_scale;
        }
        dst[static_cast<int64_t>(c) * a.page_size] = from_f32<TC>(v);
    }
}

}  // namespace

extern "C" int pulse_qkv_rows(const void* x, int x_dtype, int64_t x_stride, const void* bq, const void* bk,
                              const void* bv, const void* wq, const void* wk, int w_dtype, int norm, float eps,
                              const float* cos_t, const float* sin_t, int rotary_dim, int pairing, void* q_out,
                              int64_t q_stride, void* kcache, void* vcache, int c_dtype, const int* positions,
                              const int* token_entry, const int* block_table, int bt_width, int tokens, int nq, int nkv,
                              int d, int dv, int D, int page_size, int num_pages, int write_kv, float value_scale,
                              hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && nq > 0 && nkv > 0 && d > 0 && dv > 0, "qkv_rows: bad sizes");
    PULSE_REQUIRE(D >= d && D >= dv, "qkv_rows: the stored head width %d is below %d or %d", D, d, dv);
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype) && pulse_dtype_ok(c_dtype), "qkv_rows: bad dtype tag");
    PULSE_REQUIRE(norm == 0 || norm == 1 || norm == 2, "qkv_rows: unknown norm %d", norm);
    PULSE_REQUIRE(norm != 2 || (!wq && !wk), "qkv_rows: the norm of every head by itself has no weights");
    PULSE_REQUIRE(x && q_out && positions && token_entry, "qkv_rows: null pointer");
    PULSE_REQUIRE(!write_kv || (kcache && vcache && block_table && page_size > 0 && num_pages > 0 && bt_width > 0),
                  "qkv_rows: the cache is missing");
    const int64_t cols = static_cast<int64_t>(nq) * d + (write_kv ? static_cast<int64_t>(nkv) * (d + dv) : 0);
    PULSE_REQUIRE(x_stride >= cols && q_stride >= static_cast<int64_t>(nq) * D, "qkv_rows: rows are too short");
    PULSE_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "qkv_rows: cos and sin come together");
    PULSE_REQUIRE(!cos_t || (rotary_dim > 0 && rotary_dim % 2 == 0 && rotary_dim <= d && (pairing == 0 || pairing == 1)),
                  "qkv_rows: bad rotation (dims %d of %d, pairing %d)", rotary_dim, d, pairing);
    const size_t lds = sizeof(float) * (static_cast<size_t>(nq) * d + static_cast<size_t>(nkv) * d + nq + nkv);
    PULSE_REQUIRE(lds <= 60 * 1024, "qkv_rows: a token's q and k (%zu bytes in float32) do not fit the workgroup's memory", lds);
    if (tokens == 0) return 0;
    const int parts = tokens >= 512 ? 1 : min(16, (nq * D + 511) / 512);
    PrepArgs a;
    a.nq = nq; a.nkv = nkv; a.d = d; a.dv = dv; a.D = D; a.x_stride = x_stride; a.q_stride = q_stride;
    a.norm = norm; a.eps = eps; a.rotary_dim = cos_t ? rotary_dim : 0; a.pairing = pairing;
    a.page_size = page_size; a.num_pages = num_pages; a.bt_width = bt_width; a.write_kv = write_kv;
    a.value_scale = value_scale;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW, PULSE_DISPATCH_DTYPE(c_dtype, TC,
        hipLaunchKernelGGL((qkv_rows_kernel<TX, TW, TC>), dim3(tokens, parts), dim3(256), lds, stream,
                           static_cast<const TX*>(x), static_cast<const TW*>(bq), static_cast<const TW*>(bk),
                           static_cast<const TW*>(bv), static_cast<const TW*>(wq), static_cast<const TW*>(wk), cos_t,
                           sin_t, static_cast<TX*>(q_out), static_cast<TC*>(kcache), static_cast<TC*>(vcache), positions,
                           token_entry, block_table, a))));
    PULSE_LAUNCH_CHECK("qkv_rows");
    if (write_kv) {
        PULSE_REQUIRE(nkv < 65536, "qkv_rows: too many key/value heads");
        PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW, PULSE_DISPATCH_DTYPE(c_dtype, TC,
            hipLaunchKernelGGL((v_rows_kernel<TX, TW, TC>), dim3((tokens + 15) / 16, nkv), dim3(256), 0, stream,
                               static_cast<const TX*>(x), static_cast<const TW*>(bv), static_cast<TC*>(vcache), positions,
                               token_entry, block_table, tokens, a))));
        PULSE_LAUNCH_CHECK("qkv_rows (values)");
    }
    return 0;
}
