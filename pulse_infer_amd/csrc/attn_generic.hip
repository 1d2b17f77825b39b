// Paged causal attention for any head size, page size and storage type: one
// wavefront per (token, query head), float32 arithmetic throughout.
//
// A token at position p sees keys lo..p of its own request through the block
// table, lo = max(0, p - window + 1) when a window is set, else 0.  Keys are
// taken 64 at a time (one per lane); the softmax is the running-maximum form
// (reference: src/ops/kernels/cuda/paged_attention.cu:88-137), the scale is a
// parameter (the reference fixes rsqrt(head_size), paged_attention.cu:108), and
// query head h reads kv head h / (nq / nkv) (paged_attention.cu:61-70).
//
// With `gate` every head's output is multiplied by sigmoid(gate[token, head]) before it is stored (an output gate
// whose logits another product left, one a token and head, `gate_stride` elements from row to row); with
// `gate_width` > 0 there is a logit for each of the first `gate_width` channels of every head instead
// (gate[token, head * gate_width + channel]).  `softcap` > 0 bounds the scaled scores, s <- cap * tanh(s / cap).
// `sink` (float32, one a query head) adds exp(sink[h]) to the softmax's denominator: a term without key or value.
//
// `keep_first` > 0 (with a window): the first keep_first keys of the request stay visible whatever the window, at their
// true positions.  `all_values`: a query head's weights are applied to the values of EVERY kv head, not only its own:
// the output row of (token, head) is nkv * d wide (value head c at columns c * d ..), in float32, for a caller that
// mixes the heads' weights afterwards (a weighted sum over query heads of these rows is the same as mixing the weights
// before they meet the values).
//
// This is the kernel of the true 32-bit path and the fallback for sizes that the
// matrix-core kernels refuse.
#include "common.h"

#include <math.h>

namespace {


struct AttnArgs {
    int nq, nkv, d;
    int64_t q_stride, o_stride;
    int page_size, num_pages, bt_width;
    float scale;
    int window;  // 0: all keys
    float cap;   // > 0: a score s becomes cap * tanh(s / cap); 0: scores as they are
    int gate_per_channel;   // 0: one gate logit a head; 1: one a channel (gate [T, nq * gate_width])
    int gate_width;         // channels of a head that have a gate logit (the others are stored ungated)
    int keep_first;         // with a window: keys 0 .. keep_first - 1 stay visible
    int all_values;         // 1: the values of all kv heads side by side (nkv * d accumulators a query head)
};

template <typename TX, typename TC, typename TO, int MAX_ACC>
__global__ __launch_bounds__(64) void attn_generic_kernel(const TX* __restrict__ q, TO* __restrict__ out,
                                                          const TC* __restrict__ kcache,
                                                          const TC* __restrict__ vcache,
                                                          const int* __restrict__ positions,
                                                          const int* __restrict__ token_entry,
                                                          const int* __restrict__ block_table,
                                                          const TX* __restrict__ gate, int64_t gate_stride,
                                                          const float* __restrict__ sink, AttnArgs a) {
    extern __shared__ long long lds[];
    long long* v_s = lds;                                         // [64] value offsets of a tile's keys
    float* p_s = reinterpret_cast<float*>(lds + PULSE_WAVE);      // [64] a tile's probabilities
    float* q_s = p_s + PULSE_WAVE;                                // [d]  the scaled query

    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x;
    const int d = a.d;
    const int group = a.nq / a.nkv;
    const int kvh = h / group;
    const int pos = positions[t];
    const int* bt = block_table + static_cast<int64_t>(token_entry[t]) * a.bt_width;
    const int lo = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;
    const int n_first = min(a.keep_first, lo);        // kept keys below the window
    const int total = n_first + pos - lo + 1;         // keys this token sees
    const int width = a.all_values ? a.nkv * d : d;   // values accumulated for this query head

    const TX* qrow = q + static_cast<int64_t>(t) * a.q_stride + static_cast<int64_t>(h) * d;
    for (int e = lane; e < d; e += PULSE_WAVE) q_s[e] = to_f32<TX>(qrow[e]) * a.scale;
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[MAX_ACC];
#pragma unroll
    for (int r = 0; r < MAX_ACC; ++r) acc[r] = 0.f;

    for (int u0 = 0; u0 < total; u0 += PULSE_WAVE) {
        const int u = u0 + lane;
        const int j = u < n_first ? u : lo + u - n_first;
        float s = -INFINITY;
        long long vbase = -1;
        if (u < total) {
            const int pi = j / a.page_size;
            const int page = pi < a.bt_width ? bt[pi] : -1;
            if (page >= 0 && page < a.num_pages) {
                const int slot = j % a.page_size;
                const int64_t pg = static_cast<int64_t>(page) * a.nkv + kvh;
                const TC* krow = kcache + (pg * a.page_size + slot) * d;
                float dot = 0.f;
                for (int e = 0; e < d; ++e) dot = fmaf(q_s[e], to_f32<TC>(krow[e]), dot);
                s = a.cap > 0.f ? a.cap * tanhf(dot / a.cap) : dot;
                vbase = (a.all_values ? static_cast<int64_t>(page) * a.nkv : pg) * d * a.page_size + slot;
            }
        }
        const float tile_max = wave_max(s);
        const float m_new = fmaxf(m, tile_max);
        // every tile holds at least one visible key; were its page missing, m_new could still be -inf
        const float alpha = (m_new == -INFINITY) ? 1.f : expf(m - m_new);
        const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
        l = l * alpha + wave_sum(p);
        m = m_new;
        p_s[lane] = p;
        v_s[lane] = vbase;
        __syncthreads();
        const int nkeys = min(PULSE_WAVE, total - u0);
#pragma unroll
        for (int r = 0; r < MAX_ACC; ++r) {
            const int e = lane + r * PULSE_WAVE;
            if (e < width) {
                float sum = 0.f;
                for (int jj = 0; jj < nkeys; ++jj) {
                    const long long vb = v_s[jj];
                    if (vb >= 0) sum = fmaf(p_s[jj], to_f32<TC>(vcache[vb + static_cast<int64_t>(e) * a.page_size]), sum);
                }
                acc[r] = acc[r] * alpha + sum;
            }
        }
        __syncthreads();
    }

    TO* orow = out + static_cast<int64_t>(t) * a.o_stride + static_cast<int64_t>(h) * width;
    // a sink is one more term of the softmax's denominator, exp(sink[h]), with no key and no value
    if (sink) {
        const float sk = sink[h];
        if (m == -INFINITY) { l = 1.f; }
        else if (sk > m) { l = l * expf(m - sk) + 1.f; const float f = expf(m - sk);
#pragma unroll
            for (int r = 0; r < MAX_ACC; ++r) acc[r] *= f; }
        else l += expf(sk - m);
    }
    float inv_l = l > 0.f ? 1.0f / l : 0.f;
    const TX* grow = gate ? gate + static_cast<int64_t>(t) * gate_stride : nullptr;
    if (grow && !a.gate_per_channel) inv_l *= 1.0f / (1.0f + expf(-to_f32<TX>(grow[h])));
#pragma unroll
    for (int r = 0; r < MAX_ACC; ++r) {
        const int e = lane + r * PULSE_WAVE;
        if (e < width) {
            float v = acc[r] * inv_l;
            if (grow && a.gate_per_channel && e < a.gate_width)
                v *= 1.0f / (1.0f + expf(-to_f32<TX>(grow[static_cast<int64_t>(h) * a.gate_width + e])));
            orow[e] = from_f32<TO>(v);
        }
    }
}

template <typename TX, typename TC, typename TO>
int launch_generic(int acc, const void* q, void* out, const void* kcache, const void* vcache, const int* positions,
                   const int* token_entry, const int* block_table, const void* gate, int64_t gate_stride,
                   const float* sink, const AttnArgs& a, int tokens, size_t lds, hipStream_t stream) {
#define PULSE_GENERIC_LAUNCH(N)                                                                                      \
    hipLaunchKernelGGL((attn_generic_kernel<TX, TC, TO, N>), dim3(tokens, a.nq), dim3(64), lds, stream,              \
                       static_cast<const TX*>(q), static_cast<TO*>(out), static_cast<const TC*>(kcache),            \
                       static_cast<const TC*>(vcache), positions, token_entry, block_table,                         \
                       static_cast<const TX*>(gate), gate_stride, sink, a)
    if (acc <= 2) PULSE_GENERIC_LAUNCH(2);
    else if (acc <= 8) PULSE_GENERIC_LAUNCH(8);
    else PULSE_GENERIC_LAUNCH(32);
#undef PULSE_GENERIC_LAUNCH
    return 0;
}

}  // namespace

// `out_f32`: out is float32 whatever the storage type of q (required with `all_values`, whose rows are nkv * d wide).
extern "C" int pulse_attn_generic_ex(const void* q, int64_t q_stride, void* out, int64_t o_stride, int x_dtype,
                                     const void* kcache, const void* vcache, int c_dtype, const int* positions,
                                     const int* token_entry, const int* block_table, int bt_width, int tokens, int nq,
                                     int nkv, int d, int page_size, int num_pages, float scale, int window,
                                     const void* gate, int64_t gate_stride, int gate_width, const float* sink,
                                     float softcap, int keep_first, int all_values, int out_f32, hipStream_t stream) {
    const int width = all_values ? nkv * d : d;
    PULSE_REQUIRE(tokens >= 0 && nq > 0 && nkv > 0 && d > 0, "attn_generic: bad sizes");
    PULSE_REQUIRE(nq % nkv == 0, "attn_generic: %d query heads are not a multiple of %d kv heads", nq, nkv);
    PULSE_REQUIRE(width <= PULSE_WAVE * 32, "attn_generic: head_dim %d gives %d value channels a query head, more than %d", d,
                  width, PULSE_WAVE * 32);
    PULSE_REQUIRE(nq < 65536, "attn_generic: at most 65535 query heads, got %d", nq);
    PULSE_REQUIRE(page_size > 0 && num_pages > 0 && bt_width > 0, "attn_generic: bad cache geometry");
    PULSE_REQUIRE(window >= 0 && keep_first >= 0, "attn_generic: negative window or kept keys");
    PULSE_REQUIRE(!all_values || (out_f32 && !gate), "attn_generic: all values side by side come out in float32, ungated");
    PULSE_REQUIRE(q_stride >= static_cast<int64_t>(nq) * d && o_stride >= static_cast<int64_t>(nq) * width,
                  "attn_generic: row strides too small");
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(c_dtype), "attn_generic: bad dtype tag");
    PULSE_REQUIRE(q && out && kcache && vcache && positions && token_entry && block_table, "attn_generic: null pointer");
    PULSE_REQUIRE(gate_width >= 0 && gate_width <= d, "attn_generic: %d gated channels of a head of %d", gate_width, d);
    PULSE_REQUIRE(!gate || gate_stride >= static_cast<int64_t>(nq) * (gate_width ? gate_width : 1),
                  "attn_generic: the gate's rows are too short");
    PULSE_REQUIRE(softcap >= 0.f, "attn_generic: a negative score cap");
    if (tokens == 0) return 0;
    AttnArgs a;
    a.nq = nq; a.nkv = nkv; a.d = d; a.q_stride = q_stride; a.o_stride = o_stride;
    a.page_size = page_size; a.num_pages = num_pages; a.bt_width = bt_width; a.scale = scale; a.window = window;
    a.cap = softcap; a.gate_per_channel = gate_width > 0 ? 1 : 0; a.gate_width = gate_width;
    a.keep_first = window > 0 ? keep_first : 0; a.all_values = all_values ? 1 : 0;
    const size_t lds = static_cast<size_t>(d) * sizeof(float) + PULSE_WAVE * sizeof(float) + PULSE_WAVE * sizeof(long long);
    const int acc = (width + PULSE_WAVE - 1) / PULSE_WAVE;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(c_dtype, TC,
        if (out_f32) launch_generic<TX, TC, float>(acc, q, out, kcache, vcache, positions, token_entry, block_table, gate,
                                                   gate_stride, sink, a, tokens, lds, stream);
        else launch_generic<TX, TC, TX>(acc, q, out, kcache, vcache, positions, token_entry, block_table, gate,
                                        gate_stride, sink, a, tokens, lds, stream)));
    PULSE_LAUNCH_CHECK("attn_generic");
    return 0;
}

extern "C" int pulse_attn_generic(const void* q, int64_t q_stride, void* out, int64_t o_stride, int x_dtype,
                                  const void* kcache, const void* vcache, int c_dtype, const int* positions,
                                  const int* token_entry, const int* block_table, int bt_width, int tokens, int nq,
                                  int nkv, int d, int page_size, int num_pages, float scale, int window,
                                  const void* gate, int64_t gate_stride, int gate_width, const float* sink,
                                  float softcap, hipStream_t stream) {
    return pulse_attn_generic_ex(q, q_stride, out, o_stride, x_dtype, kcache, vcache, c_dtype, positions, token_entry,
                                 block_table, bt_width, tokens, nq, nkv, d, page_size, num_pages, scale, window, gate,
                                 gate_stride, gate_width, sink, softcap, 0, 0, 0, stream);
}
