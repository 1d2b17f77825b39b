// The two kernels of a selective state-space mixer (Mamba) that are no matrix products.
//
// A request keeps, per channel c of the mixer's inner width, a row of float32 values in its state slot:
// state[slot, c, 0 .. N) is the recurrent state S[c, :], state[slot, c, N .. N + K - 1) are the last K - 1 inputs of
// the causal convolution (oldest first).  An entry that starts at position 0 starts from zeros, whatever the slot
// holds; that is read on the device from the step's arrays.
//
// pulse_causal_conv: y[t, c] = silu(bias[c] + sum_j taps[c, j] * in[p - (K - 1) + j, c]), p the token's position;
// inputs at positions of this step come from its rows, earlier ones from the slot's tail, positions before the
// sequence's start are zeros.  A second launch then moves the tail on to the step's end.  A thread a (token, channel).
//
// pulse_selective_scan walks the tokens of every entry in order:
//     dt      = softplus(dt_raw[t, c] + dt_bias[c])
//     S[c, n] = exp(dt * A[c, n]) * S[c, n] + dt * x[t, c] * B[t, n],     A = -exp(A_log)
//     y[t, c] = (sum_n S[c, n] * C[t, n] + D[c] * x[t, c]) * silu(z[t, c])
// L lanes share a channel's N states (n = lane + L * j) and add their shares of y through lane exchanges; the
// tokens' values are staged through LDS a chunk at a time while the next chunk is fetched; the same kernel serves
// prompt portions, decoded tokens and mixed batches, so a prompt cut anywhere goes through the same arithmetic.
// State, step sizes, decays, exponentials and sums are float32 whatever the storage type of the rows.
#include "common.h"

#include <math.h>

namespace {

constexpr int MAX_TAPS = 16;
constexpr int MAX_NS = 16;   // states a lane

// silu and softplus in float32: with the library's accurate functions where the rows are float32, with the
// hardware's exponential, logarithm and reciprocal (a few units in the last place, a handful of instructions) where
// the result is rounded to bfloat16 or feeds bfloat16 rows anyway.
template <typename TX>
__device__ __forceinline__ float silu_f(float v) {
    if constexpr (sizeof(TX) == 4) return v / (1.0f + expf(-v));
    else return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
}
template <typename TX>
__device__ __forceinline__ float softplus_f(float v) {
    if constexpr (sizeof(TX) == 4) return v > 20.f ? v : log1pf(expf(v));
    else return v > 20.f ? v : __logf(1.0f + __expf(v));
}

struct ConvArgs {
    int channels, taps, n_state, state_row;   // state_row = n_state + taps - 1
    int64_t in_stride, out_stride;
    int tokens, entries;
};

template <typename TX, typename TW>
__global__ __launch_bounds__(256) void causal_conv_kernel(const TX* __restrict__ in, const TW* __restrict__ taps,
                                                          const TW* __restrict__ bias, TX* __restrict__ out,
                                                          const float* __restrict__ state,
                                                          const int* __restrict__ positions,
                                                          const int* __restrict__ token_entry,
                                                          const int* __restrict__ entry_start,
                                                          const int* __restrict__ entry_first_row,
                                                          const int* __restrict__ entry_slot, ConvArgs a) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int t = blockIdx.y;
    if (c >= a.channels) return;
    const int e = token_entry[t];
    const int start = entry_start[e], row0 = entry_first_row[e];
    const int pos = positions[t];
    const int K = a.taps;
    const float* tail = state + (static_cast<int64_t>(entry_slot[e]) * a.channels + c) * a.state_row + a.n_state;
    float acc = bias ? to_f32<TW>(bias[c]) : 0.f;
    for (int j = 0; j < K; ++j) {
        const int q = pos - (K - 1) + j;
        float v = 0.f;
        if (q >= start) v = to_f32<TX>(in[static_cast<int64_t>(row0 + q - start) * a.in_stride + c]);
        else if (q >= 0) v = tail[(K - 1) - (start - q)];   // start > 0 here
        acc = fmaf(to_f32<TW>(taps[static_cast<int64_t>(c) * K + j]), v, acc);
    }
    out[static_cast<int64_t>(t) * a.out_stride + c] = from_f32<TX>(silu_f<TX>(acc));
}

// The same for bfloat16 rows whose sizes allow 16-byte accesses and at most 8 taps: a thread takes 8 neighbouring
// channels of CONV_TOKENS consecutive tokens, with the channels' taps in registers.
constexpr int CONV_TOKENS = 8;

template <typename TW>
__global__ __launch_bounds__(256) void causal_conv_bf16x8_kernel(const bf16_t* __restrict__ in, const TW* __restrict__ taps,
                                                                 const TW* __restrict__ bias, bf16_t* __restrict__ out,
                                                                 const float* __restrict__ state,
                                                                 const int* __restrict__ positions,
                                                                 const int* __restrict__ token_entry,
                                                                 const int* __restrict__ entry_start,
                                                                 const int* __restrict__ entry_first_row,
                                                                 const int* __restrict__ entry_slot, ConvArgs a) {
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (c >= a.channels) return;
    const int K = a.taps;
    float w[8][8], b[8];   // [tap][channel]
#pragma unroll
    for (int u = 0; u < 8; ++u) {
        b[u] = bias ? to_f32<TW>(bias[c + u]) : 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j][u] = j < K ? to_f32<TW>(taps[static_cast<int64_t>(c + u) * K + j]) : 0.f;
    }
    const int t_end = min(a.tokens, static_cast<int>(blockIdx.y + 1) * CONV_TOKENS);
    for (int t = blockIdx.y * CONV_TOKENS; t < t_end; ++t) {
        const int e = token_entry[t];
        const int start = entry_start[e], row0 = entry_first_row[e];
        const int pos = positions[t];
        const float* tail = state + (static_cast<int64_t>(entry_slot[e]) * a.channels + c) * a.state_row + a.n_state;
        float acc[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc[u] = b[u];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (j >= K) continue;
            const int q = pos - (K - 1) + j;
            if (q >= start) {
                const pulse_i32x4 raw = *reinterpret_cast<const pulse_i32x4*>(in + static_cast<int64_t>(row0 + q - start) * a.in_stride + c);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const uint32_t two = static_cast<uint32_t>(raw[u]);
                    acc[2 * u] = fmaf(w[j][2 * u], __uint_as_float(two << 16), acc[2 * u]);
                    acc[2 * u + 1] = fmaf(w[j][2 * u + 1], __uint_as_float(two & 0xffff0000u), acc[2 * u + 1]);
                }
            } else if (q >= 0) {
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    acc[u] = fmaf(w[j][u], tail[static_cast<int64_t>(u) * a.state_row + (K - 1) - (start - q)], acc[u]);
            }
        }
        uint32_t packed[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            packed[u] = static_cast<uint32_t>(f32_to_bf16(silu_f<bf16_t>(acc[2 * u]))) |
                        (static_cast<uint32_t>(f32_to_bf16(silu_f<bf16_t>(acc[2 * u + 1]))) << 16);
        *reinterpret_cast<uint4*>(out + static_cast<int64_t>(t) * a.out_stride + c) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    }
}

template <typename TX>
__global__ __launch_bounds__(256) void conv_tail_kernel(const TX* __restrict__ in, float* __restrict__ state,
                                                        const int* __restrict__ entry_start,
                                                        const int* __restrict__ entry_first_row,
                                                        const int* __restrict__ entry_slot, ConvArgs a) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int e = blockIdx.y;
    if (c >= a.channels) return;
    const int start = entry_start[e], row0 = entry_first_row[e];
    const int count = entry_first_row[e + 1] - row0;
    const int K = a.taps;
    float* tail = state + (static_cast<int64_t>(entry_slot[e]) * a.channels + c) * a.state_row + a.n_state;
    const int end = start + count;
    // place jj takes the input at position end - (K - 1) + jj; an old place that is read lies above every place
    // written so far (count >= 1), so the tail moves on in place
    for (int jj = 0; jj < K - 1; ++jj) {
        const int q = end - (K - 1) + jj;
        float v = 0.f;
        if (q >= start) v = to_f32<TX>(in[static_cast<int64_t>(row0 + q - start) * a.in_stride + c]);
        else if (q >= 0) v = tail[(K - 1) - (start - q)];
        tail[jj] = v;
    }
}

struct ScanArgs {
    int channels, n_state, state_row, entries;
    int64_t x_stride, dt_stride, bc_stride, z_stride, y_stride;
    int b0, c0;   // columns of B and C in a row of bc
};

constexpr int SCAN_THREADS = 256;

// A value of every lane of a group of L neighbouring lanes (L a power of two up to 16) summed over the group, left
// in all of them: exchanges inside a quad, then mirrored halves of a row of 16 lanes (no LDS traffic).
template <int CTRL>
__device__ __forceinline__ float lane_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

template <int L>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (L >= 2) v += lane_move<0xB1>(v);    // quad_perm [1, 0, 3, 2]
    if constexpr (L >= 4) v += lane_move<0x4E>(v);    // quad_perm [2, 3, 0, 1]
    if constexpr (L >= 8) v += lane_move<0x141>(v);   // row_half_mirror: the other quad of a half row
    if constexpr (L >= 16) v += lane_move<0x140>(v);  // row_mirror: the other half of a row
    return v;
}

// exp of the recurrence: the accurate one where the rows are float32, the fast one (one instruction behind a
// multiplication, a few units in the last place) where they are bfloat16 anyway.
template <typename TX>
__device__ __forceinline__ float decay_exp(float v) {
    if constexpr (sizeof(TX) == 4) return expf(v);
    else return __expf(v);
}

// A workgroup owns CH = 256 / L neighbouring channels of one entry; the L lanes of a channel hold NS neighbouring
// states each (n = lane * NS + j; NP = L * NS >= N).  Few lanes a channel keep the work that a token costs a
// channel once (its values read, the lanes' sums brought together, the result stored) small beside the updates.
// The tokens come through LDS a chunk of CHUNK at a time, a row of W = 3 CH + 2 NP floats a token:
//   [x: CH | dt = softplus(dt_raw + bias): CH | silu(z): CH | B: NP | C: NP]
// so that step sizes and gates are computed once a (token, channel) and B and C are read from memory once a
// workgroup.  While a chunk is walked the next one is on its way into registers, as loaded (nothing is computed
// with a value before the chunk in hand is through); the chunk's outputs leave together.
template <typename TX, typename TW, int NS, int L>
__global__ __launch_bounds__(SCAN_THREADS) void selective_scan_kernel(
        const TX* __restrict__ x, const TX* __restrict__ dt_raw, const TW* __restrict__ dt_bias,
        const TW* __restrict__ a_log, const TX* __restrict__ bc, const TW* __restrict__ d_skip,
        const TX* __restrict__ z, TX* __restrict__ y, float* __restrict__ state, const int* __restrict__ entry_start,
        const int* __restrict__ entry_first_row, const int* __restrict__ entry_slot, ScanArgs a) {
    constexpr int CH = SCAN_THREADS / L;
    constexpr int NP = L * NS;
    constexpr int W = 3 * CH + 2 * NP;
    constexpr int CHUNK = L == 16 ? 16 : 1024 / CH;
    constexpr int XS = CHUNK * CH / SCAN_THREADS;                          // values of x (dt, z) a thread stages
    constexpr int BS = (CHUNK * 2 * NP + SCAN_THREADS - 1) / SCAN_THREADS;   // values of B and C
    __shared__ __attribute__((aligned(16))) float rows_s[CHUNK * W];
    __shared__ float y_s[CHUNK * CH];
    __shared__ float bias_s[CH];
    const int tid = threadIdx.x;
    const int sub = tid % L, ch = tid / L;
    const int c0 = blockIdx.x * CH;
    const int c = c0 + ch;
    const int e = blockIdx.y;
    const bool live = c < a.channels;
    const int cc = live ? c : a.channels - 1;   // idle lanes walk along (the lane exchanges want whole wavefronts)
    const int start = entry_start[e], row0 = entry_first_row[e];
    const int count = entry_first_row[e + 1] - row0;
    const int N = a.n_state;
    if (tid < CH) bias_s[tid] = (dt_bias && c0 + tid < a.channels) ? to_f32<TW>(dt_bias[c0 + tid]) : 0.f;
    float* srow = state + (static_cast<int64_t>(entry_slot[e]) * a.channels + cc) * a.state_row;
    float S[NS], A[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int n = sub * NS + j;
        A[j] = n < N ? -expf(to_f32<TW>(a_log[static_cast<int64_t>(cc) * N + n])) : 0.f;
        S[j] = (n < N && start > 0) ? srow[n] : 0.f;
    }
    const float dsk = d_skip ? to_f32<TW>(d_skip[cc]) : 0.f;

    TX sx[XS], sd[XS], sz[XS], sb[BS];
    const TX zero = from_f32<TX>(0.f);
    auto fetch = [&](int base, int tokens) {
#pragma unroll
        for (int j = 0; j < XS; ++j) {
            const int i = tid + SCAN_THREADS * j;
            const int tt = i / CH, k = c0 + i % CH;
            const bool ok = tt < tokens && k < a.channels;
            const int64_t row = row0 + base + tt;
            sx[j] = ok ? x[row * a.x_stride + k] : zero;
            sd[j] = ok ? dt_raw[row * a.dt_stride + k] : zero;
            sz[j] = (ok && z) ? z[row * a.z_stride + k] : zero;
        }
#pragma unroll
        for (int j = 0; j < BS; ++j) {
            const int i = tid + SCAN_THREADS * j;
            const int tt = i / (2 * NP), col = i % (2 * NP);
            const int n = col % NP;
            const bool ok = tt < tokens && tt < CHUNK && n < N;
            sb[j] = ok ? bc[static_cast<int64_t>(row0 + base + tt) * a.bc_stride + (col < NP ? a.b0 : a.c0) + n] : zero;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int j = 0; j < XS; ++j) {
            const int i = tid + SCAN_THREADS * j;
            float* r = rows_s + (i / CH) * W + i % CH;
            r[0] = to_f32<TX>(sx[j]);
            r[CH] = softplus_f<TX>(to_f32<TX>(sd[j]) + bias_s[i % CH]);
            r[2 * CH] = z ? silu_f<TX>(to_f32<TX>(sz[j])) : 1.f;
        }
#pragma unroll
        for (int j = 0; j < BS; ++j) {
            const int i = tid + SCAN_THREADS * j;
            if (i < CHUNK * 2 * NP) rows_s[(i / (2 * NP)) * W + 3 * CH + i % (2 * NP)] = to_f32<TX>(sb[j]);
        }
    };

    fetch(0, min(CHUNK, count));
    __syncthreads();   // bias_s
    stash();
    __syncthreads();
    for (int base = 0; base < count; base += CHUNK) {
        const int here = min(CHUNK, count - base);
        const int next = min(CHUNK, count - base - CHUNK);
        if (next > 0) fetch(base + CHUNK, next);
        for (int tt = 0; tt < here; ++tt) {
            const float* r = rows_s + tt * W;
            const float xv = r[ch], dt = r[CH + ch], gate = r[2 * CH + ch];
            const float dtx = dt * xv;
            float part = 0.f;
#pragma unroll
            for (int j = 0; j < NS; ++j) {
                S[j] = fmaf(decay_exp<TX>(dt * A[j]), S[j], dtx * r[3 * CH + sub * NS + j]);
                part = fmaf(S[j], r[3 * CH + NP + sub * NS + j], part);
            }
            part = group_sum<L>(part);
            const float out = fmaf(dsk, xv, part) * gate;
            if (sub == 0) y_s[tt * CH + ch] = out;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < XS; ++j) {
            const int i = tid + SCAN_THREADS * j;
            const int tt = i / CH, k = c0 + i % CH;
            if (tt < here && k < a.channels)
                y[static_cast<int64_t>(row0 + base + tt) * a.y_stride + k] = from_f32<TX>(y_s[i]);
        }
        if (next > 0) stash();   // (the rows in LDS have been read by everybody: the barrier above)
        __syncthreads();
    }
    if (live) {
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            const int n = sub * NS + j;
            if (n < N) srow[n] = S[j];
        }
    }
}

}  // namespace

extern "C" int pulse_causal_conv(const void* in, int64_t in_stride, int x_dtype, const void* taps, const void* bias,
                                 int w_dtype, void* out, int64_t out_stride, float* state, int slots, int n_state,
                                 const int* positions, const int* token_entry, const int* entry_start,
                                 const int* entry_first_row, const int* entry_slot, int tokens, int entries,
                                 int channels, int n_taps, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && entries >= 0 && channels > 0 && n_state >= 0 && slots > 0, "causal_conv: bad sizes");
    PULSE_REQUIRE(n_taps >= 1 && n_taps <= MAX_TAPS, "causal_conv: 1 to %d taps, got %d", MAX_TAPS, n_taps);
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype), "causal_conv: bad dtype tag");
    PULSE_REQUIRE(in && taps && out && state && positions && token_entry && entry_start && entry_first_row && entry_slot,
                  "causal_conv: null pointer");
    PULSE_REQUIRE(in_stride >= channels && out_stride >= channels, "causal_conv: rows are too short");
    PULSE_REQUIRE(tokens < 65536 && entries < 65536, "causal_conv: at most 65535 tokens a step");
    if (tokens == 0 || entries == 0) return 0;
    ConvArgs a;
    a.channels = channels; a.taps = n_taps; a.n_state = n_state; a.state_row = n_state + n_taps - 1;
    a.in_stride = in_stride; a.out_stride = out_stride; a.tokens = tokens; a.entries = entries;
    const int blocks = (channels + 255) / 256;
    // (few tokens, a decoding step: a thread a channel gives more workgroups, which is what counts there)
    const bool wide = tokens >= 64 && n_taps <= 8 && x_dtype == PULSE_BF16 && channels % 8 == 0 && in_stride % 8 == 0 && out_stride % 8 == 0 &&
                      reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    if (wide) {
        const int threads = channels / 8 >= 256 ? 256 : 64;
        PULSE_DISPATCH_DTYPE(w_dtype, TW,
            hipLaunchKernelGGL((causal_conv_bf16x8_kernel<TW>),
                               dim3((channels / 8 + threads - 1) / threads, (tokens + CONV_TOKENS - 1) / CONV_TOKENS),
                               dim3(threads), 0, stream, static_cast<const bf16_t*>(in), static_cast<const TW*>(taps),
                               static_cast<const TW*>(bias), static_cast<bf16_t*>(out), state, positions, token_entry,
                               entry_start, entry_first_row, entry_slot, a));
    } else {
        PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
            hipLaunchKernelGGL((causal_conv_kernel<TX, TW>), dim3(blocks, tokens), dim3(256), 0, stream,
                               static_cast<const TX*>(in), static_cast<const TW*>(taps), static_cast<const TW*>(bias),
                               static_cast<TX*>(out), state, positions, token_entry, entry_start, entry_first_row,
                               entry_slot, a)));
    }
    PULSE_LAUNCH_CHECK("causal_conv");
    if (n_taps > 1) {
        PULSE_DISPATCH_DTYPE(x_dtype, TX,
            hipLaunchKernelGGL((conv_tail_kernel<TX>), dim3(blocks, entries), dim3(256), 0, stream,
                               static_cast<const TX*>(in), state, entry_start, entry_first_row, entry_slot, a));
        PULSE_LAUNCH_CHECK("causal_conv (tail)");
    }
    return 0;
}

extern "C" int pulse_selective_scan(const void* x, int64_t x_stride, const void* dt_raw, int64_t dt_stride,
                                    const void* bc, int64_t bc_stride, int b0, int c0, const void* z, int64_t z_stride,
                                    void* y, int64_t y_stride, int x_dtype, const void* dt_bias, const void* a_log,
                                    const void* d_skip, int w_dtype, float* state, int slots, int state_row,
                                    const int* entry_start, const int* entry_first_row, const int* entry_slot,
                                    int entries, int channels, int n_state, hipStream_t stream) {
    PULSE_REQUIRE(entries >= 0 && channels > 0 && n_state > 0 && slots > 0, "selective_scan: bad sizes");
    PULSE_REQUIRE(state_row >= n_state, "selective_scan: a state row of %d values cannot hold %d states", state_row, n_state);
    PULSE_REQUIRE(n_state <= 16 * MAX_NS, "selective_scan: at most %d states a channel, got %d", 16 * MAX_NS, n_state);
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && pulse_dtype_ok(w_dtype), "selective_scan: bad dtype tag");
    PULSE_REQUIRE(x && dt_raw && bc && y && a_log && state && entry_start && entry_first_row && entry_slot,
                  "selective_scan: null pointer");
    PULSE_REQUIRE(x_stride >= channels && dt_stride >= channels && y_stride >= channels && (!z || z_stride >= channels),
                  "selective_scan: rows are too short");
    PULSE_REQUIRE(b0 >= 0 && c0 >= 0 && bc_stride >= b0 + n_state && bc_stride >= c0 + n_state,
                  "selective_scan: B and C do not lie inside their rows");
    PULSE_REQUIRE(entries < 65536, "selective_scan: at most 65535 entries a step");
    if (entries == 0) return 0;
    // lanes a channel: few while a lane's share of the states stays within 16 (see the kernel); more where that
    // would leave compute units without a workgroup (one long prompt: then the walk's latency is what counts, and
    // a channel's states spread over more lanes shorten it)
    int lanes = n_state == 1 ? 1 : (n_state == 2 ? 2 : (n_state <= 64 ? 4 : 16));
    const int64_t units = pulse_compute_units();
    if (lanes == 4 && n_state >= 8 && static_cast<int64_t>((channels + 63) / 64) * entries < units) lanes = 8;
    if (lanes == 8 && n_state >= 16 && static_cast<int64_t>((channels + 31) / 32) * entries < units) lanes = 16;
    if (lanes == 8 && n_state > 128) lanes = 16;
    const int ns = (n_state + lanes - 1) / lanes;
    ScanArgs a;
    a.channels = channels; a.n_state = n_state; a.state_row = state_row; a.entries = entries;
    a.x_stride = x_stride; a.dt_stride = dt_stride; a.bc_stride = bc_stride; a.z_stride = z_stride; a.y_stride = y_stride;
    a.b0 = b0; a.c0 = c0;
    const int per_block = SCAN_THREADS / lanes;
    const dim3 grid((channels + per_block - 1) / per_block, entries);
#define PULSE_SCAN(NS_, L_)                                                                                          \
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,                                              \
        hipLaunchKernelGGL((selective_scan_kernel<TX, TW, NS_, L_>), grid, dim3(SCAN_THREADS), 0, stream,           \
                           static_cast<const TX*>(x), static_cast<const TX*>(dt_raw), static_cast<const TW*>(dt_bias), \
                           static_cast<const TW*>(a_log), static_cast<const TX*>(bc), static_cast<const TW*>(d_skip), \
                           static_cast<const TX*>(z), static_cast<TX*>(y), state, entry_start, entry_first_row,       \
                           entry_slot, a)))
#define PULSE_SCAN_NS(L_)                        \
    do {                                         \
        if (ns <= 1) PULSE_SCAN(1, L_);          \
        else if (ns <= 2) PULSE_SCAN(2, L_);     \
        else if (ns <= 4) PULSE_SCAN(4, L_);     \
        else if (ns <= 8) PULSE_SCAN(8, L_);     \
        else PULSE_SCAN(16, L_);                 \
    } while (0)
    if (lanes == 1) PULSE_SCAN(1, 1);
    else if (lanes == 2) PULSE_SCAN(1, 2);
    else if (lanes == 4) PULSE_SCAN_NS(4);
    else if (lanes == 8) PULSE_SCAN_NS(8);
    else PULSE_SCAN_NS(16);
#undef PULSE_SCAN_NS
#undef PULSE_SCAN
    PULSE_LAUNCH_CHECK("selective_scan");
    return 0;
}
