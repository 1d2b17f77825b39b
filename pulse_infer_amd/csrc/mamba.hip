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
// L lanes share a channel's N states (n = lane + L * j) and add their shares of y through lane exchanges; the same
// kernel serves prompt portions, decoded tokens and mixed batches, so a prompt cut anywhere goes through the same
// arithmetic.  State, step sizes, decays, exponentials and sums are float32 whatever the storage type of the rows.
#include "common.h"

#include <math.h>

namespace {

constexpr int MAX_TAPS = 16;
constexpr int MAX_NS = 16;   // states a lane

__device__ __forceinline__ float silu_f(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }

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
    out[static_cast<int64_t>(t) * a.out_stride + c] = from_f32<TX>(silu_f(acc));
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
    int channels, n_state, state_row, lanes, entries;
    int64_t x_stride, dt_stride, bc_stride, z_stride, y_stride;
    int b0, c0;   // columns of B and C in a row of bc
};

template <typename TX, typename TW, int NS>
__global__ __launch_bounds__(256) void selective_scan_kernel(const TX* __restrict__ x, const TX* __restrict__ dt_raw,
                                                             const TW* __restrict__ dt_bias,
                                                             const TW* __restrict__ a_log, const TX* __restrict__ bc,
                                                             const TW* __restrict__ d_skip, const TX* __restrict__ z,
                                                             TX* __restrict__ y, float* __restrict__ state,
                                                             const int* __restrict__ entry_start,
                                                             const int* __restrict__ entry_first_row,
                                                             const int* __restrict__ entry_slot, ScanArgs a) {
    const int L = a.lanes;
    const int per_block = blockDim.x / L;
    const int sub = threadIdx.x % L;
    const int c = blockIdx.x * per_block + threadIdx.x / L;
    const int e = blockIdx.y;
    const bool live = c < a.channels;
    const int cc = live ? c : a.channels - 1;   // idle lanes walk along (the lane exchanges want whole wavefronts)
    const int start = entry_start[e], row0 = entry_first_row[e];
    const int count = entry_first_row[e + 1] - row0;
    const int N = a.n_state;
    float* srow = state + (static_cast<int64_t>(entry_slot[e]) * a.channels + cc) * a.state_row;
    float S[NS], A[NS];
#pragma unroll
    for (int j = 0; j < NS; ++j) {
        const int n = sub + L * j;
        A[j] = n < N ? -expf(to_f32<TW>(a_log[static_cast<int64_t>(cc) * N + n])) : 0.f;
        S[j] = (n < N && start > 0) ? srow[n] : 0.f;
    }
    const float bias = dt_bias ? to_f32<TW>(dt_bias[cc]) : 0.f;
    const float dsk = d_skip ? to_f32<TW>(d_skip[cc]) : 0.f;
    // the next token's values are asked for while this token's are worked on
    float xv, dv, zv, Bn[NS], Cn[NS];
    auto fetch = [&](int i, float& fx, float& fd, float& fz, float* fb, float* fc) {
        const int64_t row = row0 + i;
        fx = to_f32<TX>(x[row * a.x_stride + cc]);
        fd = to_f32<TX>(dt_raw[row * a.dt_stride + cc]);
        fz = z ? to_f32<TX>(z[row * a.z_stride + cc]) : 0.f;
        const TX* r = bc + row * a.bc_stride;
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            const int n = sub + L * j;
            fb[j] = n < N ? to_f32<TX>(r[a.b0 + n]) : 0.f;
            fc[j] = n < N ? to_f32<TX>(r[a.c0 + n]) : 0.f;
        }
    };
    if (count > 0) fetch(0, xv, dv, zv, Bn, Cn);
    for (int i = 0; i < count; ++i) {
        float nx = 0.f, nd = 0.f, nz = 0.f, nB[NS], nC[NS];
        if (i + 1 < count) fetch(i + 1, nx, nd, nz, nB, nC);
        const float dt = softplus_f(dv + bias);
        const float dtx = dt * xv;
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            S[j] = fmaf(expf(dt * A[j]), S[j], dtx * Bn[j]);
            part = fmaf(S[j], Cn[j], part);
        }
        for (int off = L / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, PULSE_WAVE);
        if (live && sub == 0) {
            float out = fmaf(dsk, xv, part);
            if (z) out *= silu_f(zv);
            y[static_cast<int64_t>(row0 + i) * a.y_stride + c] = from_f32<TX>(out);
        }
        if (i + 1 < count) {
            xv = nx; dv = nd; zv = nz;
#pragma unroll
            for (int j = 0; j < NS; ++j) { Bn[j] = nB[j]; Cn[j] = nC[j]; }
        }
    }
    if (live) {
#pragma unroll
        for (int j = 0; j < NS; ++j) {
            const int n = sub + L * j;
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
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((causal_conv_kernel<TX, TW>), dim3(blocks, tokens), dim3(256), 0, stream,
                           static_cast<const TX*>(in), static_cast<const TW*>(taps), static_cast<const TW*>(bias),
                           static_cast<TX*>(out), state, positions, token_entry, entry_start, entry_first_row,
                           entry_slot, a)));
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
    int lanes = 1;
    while (lanes < 16 && lanes < n_state) lanes *= 2;
    const int ns = (n_state + lanes - 1) / lanes;
    ScanArgs a;
    a.channels = channels; a.n_state = n_state; a.state_row = state_row; a.lanes = lanes; a.entries = entries;
    a.x_stride = x_stride; a.dt_stride = dt_stride; a.bc_stride = bc_stride; a.z_stride = z_stride; a.y_stride = y_stride;
    a.b0 = b0; a.c0 = c0;
    const int per_block = 256 / lanes;
    const dim3 grid((channels + per_block - 1) / per_block, entries);
#define PULSE_SCAN(NS_)                                                                                              \
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,                                              \
        hipLaunchKernelGGL((selective_scan_kernel<TX, TW, NS_>), grid, dim3(256), 0, stream,                        \
                           static_cast<const TX*>(x), static_cast<const TX*>(dt_raw), static_cast<const TW*>(dt_bias), \
                           static_cast<const TW*>(a_log), static_cast<const TX*>(bc), static_cast<const TW*>(d_skip), \
                           static_cast<const TX*>(z), static_cast<TX*>(y), state, entry_start, entry_first_row,       \
                           entry_slot, a)))
    if (ns <= 1) PULSE_SCAN(1);
    else if (ns <= 2) PULSE_SCAN(2);
    else if (ns <= 4) PULSE_SCAN(4);
    else if (ns <= 8) PULSE_SCAN(8);
    else PULSE_SCAN(16);
#undef PULSE_SCAN
    PULSE_LAUNCH_CHECK("selective_scan");
    return 0;
}
