// A residual kept in several streams (hyper-connections), and the layer norm that reads it.
//
// The residual of a token is S rows of H float32 values side by side: x [T, S, H].  A sublayer reads one row that
// is a weighted sum of the streams, and its result y goes back into every stream while the streams are mixed:
//
//     u      = sum_s in[s] x_s                                    (what the sublayer's norm reads)
//     x_t'   = sum_s mix[s, t] x_s + out[t] * y                   (all streams at once from the old ones)
//
// pulse_streams_step does, for every row r (token s = rows ? rows[r] : r), whichever of these it is handed:
//   1. the update of the token's streams with a sublayer's result y (written back in place; with a list of rows
//      the new streams are formed but not stored: whoever gathers rows reads the residual for the last time), then
//   2. u = sum_s in[s] x_s over the (new) streams (in == null: every factor is one), and the norm of u:
//        layer norm  (u - mean) / sqrt(var + eps) * w + b    (var the mean of the squared deviations), or
//        RMS norm    u / sqrt(mean(u^2) + eps) * w           (b == null and kind == 1)
//      rounded once into `out`.
// One workgroup a row; u lies in LDS, so mean and variance take two passes over exact values.  S == 1 with no
// update and no factors is a plain norm of a plain residual.  Everything is float32 up to the store.
//
// pulse_embed_streams: the embedding gather that fills all S streams of a token with the same row.
#include "common.h"

#include <math.h>

namespace {

constexpr int MAX_STREAMS = 16;

struct StreamArgs {
    int streams, hidden;
    int kind;        // 0: layer norm, 1: RMS norm
    float eps;
    int has_out;     // step 2 is wanted
};

// SC: the number of streams where it is one the kernel is compiled for (1 to 4: loops unroll, the mixing matrix
// lies in registers), 0: any number up to MAX_STREAMS, read from the arguments.
template <typename TYIN, typename TW, typename TO, int SC>
__global__ __launch_bounds__(1024) void streams_step_kernel(float* __restrict__ x, const TYIN* __restrict__ y,
                                                            const float* __restrict__ mix,
                                                            const float* __restrict__ out_w,
                                                            const float* __restrict__ in_w,
                                                            const int* __restrict__ rows, const TW* __restrict__ w,
                                                            const TW* __restrict__ b, TO* __restrict__ out,
                                                            StreamArgs a) {
    extern __shared__ float u_s[];    // [hidden]
    __shared__ float scratch[16];
    __shared__ float mix_s[MAX_STREAMS * MAX_STREAMS], ow_s[MAX_STREAMS], iw_s[MAX_STREAMS];
    constexpr int MS = SC ? SC : MAX_STREAMS;
    const int r = blockIdx.x;
    const int64_t t = rows ? rows[r] : r;
    const int S = SC ? SC : a.streams, H = a.hidden;
    if (threadIdx.x < S * S && mix) mix_s[threadIdx.x] = mix[threadIdx.x];
    if (threadIdx.x < S) {
        ow_s[threadIdx.x] = out_w ? out_w[threadIdx.x] : 0.f;
        iw_s[threadIdx.x] = in_w ? in_w[threadIdx.x] : 1.f;
    }
    __syncthreads();
    float mixr[SC ? SC * SC : 1], owr[MS], iwr[MS];
#pragma unroll
    for (int s = 0; s < MS; ++s) {
        owr[s] = s < S ? ow_s[s] : 0.f;
        iwr[s] = s < S ? iw_s[s] : 0.f;
    }
    if constexpr (SC > 0) {
#pragma unroll
        for (int i = 0; i < SC * SC; ++i) mixr[i] = y ? mix_s[i] : 0.f;
    }
    float* xrow = x + t * S * H;
    float sum = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float old[MS];
#pragma unroll
        for (int s = 0; s < MS; ++s) old[s] = s < S ? xrow[s * H + i] : 0.f;
        float u = 0.f;
        if (y) {
            const float yv = to_f32<TYIN>(y[t * H + i]);
#pragma unroll
            for (int to = 0; to < MS; ++to) {
                if (to < S) {
                    float v = 0.f;
#pragma unroll
                    for (int s = 0; s < MS; ++s)
                        if (s < S) v = fmaf(SC ? mixr[SC ? s * SC + to : 0] : mix_s[s * S + to], old[s], v);
                    v = fmaf(owr[to], yv, v);
                    if (!rows) xrow[to * H + i] = v;
                    u = fmaf(iwr[to], v, u);
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < MS; ++s)
                if (s < S) u = fmaf(iwr[s], old[s], u);
        }
        if (a.has_out) {
            u_s[i] = u;
            sum += u;
        }
    }
    if (!a.has_out) return;
    float mean = 0.f;
    if (a.kind == 0) mean = block_sum(sum, scratch) / static_cast<float>(H);
    else __syncthreads();
    float sq = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float d = u_s[i] - mean;
        sq = fmaf(d, d, sq);
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, scratch) / static_cast<float>(H) + a.eps);
    TO* orow = out + static_cast<int64_t>(r) * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = (u_s[i] - mean) * inv * to_f32<TW>(w[i]);
        if (b) v += to_f32<TW>(b[i]);
        orow[i] = from_f32<TO>(v);
    }
}

template <typename TW>
__global__ void embed_streams_kernel(const int* __restrict__ ids, const TW* __restrict__ table, float* __restrict__ out,
                                     int hidden, int vocab, int streams, int* bad_id, float scale) {
    const int t = blockIdx.x;
    const int id = ids[t];
    float* dst = out + static_cast<int64_t>(t) * hidden * streams;
    const bool bad = id < 0 || id >= vocab;
    if (bad && threadIdx.x == 0) *bad_id = 1;
    const TW* src = table + static_cast<int64_t>(bad ? 0 : id) * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
        const float v = bad ? __builtin_nanf("") : to_f32<TW>(src[i]) * scale;
        for (int s = 0; s < streams; ++s) dst[s * hidden + i] = v;
    }
}

}  // namespace

extern "C" int pulse_streams_step(float* x, int tokens, int streams, int hidden, const void* y, int y_dtype,
                                  const float* mix, const float* out_w, const float* in_w, const int* rows, int n_rows,
                                  const void* w, const void* b, int w_dtype, int kind, float eps, void* out,
                                  int out_dtype, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && n_rows >= 0 && hidden > 0 && x, "streams_step: bad sizes");
    PULSE_REQUIRE(streams >= 1 && streams <= MAX_STREAMS, "streams_step: 1 to %d streams, got %d", MAX_STREAMS, streams);
    PULSE_REQUIRE(pulse_dtype_ok(y_dtype) && pulse_dtype_ok(w_dtype) && pulse_dtype_ok(out_dtype), "streams_step: bad dtype tag");
    PULSE_REQUIRE(!y || (mix && out_w), "streams_step: an update needs the mixing matrix and the result's factors");
    PULSE_REQUIRE(!(y && rows) || out, "streams_step: an update of gathered rows is not stored, so it comes with a norm");
    PULSE_REQUIRE(y || out, "streams_step: nothing to do");
    PULSE_REQUIRE(!out || w, "streams_step: the norm's weight is missing");
    PULSE_REQUIRE(kind == 0 || kind == 1, "streams_step: unknown norm %d", kind);
    PULSE_REQUIRE(rows || n_rows == tokens, "streams_step: %d rows of %d tokens without a list of rows", n_rows, tokens);
    const size_t lds = sizeof(float) * static_cast<size_t>(hidden);
    PULSE_REQUIRE(lds <= 60 * 1024, "streams_step: rows of %d values do not fit the workgroup's memory", hidden);
    if (n_rows == 0) return 0;
    StreamArgs a;
    a.streams = streams; a.hidden = hidden; a.kind = kind; a.eps = eps; a.has_out = out ? 1 : 0;
    // few rows of a wide residual (a decoding step): wider workgroups, since there are not many of them
    const int threads = (n_rows <= 256 && hidden >= 2048) ? 1024 : 256;
#define PULSE_STREAMS(SC_)                                                                                           \
    PULSE_DISPATCH_DTYPE(y_dtype, TYIN, PULSE_DISPATCH_DTYPE(w_dtype, TW, PULSE_DISPATCH_DTYPE(out_dtype, TO,        \
        hipLaunchKernelGGL((streams_step_kernel<TYIN, TW, TO, SC_>), dim3(n_rows), dim3(threads), lds, stream, x,    \
                           static_cast<const TYIN*>(y), mix, out_w, in_w, rows, static_cast<const TW*>(w),           \
                           static_cast<const TW*>(b), static_cast<TO*>(out), a))))
    if (streams == 1) PULSE_STREAMS(1);
    else if (streams == 2) PULSE_STREAMS(2);
    else if (streams == 3) PULSE_STREAMS(3);
    else if (streams == 4) PULSE_STREAMS(4);
    else PULSE_STREAMS(0);
#undef PULSE_STREAMS
    PULSE_LAUNCH_CHECK("streams_step");
    return 0;
}

extern "C" int pulse_embed_streams(const int* ids, const void* table, int table_dtype, float* out, int tokens,
                                   int hidden, int vocab, int streams, int* bad_id, float scale, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && hidden > 0 && vocab > 0 && streams >= 1, "embed_streams: bad sizes");
    PULSE_REQUIRE(pulse_dtype_ok(table_dtype) && ids && table && out && bad_id, "embed_streams: bad arguments");
    if (tokens == 0) return 0;
    PULSE_DISPATCH_DTYPE(table_dtype, TW,
        hipLaunchKernelGGL(embed_streams_kernel<TW>, dim3(tokens), dim3(256), 0, stream, ids,
                           static_cast<const TW*>(table), out, hidden, vocab, streams, bad_id, scale));
    PULSE_LAUNCH_CHECK("embed_streams");
    return 0;
}
