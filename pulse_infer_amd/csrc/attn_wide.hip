// Paged attention on the matrix cores for query heads that gather WIDE values: the values of every kv head side by
// side (a caller that mixes the heads' weights afterwards) or one wide latent row shared by all heads; with a window
// that keeps a request's first tokens, and sinks.  bfloat16 operands, float32 everything else, float32 results.
//
// An item is R tiles of 16 rows: `hp` query heads of one kv head for 16 R / hp consecutive tokens of one request (a
// decoded token is an item of its group's heads alone).  A workgroup takes an item and a chunk of 16 CT value channels;
// its four wavefronts share the item's keys out in steps of 32 and meet in LDS at the end.  Every key and value
// operand a wavefront fetches serves all R row tiles (R = 4, CT = 8 for prompt portions: the same accumulators as R =
// 1, CT = 16 for decoded tokens, a quarter of the traffic a row).  Per step, row tile and wavefront:
//
//   S^T = K Q^T      two tiles of 16 keys x 16 rows (v_mfma_f32_16x16x32_bf16 over the head's channels): a lane then
//                    holds, for ITS row (lane % 16), the scores of keys 4 (lane / 16) + i of both tiles;
//   softmax          running maximum and sum per row (a row's lanes meet by two shuffles), scores never leave registers;
//   O^T += V^T P^T   the lane's eight weights ARE its share of the P^T operand if the step's 32 keys are taken in the
//                    order tile 0 keys 4g..4g+3, tile 1 keys 4g..4g+3 (g = lane / 16), so the V^T operand is read in
//                    that order: two 8-byte loads from the page's channel-major values.
//
// Keys come straight from the pages.  The visible keys of an item are the kept first tokens (rounded up to whole
// 16-key tiles) and the tiles from the one that holds the first row's window start to the last row's position; what a
// row must not see inside them is masked by its own position.  Values of keys behind the item's last position have
// never been written and are cleared in the operand (a weight of zero times whatever lies there must stay zero).
#include "common.h"

#include <math.h>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;

constexpr int MAX_TILES = 16;               // channel tiles of 16 a workgroup accumulates at most

struct WideArgs {
    int nq, nkv, d;       // d: stored channels of a head (keys and values alike)
    int w;                // value channels a query head gathers: nkv * d with all_values, else d
    int wv;               // of which are computed (a multiple of 16)
    int all_values, hp;
    int64_t q_stride, o_stride;
    int page_size, num_pages, bt_width;
    float scale, cap;
    int window, keep_first;
    int n_splits;         // > 1: the keys' steps are shared out over gridDim.z workgroups, whose sums go to `part`
    float* part;          // [tokens, nq, n_splits, w] sums not yet divided
    float* part_ml;       // [tokens, nq, n_splits, 2] maximum and sum of weights
};

__device__ __forceinline__ bf16x8 zeros8() {
    return __builtin_bit_cast(bf16x8, u32x4{0u, 0u, 0u, 0u});
}

template <int R, int CT>
__global__ __launch_bounds__(256, R == 1 ? 3 : 1) void attn_wide_kernel(const bf16_t* __restrict__ q, float* __restrict__ out,
                                                        const bf16_t* __restrict__ kcache,
                                                        const bf16_t* __restrict__ vcache,
                                                        const int* __restrict__ positions,
                                                        const int* __restrict__ token_entry,
                                                        const int* __restrict__ block_table,
                                                        const int* __restrict__ items, const float* __restrict__ sink,
                                                        WideArgs a) {
    __shared__ float red[2][CT][PULSE_WAVE][4];
    __shared__ float ml[4][16][2];
    const int* it = items + 4 * blockIdx.x;
    const int t0 = it[0], nt = it[1], head0 = it[2], nh = it[3];
    const int chunk0 = blockIdx.y * (16 * CT);
    const int tiles = min(CT, (a.wv - chunk0) / 16);
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
    const int r = lane % 16, g = lane / 16;
    const int d = a.d;
    bool valid[R];
    int tok[R], head[R], pos[R];
    const bf16_t* qrow[R];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const int row = 16 * rr + r, ti = row / a.hp, hi = row % a.hp;
        valid[rr] = ti < nt && hi < nh;
        tok[rr] = t0 + (valid[rr] ? ti : 0);
        head[rr] = head0 + (valid[rr] ? hi : 0);
        pos[rr] = positions[tok[rr]];
        qrow[rr] = q + static_cast<int64_t>(tok[rr]) * a.q_stride + static_cast<int64_t>(head[rr]) * d;
    }
    const int kvh = head0 / (a.nq / a.nkv);
    const int* bt = block_table + static_cast<int64_t>(token_entry[t0]) * a.bt_width;
    const int pos_first = positions[t0], pos_last = positions[t0 + nt - 1];
    const int lo = (a.window > 0 && pos_first - a.window + 1 > 0) ? pos_first - a.window + 1 : 0;
    const int lo16 = lo & ~15;
    const int nfirst = a.window > 0 ? min((a.keep_first + 15) & ~15, lo16) : 0;
    const int total = nfirst + pos_last + 1 - lo16;
    const int nsteps = (total + 31) / 32;

    float m_run[R], l_run[R];
    f32x4 acc[R][CT];
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        m_run[rr] = -INFINITY;
        l_run[rr] = 0.f;
#pragma unroll
        for (int c = 0; c < CT; ++c) acc[rr][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    const int per_split = (nsteps + a.n_splits - 1) / a.n_splits;
    const int step0 = static_cast<int>(blockIdx.z) * per_split, step1 = min(nsteps, step0 + per_split);
    // the page numbers of a step are asked for a step ahead, so that their trip lies behind the step in hand
    auto lookup = [&](int st, int t) __attribute__((always_inline)) {
        const int ub = st * 32 + 16 * t;
        const int jb = ub < nfirst ? ub : lo16 + ub - nfirst;
        const int pi = jb / a.page_size;
        return (st < step1 && ub < total && pi < a.bt_width) ? bt[pi] : -1;
    };
    int ahead[2] = {lookup(step0 + wave, 0), lookup(step0 + wave, 1)};
    for (int step = step0 + wave; step < step1; step += 4) {
        int page[2], off[2], jbase[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int ub = step * 32 + 16 * t;
            const int jb = ub < nfirst ? ub : lo16 + ub - nfirst;
            const int p = ahead[t];
            page[t] = (p >= 0 && p < a.num_pages) ? p : -1;
            off[t] = jb % a.page_size;
            jbase[t] = jb;
        }
        ahead[0] = lookup(step + 4, 0);
        ahead[1] = lookup(step + 4, 1);
        // S^T: keys x rows, for every row tile from the same key operands
        f32x4 s[R][2];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) s[rr][0] = s[rr][1] = f32x4{0.f, 0.f, 0.f, 0.f};
        const bf16_t* krow[2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
            krow[t] = page[t] >= 0 ? kcache + ((static_cast<int64_t>(page[t]) * a.nkv + kvh) * a.page_size + off[t] + r) * d
                                   : nullptr;
        for (int e0 = 0; e0 < d; e0 += 32) {
            const int e = e0 + 8 * g;
            const bool in = e < d;
            bf16x8 ka[2];
#pragma unroll
            for (int t = 0; t < 2; ++t) ka[t] = (in && krow[t]) ? *reinterpret_cast<const bf16x8*>(krow[t] + e) : zeros8();
#pragma unroll
            for (int rr = 0; rr < R; ++rr) {
                const bf16x8 qb = in ? *reinterpret_cast<const bf16x8*>(qrow[rr] + e) : zeros8();
#pragma unroll
                for (int t = 0; t < 2; ++t) s[rr][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[t], qb, s[rr][t], 0, 0, 0);
            }
        }
        // every row's scores of keys jbase[t] + 4 g + i become its weights, in the order the P^T operand wants them
        bf16x8 pb[R];
        float alpha[R];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            float v[2][4];
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int j = jbase[t] + 4 * g + i;
                    const bool seen = valid[rr] && page[t] >= 0 && j <= pos[rr] &&
                                      (a.window == 0 || pos[rr] - j < a.window || j < a.keep_first);
                    float x = s[rr][t][i] * a.scale;
                    if (a.cap > 0.f) x = a.cap * tanhf(x / a.cap);
                    v[t][i] = seen ? x : -INFINITY;
                    mx = fmaxf(mx, v[t][i]);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, PULSE_WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, PULSE_WAVE));
            const float m_new = fmaxf(m_run[rr], mx);
            alpha[rr] = (m_new == -INFINITY) ? 1.f : expf(m_run[rr] - m_new);
            float sum = 0.f;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float p = (v[t][i] == -INFINITY) ? 0.f : expf(v[t][i] - m_new);
                    sum += p;
                    pb[rr][4 * t + i] = static_cast<__bf16>(p);
                }
            l_run[rr] = l_run[rr] * alpha[rr] + sum;
            m_run[rr] = m_new;
        }
        // O^T += V^T P^T, channel tile by channel tile.  Keys of the operand that have never been stored are cleared:
        // one mask a 32-bit half of the lane's eight values, the same for every tile.
        unsigned int keep_bits[4];
        const bf16_t* vbase[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int j = jbase[t] + 4 * g;
            const bool there = page[t] >= 0;
            keep_bits[2 * t] = (there && j <= pos_last ? 0x0000FFFFu : 0u) | (there && j + 1 <= pos_last ? 0xFFFF0000u : 0u);
            keep_bits[2 * t + 1] = (there && j + 2 <= pos_last ? 0x0000FFFFu : 0u) | (there && j + 3 <= pos_last ? 0xFFFF0000u : 0u);
            // (value head c's channel e lies (c * d + e) * page_size behind kv head 0's: with all values side by side the
            // channel number is c * d + e itself)
            vbase[t] = vcache + static_cast<int64_t>(there ? page[t] : 0) * a.nkv * d * a.page_size + off[t] + 4 * g
                       + static_cast<int64_t>((a.all_values ? 0 : kvh * d) + chunk0 + r) * a.page_size;
        }
        const int tile_stride = 16 * a.page_size;
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            if (c < tiles) {
                u32x4 raw;
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const u32x2 two = *reinterpret_cast<const u32x2*>(vbase[t] + c * tile_stride);
                    raw[2 * t] = two[0] & keep_bits[2 * t];
                    raw[2 * t + 1] = two[1] & keep_bits[2 * t + 1];
                }
                const bf16x8 va = __builtin_bit_cast(bf16x8, raw);
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
                    acc[rr][c] *= alpha[rr];
                    acc[rr][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb[rr], acc[rr][c], 0, 0, 0);
                }
            }
        }
    }
    // row tile by row tile: a row's sum over the four lanes that share it; then the four wavefronts meet
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        float l = l_run[rr];
        l += __shfl_xor(l, 16, PULSE_WAVE);
        l += __shfl_xor(l, 32, PULSE_WAVE);
        __syncthreads();   // (the row tile before has been read)
        if (g == 0) { ml[wave][r][0] = m_run[rr]; ml[wave][r][1] = l; }
        __syncthreads();
        float m_all = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) m_all = fmaxf(m_all, ml[w][r][0]);
        float l_all = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) l_all += (ml[w][r][0] == -INFINITY) ? 0.f : ml[w][r][1] * expf(ml[w][r][0] - m_all);
        const float mine = (m_run[rr] == -INFINITY) ? 0.f : expf(m_run[rr] - m_all);
        // the wavefronts' sums meet in two rounds (2 and 3 into 0 and 1, then 1 into 0): half the LDS of one round
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            if (c < tiles) {
                acc[rr][c] *= mine;
                if (wave >= 2) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) red[wave - 2][c][lane][i] = acc[rr][c][i];
                }
            }
        }
        __syncthreads();
        if (wave < 2) {
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                if (c < tiles) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[rr][c][i] += red[wave][c][lane][i];
                }
            }
        }
        __syncthreads();
        if (wave == 1) {
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                if (c < tiles) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) red[0][c][lane][i] = acc[rr][c][i];
                }
            }
        }
        __syncthreads();
        if (wave == 0 && a.n_splits > 1) {
            // one of several workgroups over these keys: the sums as they are, for the merge
            if (valid[rr]) {
                const int64_t at = (static_cast<int64_t>(tok[rr]) * a.nq + head[rr]) * a.n_splits + blockIdx.z;
                if (blockIdx.y == 0 && g == 0) { a.part_ml[2 * at] = m_all; a.part_ml[2 * at + 1] = l_all; }
                float* prow = a.part + at * a.w + chunk0;
#pragma unroll
                for (int c = 0; c < CT; ++c) {
                    if (c < tiles) {
                        f32x4 sum = acc[rr][c];
#pragma unroll
                        for (int i = 0; i < 4; ++i) sum[i] += red[0][c][lane][i];
                        *reinterpret_cast<f32x4*>(prow + 16 * c + 4 * g) = sum;
                    }
                }
            }
        } else if (wave == 0) {
            // a sink is one more term of the softmax's denominator, exp(sink[h]), with no key and no value
            float scale_out = 1.f;
            if (sink) {
                const float sk = sink[head[rr]];
                if (m_all == -INFINITY) l_all = 1.f;
                else if (sk > m_all) { scale_out = expf(m_all - sk); l_all = l_all * scale_out + 1.f; }
                else l_all += expf(sk - m_all);
            }
            const float inv = l_all > 0.f ? scale_out / l_all : 0.f;
            if (valid[rr]) {
                float* orow = out + static_cast<int64_t>(tok[rr]) * a.o_stride + static_cast<int64_t>(head[rr]) * a.w + chunk0;
#pragma unroll
                for (int c = 0; c < CT; ++c) {
                    if (c < tiles) {
                        f32x4 sum = acc[rr][c];
#pragma unroll
                        for (int i = 0; i < 4; ++i) sum[i] += red[0][c][lane][i];
                        *reinterpret_cast<f32x4*>(orow + 16 * c + 4 * g) = sum * inv;
                    }
                }
            }
        }
    }
}

// The sums of the workgroups that shared a row's keys, brought together: a workgroup a (token, head).
__global__ void attn_wide_merge_kernel(const float* __restrict__ part, const float* __restrict__ part_ml,
                                       float* __restrict__ out, int64_t o_stride, const float* __restrict__ sink, int nq,
                                       int w, int wv, int n_splits) {
    const int tok = blockIdx.x, head = blockIdx.y;
    const int64_t at = (static_cast<int64_t>(tok) * nq + head) * n_splits;
    float m_all = -INFINITY;
    for (int s = 0; s < n_splits; ++s) m_all = fmaxf(m_all, part_ml[2 * (at + s)]);
    float l_all = 0.f;
    for (int s = 0; s < n_splits; ++s) {
        const float m = part_ml[2 * (at + s)];
        l_all += (m == -INFINITY) ? 0.f : part_ml[2 * (at + s) + 1] * expf(m - m_all);
    }
    float scale_out = 1.f;
    if (sink) {
        const float sk = sink[head];
        if (m_all == -INFINITY) l_all = 1.f;
        else if (sk > m_all) { scale_out = expf(m_all - sk); l_all = l_all * scale_out + 1.f; }
        else l_all += expf(sk - m_all);
    }
    const float inv = l_all > 0.f ? scale_out / l_all : 0.f;
    float* orow = out + static_cast<int64_t>(tok) * o_stride + static_cast<int64_t>(head) * w;
    for (int ch = threadIdx.x; ch < wv; ch += blockDim.x) {
        float sum = 0.f;
        for (int s = 0; s < n_splits; ++s) {
            const float m = part_ml[2 * (at + s)];
            if (m != -INFINITY) sum = fmaf(part[(at + s) * w + ch], expf(m - m_all), sum);
        }
        orow[ch] = sum * inv;
    }
}

}  // namespace

// q [tokens, q_stride] bfloat16: head h's query at h * d.  out float32 [tokens, o_stride]: head h's result at h * w,
// w = nkv * d with all_values (value head c at c * d) else d; channels 0 .. wv - 1 of it are written.  items int32
// [n_items, 4]: first token, tokens, first head, heads; row r (of 16 row_tiles, row_tiles 1 or 4) of an item is token
// r / hp, head r % hp; the items must cover every (token, head) of the `tokens` tokens.  n_splits > 1: the keys of
// every item are shared out over that many workgroups, whose sums (part float32 [tokens, nq, n_splits, w], part_ml
// [tokens, nq, n_splits, 2]) a second kernel brings together.  kcache
// [pages, nkv, page, d], vcache [pages, nkv, d, page] bfloat16, page_size a multiple of 16, d a multiple of 16.
extern "C" int pulse_attn_wide(const void* q, int64_t q_stride, float* out, int64_t o_stride, const void* kcache,
                               const void* vcache, const int* positions, const int* token_entry, const int* block_table,
                               int bt_width, const int* items, int n_items, int hp, int row_tiles, int nq, int nkv, int d, int wv,
                               int all_values, int page_size, int num_pages, float scale, int window, int keep_first,
                               const float* sink, float softcap, int n_splits, float* part, float* part_ml, int tokens,
                               hipStream_t stream) {
    PULSE_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0 && d > 0 && d % 16 == 0, "attn_wide: bad head sizes");
    PULSE_REQUIRE(page_size > 0 && page_size % 16 == 0 && num_pages > 0 && bt_width > 0, "attn_wide: pages must hold a multiple of 16 keys");
    const int w = all_values ? nkv * d : d;
    PULSE_REQUIRE(wv > 0 && wv % 16 == 0 && wv <= w, "attn_wide: %d of %d value channels", wv, w);
    PULSE_REQUIRE(hp >= 1 && hp <= 16 && n_items >= 0 && (row_tiles == 1 || row_tiles == 4), "attn_wide: bad items");
    PULSE_REQUIRE(window >= 0 && keep_first >= 0 && softcap >= 0.f, "attn_wide: bad window, kept keys or score cap");
    PULSE_REQUIRE(n_splits >= 1 && n_splits <= 64 && tokens >= 0 && (n_splits == 1 || (part && part_ml)),
                  "attn_wide: %d splits need their scratch", n_splits);
    PULSE_REQUIRE(q_stride >= static_cast<int64_t>(nq) * d && o_stride >= static_cast<int64_t>(nq) * w && o_stride % 4 == 0 &&
                  q_stride % 8 == 0, "attn_wide: row strides too small or unaligned");
    PULSE_REQUIRE(q && out && kcache && vcache && positions && token_entry && block_table && items, "attn_wide: null pointer");
    PULSE_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(kcache) % 16 == 0 && reinterpret_cast<uintptr_t>(vcache) % 16 == 0,
                  "attn_wide: operands must be 16-byte aligned");
    if (n_items == 0) return 0;
    WideArgs a;
    a.nq = nq; a.nkv = nkv; a.d = d; a.w = w; a.wv = wv; a.all_values = all_values ? 1 : 0; a.hp = hp;
    a.q_stride = q_stride; a.o_stride = o_stride; a.page_size = page_size; a.num_pages = num_pages; a.bt_width = bt_width;
    a.scale = scale; a.cap = softcap; a.window = window; a.keep_first = window > 0 ? keep_first : 0;
    a.n_splits = n_splits; a.part = part; a.part_ml = part_ml;
    if (row_tiles == 4) {
        const dim3 grid(n_items, (wv + 127) / 128, n_splits);
        hipLaunchKernelGGL((attn_wide_kernel<4, 8>), grid, dim3(256), 0, stream, static_cast<const bf16_t*>(q), out,
                           static_cast<const bf16_t*>(kcache), static_cast<const bf16_t*>(vcache), positions, token_entry,
                           block_table, items, sink, a);
    } else {
        const dim3 grid(n_items, (wv + 255) / 256, n_splits);
        hipLaunchKernelGGL((attn_wide_kernel<1, MAX_TILES>), grid, dim3(256), 0, stream, static_cast<const bf16_t*>(q), out,
                           static_cast<const bf16_t*>(kcache), static_cast<const bf16_t*>(vcache), positions, token_entry,
                           block_table, items, sink, a);
    }
    PULSE_LAUNCH_CHECK("attn_wide");
    if (n_splits > 1 && tokens > 0) {
        // (every (token, head) of the step has been written by the items: the work list covers them all)
        hipLaunchKernelGGL(attn_wide_merge_kernel, dim3(tokens, nq), dim3(256), 0, stream, part, part_ml, out, o_stride, sink,
                           nq, w, wv, n_splits);
        PULSE_LAUNCH_CHECK("attn_wide_merge");
    }
    return 0;
}
