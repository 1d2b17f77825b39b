// The experts of a routed feed-forward on the matrix cores (bfloat16): the (token, choice) pairs of a step are
// grouped by expert on the device, and every expert multiplies its own rows.
//
// pulse_moe_group (one workgroup): counts the pairs of every expert, gives each pair its place among its expert's
// (`order`: places -> pairs, the experts one after the other) and cuts every expert's pairs into tiles of TM rows:
// tile_expert, tile_row0 (first place), tile_rows, and their number.  Pairs that chose an identity expert
// (index >= experts) are in no tile.  Which place a pair gets among its expert's depends on the order in which the
// threads arrive; no result depends on it, since every row of a product is computed by itself.
//
// pulse_moe_gate_up_grouped: a workgroup of four wavefronts per (tile, 64 inner columns); a wavefront owns 16 gate
// rows and the 16 up rows beside them and walks the hidden size in steps of 32 with v_mfma_f32_16x16x32_bf16, the
// weight rows as the row operand, up to RB blocks of 16 gathered token rows as the column operand;
// act[pair, j] = silu(g) * u.
// pulse_moe_down_grouped: the same walk over the inner width with the down weights; y[pair, :] in float32.
// pulse_moe_combine: out[t] = sum over the token's choices, in their order, of weight * y[pair] (or weight * x[t]
// for an identity expert), float32.
// The launches are sized by the step's shape alone (the most tiles it can have); workgroups behind the number of
// tiles leave at once.
#include "common.h"

#include <math.h>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 zeros8() {
    bf16x8 z;
#pragma unroll
    for (int e = 0; e < 8; ++e) z[e] = (__bf16)0.0f;
    return z;
}

constexpr int GROUP_THREADS = 1024;
constexpr int MAX_EXPERTS = 1024;

__global__ __launch_bounds__(GROUP_THREADS) void moe_group_kernel(const int* __restrict__ idx, int pairs, int experts,
                                                                  int tile_rows_max, int max_tiles,
                                                                  int* __restrict__ rank, int* __restrict__ order,
                                                                  int* __restrict__ tile_expert,
                                                                  int* __restrict__ tile_row0,
                                                                  int* __restrict__ tile_rows,
                                                                  int* __restrict__ num_tiles) {
    __shared__ int count[MAX_EXPERTS];
    __shared__ int first[MAX_EXPERTS];
    const int tid = threadIdx.x;
    for (int e = tid; e < experts; e += GROUP_THREADS) count[e] = 0;
    __syncthreads();
    for (int a = tid; a < pairs; a += GROUP_THREADS) {
        const int e = idx[a];
        if (e >= 0 && e < experts) rank[a] = atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int at = 0, tiles = 0;
        for (int e = 0; e < experts; ++e) {
            first[e] = at;
            const int c = count[e];
            for (int m = 0; m < c && tiles < max_tiles; m += tile_rows_max) {
                tile_expert[tiles] = e;
                tile_row0[tiles] = at + m;
                tile_rows[tiles] = min(tile_rows_max, c - m);
                ++tiles;
            }
            at += c;
        }
        *num_tiles = tiles;
    }
    __syncthreads();
    for (int a = tid; a < pairs; a += GROUP_THREADS) {
        const int e = idx[a];
        if (e >= 0 && e < experts) order[first[e] + rank[a]] = a;
    }
}

// Tiles of 32 rows (decoding: few rows an expert) give few workgroups, each with a long walk: there the four
// wavefronts of a workgroup own the SAME 16 weight rows and a quarter of the k-steps each, and their sums meet in LDS in
// wavefront order (four times the workgroups, four times the loads in flight, the same result from run to run).
template <int NW, int RB>
__device__ __forceinline__ bool meet(f32x4 (&acc)[NW][RB], float* red, int wave, int lane) {
    // red: [4][NW * RB][64][4] floats
#pragma unroll
    for (int s = 0; s < NW; ++s)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[((wave * NW * RB + s * RB + rb) * 64 + lane) * 4 + i] = acc[s][rb][i];
    __syncthreads();
    if (wave != 0) return false;
#pragma unroll
    for (int w = 1; w < 4; ++w)
#pragma unroll
        for (int s = 0; s < NW; ++s)
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[s][rb][i] += red[((w * NW * RB + s * RB + rb) * 64 + lane) * 4 + i];
    return true;
}

// One tile of one expert against 64 weight rows: acc[rb] += W[16 rows of this wavefront] . X[16 rows of block rb]^T.
// wrow: this lane's weight row (null: beyond the weight), xrow[rb]: this lane's row of block rb (null: no such row).
template <int RB, int NW>
__device__ __forceinline__ void walk(const bf16_t* const (&wrow)[NW], const bf16_t* const (&xrow)[RB], int blocks, int K,
                                     int kg, f32x4 (&acc)[NW][RB], int share = 0, int shares = 1) {
    constexpr int U = 4;   // k-steps whose loads are asked for before the first of them is used
    // (`share` of `shares`: this wavefront takes every shares-th group of U k-steps, from group `share` on)
    for (int k0 = share * 32 * U; k0 < K; k0 += shares * 32 * U) {
        bf16x8 wa[U][NW], xb[U][RB];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kc = k0 + 32 * u + kg * 8;
            const bool kok = kc < K;   // K is a multiple of 8
#pragma unroll
            for (int s = 0; s < NW; ++s)
                wa[u][s] = (kok && wrow[s]) ? *reinterpret_cast<const bf16x8*>(wrow[s] + kc) : zeros8();
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
                xb[u][rb] = (kok && rb < blocks && xrow[rb]) ? *reinterpret_cast<const bf16x8*>(xrow[rb] + kc) : zeros8();
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                if (rb < blocks) {
#pragma unroll
                    for (int s = 0; s < NW; ++s)
                        acc[s][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[u][s], xb[u][rb], acc[s][rb], 0, 0, 0);
                }
            }
        }
    }
}

// The same walk for tiles of 128 rows (RB = 8): the tile's rows go through LDS in pieces of 64 values of k, fetched
// once by the workgroup's 256 threads (a thread half a row's piece: 64 bytes) instead of once by every wavefront, the
// next piece travelling while this one is multiplied.  src[t]: the row that thread t fetches half of (null: none).
constexpr int STAGE_K = 64;
constexpr int STAGE_ROW = STAGE_K + 8;   // values a row takes in LDS (the 8 more keep rows off each other's banks)

template <int NW>
__device__ __forceinline__ void walk_staged(const bf16_t* const (&wrow)[NW], const bf16_t* src, bf16_t* stage, int blocks,
                                            int K, int r, int kg, f32x4 (&acc)[NW][8]) {
    const int tid = threadIdx.x;
    const int frow = tid / 2, fk = (tid % 2) * 32;   // this thread fetches values fk .. fk + 31 of row frow's piece
    bf16x8 held[4];
    auto fetch = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int kc = k0 + fk + 8 * u;
            held[u] = (src && kc < K) ? *reinterpret_cast<const bf16x8*>(src + kc) : zeros8();
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += STAGE_K) {
        __syncthreads();   // the piece in LDS has been multiplied
#pragma unroll
        for (int u = 0; u < 4; ++u) *reinterpret_cast<bf16x8*>(stage + frow * STAGE_ROW + fk + 8 * u) = held[u];
        __syncthreads();
        if (k0 + STAGE_K < K) fetch(k0 + STAGE_K);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int kc = k0 + 32 * half + kg * 8;
            const bool kok = kc < K;
            bf16x8 wa[NW];
#pragma unroll
            for (int s = 0; s < NW; ++s)
                wa[s] = (kok && wrow[s]) ? *reinterpret_cast<const bf16x8*>(wrow[s] + kc) : zeros8();
#pragma unroll
            for (int rb = 0; rb < 8; ++rb) {
                if (rb < blocks) {
                    const bf16x8 xb = *reinterpret_cast<const bf16x8*>(stage + (rb * 16 + r) * STAGE_ROW + 32 * half + kg * 8);
#pragma unroll
                    for (int s = 0; s < NW; ++s)
                        acc[s][rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[s], xb, acc[s][rb], 0, 0, 0);
                }
            }
        }
    }
}

template <int RB>
__global__ __launch_bounds__(256) void moe_gate_up_grouped_kernel(const bf16_t* __restrict__ x,
                                                                  const bf16_t* __restrict__ wg,
                                                                  const bf16_t* __restrict__ wu,
                                                                  const int* __restrict__ order,
                                                                  const int* __restrict__ tile_expert,
                                                                  const int* __restrict__ tile_row0,
                                                                  const int* __restrict__ tile_rows,
                                                                  const int* __restrict__ num_tiles,
                                                                  bf16_t* __restrict__ act, int hidden, int ff, int top,
                                                                  const float* __restrict__ in_weight, int act_kind,
                                                                  float limit) {
    const int tile = blockIdx.x;
    if (tile >= *num_tiles) return;
    const int e = tile_expert[tile], row0 = tile_row0[tile], rows = tile_rows[tile];
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
    const int r = lane % 16, kg = lane / 16;
    constexpr bool SHARED_K = RB == 2;
    const int n0 = SHARED_K ? blockIdx.y * 16 : blockIdx.y * 64 + wave * 16;
    const int n = n0 + r;
    const bf16_t* wrow[2];
    wrow[0] = n < ff ? wg + (static_cast<int64_t>(e) * ff + n) * hidden : nullptr;
    wrow[1] = n < ff ? wu + (static_cast<int64_t>(e) * ff + n) * hidden : nullptr;
    const bf16_t* xrow[RB];
    int pair[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const int i = rb * 16 + r;
        pair[rb] = i < rows ? order[row0 + i] : -1;
        xrow[rb] = pair[rb] >= 0 ? x + static_cast<int64_t>(pair[rb] / top) * hidden : nullptr;
    }
    f32x4 acc[2][RB];
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[s][rb] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (RB == 8) {
        __shared__ __attribute__((aligned(16))) bf16_t stage[128 * STAGE_ROW];
        const int mine = threadIdx.x / 2;
        const int p = mine < rows ? order[row0 + mine] : -1;
        walk_staged<2>(wrow, p >= 0 ? x + static_cast<int64_t>(p / top) * hidden : nullptr, stage, (rows + 15) / 16, hidden,
                       r, kg, acc);
    } else {
        __shared__ float red[4 * 2 * RB * 64 * 4];
        walk<RB, 2>(wrow, xrow, (rows + 15) / 16, hidden, kg, acc, wave, 4);
        if (!meet<2, RB>(acc, red, wave, lane)) return;
    }
    // lane l holds inner columns 4 * (l / 16) + i of this wavefront's 16, for row l % 16 of every block
    const int j0 = n0 + 4 * kg;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        if (pair[rb] < 0) continue;
        bf16_t* dst = act + static_cast<int64_t>(pair[rb]) * ff;
        // an expert that is fed weight * x: both products are linear, so the factor goes onto their results
        const float wgt = in_weight ? in_weight[pair[rb]] : 1.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (j0 + i < ff) {
                float g = acc[0][rb][i] * wgt, u = acc[1][rb][i] * wgt;
                if (act_kind == 1) {   // clamped: min(g, limit) * sigmoid(1.702 g) * (clamp(u) + 1)
                    g = fminf(g, limit);
                    u = fminf(fmaxf(u, -limit), limit);
                    dst[j0 + i] = f32_to_bf16(g / (1.0f + expf(-1.702f * g)) * (u + 1.0f));
                } else {
                    dst[j0 + i] = f32_to_bf16(g / (1.0f + expf(-g)) * u);
                }
            }
        }
    }
}

template <int RB>
__global__ __launch_bounds__(256) void moe_down_grouped_kernel(const bf16_t* __restrict__ act,
                                                               const bf16_t* __restrict__ wd,
                                                               const int* __restrict__ order,
                                                               const int* __restrict__ tile_expert,
                                                               const int* __restrict__ tile_row0,
                                                               const int* __restrict__ tile_rows,
                                                               const int* __restrict__ num_tiles, float* __restrict__ y,
                                                               int hidden, int ff) {
    const int tile = blockIdx.x;
    if (tile >= *num_tiles) return;
    const int e = tile_expert[tile], row0 = tile_row0[tile], rows = tile_rows[tile];
    const int lane = threadIdx.x % PULSE_WAVE, wave = threadIdx.x / PULSE_WAVE;
    const int r = lane % 16, kg = lane / 16;
    constexpr bool SHARED_K = RB == 2;
    const int n0 = SHARED_K ? blockIdx.y * 16 : blockIdx.y * 64 + wave * 16;
    const int n = n0 + r;
    const bf16_t* wrow[1];
    wrow[0] = n < hidden ? wd + (static_cast<int64_t>(e) * hidden + n) * ff : nullptr;
    const bf16_t* xrow[RB];
    int pair[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const int i = rb * 16 + r;
        pair[rb] = i < rows ? order[row0 + i] : -1;
        xrow[rb] = pair[rb] >= 0 ? act + static_cast<int64_t>(pair[rb]) * ff : nullptr;
    }
    f32x4 acc[1][RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) acc[0][rb] = f32x4{0.f, 0.f, 0.f, 0.f};
    if constexpr (RB == 8) {
        __shared__ __attribute__((aligned(16))) bf16_t stage[128 * STAGE_ROW];
        const int mine = threadIdx.x / 2;
        const int p = mine < rows ? order[row0 + mine] : -1;
        walk_staged<1>(wrow, p >= 0 ? act + static_cast<int64_t>(p) * ff : nullptr, stage, (rows + 15) / 16, ff, r, kg, acc);
    } else {
        __shared__ float red[4 * 1 * RB * 64 * 4];
        walk<RB, 1>(wrow, xrow, (rows + 15) / 16, ff, kg, acc, wave, 4);
        if (!meet<1, RB>(acc, red, wave, lane)) return;
    }
    const int c0 = n0 + 4 * kg;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        if (pair[rb] < 0) continue;
        float* dst = y + static_cast<int64_t>(pair[rb]) * hidden;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (c0 + i < hidden) dst[c0 + i] = acc[0][rb][i];
    }
}

template <typename TX>
__global__ void moe_combine_kernel(const TX* __restrict__ x, const float* __restrict__ y, const int* __restrict__ idx,
                                   const float* __restrict__ weight, float* __restrict__ out, int64_t total, int hidden,
                                   int experts, int top) {
    const int64_t at = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (at >= total) return;
    const int64_t t = at / hidden;
    const int c = static_cast<int>(at % hidden);
    float acc = 0.f;
    for (int k = 0; k < top; ++k) {
        const int e = idx[t * top + k];
        const float w = weight ? weight[t * top + k] : 1.f;
        if (e >= experts) acc = fmaf(w, to_f32<TX>(x[at]), acc);
        else if (e >= 0) acc = fmaf(w, y[(t * top + k) * hidden + c], acc);
    }
    out[at] = acc;
}

}  // namespace

extern "C" int pulse_moe_group(const int* idx, int pairs, int experts, int tile_rows_max, int max_tiles, int* rank,
                               int* order, int* tile_expert, int* tile_row0, int* tile_rows, int* num_tiles,
                               hipStream_t stream) {
    PULSE_REQUIRE(pairs >= 0 && experts > 0 && experts <= MAX_EXPERTS, "moe_group: at most %d experts, got %d",
                  MAX_EXPERTS, experts);
    PULSE_REQUIRE(tile_rows_max > 0 && tile_rows_max % 16 == 0, "moe_group: tiles hold a multiple of 16 rows");
    PULSE_REQUIRE(max_tiles >= (pairs + tile_rows_max - 1) / tile_rows_max + experts,
                  "moe_group: %d tiles cannot hold %d pairs of %d experts in every case", max_tiles, pairs, experts);
    PULSE_REQUIRE(idx && rank && order && tile_expert && tile_row0 && tile_rows && num_tiles, "moe_group: null pointer");
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(GROUP_THREADS), 0, stream, idx, pairs, experts, tile_rows_max,
                       max_tiles, rank, order, tile_expert, tile_row0, tile_rows, num_tiles);
    PULSE_LAUNCH_CHECK("moe_group");
    return 0;
}

static bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

extern "C" int pulse_moe_gate_up_grouped(const void* x, const void* wg, const void* wu, const int* order,
                                         const int* tile_expert, const int* tile_row0, const int* tile_rows,
                                         const int* num_tiles, int max_tiles, int tile_rows_max, void* act, int hidden,
                                         int ff, int top, const float* in_weight, int act_kind, float limit,
                                         hipStream_t stream) {
    PULSE_REQUIRE(act_kind == 0 || act_kind == 1, "moe_gate_up_grouped: unknown activation %d", act_kind);
    PULSE_REQUIRE(hidden > 0 && ff > 0 && top > 0 && max_tiles > 0, "moe_gate_up_grouped: bad sizes");
    PULSE_REQUIRE(hidden % 8 == 0 && aligned16(x) && aligned16(wg) && aligned16(wu),
                  "moe_gate_up_grouped: rows must be multiples of 8 values and 16-byte aligned");
    PULSE_REQUIRE(tile_rows_max == 32 || tile_rows_max == 128, "moe_gate_up_grouped: tiles of 32 or 128 rows");
    PULSE_REQUIRE(x && wg && wu && order && tile_expert && tile_row0 && tile_rows && num_tiles && act,
                  "moe_gate_up_grouped: null pointer");
    PULSE_REQUIRE((ff + 15) / 16 < 65536, "moe_gate_up_grouped: an inner width of %d is too large", ff);
    const dim3 grid(max_tiles, (ff + 63) / 64);
    if (tile_rows_max == 32)
        hipLaunchKernelGGL(moe_gate_up_grouped_kernel<2>, dim3(max_tiles, (ff + 15) / 16), dim3(256), 0, stream, static_cast<const bf16_t*>(x),
                           static_cast<const bf16_t*>(wg), static_cast<const bf16_t*>(wu), order, tile_expert, tile_row0,
                           tile_rows, num_tiles, static_cast<bf16_t*>(act), hidden, ff, top, in_weight, act_kind, limit);
    else
        hipLaunchKernelGGL(moe_gate_up_grouped_kernel<8>, grid, dim3(256), 0, stream, static_cast<const bf16_t*>(x),
                           static_cast<const bf16_t*>(wg), static_cast<const bf16_t*>(wu), order, tile_expert, tile_row0,
                           tile_rows, num_tiles, static_cast<bf16_t*>(act), hidden, ff, top, in_weight, act_kind, limit);
    PULSE_LAUNCH_CHECK("moe_gate_up_grouped");
    return 0;
}

extern "C" int pulse_moe_down_grouped(const void* act, const void* wd, const int* order, const int* tile_expert,
                                      const int* tile_row0, const int* tile_rows, const int* num_tiles, int max_tiles,
                                      int tile_rows_max, float* y, int hidden, int ff, hipStream_t stream) {
    PULSE_REQUIRE(hidden > 0 && ff > 0 && max_tiles > 0, "moe_down_grouped: bad sizes");
    PULSE_REQUIRE(ff % 8 == 0 && aligned16(act) && aligned16(wd),
                  "moe_down_grouped: rows must be multiples of 8 values and 16-byte aligned");
    PULSE_REQUIRE(tile_rows_max == 32 || tile_rows_max == 128, "moe_down_grouped: tiles of 32 or 128 rows");
    PULSE_REQUIRE(act && wd && order && tile_expert && tile_row0 && tile_rows && num_tiles && y,
                  "moe_down_grouped: null pointer");
    PULSE_REQUIRE((hidden + 15) / 16 < 65536, "moe_down_grouped: a width of %d is too large", hidden);
    const dim3 grid(max_tiles, (hidden + 63) / 64);
    if (tile_rows_max == 32)
        hipLaunchKernelGGL(moe_down_grouped_kernel<2>, dim3(max_tiles, (hidden + 15) / 16), dim3(256), 0, stream, static_cast<const bf16_t*>(act),
                           static_cast<const bf16_t*>(wd), order, tile_expert, tile_row0, tile_rows, num_tiles, y, hidden, ff);
    else
        hipLaunchKernelGGL(moe_down_grouped_kernel<8>, grid, dim3(256), 0, stream, static_cast<const bf16_t*>(act),
                           static_cast<const bf16_t*>(wd), order, tile_expert, tile_row0, tile_rows, num_tiles, y, hidden, ff);
    PULSE_LAUNCH_CHECK("moe_down_grouped");
    return 0;
}

extern "C" int pulse_moe_combine(const void* x, int x_dtype, const float* y, const int* idx, const float* weight,
                                 float* out, int tokens, int hidden, int experts, int top, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && hidden > 0 && top > 0 && x && y && idx && out && pulse_dtype_ok(x_dtype),
                  "moe_combine: bad arguments");
    const int64_t total = static_cast<int64_t>(tokens) * hidden;
    if (total == 0) return 0;
    const int64_t blocks = (total + 255) / 256;
    PULSE_REQUIRE(blocks < (1ll << 31), "moe_combine: too many elements");
    PULSE_DISPATCH_DTYPE(x_dtype, TX,
        hipLaunchKernelGGL(moe_combine_kernel<TX>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                           static_cast<const TX*>(x), y, idx, weight, out, total, hidden, experts, top));
    PULSE_LAUNCH_CHECK("moe_combine");
    return 0;
}
