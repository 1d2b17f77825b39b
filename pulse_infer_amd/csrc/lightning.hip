// Linear attention with a constant decay per head ("lightning attention").
//
// Every head keeps a state S [d, dv] in float32 for each request:
//     S_t = decay_h * S_(t-1) + k_t v_t^T          o_t = S_t^T q_t
// q, k [heads, d] and v [heads, dv] are columns of one projection output, with an
// activation (silu) applied as they are read.  The state of a request lives in its
// slot and is taken as zero when the request's portion starts at position 0.
//
// pulse_lightning_scan walks the tokens of an entry in order (a single decoded token
// is the walk of one), so a prompt cut into portions, or decoded token by token, goes
// through the same arithmetic in the same order.  A wavefront owns 64 / R columns of
// one head's state; a lane holds d / R rows of one column in registers, and the R
// partial sums of an output meet through lane exchanges.  R is chosen on the host so
// that the launch has enough wavefronts.  q, k and v of 16 tokens at a time go
// through LDS, the next 16 being fetched meanwhile.
//
// pulse_gated_rmsnorm finishes the mixer: the heads' outputs of a token, taken
// together, are divided by their root mean square, multiplied by a weight and by
// sigmoid(gate), and rounded once.
#include "common.h"

#include <math.h>

namespace {

struct ScanArgs {
    int heads, d, dv;
    int64_t x_stride, o_stride;
    int q0, k0, v0;   // first columns of q, k and v in a row of x
    int act;          // 0: none, 1: silu
    // A long portion can be walked in pieces by workgroups of their own (see pulse_lightning_scan):
    int mode;             // 0: an entry a workgroup, from its slot's state to its slot's state
                          // 1: a piece from a zero state, no outputs; what it leaves goes to scratch[piece]
                          // 2: a piece from scratch[piece - 1] (or, an entry's first, from the slot); outputs; an
                          //    entry's last piece leaves the state in the slot
    const int* pieces;    // modes 1, 2: [pieces][4] = first row, tokens, entry, 1 (entry's first) | 2 (entry's last)
    float* scratch;       // [pieces, heads, d, dv]
    // q and k may be turned by the tokens' positions as they are fetched (float32, before anything else is done with
    // them): the first `rot` channels of every head, pairs (i, i + rot / 2) with pairing 1 or (2i, 2i + 1) with 0, by
    // the tables cos_t / sin_t [T, rot / 2]; k is multiplied by k_scale after the turn
    const float* cos_t;
    const float* sin_t;
    int rot, pairing;
    float k_scale;
};

__device__ __forceinline__ float activate(float z, int act) { return act == 1 ? z / (1.0f + expf(-z)) : z; }

constexpr int SCAN_TOKENS = 16;
constexpr int SCAN_THREADS = 256;

// A value of every lane of a group of 4 (R = 4) or 16 (R = 16) neighbouring lanes summed over the group, left in all
// of them: exchanges inside a quad, then rotations of a row of 16 lanes (no LDS traffic).
template <int CTRL>
__device__ __forceinline__ float lane_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

template <int R>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (R >= 4) {
        v += lane_move<0xB1>(v);   // quad_perm [1, 0, 3, 2]
        v += lane_move<0x4E>(v);   // quad_perm [2, 3, 0, 1]
    }
    if constexpr (R >= 16) {
        v += lane_move<0x124>(v);  // row_ror 4
        v += lane_move<0x128>(v);  // row_ror 8
    }
    return v;
}

// A workgroup of four wavefronts owns 4 * 64 / R neighbouring columns of one head's state; lane l of a wavefront
// holds rows (l % R) + R j of column l / R.  q, k and v of the next 16 tokens are fetched into registers while the
// 16 in LDS are walked.
template <typename TX, int D, int R>
__global__ __launch_bounds__(SCAN_THREADS) void lightning_scan_kernel(const TX* __restrict__ x, float* __restrict__ out,
                                                                      float* __restrict__ state,
                                                                      const float* __restrict__ decay,
                                                                      const int* __restrict__ entry_first_row,
                                                                      const int* __restrict__ entry_start,
                                                                      const int* __restrict__ entry_slot, ScanArgs a) {
    constexpr int TB = SCAN_TOKENS;
    constexpr int CW = PULSE_WAVE / R;            // columns of the state a wavefront owns
    constexpr int WC = 4 * CW;                    // and a workgroup
    constexpr int DR = D / R;                     // rows a lane holds
    constexpr int EQ = TB * D / SCAN_THREADS;     // values of q (and of k) a thread fetches for 16 tokens
    constexpr int EV = TB * WC / SCAN_THREADS;    // and of v
    static_assert(EQ >= 1 && EV >= 1 && DR >= 4 && DR % 4 == 0, "sizes");
    constexpr int SEG = R > 1 ? DR + 4 : DR;      // a lane's rows in LDS, set apart so that the R lanes of a column
    constexpr int DP = R * SEG;                   // read from different banks
    __shared__ __attribute__((aligned(16))) float q_s[TB][DP];
    __shared__ __attribute__((aligned(16))) float k_s[TB][DP];
    __shared__ float v_s[TB][WC];
    const int h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid % PULSE_WAVE, wave = tid / PULSE_WAVE;
    const int rg = lane % R, cl = lane / R;
    const int c = blockIdx.z * WC + wave * CW + cl;
    const bool live = c < a.dv;
    int e = blockIdx.x, row0, n, flags = 3;
    if (a.mode == 0) {
        row0 = entry_first_row[e];
        n = entry_first_row[e + 1] - row0;
    } else {
        const int* piece = a.pieces + 4 * blockIdx.x;
        row0 = piece[0]; n = piece[1]; e = piece[2]; flags = piece[3];
        if (a.mode == 1 && (flags & 2)) return;   // what an entry's last piece leaves is formed by the walk with outputs
    }
    const int64_t head = static_cast<int64_t>(a.d) * a.dv, all = head * a.heads;
    float* S = state + static_cast<int64_t>(entry_slot[e]) * all + h * head;
    const float* from = entry_start[e] == 0 ? nullptr : S;
    float* to = S;
    if (a.mode == 1) {
        from = nullptr;
        to = a.scratch + blockIdx.x * all + h * head;
    } else if (a.mode == 2) {
        if (!(flags & 1)) from = a.scratch + (static_cast<int64_t>(blockIdx.x) - 1) * all + h * head;
        if (!(flags & 2)) to = nullptr;
    }
    const bool outputs = a.mode != 1;
    float s[DR];
#pragma unroll
    for (int j = 0; j < DR; ++j) {
        const int i = rg + R * j;
        s[j] = (from && live && i < a.d) ? from[static_cast<int64_t>(i) * a.dv + c] : 0.f;
    }
    const float lam = decay[h];
    float qr[EQ], kr[EQ], vr[EV];
    auto fetch = [&](int t0) __attribute__((always_inline)) {
        const int nb = min(TB, n - t0);
#pragma unroll
        for (int u = 0; u < EQ; ++u) {
            const int idx = u * SCAN_THREADS + tid;
            const int tt = idx / D, i = idx % D;
            qr[u] = kr[u] = 0.f;
            if (tt < nb && i < a.d) {
                const TX* row = x + static_cast<int64_t>(row0 + t0 + tt) * a.x_stride;
                const TX* qh = row + a.q0 + h * a.d;
                const TX* kh = row + a.k0 + h * a.d;
                float qv = outputs ? to_f32<TX>(qh[i]) : 0.f, kv = to_f32<TX>(kh[i]);
                if (i < a.rot) {
                    const int half = a.rot / 2;
                    int pair, freq;
                    bool first;
                    if (a.pairing == 1) { first = i < half; pair = first ? i + half : i - half; freq = first ? i : i - half; }
                    else { first = (i & 1) == 0; pair = i ^ 1; freq = i >> 1; }
                    const int64_t at = static_cast<int64_t>(row0 + t0 + tt) * half + freq;
                    const float c = a.cos_t[at], sn = a.sin_t[at];
                    const float ko = to_f32<TX>(kh[pair]);
                    kv = first ? kv * c - ko * sn : kv * c + ko * sn;
                    if (outputs) {
                        const float qo = to_f32<TX>(qh[pair]);
                        qv = first ? qv * c - qo * sn : qv * c + qo * sn;
                    }
                }
                qr[u] = qv;
                kr[u] = kv * a.k_scale;
            }
        }
#pragma unroll
        for (int u = 0; u < EV; ++u) {
            const int idx = u * SCAN_THREADS + tid;
            const int tt = idx / WC, cc = blockIdx.z * WC + idx % WC;
            vr[u] = 0.f;
            if (tt < nb && cc < a.dv)
                vr[u] = to_f32<TX>(x[static_cast<int64_t>(row0 + t0 + tt) * a.x_stride + a.v0 + h * a.dv + cc]);
        }
    };
    auto step = [&](int t0, int tt) __attribute__((always_inline)) {
        const float v = v_s[tt][wave * CW + cl];
        const float4* kp = reinterpret_cast<const float4*>(&k_s[tt][rg * SEG]);
        const float4* qp = reinterpret_cast<const float4*>(&q_s[tt][rg * SEG]);
        if (!outputs) {
#pragma unroll
            for (int j4 = 0; j4 < DR / 4; ++j4) {
                const float4 k4 = kp[j4];
                const float kk[4] = {k4.x, k4.y, k4.z, k4.w};
#pragma unroll
                for (int u = 0; u < 4; ++u) s[4 * j4 + u] = fmaf(lam, s[4 * j4 + u], kk[u] * v);
            }
            return;
        }
        float o = 0.f;
#pragma unroll
        for (int j4 = 0; j4 < DR / 4; ++j4) {
            const float4 k4 = kp[j4], q4 = qp[j4];
            const float kk[4] = {k4.x, k4.y, k4.z, k4.w}, qq[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                s[4 * j4 + u] = fmaf(lam, s[4 * j4 + u], kk[u] * v);
                o = fmaf(s[4 * j4 + u], qq[u], o);
            }
        }
        o = group_sum<R>(o);
        if (live && rg == 0) out[static_cast<int64_t>(row0 + t0 + tt) * a.o_stride + h * a.dv + c] = o;
    };
    if (n > 0) fetch(0);
    for (int t0 = 0; t0 < n; t0 += TB) {
        __syncthreads();   // the tokens in LDS have been walked
#pragma unroll
        for (int u = 0; u < EQ; ++u) {
            const int idx = u * SCAN_THREADS + tid;
            const int i = idx % D, at = (i % R) * SEG + i / R;   // a lane's rows lie side by side: it reads them 16 bytes at a time
            q_s[idx / D][at] = activate(qr[u], a.act);   // (a value beyond the tokens or the head is zero and stays zero)
            k_s[idx / D][at] = activate(kr[u], a.act);
        }
#pragma unroll
        for (int u = 0; u < EV; ++u) {
            const int idx = u * SCAN_THREADS + tid;
            v_s[idx / WC][idx % WC] = activate(vr[u], a.act);
        }
        __syncthreads();
        if (t0 + TB < n) fetch(t0 + TB);
        const int nb = min(TB, n - t0);
        if (nb == TB) {
#pragma unroll
            for (int tt = 0; tt < TB; ++tt) step(t0, tt);
        } else {
            for (int tt = 0; tt < nb; ++tt) step(t0, tt);
        }
    }
    if (live && to) {
#pragma unroll
        for (int j = 0; j < DR; ++j) {
            const int i = rg + R * j;
            if (i < a.d) to[static_cast<int64_t>(i) * a.dv + c] = s[j];
        }
    }
}

// Between the two walks of a portion in pieces: scratch[p] holds what piece p alone adds to a state; it becomes the
// state behind piece p, state_(p) = decay^tokens(p) * state_(p-1) + scratch[p], starting at an entry's first piece
// from the slot's state (zero for an entry that starts at position 0).  One thread a state element.
__global__ void lightning_combine_kernel(float* __restrict__ scratch, const float* __restrict__ state,
                                         const float* __restrict__ decay, const int* __restrict__ pieces, int n_pieces,
                                         const int* __restrict__ entry_start, const int* __restrict__ entry_slot,
                                         int64_t head, int64_t all) {
    const int64_t g = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (g >= all) return;
    const float lam = decay[g / head];
    float carry = 0.f;
    for (int p = 0; p < n_pieces; ++p) {
        const int* piece = pieces + 4 * p;
        const int flags = piece[3];
        if (flags & 1) carry = entry_start[piece[2]] == 0 ? 0.f : state[static_cast<int64_t>(entry_slot[piece[2]]) * all + g];
        if (flags & 2) continue;
        carry = fmaf(powf(lam, static_cast<float>(piece[1])), carry, scratch[p * all + g]);
        scratch[p * all + g] = carry;
    }
}

// ------------------------------------------------------- gated norm of heads
template <typename TX, typename TW>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ o, int64_t o_stride, const TW* __restrict__ w,
                                     const TX* __restrict__ gate, int64_t gate_stride, TX* __restrict__ y,
                                     int64_t y_stride, int n, float eps, float scale) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const float* row = o + static_cast<int64_t>(t) * o_stride;
    float ss = 0.f;
#pragma unroll 4
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss = fmaf(row[i], row[i], ss);
    const float total = block_sum(ss, scratch);
    const float inv = scale / sqrtf(total / static_cast<float>(n) + eps);
    const TX* g = gate ? gate + static_cast<int64_t>(t) * gate_stride : nullptr;
    TX* dst = y + static_cast<int64_t>(t) * y_stride;
#pragma unroll 4
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        float v = row[i] * inv * to_f32<TW>(w[i]);
        if (g) v *= 1.0f / (1.0f + expf(-to_f32<TX>(g[i])));
        dst[i] = from_f32<TX>(v);
    }
}

template <typename TX, int D, int R>
int launch_scan(const void* x, float* out, float* state, const float* decay, const int* first_row, const int* start,
                const int* slot, int entries, const ScanArgs& a, hipStream_t stream) {
    constexpr int WC = 4 * PULSE_WAVE / R;
    const dim3 grid(entries, a.heads, (a.dv + WC - 1) / WC);
    hipLaunchKernelGGL((lightning_scan_kernel<TX, D, R>), grid, dim3(SCAN_THREADS), 0, stream, static_cast<const TX*>(x), out, state,
                       decay, first_row, start, slot, a);
    return 0;
}

template <typename TX, int D>
int launch_scan_d(int r, const void* x, float* out, float* state, const float* decay, const int* first_row,
                  const int* start, const int* slot, int entries, const ScanArgs& a, hipStream_t stream) {
    if constexpr (D >= 64) {
        if (r >= 16) return launch_scan<TX, D, 16>(x, out, state, decay, first_row, start, slot, entries, a, stream);
    }
    if (r >= 4) return launch_scan<TX, D, 4>(x, out, state, decay, first_row, start, slot, entries, a, stream);
    return launch_scan<TX, D, 1>(x, out, state, decay, first_row, start, slot, entries, a, stream);
}

}  // namespace

// x [T, x_stride]: the projection output that holds q, k (heads x d each) and v (heads x dv) from columns q0, k0, v0;
// out [T, o_stride] float32 receives the heads' outputs (heads x dv); state [slots, heads, d, dv] float32;
// decay [heads] float32; the entries' first rows [entries + 1], start positions and slots are read on the device.
// row_groups: over how many lanes a column's rows are shared out (1, 4 or 16; 16 from 64 key channels a head on).
// mode 0: a workgroup walks an entry.  Modes 1 and 2 walk `n_pieces` pieces of entries (see ScanArgs): a long portion
// is walked twice, first every piece from a zero state (mode 1), then, after pulse_lightning_combine has turned what the
// pieces left into the states between them, every piece with its outputs (mode 2); all pieces run at the same time.
// cos_t / sin_t (float32 [T, rot / 2]; null: no turn), rot, pairing, k_scale: see ScanArgs.
extern "C" int pulse_lightning_scan_turned(const void* x, int x_dtype, int64_t x_stride, int q0, int k0, int v0, float* out,
                                           int64_t o_stride, float* state, int slots, const float* decay,
                                           const int* entry_first_row, const int* entry_start, const int* entry_slot,
                                           int entries, int heads, int d, int dv, int act, int row_groups, int mode,
                                           const int* pieces, int n_pieces, float* scratch, const float* cos_t,
                                           const float* sin_t, int rot, int pairing, float k_scale, hipStream_t stream) {
    PULSE_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= d && (rot == 0 || (cos_t && sin_t && act == 0)) &&
                  (pairing == 0 || pairing == 1), "lightning_scan: bad rotation (%d of %d channels)", rot, d);
    PULSE_REQUIRE(mode >= 0 && mode <= 2 && (mode == 0 || (pieces && scratch && n_pieces > 0)),
                  "lightning_scan: a walk in pieces needs its pieces and scratch");
    PULSE_REQUIRE(entries >= 0 && heads > 0 && d > 0 && dv > 0 && slots > 0, "lightning_scan: bad sizes");
    PULSE_REQUIRE(d <= 256, "lightning_scan: at most 256 key channels a head, got %d", d);
    PULSE_REQUIRE(heads < 65536 && dv < 65536 * 4, "lightning_scan: too many heads or value channels");
    PULSE_REQUIRE(pulse_dtype_ok(x_dtype) && (act == 0 || act == 1), "lightning_scan: bad dtype tag or activation");
    PULSE_REQUIRE(x && out && state && decay && entry_first_row && entry_start && entry_slot, "lightning_scan: null pointer");
    PULSE_REQUIRE(q0 >= 0 && k0 >= 0 && v0 >= 0 && x_stride >= static_cast<int64_t>(q0) + heads * d &&
                  x_stride >= static_cast<int64_t>(k0) + heads * d && x_stride >= static_cast<int64_t>(v0) + heads * dv &&
                  o_stride >= static_cast<int64_t>(heads) * dv, "lightning_scan: rows are too short for their columns");
    if (entries == 0) return 0;
    ScanArgs a;
    a.heads = heads; a.d = d; a.dv = dv; a.x_stride = x_stride; a.o_stride = o_stride;
    a.q0 = q0; a.k0 = k0; a.v0 = v0; a.act = act;
    a.mode = mode; a.pieces = pieces; a.scratch = scratch;
    a.cos_t = cos_t; a.sin_t = sin_t; a.rot = cos_t ? rot : 0; a.pairing = pairing; a.k_scale = k_scale;
    if (mode != 0) entries = n_pieces;   // workgroups along x
    int rc = 0;
#define PULSE_SCAN_CASE(DD)                                                                                            \
    PULSE_DISPATCH_DTYPE(x_dtype, TX, rc = launch_scan_d<TX, DD>(row_groups, x, out, state, decay, entry_first_row,     \
                                                                 entry_start, entry_slot, entries, a, stream))
    if (d <= 16) PULSE_SCAN_CASE(16);
    else if (d <= 32) PULSE_SCAN_CASE(32);
    else if (d <= 64) PULSE_SCAN_CASE(64);
    else if (d <= 128) PULSE_SCAN_CASE(128);
    else PULSE_SCAN_CASE(256);
#undef PULSE_SCAN_CASE
    if (rc) return rc;
    PULSE_LAUNCH_CHECK("lightning_scan");
    return 0;
}

extern "C" int pulse_lightning_scan(const void* x, int x_dtype, int64_t x_stride, int q0, int k0, int v0, float* out,
                                    int64_t o_stride, float* state, int slots, const float* decay,
                                    const int* entry_first_row, const int* entry_start, const int* entry_slot,
                                    int entries, int heads, int d, int dv, int act, int row_groups, int mode,
                                    const int* pieces, int n_pieces, float* scratch, hipStream_t stream) {
    return pulse_lightning_scan_turned(x, x_dtype, x_stride, q0, k0, v0, out, o_stride, state, slots, decay, entry_first_row,
                                       entry_start, entry_slot, entries, heads, d, dv, act, row_groups, mode, pieces,
                                       n_pieces, scratch, nullptr, nullptr, 0, 0, 1.0f, stream);
}

extern "C" int pulse_lightning_combine(float* scratch, const float* state, const float* decay, const int* pieces,
                                       int n_pieces, const int* entry_start, const int* entry_slot, int heads, int d,
                                       int dv, hipStream_t stream) {
    PULSE_REQUIRE(scratch && state && decay && pieces && entry_start && entry_slot && n_pieces > 0 && heads > 0 && d > 0 &&
                  dv > 0, "lightning_combine: bad arguments");
    const int64_t head = static_cast<int64_t>(d) * dv, all = head * heads;
    const int64_t blocks = (all + 255) / 256;
    PULSE_REQUIRE(blocks < (1ll << 31), "lightning_combine: the state is too large");
    hipLaunchKernelGGL(lightning_combine_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, scratch, state,
                       decay, pieces, n_pieces, entry_start, entry_slot, head, all);
    PULSE_LAUNCH_CHECK("lightning_combine");
    return 0;
}

// y[t, i] = scale * o[t, i] / sqrt(mean_i(o[t]^2) + eps) * w[i] * sigmoid(gate[t, i]), one rounding; gate may be null.
extern "C" int pulse_gated_rmsnorm(const float* o, int64_t o_stride, const void* w, int w_dtype, const void* gate,
                                   int64_t gate_stride, void* y, int64_t y_stride, int x_dtype, int tokens, int n,
                                   float eps, float scale, hipStream_t stream) {
    PULSE_REQUIRE(tokens >= 0 && n > 0 && o && w && y, "gated_rmsnorm: bad arguments");
    PULSE_REQUIRE(pulse_dtype_ok(w_dtype) && pulse_dtype_ok(x_dtype), "gated_rmsnorm: bad dtype tag");
    PULSE_REQUIRE(o_stride >= n && y_stride >= n && (!gate || gate_stride >= n), "gated_rmsnorm: rows are too short");
    if (tokens == 0) return 0;
    const int threads = n >= 1024 ? (tokens <= 64 ? 1024 : 256) : 128;
    PULSE_DISPATCH_DTYPE(x_dtype, TX, PULSE_DISPATCH_DTYPE(w_dtype, TW,
        hipLaunchKernelGGL((gated_rmsnorm_kernel<TX, TW>), dim3(tokens), dim3(threads), 0, stream, o, o_stride,
                           static_cast<const TW*>(w), static_cast<const TX*>(gate), gate_stride, static_cast<TX*>(y),
                           y_stride, n, eps, scale)));
    PULSE_LAUNCH_CHECK("gated_rmsnorm");
    return 0;
}
