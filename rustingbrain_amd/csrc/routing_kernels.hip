// Router, dispatch and combine kernels of the mixture-of-experts forward pass
// for gfx950 (wave64).
//
//   logits_kernel   router logits in the reference's eight-lane `dot` order
//   router_kernel   softmax, log-sum-exp, deterministic top-k, per-block ranks
//                   and histogram, per-block partial sums for the auxiliary losses
//   dispatch_kernel prefix scan over blocks and experts, stable permutation
//                   (slot -> position), optional row gather; block 0 also writes
//                   the tile table of the grouped products and the two losses
//   combine_kernel  gate-weighted sum in ascending expert order, then the
//                   shared expert, then the optional residual
//
// Nothing here uses floating-point atomics: every sum has a fixed order, so two
// runs give the same bits.
#include <atomic>
#include <cstdlib>
#include <type_traits>

#include "rbmoe_kernels.h"

namespace rbmoe {


// Dynamic LDS layout of router_kernel (floats / ints, in this order):
//   prob   [TB][ES]   logits, then exp, then probabilities   (ES = E | 1)
//   lsev   [TB]       log-sum-exp per token
//   gates  [TB][k]    selected probabilities, then gates
//   lexp   [TB][k]    selected expert per local slot (-1 = unrouted)
//   wcount [waves][E] per-wave match counts of one ranking round
//   running[E]        slots already ranked per expert
__host__ __device__ static size_t router_fixed_bytes(int E, int k) {
    const int ES = E | 1;
    size_t n = (size_t)kRouterTokens * ES + kRouterTokens + 2 * (size_t)kRouterTokens * k + (size_t)kRouterWaves * E + E;
    return (n * 4 + 15) & ~(size_t)15;
}

size_t router_lds_bytes(int E, int k) {
    return router_fixed_bytes(E, k);
}

// ---------------------------------------------------------------------------
// logits_kernel: logits[t, e] = dot(x[t, :], w[e, :]) (+ bias[e]) in the order of the
// reference's eight-lane `dot` (src/matrix.rs:26-40): lanes[c % 8] += x[c] * w[c] in
// increasing c (a rounded multiply, then a rounded add), a scalar `rest` for the columns
// past the last multiple of 8, lanes folded left to right, rest added last.
//
// A workgroup owns 64 tokens x 8 experts: 8 waves, lane = token, one expert per wave, so a
// router row is wave-uniform and is fetched with scalar loads (it costs neither vector
// memory bandwidth nor LDS), 64 columns at a time so that their latency is paid once per
// batch.  The token rows are staged through LDS in slices of kLogitChunk columns (16-byte
// pieces, rows padded by one piece so that a wave's 64 row reads spread over all banks).
// ---------------------------------------------------------------------------
constexpr int kLogitTokens = 64;
constexpr int kLogitChunk = 256;
constexpr int kLogitBatch = 8;  // pieces (of 8 columns) per batch of scalar loads

template <typename XT>
struct XPiece;  // 8 consecutive elements of a token row
template <>
struct XPiece<bf16_t> {
    typedef uint4 raw_t;
    static __device__ __forceinline__ void widen(const raw_t& a, float (&v)[8]) {
        v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
        v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
        v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xffff0000u);
        v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xffff0000u);
    }
};
template <>
struct XPiece<float> {
    struct raw_t {
        float4 a, b;
    };
    static __device__ __forceinline__ void widen(const raw_t& r, float (&v)[8]) {
        v[0] = r.a.x; v[1] = r.a.y; v[2] = r.a.z; v[3] = r.a.w;
        v[4] = r.b.x; v[5] = r.b.y; v[6] = r.b.z; v[7] = r.b.w;
    }
};

// NE = experts (= waves) per workgroup.
// (bf16 without AHEAD: 6 waves per SIMD, i.e. three workgroups on a compute unit, is what the launches of many
// workgroups are tuned for - the bound keeps a later edit from quietly costing one of them)
// `rows16` (f32 rows only, or null): a bf16 copy of the rows, rounded to nearest even, for the expert products of a
// layer whose weights are bf16 or int8 - written on the way by the workgroups of the first group of experts, which
// have every piece of their rows in hand anyway (widths that are multiples of 8).
// WIDE (bf16 rows): the rows are widened to f32 once, on their way into LDS, instead of by each of the NE waves
// that read them (one of the three vector instructions per element); a slice is then half as many columns, so
// that a workgroup takes no more LDS and as many of them fit a compute unit.
template <typename XT, int NE, bool AHEAD, bool WIDE = false>
__global__ __launch_bounds__(NE * 64, (!AHEAD && sizeof(XT) == 2) ? 6 : 2) void logits_kernel(const XT* __restrict__ x,
                                                                const float* __restrict__ wr,
                                                                const float* __restrict__ bias, int T, int d, int E,
                                                                float* __restrict__ logits,
                                                                bf16_t* __restrict__ rows16) {
    static_assert(!WIDE || sizeof(XT) == 2, "only bf16 rows are widened");
    typedef typename XPiece<XT>::raw_t piece_t;
    typedef typename std::conditional<WIDE, float, XT>::type ST;  // the element type of the staged rows
    typedef typename XPiece<ST>::raw_t spiece_t;
    constexpr int kChunk = WIDE ? kLogitChunk / 2 : kLogitChunk;
    constexpr int PIECES = kChunk / 8;  // pieces per row per slice
    constexpr int ROWB = PIECES * (int)sizeof(spiece_t) + 16;  // bytes of a staged row: 16 of padding, so that the lanes' rows start in different banks
    __shared__ __align__(16) unsigned char xs_raw[kLogitTokens * ROWB];
    auto staged = [&](int r, int q) -> spiece_t* {
        return reinterpret_cast<spiece_t*>(xs_raw + (size_t)r * ROWB + (size_t)q * sizeof(spiece_t));
    };
    auto put = [&](int r, int q, const piece_t& v) {
        if constexpr (WIDE) {
            float f[8];
            XPiece<XT>::widen(v, f);
            spiece_t o;
            o.a = make_float4(f[0], f[1], f[2], f[3]);
            o.b = make_float4(f[4], f[5], f[6], f[7]);
            *staged(r, q) = o;
        } else {
            *staged(r, q) = v;
        }
    };
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t0 = blockIdx.x * kLogitTokens;
    const int nt = min(kLogitTokens, T - t0);
    constexpr int kLogitThreads = NE * 64;
    const int e = blockIdx.y * NE + wave;  // this wave's expert
    const bool has = e < E;
    const float* w0 = wr + (size_t)(has ? e : 0) * d;
    const int tail = d - d % 8;
    float la[8];
#pragma unroll
    for (int l = 0; l < 8; ++l) la[l] = 0.0f;
    const bool vec = d % 8 == 0;
    // A slice's pieces travel global -> registers -> LDS.  AHEAD: the loads of the next slice are issued
    // before the products of the current one, so their latency is covered by arithmetic - for launches of few
    // workgroups; with several workgroups on a compute unit they cover for each other, and the registers the
    // pieces in flight occupy would cost one of them.
    constexpr int MAXP = (kLogitTokens * PIECES + kLogitThreads - 1) / kLogitThreads;
    piece_t pre[MAXP];
    const bool copy16 = sizeof(XT) == 4 && rows16 != nullptr && blockIdx.y == 0;
    auto load_piece = [&](int r, int c) {  // eight elements of row r from column c (zeros past the last row)
        piece_t v = {};
        if (r < nt) {
            const XT* src = x + (size_t)(t0 + r) * d + c;
            if (vec) {
                v = *reinterpret_cast<const piece_t*>(src);
                if constexpr (sizeof(XT) == 4) {
                    if (copy16) {
                        float f[8];
                        XPiece<XT>::widen(v, f);
                        uint4 o;
                        o.x = f32_to_bf16_bits(f[0]) | ((uint32_t)f32_to_bf16_bits(f[1]) << 16);
                        o.y = f32_to_bf16_bits(f[2]) | ((uint32_t)f32_to_bf16_bits(f[3]) << 16);
                        o.z = f32_to_bf16_bits(f[4]) | ((uint32_t)f32_to_bf16_bits(f[5]) << 16);
                        o.w = f32_to_bf16_bits(f[6]) | ((uint32_t)f32_to_bf16_bits(f[7]) << 16);
                        *reinterpret_cast<uint4*>(rows16 + (size_t)(t0 + r) * d + c) = o;
                    }
                }
            } else {  // rows are not 16-byte aligned: gather the eight elements
                XT tmp[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) tmp[j] = src[j];
                v = *reinterpret_cast<const piece_t*>(tmp);
            }
        }
        return v;
    };
    auto fetch = [&](int c0) {
        const int np = min(PIECES, (tail - c0) / 8);
#pragma unroll
        for (int u = 0; u < MAXP; ++u) {
            const int idx = tid + u * kLogitThreads;  // over the full 64 x PIECES grid: no division by np
            const int r = idx / PIECES, q = idx % PIECES;
            pre[u] = (r < kLogitTokens && q < np) ? load_piece(r, c0 + 8 * q) : piece_t{};
        }
    };
    if (AHEAD && tail > 0) fetch(0);
    for (int c0 = 0; c0 < tail; c0 += kChunk) {
        const int np = min(PIECES, (tail - c0) / 8);  // pieces in this slice
        __syncthreads();
        if (AHEAD) {
#pragma unroll
            for (int u = 0; u < MAXP; ++u) {
                const int idx = tid + u * kLogitThreads;
                const int r = idx / PIECES, q = idx % PIECES;
                if (r < kLogitTokens && q < np) put(r, q, pre[u]);
            }
        } else {
            for (int idx = tid; idx < kLogitTokens * np; idx += kLogitThreads) {
                const int r = idx / np, q = idx - r * np;
                put(r, q, load_piece(r, c0 + 8 * q));
            }
        }
        __syncthreads();
        if (AHEAD && c0 + kChunk < tail) fetch(c0 + kChunk);
        if (has) {
            const float* wa = w0 + c0;
            int q = 0;
            for (; q + kLogitBatch <= np; q += kLogitBatch) {
                // one batch: 32 router weights into scalar registers, 4 token pieces from LDS
                float wv[8 * kLogitBatch];
#pragma unroll
                for (int j = 0; j < 8 * kLogitBatch; ++j) wv[j] = wa[8 * q + j];
                spiece_t xp[kLogitBatch];
#pragma unroll
                for (int b = 0; b < kLogitBatch; ++b) xp[b] = *staged(lane, q + b);
#pragma unroll
                for (int b = 0; b < kLogitBatch; ++b) {
                    float xv[8];
                    XPiece<ST>::widen(xp[b], xv);
#pragma unroll
                    for (int l = 0; l < 8; ++l) la[l] = __fadd_rn(la[l], __fmul_rn(xv[l], wv[8 * b + l]));
                }
            }
            for (; q < np; ++q) {
                float xv[8];
                XPiece<ST>::widen(*staged(lane, q), xv);
#pragma unroll
                for (int l = 0; l < 8; ++l) la[l] = __fadd_rn(la[l], __fmul_rn(xv[l], wa[8 * q + l]));
            }
        }
    }
    if (lane < nt && has) {
        const XT* xr = x + (size_t)(t0 + lane) * d;
        float rest = 0.0f;
        for (int c = tail; c < d; ++c) rest = __fadd_rn(rest, __fmul_rn(to_f32(xr[c]), w0[c]));
        float sum = 0.0f;
#pragma unroll
        for (int l = 0; l < 8; ++l) sum = __fadd_rn(sum, la[l]);
        float v = __fadd_rn(sum, rest);
        if (bias) v = __fadd_rn(v, bias[e]);
        logits[(size_t)(t0 + lane) * E + e] = v;
    }
}

// softmax, log-sum-exp and the k argmax rounds for the tokens of one wave of a router block (see router_tail).
// Everything order-sensitive keeps the reference's order: the maximum ignores NaN (f32::max), exp(v - max) is
// summed one expert after the other in index order, the k argmax rounds prefer the lower index on equal
// probabilities, and the gates are summed in rank order.
// The sum: lane l of a group ends with ((ex_0 + ex_1) + ... ) + ex_l after l steps of "take the lane below's sum,
// add your own value" (a shift of the whole wave by one lane inside the add; a group's first lane keeps the sum
// carried over from the experts of the slices before) - the reference's chain, one rounded add per expert, with
// no trip through LDS; lanes past the last expert add zeros.  An argmax round is two reductions of 32 bits: the
// greatest probability bits (probabilities are never negative, so the bits order like the values), then the
// lowest expert index among the lanes that hold them.
// NQ = turns a wave needs for its tokens (64 / G tokens a turn); the NQ turns share no data and run interleaved.
template <int MAXJ, int NQ>
__device__ __forceinline__ void softmax_topk(float* __restrict__ prob, float* __restrict__ lsev,
                                             float* __restrict__ gates, int* __restrict__ lexp, int G, int t0, int nt,
                                             int ES, const uint8_t* __restrict__ valid, int E, int k) {
    constexpr int TB = kRouterTokens;
    constexpr int TW = TB / kRouterWaves;  // tokens of a wave
    const int lane_ = threadIdx.x & 63, wave_ = threadIdx.x >> 6;
    const int lig = lane_ & (G - 1);          // lane in group
    const int gbase = lane_ & ~(G - 1);       // first lane of the group
    const int tpw = 64 / G;                   // tokens a wave handles in one turn
    const unsigned long long gmask = (G == 64 ? ~0ull : ((1ull << G) - 1ull)) << gbase;
    const float neg_inf = __uint_as_float(0xff800000u);
    int tok[NQ];
    bool live[NQ], ok[NQ];
    float* row[NQ];
    float pv[NQ][MAXJ], mx[NQ], sum[NQ], total[NQ];
    unsigned taken_bits[NQ];  // bit j: expert lig + G j is taken
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        tok[q] = wave_ * TW + q * tpw + lane_ / G;  // token of this group in turn q
        live[q] = tok[q] < nt && tok[q] < (wave_ + 1) * TW && q * tpw < TW;
        row[q] = prob + (live[q] ? tok[q] : 0) * ES;
        mx[q] = neg_inf;
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
            const int e = lig + G * j;
            pv[q][j] = (live[q] && e < E) ? row[q][e] : neg_inf;
            const float vv = (pv[q][j] == pv[q][j]) ? pv[q][j] : neg_inf;  // a NaN never becomes the maximum
            mx[q] = vv > mx[q] ? vv : mx[q];
        }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) mx[q] = group_fmax(mx[q], G);
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
            const int e = lig + G * j;
            // lanes without an expert carry +0 through the sums below
            pv[q][j] = (live[q] && e < E) ? rb_expf(__fadd_rn(pv[q][j], -mx[q])) : 0.0f;
        }
    }
    // the sums: one chain of adds per token in index order, slice after slice
    {
        float carry[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) carry[q] = 0.0f;
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
            if (G * j >= E) break;  // uniform
            float acc[NQ], seed[NQ];
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                seed[q] = __fadd_rn(carry[q], pv[q][j]);  // what a group's first lane holds: 0 + ex_0 = ex_0 in the first slice
                acc[q] = lig == 0 ? seed[q] : pv[q][j];
            }
            for (int st = 1; st < G; ++st) {
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    const float below = __uint_as_float(lanes_from<0x138>(__float_as_uint(acc[q])));  // wave_shr:1
                    const float next = __fadd_rn(below, pv[q][j]);
                    acc[q] = lig == 0 ? seed[q] : next;
                }
            }
#pragma unroll
            for (int q = 0; q < NQ; ++q) carry[q] = __shfl(acc[q], gbase + G - 1);
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q) sum[q] = carry[q];
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        if (live[q] && lig == 0) lsev[tok[q]] = __fadd_rn(mx[q], rb_logf(sum[q]));
#pragma unroll
        for (int j = 0; j < MAXJ; ++j) {
            const int e = lig + G * j;
            if (live[q] && e < E) {
                if (sum[q] > 0.0f) pv[q][j] = __fdiv_rn(pv[q][j], sum[q]);
                row[q][e] = pv[q][j];
            }
        }
        ok[q] = live[q] && ((valid == nullptr) || (valid[t0 + tok[q]] != 0));
        taken_bits[q] = 0;
        total[q] = 0.0f;
    }
    // ---- k rounds of argmax over the experts not yet taken ----
    for (int r = 0; r < k; ++r) {
        int first[NQ];
        uint32_t lbits[NQ], le[NQ];  // this lane's best candidate: probability bits and expert index
        bool has[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            // First expert not yet taken: the lowest set bit of a ballot over the group, taking
            // the expert slices j in increasing order (slice j holds experts G j .. G j + G - 1).
            first[q] = 0x7fffffff;
#pragma unroll
            for (int j = MAXJ - 1; j >= 0; --j) {
                const int e = lig + G * j;
                const unsigned long long m = __ballot(e < E && !((taken_bits[q] >> j) & 1u)) & gmask;
                if (m != 0ull) first[q] = (__ffsll((long long)m) - 1 - gbase) + G * j;
            }
            // best candidate of this lane: not taken, not NaN; greater probability, then lower index
            has[q] = false;
            lbits[q] = 0;
            le[q] = 0x7fffffffu;
#pragma unroll
            for (int j = 0; j < MAXJ; ++j) {
                const int e = lig + G * j;
                if (live[q] && e < E && !((taken_bits[q] >> j) & 1u) && pv[q][j] == pv[q][j]) {
                    const uint32_t bits = __float_as_uint(pv[q][j]);
                    if (!has[q] || bits > lbits[q]) {  // slices in increasing index order: a tie keeps the lower index
                        lbits[q] = bits;
                        le[q] = (uint32_t)e;
                    }
                    has[q] = true;
                }
            }
        }
        uint32_t mbits[NQ], ci[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) mbits[q] = group_umax(has[q] ? lbits[q] : 0u, G);
#pragma unroll
        for (int q = 0; q < NQ; ++q) ci[q] = group_umin((has[q] && lbits[q] == mbits[q]) ? le[q] : 0x7fffffffu, G);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            // the reference starts from the first untaken expert and replaces it only on a
            // strictly greater probability: if that first one is NaN nothing replaces it
            bool first_nan = false;
#pragma unroll
            for (int j = 0; j < MAXJ; ++j)
                if (lig + G * j == first[q] && pv[q][j] != pv[q][j]) first_nan = true;
            const bool nan_wins = (__ballot(first_nan) & gmask) != 0ull;
            const bool use_first = nan_wins || ci[q] == 0x7fffffffu;
            const int best = use_first ? first[q] : (int)ci[q];
            float mine = 0.0f;
#pragma unroll
            for (int j = 0; j < MAXJ; ++j)
                if (lig + G * j == best) {
                    mine = pv[q][j];
                    taken_bits[q] |= 1u << j;
                }
            // the winner's probability is the greatest bits themselves; only a NaN first expert has to be fetched
            float bestv = __uint_as_float(mbits[q]);
            if (__ballot(use_first) != 0ull) {  // uniform over the wave
                const float fv = __shfl(mine, gbase + (best & (G - 1)));
                if (use_first) bestv = fv;
            }
            total[q] = __fadd_rn(total[q], bestv);
            if (live[q] && lig == 0) {
                lexp[tok[q] * k + r] = ok[q] ? best : -1;
                gates[tok[q] * k + r] = ok[q] ? bestv : 0.0f;
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q = 0; q < NQ; ++q)
        if (ok[q] && total[q] > 0.0f)
            for (int r = lig; r < k; r += G) gates[tok[q] * k + r] = __fdiv_rn(gates[tok[q] * k + r], total[q]);
}

// router_tail: everything behind the logits for the 32 tokens of router block `blk` - softmax, log-sum-exp, top-k,
// gates, ranks, block histogram, partial sums of the losses.  LOADED = false: the logits are read from P;
// true: the caller has put them into the `prob` array of `lds_raw` (row pitch E | 1) and met at a barrier.
// MAXJ = experts a lane may own: 1 when E <= 64 (a lane owns one expert), kMaxExperts / 64 otherwise.
template <int MAXJ, bool LOADED>
__device__ __forceinline__ void router_tail(
    unsigned char* __restrict__ lds_raw, int blk, const uint8_t* __restrict__ valid, int T, int E, int k,
    float* __restrict__ P, float* __restrict__ lse, int* __restrict__ expert_of, float* __restrict__ gate_of,
    int* __restrict__ rank_in_block, int* __restrict__ blockcnt, float* __restrict__ partial) {
    constexpr int TB = kRouterTokens;
    const int ES = E | 1;
    float* prob = reinterpret_cast<float*>(lds_raw);
    float* lsev = prob + TB * ES;
    float* gates = lsev + TB;
    int* lexp = reinterpret_cast<int*>(gates + TB * k);
    int* wcount = lexp + TB * k;
    int* running = wcount + kRouterWaves * E;

    const int tid = threadIdx.x;
    const int t0 = blk * TB;
    const int nt = min(TB, T - t0);

    // ---- logits were written to P by logits_kernel ------------------------------
    if constexpr (!LOADED) {
        for (int idx = tid; idx < nt * E; idx += kRouterThreads) {
            const int i = idx / E;
            prob[i * ES + (idx - i * E)] = P[(size_t)t0 * E + idx];
        }
    }
    for (int idx = tid; idx < E; idx += kRouterThreads) running[idx] = 0;
    __syncthreads();

    // ---- softmax + top-k: G lanes per token, lane j of a group owns experts j, j + G, ... ----
    {
        int G = 1;
        while (G < E && G < 64) G <<= 1;
        // a wave's four tokens: all at once with up to 16 lanes per token, in two or four turns with 32 or 64 - the
        // turns are worked on side by side (one instruction stream), because each is a chain of dependent steps
        if (G == 64) softmax_topk<MAXJ, 4>(prob, lsev, gates, lexp, G, t0, nt, ES, valid, E, k);
        else if (G == 32) softmax_topk<MAXJ, 2>(prob, lsev, gates, lexp, G, t0, nt, ES, valid, E, k);
        else softmax_topk<MAXJ, 1>(prob, lsev, gates, lexp, G, t0, nt, ES, valid, E, k);
    }
    __syncthreads();

    // ---- write probabilities, lse, assignments (coalesced) ----------------
    for (int idx = tid; idx < nt * E; idx += kRouterThreads) {
        const int i = idx / E;
        const int e = idx - i * E;
        P[(size_t)t0 * E + idx] = prob[i * ES + e];
    }
    if (tid < nt) lse[t0 + tid] = lsev[tid];
    const int nls = nt * k;
    for (int ls = tid; ls < nls; ls += kRouterThreads) {
        expert_of[(size_t)t0 * k + ls] = lexp[ls];
        gate_of[(size_t)t0 * k + ls] = gates[ls];
    }

    // ---- partial sums for the auxiliary losses (fixed order): the waves behind the first, which ranks the slots
    // at the same time -----------------------------------------------------------
    const bool one_wave_ranks = nls <= 64;
    const int pfirst = one_wave_ranks ? 64 : 0;  // first thread that takes partial sums
    for (int e = tid - pfirst; e >= 0 && e <= E; e += kRouterThreads - pfirst) {
        float s = 0.0f;
        for (int i0 = 0; i0 < nt; i0 += 8) {
            float pvv[8];
            int okv[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i = min(i0 + u, nt - 1);
                okv[u] = lexp[i * k];
                pvv[u] = e < E ? prob[i * ES + e] : lsev[i] * lsev[i];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (i0 + u < nt && okv[u] >= 0) s += pvv[u];
        }
        partial[(size_t)blk * (E + 1) + e] = s;
    }

    // ---- rank of every local slot among earlier slots of the same expert --
    const int lane = tid & 63;
    const int wave = tid >> 6;
    int ebits = 0;
    while ((1 << ebits) < E) ++ebits;
    if (one_wave_ranks) {
        // every slot of the block in one wave: a slot's rank is the number of lower lanes with its expert, an
        // expert's count the size of its group - no barrier, no second pass
        if (wave == 0) {
            const int e = (lane < nls) ? lexp[lane] : -1;
            unsigned long long mask = __ballot(e >= 0);
            for (int b = 0; b < ebits; ++b) {
                const bool bit = (e >> b) & 1;
                const unsigned long long bb = __ballot(bit);
                mask &= bit ? bb : ~bb;
            }
            const int rank_w = __popcll(mask & ((1ull << lane) - 1ull));
            if (e >= 0) {
                rank_in_block[(size_t)t0 * k + lane] = rank_w;
                if (rank_w == 0) running[e] = __popcll(mask);  // zero so far (cleared at the top)
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's LDS writes have landed
            __builtin_amdgcn_wave_barrier();
            for (int idx = lane; idx < E; idx += 64) blockcnt[(size_t)blk * E + idx] = running[idx];
        }
        return;
    }
    const int rounds = (nls + kRouterThreads - 1) / kRouterThreads;
    for (int rd = 0; rd < rounds; ++rd) {
        for (int idx = tid; idx < kRouterWaves * E; idx += kRouterThreads) wcount[idx] = 0;
        __syncthreads();
        const int ls = rd * kRouterThreads + tid;
        const int e = (ls < nls) ? lexp[ls] : -1;
        unsigned long long mask = __ballot(e >= 0);
        for (int b = 0; b < ebits; ++b) {
            const bool bit = (e >> b) & 1;
            const unsigned long long bb = __ballot(bit);
            mask &= bit ? bb : ~bb;
        }
        const int rank_w = __popcll(mask & ((1ull << lane) - 1ull));
        if (e >= 0 && rank_w == 0) wcount[wave * E + e] = __popcll(mask);
        __syncthreads();
        if (e >= 0) {
            int pre = running[e];
            for (int w = 0; w < wave; ++w) pre += wcount[w * E + e];
            rank_in_block[(size_t)t0 * k + ls] = pre + rank_w;
        }
        __syncthreads();
        for (int idx = tid; idx < E; idx += kRouterThreads)
            for (int w = 0; w < kRouterWaves; ++w) running[idx] += wcount[w * E + idx];
        __syncthreads();
    }
    for (int idx = tid; idx < E; idx += kRouterThreads) blockcnt[(size_t)blk * E + idx] = running[idx];
}

// ---------------------------------------------------------------------------
// logits_q8_kernel: the logits of a quantized router, one thread per (token, expert).  The reference's order
// (dot_lanes::<32>, src/quantized.rs:154-177, taken on machines with AVX2, :179-196): lanes[c % 32] += x[c] * f32(q[c])
// over the whole chunks of 32 columns, a scalar rest over the tail, the lanes folded from 0.0 in lane order, plus the
// rest, times the row's scale (:61); every product and every sum rounded by itself.  Any width; not tuned (a
// quantized layer's router is a few hundred kilobytes and this kernel a few percent of its forward).
// ---------------------------------------------------------------------------
template <typename XT>
__global__ __launch_bounds__(256) void logits_q8_kernel(const XT* __restrict__ x, const int8_t* __restrict__ q,
                                                        const float* __restrict__ scale, const float* __restrict__ bias,
                                                        int T, int d, int E, float* __restrict__ P) {
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)T * E) return;
    const int t = (int)(idx / E), e = (int)(idx - (long long)t * E);
    const XT* const xr = x + (size_t)t * d;
    const int8_t* const qr = q + (size_t)e * d;
    float lanes[32];
#pragma unroll
    for (int l = 0; l < 32; ++l) lanes[l] = 0.0f;
    const int tail = d - d % 32;
    for (int c = 0; c < tail; c += 32) {
#pragma unroll
        for (int l = 0; l < 32; ++l)
            lanes[l] = __fadd_rn(lanes[l], __fmul_rn(to_f32(xr[c + l]), (float)qr[c + l]));
    }
    float rest = 0.0f;
    for (int c = tail; c < d; ++c) rest = __fadd_rn(rest, __fmul_rn(to_f32(xr[c]), (float)qr[c]));
    float sum = 0.0f;
#pragma unroll
    for (int l = 0; l < 32; ++l) sum = __fadd_rn(sum, lanes[l]);
    float v = __fmul_rn(__fadd_rn(sum, rest), scale[e]);
    if (bias) v = __fadd_rn(v, bias[e]);
    P[idx] = v;
}

// ---------------------------------------------------------------------------
// route_fused_kernel: the logits AND everything behind them for the 32 tokens of a router block, in one workgroup
// - one launch and one trip of the logits through memory less than logits_kernel + router_kernel.  A workgroup
// must then hold every expert of its tokens, and with 32 tokens a wave's 64 lanes are two experts side by side:
// lane = (token, half), wave w takes the experts 2 w + half (+ 16, + 32, ... for more than 16 experts).  The router
// rows are no longer uniform over a wave, so they are staged in LDS beside the token rows, a slice of columns at a
// time, and read from there (one address per half-wave: a broadcast).  The arithmetic is logits_kernel's, element by
// element: lanes[c % 8] += x[c] * w[c] in increasing c, a rounded multiply and a rounded add, the lanes folded left
// to right (widths that are multiples of 8: no tail).
// Dynamic LDS: the arrays of router_tail, then 32 token rows and E router rows of one slice.
// NI = experts per lane = ceil(E / 16).
// ---------------------------------------------------------------------------
__host__ __device__ static size_t fused_lds_bytes(int E, int k, int cols, size_t xsize) {
    return router_fixed_bytes(E, k) + (size_t)kRouterTokens * (cols * xsize + 16) + (size_t)E * (cols * 4 + 16);
}

// LDS reads of 16 bytes each that stay where they are written.
template <typename V>
__device__ __forceinline__ V lds_load_ahead(const unsigned char* p) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    static_assert(sizeof(V) % 16 == 0, "16-byte pieces");
    struct Raw {
        u32x4 v[sizeof(V) / 16];
    } raw;
#pragma unroll
    for (size_t i = 0; i < sizeof(V) / 16; ++i)
        raw.v[i] = *(const volatile __attribute__((address_space(3))) u32x4*)(const __attribute__((address_space(3))) void*)(p + 16 * i);
    return __builtin_bit_cast(V, raw);
}

// WIDE (bf16 rows): the token rows are widened to f32 once, on their way into LDS, instead of by each of the 16
// lanes that read an element (a shift or a mask per element and lane: a fifth of the kernel's vector
// instructions); the staged slice then takes twice the LDS, so the launcher asks for it only where that fits.
template <typename XT, int NI, bool WIDE>
__global__ __launch_bounds__(kRouterThreads) void route_fused_kernel(
    const XT* __restrict__ x, const float* __restrict__ wr, const float* __restrict__ bias,
    const uint8_t* __restrict__ valid, int T, int d, int E, int k, int cols, float* __restrict__ P,
    float* __restrict__ lse, int* __restrict__ expert_of, float* __restrict__ gate_of,
    int* __restrict__ rank_in_block, int* __restrict__ blockcnt, float* __restrict__ partial,
    bf16_t* __restrict__ rows16) {
    typedef typename XPiece<XT>::raw_t piece_t;
    typedef typename std::conditional<WIDE, float, XT>::type ST;  // the element type of the staged token rows
    typedef typename XPiece<ST>::raw_t spiece_t;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    constexpr int TB = kRouterTokens;
    const int ES = E | 1;
    float* const prob = reinterpret_cast<float*>(lds_raw);
    const int xpitch = cols * (int)sizeof(ST) + 16, wpitch = cols * 4 + 16;  // bytes; + 16: rows start in different banks
    unsigned char* const xs = lds_raw + router_fixed_bytes(E, k);
    unsigned char* const ws = xs + (size_t)TB * xpitch;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t = lane & 31, half = lane >> 5;
    const int blk = blockIdx.x;
    const int t0 = blk * TB;
    const int nt = min(TB, T - t0);

    float la[NI][8];
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int l = 0; l < 8; ++l) la[i][l] = 0.0f;

    // A slice travels global -> registers -> LDS; the loads of the next slice are issued before the products of the
    // current one, so that their latency is covered by arithmetic.  A thread moves up to MAXX pieces of token rows
    // (32 rows x 32 pieces at most) and MAXW 16-byte pieces of router rows (E rows x 64 at most) per slice.
    constexpr int MAXX = (kRouterTokens * 32 + kRouterThreads - 1) / kRouterThreads;
    constexpr int MAXW = (NI * 16 * 64 + kRouterThreads - 1) / kRouterThreads;
    piece_t pre_x[MAXX];
    float4 pre_w[MAXW];
    auto fetch = [&](int c0) {
        const int nc = min(cols, d - c0);
        const int np = nc / 8, nq = nc / 4;
#pragma unroll
        for (int u = 0; u < MAXX; ++u) {
            const int idx = tid + u * kRouterThreads;
            const int r = idx / np, q = idx - r * np;
            pre_x[u] = (idx < TB * np && r < nt) ? *reinterpret_cast<const piece_t*>(x + (size_t)(t0 + r) * d + c0 + 8 * q)
                                                 : piece_t{};
        }
#pragma unroll
        for (int u = 0; u < MAXW; ++u) {
            const int idx = tid + u * kRouterThreads;
            const int e = idx / nq, j = idx - e * nq;
            pre_w[u] = idx < E * nq ? *reinterpret_cast<const float4*>(wr + (size_t)e * d + c0 + 4 * j)
                                    : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
    };
    auto stage = [&](int c0) {
        const int nc = min(cols, d - c0);
        const int np = nc / 8, nq = nc / 4;
#pragma unroll
        for (int u = 0; u < MAXX; ++u) {
            const int idx = tid + u * kRouterThreads;
            if (idx < TB * np) {
                const int r = idx / np, q = idx - r * np;
                if constexpr (WIDE && sizeof(XT) == 2) {
                    float f[8];
                    XPiece<XT>::widen(pre_x[u], f);
                    float4* const to = reinterpret_cast<float4*>(xs + (size_t)r * xpitch + (size_t)q * sizeof(spiece_t));
                    to[0] = make_float4(f[0], f[1], f[2], f[3]);
                    to[1] = make_float4(f[4], f[5], f[6], f[7]);
                } else {
                    *reinterpret_cast<piece_t*>(xs + (size_t)r * xpitch + (size_t)q * sizeof(piece_t)) = pre_x[u];
                }
                if constexpr (sizeof(XT) == 4) {
                    if (rows16 != nullptr && r < nt) {  // the bf16 copy of f32 rows for the expert products (see logits_kernel)
                        float f[8];
                        XPiece<XT>::widen(pre_x[u], f);
                        uint4 o;
                        o.x = f32_to_bf16_bits(f[0]) | ((uint32_t)f32_to_bf16_bits(f[1]) << 16);
                        o.y = f32_to_bf16_bits(f[2]) | ((uint32_t)f32_to_bf16_bits(f[3]) << 16);
                        o.z = f32_to_bf16_bits(f[4]) | ((uint32_t)f32_to_bf16_bits(f[5]) << 16);
                        o.w = f32_to_bf16_bits(f[6]) | ((uint32_t)f32_to_bf16_bits(f[7]) << 16);
                        *reinterpret_cast<uint4*>(rows16 + (size_t)(t0 + r) * d + c0 + 8 * q) = o;
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < MAXW; ++u) {
            const int idx = tid + u * kRouterThreads;
            if (idx < E * nq) {
                const int e = idx / nq, j = idx - e * nq;
                *reinterpret_cast<float4*>(ws + (size_t)e * wpitch + 16 * j) = pre_w[u];
            }
        }
    };
    fetch(0);
    for (int c0 = 0; c0 < d; c0 += cols) {
        const int nc = min(cols, d - c0);
        const int np = nc / 8;  // pieces of 8 columns in this slice
        __syncthreads();        // the slice before has been consumed
        stage(c0);
        __syncthreads();
        if (c0 + cols < d) fetch(c0 + cols);
        // The LDS reads of piece q + 1 are issued before the arithmetic of piece q, so that their latency is covered
        // by it (two waves on a SIMD do not cover it by themselves).  An expert index past E is clamped: its sums
        // are computed and dropped, which keeps branches out of the loop.
        const unsigned char* const xrow = xs + (size_t)t * xpitch;
        const unsigned char* wrow[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i) wrow[i] = ws + (size_t)min(2 * wave + half + 16 * i, E - 1) * wpitch;
        struct Operands {
            spiece_t x;
            float4 wa[NI], wb[NI];
        };
        auto read = [&](Operands& o, int q) {
            o.x = lds_load_ahead<spiece_t>(xrow + (size_t)q * sizeof(spiece_t));
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                o.wa[i] = lds_load_ahead<float4>(wrow[i] + 32 * q);
                o.wb[i] = lds_load_ahead<float4>(wrow[i] + 32 * q + 16);
            }
            __builtin_amdgcn_sched_barrier(0);  // the reads stay in front of the arithmetic that follows
        };
        auto multiply = [&](const Operands& o) {
            float xv[8];
            XPiece<ST>::widen(o.x, xv);
#pragma unroll
            for (int i = 0; i < NI; ++i) {
                la[i][0] = __fadd_rn(la[i][0], __fmul_rn(xv[0], o.wa[i].x));
                la[i][1] = __fadd_rn(la[i][1], __fmul_rn(xv[1], o.wa[i].y));
                la[i][2] = __fadd_rn(la[i][2], __fmul_rn(xv[2], o.wa[i].z));
                la[i][3] = __fadd_rn(la[i][3], __fmul_rn(xv[3], o.wa[i].w));
                la[i][4] = __fadd_rn(la[i][4], __fmul_rn(xv[4], o.wb[i].x));
                la[i][5] = __fadd_rn(la[i][5], __fmul_rn(xv[5], o.wb[i].y));
                la[i][6] = __fadd_rn(la[i][6], __fmul_rn(xv[6], o.wb[i].z));
                la[i][7] = __fadd_rn(la[i][7], __fmul_rn(xv[7], o.wb[i].w));
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        // two sets of operand registers take turns, so that nothing is copied between the trips
        Operands oa, ob;
        read(oa, 0);
        for (int q = 0; q < np; q += 2) {
            read(ob, min(q + 1, np - 1));
            multiply(oa);
            read(oa, min(q + 2, np - 1));
            if (q + 1 < np) multiply(ob);
        }
    }
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int e = 2 * wave + half + 16 * i;
        if (e < E && t < nt) {
            float sum = 0.0f;
#pragma unroll
            for (int l = 0; l < 8; ++l) sum = __fadd_rn(sum, la[i][l]);
            float v = __fadd_rn(sum, 0.0f);  // the reference adds its (empty) scalar rest: sum + 0
            if (bias) v = __fadd_rn(v, bias[e]);
            prob[t * ES + e] = v;
        }
    }
    __syncthreads();
    router_tail<1, true>(lds_raw, blk, valid, T, E, k, P, lse, expert_of, gate_of, rank_in_block, blockcnt, partial);
}

template <typename XT, int MAXJ>
__global__ __launch_bounds__(kRouterThreads) void router_kernel(
    const XT* __restrict__ x, const float* __restrict__ wr, const float* __restrict__ bias,
    const uint8_t* __restrict__ valid, int T, int d, int E, int k, float* __restrict__ P,
    float* __restrict__ lse, int* __restrict__ expert_of, float* __restrict__ gate_of,
    int* __restrict__ rank_in_block, int* __restrict__ blockcnt, float* __restrict__ partial) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    router_tail<MAXJ, false>(lds_raw, blockIdx.x, valid, T, E, k, P, lse, expert_of, gate_of, rank_in_block, blockcnt,
                             partial);
}

// ---------------------------------------------------------------------------
// dispatch_kernel: block b owns the same 32 tokens as router block b.
//
// Prologue (every block, redundantly — the table is a few KB and sits in L2): column sums
// of the per-block histogram give counts[e], their exclusive prefix gives offsets[e], and
// the sums over the blocks before b give this block's base per expert.  Block 0 also
// writes counts / offsets, the tile table of the grouped products (tile i = rows
// [tile_row0[i], tile_row0[i] + tile_rows[i]) of expert tile_expert[i]; a tile never spans
// two experts) and the two auxiliary losses (reference src/moe.rs:602-639), folding the
// per-block partial sums in a fixed order.
//
// Position of a routed slot = offsets[e] + base[e] + rank_in_block[slot]: slots are numbered
// token-major, so this is exactly the order in which the reference appends slots to an
// expert's list (src/moe.rs:266-274).  The optional row copy is `gather_rows`
// (src/moe.rs:658-664); rows move as 16-byte pieces.
// ---------------------------------------------------------------------------
// dispatch_fused_kernel: for a modest number of router blocks the layout scan is folded into the
// dispatch launch: every block re-derives counts, offsets and its own base from all the block
// histograms (O(blocks^2 x experts) reads in total, but one launch less on the critical path);
// block 0 also writes counts, offsets and the tile table, the last block the losses.
size_t dispatch_fused_lds_bytes(int E, int k) {
    const int parts = 256 / E;
    return ((size_t)2 * parts * E + (size_t)parts * (E + 1) + 4 * (size_t)(E + 1) + (size_t)kRouterTokens * k) * 4;
}

template <typename XT>
__global__ __launch_bounds__(256) void dispatch_fused_kernel(
    const XT* __restrict__ x, const int* __restrict__ expert_of, const int* __restrict__ rank_in_block,
    const int* __restrict__ blockcnt, const float* __restrict__ partial, int T, int d, int E, int k,
    float w_aux, float w_z, int tile_m, int* __restrict__ counts, int* __restrict__ offsets,
    int* __restrict__ tile_expert, int* __restrict__ tile_row0, int* __restrict__ tile_rows,
    int* __restrict__ ntiles, float* __restrict__ losses, int* __restrict__ perm_slot,
    int* __restrict__ perm_token, int* __restrict__ inv_pos, XT* __restrict__ xg) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    constexpr int TB = kRouterTokens;
    const int parts = 256 / E;  // E <= 256
    int* part_all = reinterpret_cast<int*>(lds_raw);           // [parts][E]
    int* part_before = part_all + parts * E;                   // [parts][E]
    float* part_mass = reinterpret_cast<float*>(part_before + parts * E);  // [parts][E+1] (block 0)
    int* cnt = reinterpret_cast<int*>(part_mass + parts * (E + 1));        // [E+1]
    int* base = cnt + (E + 1);                                 // [E+1]
    int* off = base + (E + 1);                                 // [E+1]
    float* mass = reinterpret_cast<float*>(off + (E + 1));     // [E+1]
    int* lpos = reinterpret_cast<int*>(mass + (E + 1));        // [TB * k]

    const int tid = threadIdx.x;
    const int blk = blockIdx.x;
    const int nb = (T + TB - 1) / TB;
    const int len = (nb + parts - 1) / parts;
    const int p = tid / E;
    const int e = tid - p * E;
    const bool active = p < parts;
    // Block 0 writes counts, offsets and the tile table; the two losses are the work of another block (the last
    // one), so that neither of the two is the launch's long pole.  That block fetches the partial sums in the same
    // batch of loads as the histograms.
    const bool loss_blk = blk == nb - 1;
    // this thread's first slot does not depend on the scan: fetch it before anything else
    const int t0 = blk * TB;
    const int nt = min(TB, T - t0);
    const int nls = nt * k;
    int ex_first = -1, rank_first = 0;
    if (tid < nls) {
        ex_first = expert_of[(size_t)t0 * k + tid];
        rank_first = rank_in_block[(size_t)t0 * k + tid];
    }
    if (active) {
        const int b0 = min(nb, p * len), b1 = min(nb, b0 + len);
        // Loads in batches of 16 that do not depend on one another: one round trip to L2 per
        // batch instead of one per block.
        int s_all = 0, s_before = 0;
        float m = 0.0f, zs = 0.0f;
        for (int b = b0; b < b1; b += 16) {
            int c[16];
            float v[16], z[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) c[u] = b + u < b1 ? blockcnt[(size_t)(b + u) * E + e] : 0;
            if (loss_blk) {
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    v[u] = b + u < b1 ? partial[(size_t)(b + u) * (E + 1) + e] : 0.0f;
                    z[u] = (e == 0 && b + u < b1) ? partial[(size_t)(b + u) * (E + 1) + E] : 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                s_all += c[u];
                s_before += b + u < blk ? c[u] : 0;
            }
            if (loss_blk) {
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    if (b + u < b1) {
                        m += v[u];
                        zs += z[u];
                    }
                }
            }
        }
        part_all[p * E + e] = s_all;
        part_before[p * E + e] = s_before;
        if (loss_blk) {
            part_mass[p * (E + 1) + e] = m;
            if (e == 0) part_mass[p * (E + 1) + E] = zs;
        }
    }
    __syncthreads();
    if (tid < E) {
        int ca = 0, cb = 0;
        float m = 0.0f;
        for (int q = 0; q < parts; ++q) {
            ca += part_all[q * E + tid];
            cb += part_before[q * E + tid];
            if (loss_blk) m += part_mass[q * (E + 1) + tid];
        }
        cnt[tid] = ca;
        base[tid] = cb;
        mass[tid] = m;
    }
    // the sum of lse^2 over the parts: by the last thread of the workgroup, which exists for every expert count
    // (a thread numbered E does not when E is the workgroup size) and owns no expert column unless E is 256
    if (loss_blk && tid == 255) {
        float zs = 0.0f;
        for (int q = 0; q < parts; ++q) zs += part_mass[q * (E + 1) + E];
        mass[E] = zs;
    }
    __syncthreads();
    if (E <= 64) {  // exclusive prefix over the experts: one wave, log2(64) shuffle steps
        if (tid < 64) {
            const int c = tid < E ? cnt[tid] : 0;
            int incl = c;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(incl, o);
                if (tid >= o) incl += up;
            }
            if (tid < E) off[tid] = incl - c;
            if (tid == E - 1) off[E] = incl;
        }
    } else if (tid == 0) {
        int run = 0;
        for (int q = 0; q < E; ++q) {
            off[q] = run;
            run += cnt[q];
        }
        off[E] = run;
    }
    __syncthreads();
    if (blk == 0) {
        if (tid < E) {
            counts[tid] = cnt[tid];
            offsets[tid] = off[tid];
            // tiles of this expert start after the tiles of the experts before it
            int first = 0;
            for (int q = 0; q < tid; ++q) first += (cnt[q] + tile_m - 1) / tile_m;
            const int n = (cnt[tid] + tile_m - 1) / tile_m;
            for (int i = 0; i < n; ++i) {
                tile_expert[first + i] = tid;
                tile_row0[first + i] = off[tid] + i * tile_m;
                tile_rows[first + i] = min(tile_m, cnt[tid] - i * tile_m);
            }
            if (tid == E - 1) ntiles[0] = first + n;
        }
        if (tid == 0) offsets[E] = off[E];
    }
    if (loss_blk) {
        // every valid token routes exactly k slots, so the valid-token count is routed / k.  The experts' terms
        // (two divisions and a product each) side by side, then their sum in expert order by one thread.
        const int V = off[E] / k;
        const float tokens = (float)V;
        const float slots = (float)V * (float)k;
        float* const term = part_mass;  // [E]: the parts' sums are used up
        if (tid < E && V > 0) term[tid] = ((float)cnt[tid] / slots) * (mass[tid] / tokens);
        __syncthreads();
        if (tid == 0) {
            float aux = 0.0f, z = 0.0f;
            if (V > 0) {
                for (int q = 0; q < E; ++q) aux = aux + term[q];
                aux = aux * ((float)E * w_aux);
                z = w_z * mass[E] / tokens;
            }
            losses[0] = aux;
            losses[1] = z;
        }
    }

    for (int ls = tid; ls < nls; ls += 256) {
        const int s = t0 * k + ls;
        const int ex = ls == tid ? ex_first : expert_of[s];
        int pos = -1;
        if (ex >= 0) {
            pos = off[ex] + base[ex] + (ls == tid ? rank_first : rank_in_block[s]);
            perm_slot[pos] = s;
            perm_token[pos] = s / k;
        }
        inv_pos[s] = pos;
        lpos[ls] = pos;
    }
    __syncthreads();
    if (xg == nullptr) return;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    constexpr int VE = 16 / (int)sizeof(XT);  // elements per 16 bytes
    const bool vec = (d % VE == 0);
    for (int ls = wave; ls < nls; ls += 4) {
        const int pos = lpos[ls];
        if (pos < 0) continue;
        const XT* src = x + (size_t)(t0 + ls / k) * d;
        XT* dst = xg + (size_t)pos * d;
        if (vec) {
            const uint4* s4 = reinterpret_cast<const uint4*>(src);
            uint4* d4 = reinterpret_cast<uint4*>(dst);
            for (int c = lane; c < d / VE; c += 64) d4[c] = s4[c];
        } else {
            for (int c = lane; c < d; c += 64) dst[c] = src[c];
        }
    }
}


// layout_scan_kernel: one workgroup turns the per-block histograms into the global layout in
// O(blocks x experts): counts and offsets per expert, for every router block the number of
// slots of each expert routed by the blocks before it, the tile table of the grouped
// products, and the two auxiliary losses (src/moe.rs:602-639) from the per-block partial sums.
constexpr int kScanThreads = 1024;
// router blocks x experts up to which the scan is folded into the dispatch launch
constexpr long long kFusedScanLimit = 4096;

// the blocks are cut into at most 16 consecutive parts: their partial results are folded serially
__host__ __device__ static int scan_parts(int E) { return kScanThreads / E < 16 ? kScanThreads / E : 16; }

size_t scan_lds_bytes(int E) {
    const int parts = scan_parts(E);
    return ((size_t)parts * E + (size_t)parts * (E + 1) + 3 * (size_t)(E + 1)) * 4;
}

__global__ __launch_bounds__(kScanThreads) void layout_scan_kernel(
    const int* __restrict__ blockcnt, const float* __restrict__ partial, int nb, int E, int k, float w_aux,
    float w_z, int tile_m, int* __restrict__ blockbase, int* __restrict__ counts, int* __restrict__ offsets,
    int* __restrict__ tile_expert, int* __restrict__ tile_row0, int* __restrict__ tile_rows,
    int* __restrict__ ntiles, float* __restrict__ losses) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int parts = scan_parts(E);  // E <= 256: at least 4 parts
    int* part_sum = reinterpret_cast<int*>(lds_raw);                      // [parts][E]
    float* part_mass = reinterpret_cast<float*>(part_sum + parts * E);   // [parts][E+1]
    int* cnt = reinterpret_cast<int*>(part_mass + parts * (E + 1));      // [E+1]
    int* off = cnt + (E + 1);                                             // [E+1]
    float* mass = reinterpret_cast<float*>(off + (E + 1));               // [E+1]

    const int tid = threadIdx.x;
    const int len = (nb + parts - 1) / parts;
    const int p = tid / E;
    const int e = tid - p * E;
    const bool active = p < parts;
    const int b0 = min(nb, p * len), b1 = min(nb, b0 + len);
    // Loads come in batches of 8 that do not depend on one another: one round trip per batch.
    // The first kKeep histogram entries of a thread stay in registers for the second pass.
    constexpr int kKeep = 32;
    int keep[kKeep];
    if (active) {
        int sc = 0;
        float m = 0.0f, zs = 0.0f;
#pragma unroll
        for (int i = 0; i < kKeep; i += 8) {
            float v[8], z[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int bb = max(0, min(b0 + i + u, nb - 1));  // always a valid row: no branch around the loads
                keep[i + u] = blockcnt[(size_t)bb * E + e];
                v[u] = partial[(size_t)bb * (E + 1) + e];
                z[u] = partial[(size_t)bb * (E + 1) + E];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (b0 + i + u < b1) {
                    sc += keep[i + u];
                    m += v[u];
                    zs += z[u];
                }
            }
        }
        for (int b = b0 + kKeep; b < b1; b += 8) {
            int c[8];
            float v[8], z[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int bb = min(b + u, b1 - 1);
                c[u] = blockcnt[(size_t)bb * E + e];
                v[u] = partial[(size_t)bb * (E + 1) + e];
                z[u] = partial[(size_t)bb * (E + 1) + E];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (b + u < b1) {
                    sc += c[u];
                    m += v[u];
                    zs += z[u];
                }
            }
        }
        part_sum[p * E + e] = sc;
        part_mass[p * (E + 1) + e] = m;
        if (e == 0) part_mass[p * (E + 1) + E] = zs;
    }
    __syncthreads();
    if (tid < E) {  // exclusive prefix over the parts, per expert
        int run = 0;
        float m = 0.0f;
        for (int q = 0; q < parts; ++q) {
            const int c = part_sum[q * E + tid];
            part_sum[q * E + tid] = run;
            run += c;
            m += part_mass[q * (E + 1) + tid];
        }
        cnt[tid] = run;
        mass[tid] = m;
    }
    if (tid == E) {
        float zs = 0.0f;
        for (int q = 0; q < parts; ++q) zs += part_mass[q * (E + 1) + E];
        mass[E] = zs;
    }
    __syncthreads();
    if (E <= 64) {  // exclusive prefix over the experts: one wave, log2(64) shuffle steps
        if (tid < 64) {
            const int c = tid < E ? cnt[tid] : 0;
            int incl = c;
#pragma unroll
            for (int o = 1; o < 64; o <<= 1) {
                const int up = __shfl_up(incl, o);
                if (tid >= o) incl += up;
            }
            if (tid < E) off[tid] = incl - c;
            if (tid == E - 1) off[E] = incl;
        }
    } else if (tid == 0) {
        int run = 0;
        for (int q = 0; q < E; ++q) {
            off[q] = run;
            run += cnt[q];
        }
        off[E] = run;
    }
    __syncthreads();
    if (active) {  // slots of expert e routed by the blocks before block b
        int run = part_sum[p * E + e];
#pragma unroll
        for (int i = 0; i < kKeep; ++i) {
            if (b0 + i < b1) {
                blockbase[(size_t)(b0 + i) * E + e] = run;
                run += keep[i];
            }
        }
        for (int b = b0 + kKeep; b < b1; b += 8) {
            int c[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) c[u] = blockcnt[(size_t)min(b + u, b1 - 1) * E + e];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (b + u < b1) {
                    blockbase[(size_t)(b + u) * E + e] = run;
                    run += c[u];
                }
            }
        }
    }
    if (tid < E) {
        counts[tid] = cnt[tid];
        offsets[tid] = off[tid];
        // tiles of this expert start after the tiles of the experts before it
        int first = 0;
        for (int q = 0; q < tid; ++q) first += (cnt[q] + tile_m - 1) / tile_m;
        const int n = (cnt[tid] + tile_m - 1) / tile_m;
        for (int i = 0; i < n; ++i) {
            tile_expert[first + i] = tid;
            tile_row0[first + i] = off[tid] + i * tile_m;
            tile_rows[first + i] = min(tile_m, cnt[tid] - i * tile_m);
        }
        if (tid == E - 1) ntiles[0] = first + n;
    }
    // every valid token routes exactly k slots, so the valid-token count is routed / k.  The experts' terms (two
    // divisions and a product each) side by side, then their sum in expert order by one thread.
    const int V = off[E] / k;
    const float tokens = (float)V;
    const float slots = (float)V * (float)k;
    float* const term = part_mass;  // [E]: the parts' sums are used up
    if (tid < E && V > 0) term[tid] = ((float)cnt[tid] / slots) * (mass[tid] / tokens);
    __syncthreads();
    if (tid == 0) {
        offsets[E] = off[E];
        float aux = 0.0f, z = 0.0f;
        if (V > 0) {
            for (int q = 0; q < E; ++q) aux = aux + term[q];
            aux = aux * ((float)E * w_aux);
            z = w_z * mass[E] / tokens;
        }
        losses[0] = aux;
        losses[1] = z;
    }
}

// ---------------------------------------------------------------------------
// dispatch_kernel: block b owns the same 32 tokens as router block b:
// position = offsets[e] + blockbase[b][e] + rank in block.
// ---------------------------------------------------------------------------
size_t dispatch_lds_bytes(int E, int k) {
    return ((size_t)2 * (E + 1) + (size_t)kRouterTokens * k) * 4;
}

template <typename XT>
__global__ __launch_bounds__(256) void dispatch_kernel(
    const XT* __restrict__ x, const int* __restrict__ expert_of, const int* __restrict__ rank_in_block,
    const int* __restrict__ blockbase, const int* __restrict__ offsets, int T, int d, int E, int k,
    int* __restrict__ perm_slot, int* __restrict__ perm_token, int* __restrict__ inv_pos, XT* __restrict__ xg) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    constexpr int TB = kRouterTokens;
    int* base = reinterpret_cast<int*>(lds_raw);  // [E+1] slots of each expert routed by earlier blocks
    int* off = base + (E + 1);                    // [E+1] first row of each expert group
    int* lpos = off + (E + 1);                    // [TB * k]

    const int tid = threadIdx.x;
    const int blk = blockIdx.x;
    const int t0 = blk * TB;
    const int nt = min(TB, T - t0);
    const int nls = nt * k;
    // this thread's first slot and the block's two table rows are independent loads
    int ex_first = -1, rank_first = 0;
    if (tid < nls) {
        ex_first = expert_of[(size_t)t0 * k + tid];
        rank_first = rank_in_block[(size_t)t0 * k + tid];
    }
    for (int q = tid; q < E; q += 256) {
        base[q] = blockbase[(size_t)blk * E + q];
        off[q] = offsets[q];
    }
    __syncthreads();

    for (int ls = tid; ls < nls; ls += 256) {
        const int s = t0 * k + ls;
        const int ex = ls == tid ? ex_first : expert_of[s];
        int pos = -1;
        if (ex >= 0) {
            pos = off[ex] + base[ex] + (ls == tid ? rank_first : rank_in_block[s]);
            perm_slot[pos] = s;
            perm_token[pos] = s / k;
        }
        inv_pos[s] = pos;
        lpos[ls] = pos;
    }
    __syncthreads();
    if (xg == nullptr) return;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    constexpr int VE = 16 / (int)sizeof(XT);  // elements per 16 bytes
    const bool vec = (d % VE == 0);
    for (int ls = wave; ls < nls; ls += 4) {
        const int pos = lpos[ls];
        if (pos < 0) continue;
        const XT* src = x + (size_t)(t0 + ls / k) * d;
        XT* dst = xg + (size_t)pos * d;
        if (vec) {
            const uint4* s4 = reinterpret_cast<const uint4*>(src);
            uint4* d4 = reinterpret_cast<uint4*>(dst);
            for (int c = lane; c < d / VE; c += 64) d4[c] = s4[c];
        } else {
            for (int c = lane; c < d; c += 64) dst[c] = src[c];
        }
    }
}

// ---------------------------------------------------------------------------
// combine_kernel: out[t,:] = sum over the token's slots in ascending expert
// order of gate * y[pos,:] (a rounded multiply then a rounded add, as
// src/moe.rs:294-311), then + shared[t,:] (src/moe.rs:313-319), then
// + residual[t,:].  Ascending expert order is ascending position order.
// One thread per (token, 16-byte column piece); the token's slots are sorted
// by position in registers when k <= KMAX, otherwise found by repeated search.
// ---------------------------------------------------------------------------
// VN consecutive elements of an expert row, as raw bits and widened: the rows are of the layer's activation type, or
// bf16 under f32 activations (a layer whose bf16 / int8 expert products run on the matrix cores).
template <typename YT, typename XT>
struct RowPiece {  // rows of the activation type itself
    typedef uint4 raw_t;
    static __device__ __forceinline__ raw_t load_raw(const YT* p) { return Vec16<YT>::load_raw(p); }
    static __device__ __forceinline__ void widen(const raw_t& a, float (&v)[Vec16<YT>::N]) { Vec16<YT>::widen(a, v); }
};
template <>
struct RowPiece<bf16_t, float> {  // four bf16 elements beside four f32 ones
    typedef uint2 raw_t;
    static __device__ __forceinline__ raw_t load_raw(const bf16_t* p) { return *reinterpret_cast<const uint2*>(p); }
    static __device__ __forceinline__ void widen(const raw_t& a, float (&v)[4]) {
        v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
        v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
    }
};

template <typename XT, typename YT, int KMAX>
__global__ __launch_bounds__(256) void combine_vec_kernel(
    const YT* __restrict__ y, const YT* __restrict__ yshared, const XT* __restrict__ residual,
    const int* __restrict__ inv_pos, const float* __restrict__ gate_of, int T, int d, int k,
    XT* __restrict__ out) {
    constexpr int VN = Vec16<XT>::N;
    typedef RowPiece<YT, XT> YP;
    const int pieces = d / VN;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)T * pieces) return;
    const int t = (int)(idx / pieces);
    const int c = (int)(idx - (long long)t * pieces) * VN;
    // the token's routed slots, sorted by position (insertion sort on registers)
    int pos[KMAX];
    float gate[KMAX];
    int n = 0;
#pragma unroll
    for (int r = 0; r < KMAX; ++r) {
        pos[r] = 0x7fffffff;
        gate[r] = 0.0f;
    }
    // (all positions and gates are requested before the first is looked at, from addresses that do not depend on
    // one another - a slot past k repeats the last one: loads under a branch would follow one another, two trips to
    // memory a slot in front of the rows')
    int p_in[KMAX];
    float g_in[KMAX];
#pragma unroll
    for (int r = 0; r < KMAX; ++r) {
        const int rr = r < k ? r : k - 1;
        p_in[r] = inv_pos[(size_t)t * k + rr];
        g_in[r] = gate_of[(size_t)t * k + rr];
    }
#pragma unroll
    for (int r = 0; r < KMAX; ++r) {
        int p = p_in[r];
        float g = g_in[r];
        if (r < k && p >= 0) {
            ++n;
#pragma unroll
            for (int q = 0; q < KMAX; ++q) {
                if (p < pos[q]) {
                    const int tp = pos[q];
                    const float tg = gate[q];
                    pos[q] = p;
                    gate[q] = g;
                    p = tp;
                    g = tg;
                }
            }
        }
    }
    float acc[VN];
#pragma unroll
    for (int i = 0; i < VN; ++i) acc[i] = 0.0f;
    // every row piece is fetched before the first add (no branch around a load: an unused slot
    // re-reads row 0), so the k loads of a token are one round trip instead of k
    typename YP::raw_t raw[KMAX], raw_s = {};
    uint4 raw_r = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < KMAX; ++r) raw[r] = YP::load_raw(y + (size_t)(r < n ? pos[r] : 0) * d + c);
    if (yshared) raw_s = YP::load_raw(yshared + (size_t)t * d + c);    // uniform over the launch
    if (residual) raw_r = Vec16<XT>::load_raw(residual + (size_t)t * d + c);
#pragma unroll
    for (int r = 0; r < KMAX; ++r) {
        if (r < n) {
            float v[VN];
            YP::widen(raw[r], v);
#pragma unroll
            for (int i = 0; i < VN; ++i) acc[i] = __fadd_rn(acc[i], __fmul_rn(gate[r], v[i]));
        }
    }
    if (yshared) {
        float v[VN];
        YP::widen(raw_s, v);
#pragma unroll
        for (int i = 0; i < VN; ++i) acc[i] = __fadd_rn(acc[i], v[i]);
    }
    if (residual) {
        float v[VN];
        Vec16<XT>::widen(raw_r, v);
#pragma unroll
        for (int i = 0; i < VN; ++i) acc[i] = __fadd_rn(acc[i], v[i]);
    }
    Vec16<XT>::store(out + (size_t)t * d + c, acc);
}

// Any k, any d: one wave per token, one column per lane per step.
template <typename XT, typename YT>
__global__ __launch_bounds__(256) void combine_any_kernel(
    const YT* __restrict__ y, const YT* __restrict__ yshared, const XT* __restrict__ residual,
    const int* __restrict__ inv_pos, const float* __restrict__ gate_of, int T, int d, int k,
    XT* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const int* ip = inv_pos + (size_t)t * k;
    const float* gp = gate_of + (size_t)t * k;
    for (int c = lane; c < d; c += 64) {
        float acc = 0.0f;
        int last = -1;
        for (int r = 0; r < k; ++r) {
            int best = 0x7fffffff, bi = -1;  // next smallest position greater than `last`
            for (int q = 0; q < k; ++q) {
                const int p = ip[q];
                if (p > last && p < best) {
                    best = p;
                    bi = q;
                }
            }
            if (bi < 0) break;
            last = best;
            acc = __fadd_rn(acc, __fmul_rn(gp[bi], to_f32(y[(size_t)best * d + c])));
        }
        if (yshared) acc = __fadd_rn(acc, to_f32(yshared[(size_t)t * d + c]));
        if (residual) acc = __fadd_rn(acc, to_f32(residual[(size_t)t * d + c]));
        out[(size_t)t * d + c] = from_f32<XT>(acc);
    }
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
// Whether route_fused_kernel takes the call: every expert of a token in one workgroup (at most 64, four per lane),
// rows of whole 8-element pieces on 16-byte boundaries, and a slice of columns that fits LDS.
// Large launches take the two-launch sequence: logits_kernel fetches the router rows with scalar loads and keeps six
// waves on a SIMD, which per (token, expert) pair is the faster arithmetic once the launch fills the chip several
// times over (16 384 tokens x 64 experts: 126 us for both launches against 153 us fused); up to 256 K pairs the
// saved launch and the saved trip of the logits through memory weigh more (8192 x 16: 22 against 25 us).
static int fused_cols(const RouterArgs& a, size_t xsize) {
    if (!a.allow_fused || a.E > 64 || a.d % 8 != 0 || a.d < 8) return 0;
    if ((long long)a.T * a.E > 256 * 1024) return 0;
    if ((reinterpret_cast<uintptr_t>(a.x) & 15) || (reinterpret_cast<uintptr_t>(a.wr) & 15)) return 0;
    if (((size_t)a.d * xsize) % 16 != 0) return 0;
    const int cols = a.E <= 32 ? 256 : 128;
    return fused_lds_bytes(a.E, a.k, cols, xsize) <= 64 * 1024 ? cols : 0;
}

template <typename XT>
static hipError_t launch_router_t(const RouterArgs& a, hipStream_t s) {
    const int nb = (a.T + kRouterTokens - 1) / kRouterTokens;
    if (const int cols = a.wq ? 0 : fused_cols(a, sizeof(XT))) {
        // bf16 rows staged as f32 where a slice of the same width then still fits
        const bool wide = sizeof(XT) == 2 && fused_cols(a, 4) == cols;
        const size_t lds = fused_lds_bytes(a.E, a.k, cols, wide ? 4 : sizeof(XT));
        auto go = [&](auto ni, auto wide_tag) {
            RB_LAUNCH((route_fused_kernel<XT, decltype(ni)::value, decltype(wide_tag)::value>), dim3(nb),
                               dim3(kRouterThreads), lds, s,
                               static_cast<const XT*>(a.x), a.wr, a.bias, a.valid, a.T, a.d, a.E, a.k, cols, a.P, a.lse,
                               a.expert_of, a.gate_of, a.rank_in_block, a.blockcnt, a.partial,
                               static_cast<bf16_t*>(a.rows16));
        };
        auto pick = [&](auto wide_tag) {
            if (a.E <= 16) go(std::integral_constant<int, 1>{}, wide_tag);
            else if (a.E <= 32) go(std::integral_constant<int, 2>{}, wide_tag);
            else go(std::integral_constant<int, 4>{}, wide_tag);
        };
        if constexpr (sizeof(XT) == 2) {
            if (wide) pick(std::true_type{});
            else pick(std::false_type{});
        } else {
            pick(std::false_type{});
        }
        return hipGetLastError();
    }
    static std::atomic<unsigned long long> attr_set{0};
    {  // allow more than the default 64 KiB of dynamic LDS (gfx950 has 160 KiB per CU)
        const hipError_t e = once_per_device(attr_set, [] {
            hipError_t r = hipFuncSetAttribute(reinterpret_cast<const void*>(router_kernel<XT, 1>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kMaxRouterLds);
            if (r == hipSuccess)
                r = hipFuncSetAttribute(reinterpret_cast<const void*>(router_kernel<XT, kMaxExperts / 64>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, kMaxRouterLds);
            return r;
        });
        if (e != hipSuccess) return e;
    }
    // eight experts (waves) per workgroup share one staged slice of 64 token rows
    constexpr int NE = 8;
    const int tiles_t = (a.T + kLogitTokens - 1) / kLogitTokens;
    const dim3 lgrid(tiles_t, (a.E + NE - 1) / NE);
    if (a.wq) {
        if (a.rows16 || !a.wscale) return hipErrorInvalidValue;  // (the caller casts f32 rows itself on this path)
        const long long pairs = (long long)a.T * a.E;
        RB_LAUNCH(logits_q8_kernel<XT>, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, s,
                  static_cast<const XT*>(a.x), a.wq, a.wscale, a.bias, a.T, a.d, a.E, a.P);
    } else if ((long long)lgrid.x * lgrid.y <= 512)  // at most two workgroups on a compute unit
        RB_LAUNCH((logits_kernel<XT, NE, true>), lgrid, dim3(NE * 64), 0, s, static_cast<const XT*>(a.x),
                           a.wr, a.bias, a.T, a.d, a.E, a.P, static_cast<bf16_t*>(a.rows16));
    else
        RB_LAUNCH((logits_kernel<XT, NE, false, sizeof(XT) == 2>), lgrid, dim3(NE * 64), 0, s, static_cast<const XT*>(a.x),
                           a.wr, a.bias, a.T, a.d, a.E, a.P, static_cast<bf16_t*>(a.rows16));
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (a.E <= 64)
        RB_LAUNCH((router_kernel<XT, 1>), dim3(nb), dim3(kRouterThreads), router_lds_bytes(a.E, a.k), s,
                           static_cast<const XT*>(a.x), a.wr, a.bias, a.valid, a.T, a.d, a.E, a.k, a.P, a.lse,
                           a.expert_of, a.gate_of, a.rank_in_block, a.blockcnt, a.partial);
    else
        RB_LAUNCH((router_kernel<XT, kMaxExperts / 64>), dim3(nb), dim3(kRouterThreads),
                           router_lds_bytes(a.E, a.k), s, static_cast<const XT*>(a.x), a.wr, a.bias, a.valid, a.T, a.d,
                           a.E, a.k, a.P, a.lse, a.expert_of, a.gate_of, a.rank_in_block, a.blockcnt, a.partial);
    return hipGetLastError();
}

hipError_t launch_router(const RouterArgs& a, bool bf16, hipStream_t s) {
    if (a.T <= 0) return hipSuccess;
    if (a.rows16 && (bf16 || a.d % 8 != 0)) return hipErrorInvalidValue;  // the copy rides on the 8-element pieces
    return bf16 ? launch_router_t<bf16_t>(a, s) : launch_router_t<float>(a, s);
}

template <typename XT>
static hipError_t launch_dispatch_t(const DispatchArgs& a, hipStream_t s) {
    const int nb = (a.T + kRouterTokens - 1) / kRouterTokens;
    if ((long long)nb * a.E <= kFusedScanLimit) {
        RB_LAUNCH(dispatch_fused_kernel<XT>, dim3(nb > 0 ? nb : 1), dim3(256),
                           dispatch_fused_lds_bytes(a.E, a.k), s, static_cast<const XT*>(a.x), a.expert_of,
                           a.rank_in_block, a.blockcnt, a.partial, a.T, a.d, a.E, a.k, a.w_aux, a.w_z, a.tile_m,
                           a.counts, a.offsets, a.tile_expert, a.tile_row0, a.tile_rows, a.ntiles, a.losses,
                           a.perm_slot, a.perm_token, a.inv_pos, static_cast<XT*>(a.xg));
        return hipGetLastError();
    }
    static std::atomic<unsigned long long> attr_set{0};
    {
        const hipError_t e = once_per_device(attr_set, [] {
            return hipFuncSetAttribute(reinterpret_cast<const void*>(layout_scan_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
        });
        if (e != hipSuccess) return e;
    }
    // runs for T == 0 too: it then writes zero counts, an empty tile table and zero losses
    RB_LAUNCH(layout_scan_kernel, dim3(1), dim3(kScanThreads), scan_lds_bytes(a.E), s, a.blockcnt, a.partial,
                       nb, a.E, a.k, a.w_aux, a.w_z, a.tile_m, a.blockbase, a.counts, a.offsets, a.tile_expert,
                       a.tile_row0, a.tile_rows, a.ntiles, a.losses);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || nb == 0) return e;
    RB_LAUNCH(dispatch_kernel<XT>, dim3(nb), dim3(256), dispatch_lds_bytes(a.E, a.k), s,
                       static_cast<const XT*>(a.x), a.expert_of, a.rank_in_block, a.blockbase, a.offsets, a.T, a.d,
                       a.E, a.k, a.perm_slot, a.perm_token, a.inv_pos, static_cast<XT*>(a.xg));
    return hipGetLastError();
}

hipError_t launch_dispatch(const DispatchArgs& a, bool bf16, hipStream_t s) {
    return bf16 ? launch_dispatch_t<bf16_t>(a, s) : launch_dispatch_t<float>(a, s);
}

template <typename XT, typename YT>
static hipError_t launch_combine_t(const CombineArgs& a, hipStream_t s) {
    const YT* y = static_cast<const YT*>(a.y);
    const YT* ys = static_cast<const YT*>(a.yshared);
    const XT* res = static_cast<const XT*>(a.residual);
    XT* out = static_cast<XT*>(a.out);
    constexpr int VN = Vec16<XT>::N;
    if (a.d % VN == 0 && a.k <= 8) {
        const long long total = (long long)a.T * (a.d / VN);
        const dim3 grid((unsigned)((total + 255) / 256)), block(256);
        if (a.k <= 2)
            RB_LAUNCH((combine_vec_kernel<XT, YT, 2>), grid, block, 0, s, y, ys, res, a.inv_pos, a.gate_of, a.T, a.d, a.k, out);
        else if (a.k <= 4)
            RB_LAUNCH((combine_vec_kernel<XT, YT, 4>), grid, block, 0, s, y, ys, res, a.inv_pos, a.gate_of, a.T, a.d, a.k, out);
        else
            RB_LAUNCH((combine_vec_kernel<XT, YT, 8>), grid, block, 0, s, y, ys, res, a.inv_pos, a.gate_of, a.T, a.d, a.k, out);
    } else {
        RB_LAUNCH((combine_any_kernel<XT, YT>), dim3((a.T + 3) / 4), dim3(256), 0, s, y, ys, res, a.inv_pos,
                           a.gate_of, a.T, a.d, a.k, out);
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// RmsNorm::forward (src/norm.rs:41-61, inverse_rms :128-131) in front of the layer
// (feed_forward_norm, src/transformer_block.rs:216).  The sum of squares of a row is the
// reference's sequential f32 sum in index order, so the normed rows (and with them the routing)
// come out identical; the output is (value * inverse_rms) * weight, two separately rounded
// products as in the reference.
//
// The chain of d dependent additions per row is the floor of this kernel.  To keep memory
// latency off that chain, a block first copies its R rows into LDS with every lane's loads in
// flight at once (the rows of a block are one contiguous range), then lane r of the first wave
// walks row r in LDS (pitch padded by 16 bytes: lanes fall into different banks), then the whole
// block writes the normed rows from the LDS copy - the input is read from memory once.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float inverse_rms_of(float sum, int d, float eps) {
    const float mean_square = __fdiv_rn(sum, (float)d);
    // The root must be the correctly rounded one (the reference's f32::sqrt): taken in double and rounded once,
    // which is exact for a square root; the single-precision root instruction alone is not.
    const float root = (float)sqrt((double)__fadd_rn(mean_square, eps));
    return __fdiv_rn(1.0f, root);
}

template <typename XT>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const XT* __restrict__ x, const float* __restrict__ weight,
                                                           float eps, int T, int d, int R, int pitch,
                                                           XT* __restrict__ out) {
    constexpr int VN = Vec16<XT>::N;
    extern __shared__ __attribute__((aligned(16))) char smem[];  // R rows of `pitch` bytes, then R floats
    float* const inv = reinterpret_cast<float*>(smem + (size_t)R * pitch);
    const int tid = threadIdx.x;
    const int row0 = blockIdx.x * R;
    const int nrows = min(R, T - row0);
    const int pieces = d / VN;  // d is a multiple of VN (checked by the launcher)
    const XT* const src = x + (size_t)row0 * d;
    for (int idx = tid; idx < nrows * pieces; idx += 256) {
        const int r = idx / pieces, p = idx - r * pieces;
        *reinterpret_cast<uint4*>(smem + (size_t)r * pitch + p * 16) =
            *reinterpret_cast<const uint4*>(src + (size_t)idx * VN);
    }
    __syncthreads();
    if (tid < nrows) {
        const XT* const row = reinterpret_cast<const XT*>(smem + (size_t)tid * pitch);
        float sum = 0.0f;
#pragma unroll 4
        for (int c = 0; c < d; c += VN) {
            float v[VN];
            Vec16<XT>::load(row + c, v);
#pragma unroll
            for (int i = 0; i < VN; ++i) sum = __fadd_rn(sum, __fmul_rn(v[i], v[i]));
        }
        inv[tid] = inverse_rms_of(sum, d, eps);
    }
    __syncthreads();
    XT* const dst = out + (size_t)row0 * d;
    for (int idx = tid; idx < nrows * pieces; idx += 256) {
        const int r = idx / pieces, p = idx - r * pieces;
        float v[VN], o[VN];
        Vec16<XT>::load(reinterpret_cast<const XT*>(smem + (size_t)r * pitch + p * 16), v);
        const float s = inv[r];
        const float4* w = reinterpret_cast<const float4*>(weight + p * VN);
#pragma unroll
        for (int q = 0; q < VN / 4; ++q) {
            const float4 wv = w[q];
            o[4 * q + 0] = __fmul_rn(__fmul_rn(v[4 * q + 0], s), wv.x);
            o[4 * q + 1] = __fmul_rn(__fmul_rn(v[4 * q + 1], s), wv.y);
            o[4 * q + 2] = __fmul_rn(__fmul_rn(v[4 * q + 2], s), wv.z);
            o[4 * q + 3] = __fmul_rn(__fmul_rn(v[4 * q + 3], s), wv.w);
        }
        Vec16<XT>::store(dst + (size_t)idx * VN, o);
    }
}

// Any width, rows straight from memory: one thread per row for the sum, then the block walks its 64 rows.
template <typename XT>
__global__ __launch_bounds__(64) void rmsnorm_rows_direct_kernel(const XT* __restrict__ x,
                                                                 const float* __restrict__ weight, float eps, int T,
                                                                 int d, XT* __restrict__ out) {
    __shared__ float inv[64];
    const int lane = threadIdx.x;
    const int row0 = blockIdx.x * 64;
    const int my = min(row0 + lane, T - 1);  // rows past the end: a valid row, result unused
    const XT* xr = x + (size_t)my * d;
    float sum = 0.0f;
    for (int c = 0; c < d; ++c) {
        const float v = to_f32(xr[c]);
        sum = __fadd_rn(sum, __fmul_rn(v, v));
    }
    inv[lane] = inverse_rms_of(sum, d, eps);
    __syncthreads();
    const int nrows = min(64, T - row0);
    for (int idx = lane; idx < nrows * d; idx += 64) {
        const int r = idx / d, c = idx - r * d;
        const float v = to_f32(x[(size_t)(row0 + r) * d + c]);
        out[(size_t)(row0 + r) * d + c] = from_f32<XT>(__fmul_rn(__fmul_rn(v, inv[r]), weight[c]));
    }
}

template <typename XT>
hipError_t launch_rmsnorm_t(const XT* x, const float* weight, float eps, int T, int d, XT* out, hipStream_t s) {
    constexpr int VN = Vec16<XT>::N;
    const int pitch = d * (int)sizeof(XT) + 16;
    const bool pieces_ok = d % VN == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
                           (reinterpret_cast<uintptr_t>(out) & 15) == 0 && (reinterpret_cast<uintptr_t>(weight) & 15) == 0;
    if (pieces_ok && pitch + 4 <= 40 * 1024) {
        const int R = std::max(1, std::min(64, (32 * 1024) / pitch));
        const size_t lds = (size_t)R * pitch + (size_t)R * 4;
        RB_LAUNCH(rmsnorm_rows_kernel<XT>, dim3((T + R - 1) / R), dim3(256), lds, s, x, weight, eps, T, d, R,
                           pitch, out);
    } else {
        RB_LAUNCH(rmsnorm_rows_direct_kernel<XT>, dim3((T + 63) / 64), dim3(64), 0, s, x, weight, eps, T, d,
                           out);
    }
    return hipGetLastError();
}

hipError_t launch_rmsnorm(const void* x, const float* weight, float eps, int T, int d, void* out, bool bf16,
                          hipStream_t s) {
    if (T <= 0) return hipSuccess;
    return bf16 ? launch_rmsnorm_t(static_cast<const bf16_t*>(x), weight, eps, T, d, static_cast<bf16_t*>(out), s)
                : launch_rmsnorm_t(static_cast<const float*>(x), weight, eps, T, d, static_cast<float*>(out), s);
}

hipError_t launch_combine(const CombineArgs& a, bool bf16, hipStream_t s) {
    if (a.T <= 0) return hipSuccess;
    if (bf16) return launch_combine_t<bf16_t, bf16_t>(a, s);
    return a.rows_bf16 ? launch_combine_t<float, bf16_t>(a, s) : launch_combine_t<float, float>(a, s);
}

}  // namespace rbmoe
