// Decode-shaped forward (a few tokens): the layer is bound by streaming the touched experts'
// weights once from HBM and by launch latency.  The work is cut into four launches
//
//   route_small_kernel   one workgroup: logits, softmax, top-k, counting sort, tile table,
//                        auxiliary losses (MoeLayer::forward_train, src/moe.rs:243-341, up to
//                        the bucket loop; route src/moe.rs:553-593; losses src/moe.rs:325-337)
//   decode_gemm_kernel   gate/up + SwiGLU of every routed tile and of the shared expert
//   decode_gemm_kernel   down product of both
//   combine              (the same kernel as the large path)
//
// which the layer folds into fewer where the call allows it: the combine into the down launch (the last
// workgroup of a block of output columns to finish sums it), and - when most experts are about to be touched -
// the routing into the gate/up launch (decode_front_kernel), behind which the down launch has one row of
// workgroups per expert (decode_down_by_expert_kernel): two launches.  The products are spread over (tile,
// 32-feature block) workgroups whose waves split the reduction dimension, so that a few hundred kilobytes of
// weight fragments are in flight per CU and every byte of a touched expert is fetched exactly once per 32-row tile.
#include <type_traits>

#include "rbmoe_kernels.h"

namespace rbmoe {

// ---------------------------------------------------------------------------
// route_small_kernel.  Everything is written the way the reference walks it, one token or
// one expert per thread, because at this size the order of operations matters and the time
// does not: logits in the order of the eight-lane `dot` (src/matrix.rs:26-40) with the
// eight lanes of a pair on eight neighbouring threads, softmax_rows and route per token,
// the bucket loop per expert (a stable counting sort), losses per expert in token order.
// ---------------------------------------------------------------------------
constexpr int kSmallThreads = 512;
constexpr int kStageBytes = 96 * 1024;  // LDS for the staged router and token rows (gfx950: 160 KiB per workgroup)
// LDS of the routing code behind the staging area: prob, lsev, sexp, cnt, off, aux_term (see route_small_body)
constexpr int kRouteFixedBytes = (kSmallRouteMaxPairs + kSmallRouteMaxTokens + kSmallRouteMaxTokens * kMaxTopK +
                                  2 * (kMaxExperts + 1) + kMaxExperts) * 4 + 64;
// The launch that runs the routing beside the gate/up products (decode_front_kernel) keeps two workgroups on a
// compute unit: 80 KiB each, of which the routing workgroup stages rows in this much.
constexpr int kFrontLdsBytes = 80 * 1024;
constexpr int kFrontStageBytes = (kFrontLdsBytes - kRouteFixedBytes) / 16 * 16;

// softmax_rows (src/moe.rs, softmax over one row) and route (src/moe.rs:553-593) of one token, by one
// thread, the row used where it lies in LDS: the path for more experts than a wave has lanes.
__device__ __forceinline__ void token_phase_serial(float* row, int t, int E, int k, const uint8_t* valid, float* P,
                                                   float* lse, float* lsev, int* sexp, int* expert_of, float* gate_of) {
    const float neg_inf = __uint_as_float(0xff800000u);
    float mx = neg_inf;
    for (int e = 0; e < E; ++e)
        if (row[e] > mx) mx = row[e];  // a NaN never replaces the maximum
    float sum = 0.0f;
    for (int e = 0; e < E; ++e) {
        row[e] = rb_expf(__fadd_rn(row[e], -mx));
        sum = __fadd_rn(sum, row[e]);
    }
    const float l = __fadd_rn(mx, rb_logf(sum));
    lsev[t] = l;
    lse[t] = l;
    for (int e = 0; e < E; ++e) {
        if (sum > 0.0f) row[e] = __fdiv_rn(row[e], sum);
        P[(size_t)t * E + e] = row[e];
    }

    int* eo = sexp + t * k;
    const bool ok = (valid == nullptr) || (valid[t] != 0);
    if (!ok) {
        for (int r = 0; r < k; ++r) {
            eo[r] = -1;
            expert_of[t * k + r] = -1;
            gate_of[t * k + r] = 0.0f;
        }
        return;
    }
    float total = 0.0f;
    for (int r = 0; r < k; ++r) {
        int best = -1;
        float bestv = 0.0f;
        for (int e = 0; e < E; ++e) {
            bool taken = false;
            for (int q = 0; q < r; ++q) taken = taken || (eo[q] == e);
            if (taken) continue;
            const float v = row[e];
            if (best < 0 || v > bestv) {
                best = e;
                bestv = v;
            }
        }
        eo[r] = best;
        total = __fadd_rn(total, bestv);
        gate_of[t * k + r] = bestv;  // rewritten below once the sum is known
        expert_of[t * k + r] = best;
    }
    if (total > 0.0f)
        for (int r = 0; r < k; ++r) gate_of[t * k + r] = __fdiv_rn(row[eo[r]], total);
}

// The same two steps with G lanes per token (G = 16 or 64, E <= G), lane j holding expert j: the
// exponentials, divisions and the argmax of every round run side by side, and only what the reference
// does in sequence stays a sequence - the sum of the exponentials in index order (every lane of the group
// adds the E values up in the same order, fetching them with shuffles) and the running sum of the selected
// probabilities.  A round's winner is the largest 64-bit key (probability bits above the inverted index:
// probabilities are >= +0, so their bit patterns order like their values, and among equal ones the lower
// index wins, as the reference's strict `>` scan does); a taken expert's key is 0, and so is a NaN's, which the
// scan never prefers to anything and never replaces once it is the candidate.
// softmax_rows and route of one token by a group of G lanes (16 or 64), lane j owning expert j: the reductions
// run through lane-permuting operands and the ordered sum as a lane-shift chain (see softmax_topk in
// routing_kernels.hip for both), so the phase makes two trips to LDS instead of dozens.
template <int G>
__device__ __forceinline__ void token_phase_lanes(float* row_lds, int t, int j, int E, int k, const uint8_t* valid,
                                                  float* P, float* lse, float* lsev, int* sexp, int* expert_of,
                                                  float* gate_of) {
    const int lane = threadIdx.x & 63;
    const int base = lane - j;  // first lane of the group
    const bool mine = j < E;
    const float neg_inf = __uint_as_float(0xff800000u);
    const float v = mine ? row_lds[j] : neg_inf;
    const float mx = group_fmax((v == v) ? v : neg_inf, G);  // a NaN never replaces the maximum
    const float ex = mine ? rb_expf(__fadd_rn(v, -mx)) : 0.0f;   // lanes without an expert carry +0 through the sum
    // ((ex_0 + ex_1) + ex_2) + ...: lane l holds the sum through expert l after l steps
    float acc = ex;
    for (int st = 1; st < G; ++st) {
        const float below = __uint_as_float(lanes_from<0x138>(__float_as_uint(acc)));  // wave_shr:1
        const float next = __fadd_rn(below, ex);
        acc = j == 0 ? ex : next;
    }
    const float sum = __shfl(acc, base + G - 1);
    const float l = __fadd_rn(mx, rb_logf(sum));
    const float p = sum > 0.0f ? __fdiv_rn(ex, sum) : ex;
    if (mine) {
        P[(size_t)t * E + j] = p;
        row_lds[j] = p;  // the loss phase reads the probabilities from LDS
    }
    if (j == 0) {
        lsev[t] = l;
        lse[t] = l;
    }
    const bool ok = (valid == nullptr) || (valid[t] != 0);
    if (!ok) {
        if (j < k) {
            sexp[t * k + j] = -1;
            expert_of[t * k + j] = -1;
            gate_of[t * k + j] = 0.0f;
        }
        return;
    }
    // A NaN is never greater than anything and nothing is greater than a NaN (src/moe.rs:566-581): a NaN takes
    // part in no comparison - it is selected only when it is the first expert not yet taken, and then nothing
    // replaces it.
    const bool is_nan = p != p;
    bool taken = !mine;
    const unsigned long long gmask = G == 64 ? ~0ull : ((1ull << G) - 1ull);
    float total = 0.0f;
    float my_p = 0.0f;  // lane r keeps round r's probability
    int my_e = -1;
    for (int r = 0; r < k; ++r) {
        // greatest probability bits among the experts not yet taken (probabilities are never negative), then the
        // lowest index among the lanes that hold them
        const bool cand = !taken && !is_nan;
        const uint32_t mbits = group_umax(cand ? __float_as_uint(p) : 0u, G);
        const uint32_t ci = group_umin((cand && __float_as_uint(p) == mbits) ? (uint32_t)j : 0x7fffffffu, G);
        const unsigned long long untaken = (__ballot(!taken) >> base) & gmask;
        const unsigned long long nans = (__ballot(!taken && is_nan) >> base) & gmask;
        const int first = __ffsll((long long)untaken) - 1;  // k <= E: some expert is always left
        const bool first_nan = ((nans >> first) & 1ull) != 0ull;
        const bool use_first = first_nan || ci == 0x7fffffffu;
        const int be = use_first ? first : (int)ci;
        float bv = __uint_as_float(mbits);  // the winner's probability is the greatest bits themselves
        if (__ballot(use_first) != 0ull) {  // uniform over the wave: only a NaN first expert has to be fetched
            const float fv = __shfl(p, base + be);
            if (use_first) bv = fv;
        }
        total = __fadd_rn(total, bv);
        if (j == be) taken = true;
        if (j == r) {
            my_p = bv;
            my_e = be;
        }
    }
    if (j < k) {
        sexp[t * k + j] = my_e;
        expert_of[t * k + j] = my_e;
        gate_of[t * k + j] = total > 0.0f ? __fdiv_rn(my_p, total) : my_p;
    }
}

// STAGE = bytes of `smem` for the staged router and token rows; the routing arrays follow them.
template <typename XT, int STAGE>
__device__ __forceinline__ void route_small_body(
    unsigned char* __restrict__ smem,
    const XT* __restrict__ x, const float* __restrict__ wr, const float* __restrict__ bias,
    const uint8_t* __restrict__ valid, int T, int d, int E, int k, float w_aux, float w_z, int tile_m,
    float* __restrict__ P, float* __restrict__ lse, int* __restrict__ expert_of, float* __restrict__ gate_of,
    int* __restrict__ counts, int* __restrict__ offsets, int* __restrict__ tile_expert,
    int* __restrict__ tile_row0, int* __restrict__ tile_rows, int* __restrict__ ntiles,
    float* __restrict__ losses, int* __restrict__ perm_slot, int* __restrict__ perm_token,
    int* __restrict__ inv_pos, const float* __restrict__ norm_w, float norm_eps, XT* __restrict__ xn_out,
    bf16_t* __restrict__ rows16, unsigned int* __restrict__ expert_tokens = nullptr) {
    static_assert(STAGE % 16 == 0, "the arrays behind the staging area stay aligned");
    unsigned char* const stage = smem;
    float* const prob = reinterpret_cast<float*>(smem + STAGE);                 // [kSmallRouteMaxPairs]
    float* const lsev = prob + kSmallRouteMaxPairs;                             // [kSmallRouteMaxTokens]
    int* const sexp = reinterpret_cast<int*>(lsev + kSmallRouteMaxTokens);      // [kSmallRouteMaxTokens * kMaxTopK]
    int* const cnt = sexp + kSmallRouteMaxTokens * kMaxTopK;                    // [kMaxExperts + 1]
    int* const off = cnt + (kMaxExperts + 1);                                   // [kMaxExperts + 1]
    float* const aux_term = reinterpret_cast<float*>(off + (kMaxExperts + 1));  // [kMaxExperts]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int S = T * k;

    // ---- logits ---------------------------------------------------------------
    // When they fit, the router rows and the token rows are first copied to LDS with wide
    // coalesced loads (one round trip to memory instead of one per batch of columns); rows are
    // padded by 8 elements so that the eight pairs a wave works on fall into different banks.
    const int ds = d + 8;
    const bool staged = (d % 8 == 0) && ((size_t)E * ds * 4 + (size_t)T * ds * sizeof(XT) <= (size_t)STAGE) &&
                        (reinterpret_cast<uintptr_t>(x) % 16 == 0) && (reinterpret_cast<uintptr_t>(wr) % 16 == 0);
    if (staged) {
        float* ws = reinterpret_cast<float*>(stage);
        XT* xs = reinterpret_cast<XT*>(stage + (size_t)E * ds * 4);
        const int wp = d / 4, xp = d * (int)sizeof(XT) / 16;  // 16-byte pieces per row
        const int nw = E * wp, nx = T * xp;
        const uint4* wsrc = reinterpret_cast<const uint4*>(wr);
        const uint4* xsrc = reinterpret_cast<const uint4*>(x);
        // One load a piece from a chosen address (not a chosen one of two loads: loads under a branch stay in front
        // of their own stores, and the round trips follow one another), into variables of their own (an array of
        // pieces ends up in scratch memory).
        auto fetch = [&](int i) -> uint4 {
            i = min(i, nw + nx - 1);
            const uint4* const from = i < nw ? wsrc + i : xsrc + (i - nw);
            return *from;
        };
        auto put = [&](int i, const uint4& v) {
            if (i < nw) {
                const int r = i / wp, c = i - r * wp;
                *reinterpret_cast<uint4*>(ws + (size_t)r * ds + 4 * c) = v;
            } else if (i < nw + nx) {
                const int r = (i - nw) / xp, c = (i - nw) - r * xp;
                *reinterpret_cast<uint4*>(reinterpret_cast<char*>(xs + (size_t)r * ds) + 16 * c) = v;
            }
        };
        // eight pieces a thread are requested before the first is stored: 64 KB a round trip (36 KB for 8 tokens,
        // 8 experts and 768 columns: one)
        constexpr int NT = kSmallThreads;
        for (int i = tid; i < nw + nx; i += 8 * NT) {
            const uint4 v0 = fetch(i), v1 = fetch(i + NT), v2 = fetch(i + 2 * NT), v3 = fetch(i + 3 * NT);
            const uint4 v4 = fetch(i + 4 * NT), v5 = fetch(i + 5 * NT), v6 = fetch(i + 6 * NT), v7 = fetch(i + 7 * NT);
            __builtin_amdgcn_sched_barrier(0);
            put(i, v0); put(i + NT, v1); put(i + 2 * NT, v2); put(i + 3 * NT, v3);
            put(i + 4 * NT, v4); put(i + 5 * NT, v5); put(i + 6 * NT, v6); put(i + 7 * NT, v7);
        }
        __syncthreads();
        if (norm_w != nullptr) {
            // RmsNorm::forward (src/norm.rs:41-61) on the staged rows, in place: thread t adds up the squares
            // of row t in index order (the reference's sequential sum), then the block scales the rows with two
            // separately rounded products, rounds them to the activation type, and writes them out for the
            // kernels that follow.  (The launcher passes the norm only when the rows are staged.)
            float* const inv = lsev;  // free until the token phase
            constexpr int VN = Vec16<XT>::N;  // d is a multiple of 8 here, rows start on 16-byte boundaries
            if (tid < T) {
                const XT* row = xs + (size_t)tid * ds;
                float sum = 0.0f;
#pragma unroll 4
                for (int c = 0; c < d; c += VN) {
                    float v[VN];
                    Vec16<XT>::load(row + c, v);
#pragma unroll
                    for (int i = 0; i < VN; ++i) sum = __fadd_rn(sum, __fmul_rn(v[i], v[i]));
                }
                const float mean_square = __fdiv_rn(sum, (float)d);
                // correctly rounded root: in double, rounded once (the f32 root instruction is not)
                inv[tid] = __fdiv_rn(1.0f, (float)sqrt((double)__fadd_rn(mean_square, norm_eps)));
            }
            __syncthreads();
            const int pieces = d / VN;
            for (int i = tid; i < T * pieces; i += kSmallThreads) {
                const int t = i / pieces, c = (i - t * pieces) * VN;
                float v[VN], o[VN];
                Vec16<XT>::load(xs + (size_t)t * ds + c, v);
                const float sc = inv[t];
#pragma unroll
                for (int q = 0; q < VN; ++q) o[q] = __fmul_rn(__fmul_rn(v[q], sc), norm_w[c + q]);
                Vec16<XT>::store(xs + (size_t)t * ds + c, o);
                Vec16<XT>::store(xn_out + (size_t)t * d + c, o);
            }
            __syncthreads();
        }
        if constexpr (sizeof(XT) == 4) {
            // f32 rows of a layer whose expert products run on the bf16 matrix cores: their bf16 copy (nearest
            // even), from the staged - and, with a norm, normed - rows
            if (rows16 != nullptr) {
                for (int i = tid; i < T * (d / 8); i += kSmallThreads) {
                    const int t = i / (d / 8), c = (i - t * (d / 8)) * 8;
                    const float* src = reinterpret_cast<const float*>(xs) + (size_t)t * ds + c;
                    uint4 o;
                    o.x = f32_to_bf16_bits(src[0]) | ((uint32_t)f32_to_bf16_bits(src[1]) << 16);
                    o.y = f32_to_bf16_bits(src[2]) | ((uint32_t)f32_to_bf16_bits(src[3]) << 16);
                    o.z = f32_to_bf16_bits(src[4]) | ((uint32_t)f32_to_bf16_bits(src[5]) << 16);
                    o.w = f32_to_bf16_bits(src[6]) | ((uint32_t)f32_to_bf16_bits(src[7]) << 16);
                    *reinterpret_cast<uint4*>(rows16 + (size_t)t * d + c) = o;
                }
            }
        }
        const int tasks = T * E * 8;
        for (int base = 0; base < tasks; base += kSmallThreads) {
            const int task = base + tid;
            const bool live = task < tasks;
            const int pair = live ? task >> 3 : 0;
            const int j = task & 7;
            const int t = pair / E;
            const int e = pair - t * E;
            const XT* xr = xs + (size_t)t * ds;
            const float* wrow = ws + (size_t)e * ds;
            const float bv = (bias && live && j == 0) ? bias[e] : 0.0f;  // fetched while the dot product runs
            float acc = 0.0f;
            if (live) {
#pragma unroll 16
                for (int c = j; c < d; c += 8) acc = __fadd_rn(acc, __fmul_rn(to_f32(xr[c]), wrow[c]));
            }
            float sum = 0.0f;
#pragma unroll
            for (int l = 0; l < 8; ++l) sum = __fadd_rn(sum, __shfl(acc, (lane & ~7) + l));
            if (live && j == 0) {
                float v = __fadd_rn(sum, 0.0f);  // the reference adds its (empty) scalar rest: sum + 0
                if (bias) v = __fadd_rn(v, bv);
                prob[pair] = v;
            }
        }
    } else {
        const int tail = d - d % 8;
        const int tasks = T * E * 8;
        for (int base = 0; base < tasks; base += kSmallThreads) {
            const int task = base + tid;
            const bool live = task < tasks;
            const int pair = live ? task >> 3 : 0;
            const int j = task & 7;
            const int t = pair / E;
            const int e = pair - t * E;
            const XT* xr = x + (size_t)t * d;
            const float* wrow = wr + (size_t)e * d;
            // lane j of the pair: columns j, j + 8, ... in increasing order.  The loads of 32 steps
            // are issued together (they do not depend on one another); the adds stay a chain.
            float acc = 0.0f;
            if (live) {
                constexpr int U = 32;
                for (int c0 = j; c0 < tail; c0 += 8 * U) {
                    float xv[U], wv[U];
    #pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int c = c0 + 8 * u;
                        const int cc = c < tail ? c : j;  // always a valid column: no branch around the load
                        xv[u] = to_f32(xr[cc]);
                        wv[u] = wrow[cc];
                    }
    #pragma unroll
                    for (int u = 0; u < U; ++u)
                        if (c0 + 8 * u < tail) acc = __fadd_rn(acc, __fmul_rn(xv[u], wv[u]));
                }
            }
            // lanes folded left to right, by the first thread of the group of eight
            float sum = 0.0f;
    #pragma unroll
            for (int l = 0; l < 8; ++l) sum = __fadd_rn(sum, __shfl(acc, (lane & ~7) + l));
            if (live && j == 0) {
                float rest = 0.0f;
                for (int c = tail; c < d; ++c) rest = __fadd_rn(rest, __fmul_rn(to_f32(xr[c]), wrow[c]));
                float v = __fadd_rn(sum, rest);
                if (bias) v = __fadd_rn(v, bias[e]);
                prob[pair] = v;
            }
        }
    }
    __syncthreads();

    // ---- softmax_rows and route: one token per thread --------------------------
    // Up to 64 experts: a group of lanes per token; more: one thread per token.
    if (E <= 16 && k <= 16) {
        // 16 lanes per token, 32 tokens per pass of the block
        for (int t = tid >> 4; t < T; t += kSmallThreads / 16)
            token_phase_lanes<16>(prob + t * E, t, tid & 15, E, k, valid, P, lse, lsev, sexp, expert_of, gate_of);
    } else if (E <= 64) {
        // a wave per token (k <= 32 < 64 always)
        for (int t = tid >> 6; t < T; t += kSmallThreads / 64)
            token_phase_lanes<64>(prob + t * E, t, tid & 63, E, k, valid, P, lse, lsev, sexp, expert_of, gate_of);
    } else if (tid < T) {
        token_phase_serial(prob + tid * E, tid, E, k, valid, P, lse, lsev, sexp, expert_of, gate_of);
    }
    __syncthreads();

    // ---- bucket loop: a stable counting sort of the slots by expert ----------------
    // With at most 64 slots and 64 experts the first wave sorts and the second wave works out the two losses beside
    // it (same formulas and orders as the general code at the end; the per-expert counts it needs are ballots of
    // its own), and nothing is left to wait for.
    const bool side_losses = S <= 64 && E <= 64;
    if (side_losses && tid >= 64 && tid < 128) {
        const int ln = tid - 64;
        const int my = ln < S ? sexp[ln] : -1;
        int c_mine = 0;  // lane e: slots of expert e
        for (int e = 0; e < E; ++e) {
            const int c = __popcll(__ballot(my == e));
            if (ln == e) c_mine = c;
        }
        int V = 0;
        for (int t = 0; t < T; ++t) V += ((valid == nullptr) || valid[t]) ? 1 : 0;
        if (ln < E) {
            float term = 0.0f;
            if (V > 0) {
                const float load = (float)c_mine / ((float)V * (float)k);
                float mass = 0.0f;
                for (int t = 0; t < T; ++t)
                    if ((valid == nullptr) || valid[t]) mass = mass + prob[t * E + ln];
                mass = mass / (float)V;
                term = load * mass;
            }
            aux_term[ln] = term;
        }
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's LDS writes have landed
        __builtin_amdgcn_wave_barrier();
        if (ln == 0) {
            float aux = 0.0f, z = 0.0f;
            if (V > 0) {
                for (int e = 0; e < E; ++e) aux = aux + aux_term[e];
                aux = aux * ((float)E * w_aux);
                float zs = 0.0f;
                for (int t = 0; t < T; ++t)
                    if ((valid == nullptr) || valid[t]) zs = zs + lsev[t] * lsev[t];
                z = w_z * zs / (float)V;
            }
            losses[0] = aux;
            losses[1] = z;
        }
    }
    if (S <= 64) {
        // one wave, slot = lane: a ballot per expert gives its count and every slot's rank
        if (tid < 64) {
            const int my = tid < S ? sexp[tid] : -1;
            int run = 0, tiles = 0;
            if (expert_tokens != nullptr) {
                // the tokens of every expert, one bit a token (its rows are these tokens in ascending order: the sort
                // is stable and a token names an expert at most once), gathered in LDS (`off` is free on this path)
                for (int e = tid; e < E; e += 64) off[e] = 0;
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
                __builtin_amdgcn_wave_barrier();
                if (my >= 0) atomicOr(reinterpret_cast<unsigned int*>(&off[my]), 1u << (tid / k));
                __builtin_amdgcn_s_waitcnt(0xc07f);
                __builtin_amdgcn_wave_barrier();
                for (int e = tid; e < E; e += 64) expert_tokens[e] = (unsigned int)off[e];
            }
            if (E <= 64) {
                // the loop keeps everything in registers - slot `tid` its position, lane e expert e's count, first
                // position and first tile - and every store follows it, side by side
                int pos = -1, e_cnt = 0, e_off = 0, e_tile0 = 0;
                for (int e = 0; e < E; ++e) {
                    const unsigned long long mask = __ballot(my == e);
                    const int c = __popcll(mask);
                    pos = my == e ? run + __popcll(mask & ((1ull << tid) - 1ull)) : pos;
                    e_cnt = tid == e ? c : e_cnt;
                    e_off = tid == e ? run : e_off;
                    e_tile0 = tid == e ? tiles : e_tile0;
                    run += c;
                    tiles += c <= tile_m ? (c > 0 ? 1 : 0) : (c + tile_m - 1) / tile_m;
                }
                if (my >= 0) {
                    perm_slot[pos] = tid;
                    perm_token[pos] = tid / k;
                    inv_pos[tid] = pos;
                }
                if (tid < E) {
                    cnt[tid] = e_cnt;
                    counts[tid] = e_cnt;
                    offsets[tid] = e_off;
                    for (int r0 = 0, ti = e_tile0; r0 < e_cnt; r0 += tile_m, ++ti) {
                        tile_expert[ti] = tid;
                        tile_row0[ti] = e_off + r0;
                        tile_rows[ti] = min(tile_m, e_cnt - r0);
                    }
                }
            } else
            for (int e = 0; e < E; ++e) {
                const unsigned long long mask = __ballot(my == e);
                const int c = __popcll(mask);
                if (my == e) {
                    const int pos = run + __popcll(mask & ((1ull << tid) - 1ull));
                    perm_slot[pos] = tid;
                    perm_token[pos] = tid / k;
                    inv_pos[tid] = pos;
                }
                if (tid == 0) {
                    cnt[e] = c;
                    counts[e] = c;
                    offsets[e] = run;
                    for (int r0 = 0; r0 < c; r0 += tile_m) {
                        tile_expert[tiles] = e;
                        tile_row0[tiles] = run + r0;
                        tile_rows[tiles] = min(tile_m, c - r0);
                        ++tiles;
                    }
                }
                run += c;
            }
            if (tid < S && my < 0) inv_pos[tid] = -1;
            if (tid == 0) {
                offsets[E] = run;
                ntiles[0] = tiles;
            }
        }
    } else {
        // one expert per thread, slots in increasing order
        for (int e = tid; e < E; e += kSmallThreads) {
            int c = 0;
            for (int s = 0; s < S; ++s) c += (sexp[s] == e) ? 1 : 0;
            cnt[e] = c;
        }
        __syncthreads();
        if (tid == 0) {
            int run = 0, tiles = 0;
            for (int e = 0; e < E; ++e) {
                off[e] = run;
                counts[e] = cnt[e];
                offsets[e] = run;
                for (int r0 = 0; r0 < cnt[e]; r0 += tile_m) {
                    tile_expert[tiles] = e;
                    tile_row0[tiles] = run + r0;
                    tile_rows[tiles] = min(tile_m, cnt[e] - r0);
                    ++tiles;
                }
                run += cnt[e];
            }
            off[E] = run;
            offsets[E] = run;
            ntiles[0] = tiles;
        }
        for (int s = tid; s < S; s += kSmallThreads)
            if (sexp[s] < 0) inv_pos[s] = -1;
        __syncthreads();
        for (int e = tid; e < E; e += kSmallThreads) {
            int pos = off[e];
            unsigned int tokens = 0u;
            for (int s = 0; s < S; ++s)
                if (sexp[s] == e) {
                    perm_slot[pos] = s;
                    perm_token[pos] = s / k;
                    inv_pos[s] = pos;
                    tokens |= 1u << (s / k);
                    ++pos;
                }
            if (expert_tokens != nullptr) expert_tokens[e] = tokens;
        }
    }
    if (side_losses) return;
    __syncthreads();

    // ---- auxiliary losses (src/moe.rs:325-337): per expert in token order ---------
    int V = 0;
    for (int t = 0; t < T; ++t) V += ((valid == nullptr) || valid[t]) ? 1 : 0;
    for (int e = tid; e < E; e += kSmallThreads) {
        float term = 0.0f;
        if (V > 0) {
            const float load = (float)cnt[e] / ((float)V * (float)k);
            float mass = 0.0f;
            for (int t = 0; t < T; ++t)
                if ((valid == nullptr) || valid[t]) mass = mass + prob[t * E + e];
            mass = mass / (float)V;
            term = load * mass;
        }
        aux_term[e] = term;
    }
    __syncthreads();
    if (tid == 0) {
        float aux = 0.0f, z = 0.0f;
        if (V > 0) {
            for (int e = 0; e < E; ++e) aux = aux + aux_term[e];
            aux = aux * ((float)E * w_aux);
            float zs = 0.0f;
            for (int t = 0; t < T; ++t)
                if ((valid == nullptr) || valid[t]) zs = zs + lsev[t] * lsev[t];
            z = w_z * zs / (float)V;
        }
        losses[0] = aux;
        losses[1] = z;
    }
}

template <typename XT>
__global__ __launch_bounds__(kSmallThreads) void route_small_kernel(
    const XT* __restrict__ x, const float* __restrict__ wr, const float* __restrict__ bias,
    const uint8_t* __restrict__ valid, int T, int d, int E, int k, float w_aux, float w_z, int tile_m,
    float* __restrict__ P, float* __restrict__ lse, int* __restrict__ expert_of, float* __restrict__ gate_of,
    int* __restrict__ counts, int* __restrict__ offsets, int* __restrict__ tile_expert,
    int* __restrict__ tile_row0, int* __restrict__ tile_rows, int* __restrict__ ntiles,
    float* __restrict__ losses, int* __restrict__ perm_slot, int* __restrict__ perm_token,
    int* __restrict__ inv_pos, const float* __restrict__ norm_w, float norm_eps, XT* __restrict__ xn_out,
    bf16_t* __restrict__ rows16) {
    __shared__ __align__(16) unsigned char smem[kStageBytes + kRouteFixedBytes];
    route_small_body<XT, kStageBytes>(smem, x, wr, bias, valid, T, d, E, k, w_aux, w_z, tile_m, P, lse, expert_of, gate_of,
                                      counts, offsets, tile_expert, tile_row0, tile_rows, ntiles, losses, perm_slot,
                                      perm_token, inv_pos, norm_w, norm_eps, xn_out, rows16);
}

bool small_route_ok(int T, int E, int k) {
    return T >= 1 && T <= kSmallRouteMaxTokens && E <= kMaxExperts && k <= kMaxTopK &&
           T * E <= kSmallRouteMaxPairs;
}

// Whether route_small_kernel copies the router and the token rows into LDS for this call (the condition the
// kernel itself evaluates); only then can it apply the norm in front of the layer.
bool small_route_stages_rows(const void* x, const float* wr, int T, int d, int E, bool bf16) {
    const size_t ds = (size_t)d + 8;
    return d % 8 == 0 && (size_t)E * ds * 4 + (size_t)T * ds * (bf16 ? 2 : 4) <= (size_t)kStageBytes &&
           reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(wr) % 16 == 0;
}

hipError_t launch_route_small(const SmallRouteArgs& a, bool bf16, hipStream_t s) {
    if (!small_route_ok(a.T, a.E, a.k)) return hipErrorInvalidValue;
    if (a.norm_w && (!a.xn_out || !small_route_stages_rows(a.x, a.wr, a.T, a.d, a.E, bf16))) return hipErrorInvalidValue;
    if (a.rows16 && (bf16 || !small_route_stages_rows(a.x, a.wr, a.T, a.d, a.E, bf16))) return hipErrorInvalidValue;
    if (bf16)
        RB_LAUNCH(route_small_kernel<bf16_t>, dim3(1), dim3(kSmallThreads), 0, s,
                           static_cast<const bf16_t*>(a.x), a.wr, a.bias, a.valid, a.T, a.d, a.E, a.k, a.w_aux, a.w_z,
                           a.tile_m, a.P, a.lse, a.expert_of, a.gate_of, a.counts, a.offsets, a.tile_expert,
                           a.tile_row0, a.tile_rows, a.ntiles, a.losses, a.perm_slot, a.perm_token, a.inv_pos,
                           a.norm_w, a.norm_eps, static_cast<bf16_t*>(a.xn_out), nullptr);
    else
        RB_LAUNCH(route_small_kernel<float>, dim3(1), dim3(kSmallThreads), 0, s,
                           static_cast<const float*>(a.x), a.wr, a.bias, a.valid, a.T, a.d, a.E, a.k, a.w_aux, a.w_z,
                           a.tile_m, a.P, a.lse, a.expert_of, a.gate_of, a.counts, a.offsets, a.tile_expert,
                           a.tile_row0, a.tile_rows, a.ntiles, a.losses, a.perm_slot, a.perm_token, a.inv_pos,
                           a.norm_w, a.norm_eps, static_cast<float*>(a.xn_out), static_cast<bf16_t*>(a.rows16));
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// decode_gemm_kernel: out[row, n] for one tile of at most 32 rows and one block of 32
// output features (gate/up: 32 gate rows and the matching 32 up rows of the packed weights).
// The waves of a workgroup take an equal share of the reduction steps each; a wave fetches
// its weight fragments (1 KB per step and row block, straight from the packed layout) in
// batches of kBatch steps so that tens of kilobytes are in flight, multiplies them on the
// matrix cores against token fragments read from global memory (32 rows x K: they stay in
// L2), and the partial sums meet in LDS, in a fixed order.
// blockIdx.y < max_tiles: routed tiles (those past *ntiles exit); the rest: 32-row blocks of
// the shared expert, which takes every token.
// ---------------------------------------------------------------------------
constexpr int kBatch = 12;

struct DecodeSide {
    const bf16_t* a;
    const int* row_index;
    const char* w;
    const float* scales;
    bf16_t* out;
    int N, K, row0, rows;
    int a_row0;    // added to a row's number in `a` (rows of one expert inside a per-expert array)
    int out_row0;  // first output row is out_row0 + row0
    // The rows are read again inside this launch by a workgroup that may sit on another XCD (the folded combine): the
    // XCDs' L2 caches are not coherent with one another, so such rows are stored with device-scope stores, which
    // go through to memory, and read back with device-scope loads.
    bool coherent_out = false;
};

// NW = waves of a workgroup, each with 1 / NW of the reduction steps: 4 for the gate/up product, 8 for the
// down product (a third of the workgroups and twice the reduction length: with 8 waves every weight byte of
// the launch is requested before the first multiply there as well).
// The rows of a routed expert as the routing leaves them for a launch with one workgroup row per expert
// (decode_down_by_expert_kernel): the tokens the expert takes, one bit a token, and the position of its first row.
// The words are fetched behind the first weight loads (LATE_ROWS): nothing the weights' addresses need waits for them.
struct LateRows {
    const unsigned int* tokens;  // the expert's word
    const int* first;            // the expert's word
    const int* with_rows;        // experts with rows (one word for the launch)
    bool routed;  // false: the side's rows are sd.row0 / sd.rows as they stand (the shared expert)
    int with_rows_out = 0;
};

template <bool SWIGLU, bool I8, int NW, int BATCH, int TEAMS = 1, bool LATE_ROWS = false>
__device__ __forceinline__ void decode_gemm_body(DecodeSide& sd, int fb, float* red_raw, LateRows* late = nullptr);

// The combine of a decode-shaped call, for the 32 output features of block `fb` and every token: what
// combine_vec_kernel computes, element by element in the same order (the token's expert rows by ascending position,
// i.e. ascending expert; gate * row as a rounded multiply, then a rounded add; then the shared expert's row; then
// the residual).  Run by the last workgroup of the block's column to finish; the rows were stored with device-scope
// stores and are read with device-scope loads (see DecodeSide::coherent_out).
template <typename XT>
__device__ __forceinline__ void decode_combine_block(const DecodeGemmArgs& g, int fb, int nthreads) {
    const bf16_t* const y = static_cast<const bf16_t*>(g.out);
    const bf16_t* const ys = g.a_shared ? static_cast<const bf16_t*>(g.out_shared) : nullptr;
    const XT* const res = static_cast<const XT*>(g.cmb_residual);
    XT* const out = static_cast<XT*>(g.cmb_out);
    const int d = g.N, k = g.cmb_k;
    for (int idx = threadIdx.x; idx < g.cmb_T * 16; idx += nthreads) {
        const int t = idx >> 4;
        const int c = fb * 32 + 2 * (idx & 15);
        const int* const ip = g.cmb_inv_pos + (size_t)t * k;
        const float* const gp = g.cmb_gate_of + (size_t)t * k;
        float a0 = 0.0f, a1 = 0.0f;
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
            const uint32_t v = __hip_atomic_load(reinterpret_cast<const uint32_t*>(y + (size_t)best * d + c),
                                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const float gt = gp[bi];
            a0 = __fadd_rn(a0, __fmul_rn(gt, __uint_as_float(v << 16)));
            a1 = __fadd_rn(a1, __fmul_rn(gt, __uint_as_float(v & 0xffff0000u)));
        }
        if (ys) {
            const uint32_t v = __hip_atomic_load(reinterpret_cast<const uint32_t*>(ys + (size_t)t * d + c),
                                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            a0 = __fadd_rn(a0, __uint_as_float(v << 16));
            a1 = __fadd_rn(a1, __uint_as_float(v & 0xffff0000u));
        }
        if (res) {
            a0 = __fadd_rn(a0, to_f32(res[(size_t)t * d + c]));
            a1 = __fadd_rn(a1, to_f32(res[(size_t)t * d + c + 1]));
        }
        out[(size_t)t * d + c] = from_f32<XT>(a0);
        out[(size_t)t * d + c + 1] = from_f32<XT>(a1);
    }
}

// What a thread of the folded combine can fetch before its workgroup has multiplied anything: the positions of its
// token's expert rows in ascending order with their gates (at most four slots a token), and the residual.
constexpr int kCombineEarlySlots = 4;
struct CombineEarly {
    int pos[kCombineEarlySlots];  // as the routing wrote them; slots past k repeat the last one
    float gate[kCombineEarlySlots];
    uint32_t res[2];  // the residual's two elements as they lie in memory: one word of two bf16, or two f32
};

__device__ __forceinline__ void decode_combine_fetch(const DecodeGemmArgs& g, int fb, CombineEarly& ce) {
    // loads only, none of them looked at here and no branch between them: they return while the weights stream in
    const int t = min((int)threadIdx.x >> 4, g.cmb_T - 1), c = fb * 32 + 2 * ((int)threadIdx.x & 15), k = g.cmb_k;
    const int* const ip = g.cmb_inv_pos + (size_t)t * k;
    const float* const gp = g.cmb_gate_of + (size_t)t * k;
#pragma unroll
    for (int q = 0; q < kCombineEarlySlots; ++q) {
        ce.pos[q] = ip[min(q, k - 1)];
        ce.gate[q] = gp[min(q, k - 1)];
    }
    // (without a residual the words of the output's own place are fetched and never used; bf16: the second word is
    // the first again)
    const int es = g.cmb_f32 ? 4 : 2;
    const char* const base = static_cast<const char*>(g.cmb_residual ? g.cmb_residual : g.cmb_out);
    const char* const at = base + ((size_t)t * g.N + c) * es;
    ce.res[0] = *reinterpret_cast<const uint32_t*>(at);
    ce.res[1] = *reinterpret_cast<const uint32_t*>(at + (g.cmb_f32 ? 4 : 0));
}

// decode_combine_block for a workgroup of 512 threads (one element pair a thread) that fetched `ce` beforehand: the
// expert rows' loads go out side by side, the sums are taken in the same order.
template <typename XT>
__device__ __forceinline__ void decode_combine_block_early(const DecodeGemmArgs& g, int fb, CombineEarly ce) {
    const int t = (int)threadIdx.x >> 4, c = fb * 32 + 2 * ((int)threadIdx.x & 15);
    if (t >= g.cmb_T) return;
    // ascending positions (they are distinct; a padding token's slots and the slots past k have no row): five
    // exchanges sort four
#pragma unroll
    for (int q = 0; q < kCombineEarlySlots; ++q)
        if (q >= g.cmb_k || ce.pos[q] < 0) ce.pos[q] = 0x7fffffff;
    auto order = [&](int a, int b) {
        if (ce.pos[b] < ce.pos[a]) {
            const int p = ce.pos[a]; ce.pos[a] = ce.pos[b]; ce.pos[b] = p;
            const float w = ce.gate[a]; ce.gate[a] = ce.gate[b]; ce.gate[b] = w;
        }
    };
    order(0, 1); order(2, 3); order(0, 2); order(1, 3); order(1, 2);
    const bf16_t* const y = static_cast<const bf16_t*>(g.out);
    const int d = g.N;
    uint32_t v[kCombineEarlySlots], vs = 0u;
#pragma unroll
    for (int q = 0; q < kCombineEarlySlots; ++q)
        v[q] = ce.pos[q] != 0x7fffffff
                   ? __hip_atomic_load(reinterpret_cast<const uint32_t*>(y + (size_t)ce.pos[q] * d + c), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT)
                   : 0u;
    if (g.a_shared)
        vs = __hip_atomic_load(reinterpret_cast<const uint32_t*>(static_cast<const bf16_t*>(g.out_shared) + (size_t)t * d + c),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
    for (int q = 0; q < kCombineEarlySlots; ++q)
        if (ce.pos[q] != 0x7fffffff) {
            a0 = __fadd_rn(a0, __fmul_rn(ce.gate[q], __uint_as_float(v[q] << 16)));
            a1 = __fadd_rn(a1, __fmul_rn(ce.gate[q], __uint_as_float(v[q] & 0xffff0000u)));
        }
    if (g.a_shared) {
        a0 = __fadd_rn(a0, __uint_as_float(vs << 16));
        a1 = __fadd_rn(a1, __uint_as_float(vs & 0xffff0000u));
    }
    if (g.cmb_residual) {
        if constexpr (sizeof(XT) == 4) {
            a0 = __fadd_rn(a0, __uint_as_float(ce.res[0]));
            a1 = __fadd_rn(a1, __uint_as_float(ce.res[1]));
        } else {
            a0 = __fadd_rn(a0, __uint_as_float(ce.res[0] << 16));
            a1 = __fadd_rn(a1, __uint_as_float(ce.res[0] & 0xffff0000u));
        }
    }
    XT* const out = static_cast<XT*>(g.cmb_out);
    out[(size_t)t * d + c] = from_f32<XT>(a0);
    out[(size_t)t * d + c + 1] = from_f32<XT>(a1);
}

template <bool SWIGLU, bool I8, int NW>
__global__ __launch_bounds__(NW * 64) void decode_gemm_kernel(DecodeGemmArgs g) {
    __shared__ float red[NW * (SWIGLU ? 2 : 1) * 16 * 64];
    __shared__ int last_of_block;
    const int fb = blockIdx.x;
    const int ty = blockIdx.y;
    DecodeSide sd;
    sd.a_row0 = 0;
    sd.out_row0 = 0;
    // One round trip for the whole tile table: the four entries are fetched side by side (a stale entry past
    // *ntiles is read and dropped), not one after the other - with cold caches every dependent scalar load in
    // front of the first weight load is a few hundred nanoseconds of a launch that lasts ten microseconds.
    const bool routed = ty < g.max_tiles;
    const int tix = routed ? ty : 0;
    const int live_tiles = *g.ntiles;
    const int t_expert = g.tile_expert[tix], t_row0 = g.tile_row0[tix], t_rows = g.tile_rows[tix];
    asm volatile("" ::"s"(live_tiles), "s"(t_expert), "s"(t_row0), "s"(t_rows));  // all four here, not sunk into the branches
    // workgroups that write rows of this feature block's columns: the live routed tiles and the shared expert's
    const int writers = live_tiles + (g.a_shared ? (g.T_shared + 31) / 32 : 0);
    bool works = true;
    if (routed) {
        if (ty >= live_tiles) works = false;
        const int expert = t_expert;
        sd.a = static_cast<const bf16_t*>(g.a);
        sd.row_index = g.row_index;
        sd.w = static_cast<const char*>(g.w) + (size_t)expert * g.w_expert_stride * (I8 ? 1 : 2);
        sd.scales = I8 ? g.scales + (size_t)expert * g.s_expert_stride : nullptr;
        sd.out = static_cast<bf16_t*>(g.out);
        sd.N = g.N;
        sd.K = g.K;
        sd.row0 = t_row0;
        sd.rows = t_rows;
        sd.a_row0 = expert * g.a_expert_rows;
    } else {
        const int st = ty - g.max_tiles;
        sd.a = static_cast<const bf16_t*>(g.a_shared);
        sd.row_index = nullptr;
        sd.w = static_cast<const char*>(g.w_shared);
        sd.scales = I8 ? g.scales_shared : nullptr;
        sd.out = static_cast<bf16_t*>(g.out_shared);
        sd.N = g.N_shared;
        sd.K = g.K_shared;
        sd.row0 = st * 32;
        sd.rows = min(32, g.T_shared - sd.row0);
    }
    if (fb * 32 >= sd.N) return;
    if constexpr (!SWIGLU) {
        if (g.cmb_out != nullptr) {  // uniform over the launch
            // eight waves and at most four slots a token: what the combine needs of the routing is fetched now
            const bool early = NW == 8 && g.cmb_k <= kCombineEarlySlots;
            CombineEarly ce;
            if (early) decode_combine_fetch(g, fb, ce);
            if (!works) {
                // nothing to multiply here; with no writer at all (every row is padding and there is no shared
                // expert) the first of these workgroups still owes the block its combine
                if (writers != 0 || ty != 0) return;
            } else {
                sd.coherent_out = true;
                decode_gemm_body<SWIGLU, I8, NW, kBatch>(sd, fb, red);
                // every wave waits until its row stores have been acknowledged (they are device-scope stores: they
                // go through to memory) before the workgroup's arrival is counted behind the barrier - a barrier
                // alone does not wait for stores.  No device-scope fence: that would write back this XCD's whole
                // L2, once per workgroup.
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (threadIdx.x == 0) {
                    const int before = atomicAdd(&g.cmb_counter[fb * kDecodeCombineCounterStride], 1);
                    last_of_block = before == writers - 1;
                    if (before == writers - 1) atomicExch(&g.cmb_counter[fb * kDecodeCombineCounterStride], 0);  // every writer has arrived: ready for the next launch
                }
                __syncthreads();
                if (!last_of_block) return;
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            }
            if (early) {
                if (g.cmb_f32) decode_combine_block_early<float>(g, fb, ce);
                else decode_combine_block_early<bf16_t>(g, fb, ce);
            } else {
                if (g.cmb_f32) decode_combine_block<float>(g, fb, NW * 64);
                else decode_combine_block<bf16_t>(g, fb, NW * 64);
            }
            return;
        }
    }
    if (!works) return;
    decode_gemm_body<SWIGLU, I8, NW, kBatch>(sd, fb, red);
}

// ---------------------------------------------------------------------------
// decode_down_by_expert_kernel: the down product and the folded combine behind decode_front_kernel, blockIdx.y =
// expert (then the shared expert's 32-row blocks).  decode_gemm_kernel learns its expert from the tile table and
// its rows from the row index - two dependent trips to memory in front of the weight loads and the token loads;
// here the weights' address follows from the grid, and the three words that say which rows the expert has (its
// token bits, its first position, the number of experts with rows) are requested before the weights and looked at
// behind them.  Every thread also fetches what the combine will need of the routing (positions, gates, residual)
// before the product, so that the last workgroup of a block has only the expert rows left to load.
// Same products, same order of sums: the outputs are decode_gemm_kernel's bit for bit.
// ---------------------------------------------------------------------------
template <bool I8>
__global__ __launch_bounds__(512) void decode_down_by_expert_kernel(DecodeGemmArgs g, const unsigned int* __restrict__ expert_tokens,
                                                                    const int* __restrict__ offsets, int E) {
    __shared__ float red[8 * 16 * 64];
    __shared__ int last_of_block;
    const int fb = blockIdx.x, side = blockIdx.y;
    const bool routed = side < E;
    LateRows late;
    late.routed = routed;
    late.tokens = expert_tokens + (routed ? side : 0);
    late.first = offsets + (routed ? side : 0);
    late.with_rows = g.ntiles;  // one tile an expert: the experts with rows
    const int shared_tiles = g.a_shared ? (g.T_shared + 31) / 32 : 0;
    DecodeSide sd;
    sd.row_index = nullptr;
    sd.a_row0 = 0;
    sd.out_row0 = 0;
    sd.row0 = 0;
    sd.rows = 0;
    sd.coherent_out = true;
    if (routed) {
        sd.a = static_cast<const bf16_t*>(g.a);
        sd.a_row0 = side * g.a_expert_rows;
        sd.w = static_cast<const char*>(g.w) + (size_t)side * g.w_expert_stride * (I8 ? 1 : 2);
        sd.scales = I8 ? g.scales + (size_t)side * g.s_expert_stride : nullptr;
        sd.out = static_cast<bf16_t*>(g.out);
        sd.N = g.N;
        sd.K = g.K;
    } else {
        const int st = side - E;
        sd.a = static_cast<const bf16_t*>(g.a_shared);
        sd.w = static_cast<const char*>(g.w_shared);
        sd.scales = I8 ? g.scales_shared : nullptr;
        sd.out = static_cast<bf16_t*>(g.out_shared);
        sd.N = g.N_shared;
        sd.K = g.K_shared;
        sd.row0 = st * 32;
        sd.rows = min(32, g.T_shared - sd.row0);
    }
    CombineEarly ce;
    decode_combine_fetch(g, fb, ce);
    decode_gemm_body<false, I8, 8, kBatch, 1, true>(sd, fb, red, &late);
    const bool works = sd.rows > 0;
    const int writers = late.with_rows_out + shared_tiles;
    if (!works) {
        // nothing to multiply here; with no writer at all (every row is padding and there is no shared expert) the
        // first side's workgroups still owe their blocks the combine
        if (writers != 0 || side != 0) return;
    } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the row stores have been acknowledged
        __syncthreads();
        if (threadIdx.x == 0) {
            const int before = atomicAdd(&g.cmb_counter[fb * kDecodeCombineCounterStride], 1);
            last_of_block = before == writers - 1;
            if (before == writers - 1) atomicExch(&g.cmb_counter[fb * kDecodeCombineCounterStride], 0);  // every writer has arrived: ready for the next launch
        }
        __syncthreads();
        if (!last_of_block) return;
    }
    if (g.cmb_f32) decode_combine_block_early<float>(g, fb, ce);
    else decode_combine_block_early<bf16_t>(g, fb, ce);
}

// red_raw: TEAMS * NW * (SWIGLU ? 2 : 1) * 1024 floats of LDS; BATCH: reduction steps whose loads a wave issues together.
// TEAMS > 1: the workgroup is TEAMS teams of NW waves, each with a feature block `fb` of its own (the caller hands
// every team its block; a team without one has left the kernel before: the barrier below counts the waves that
// are still there).
// LATE_ROWS: which rows the side has is looked at behind the first weight loads (`late`); a side without rows leaves
// with sd.rows == 0 and nothing stored.
template <bool SWIGLU, bool I8, int NW, int BATCH, int TEAMS, bool LATE_ROWS>
__device__ __forceinline__ void decode_gemm_body(DecodeSide& sd, int fb, float* red_raw, LateRows* late) {
    const int team = TEAMS > 1 ? (int)threadIdx.x / (NW * 64) : 0;
    float (*red)[SWIGLU ? 2 : 1][16][64] =
        reinterpret_cast<float (*)[SWIGLU ? 2 : 1][16][64]>(red_raw + (size_t)team * NW * (SWIGLU ? 2 : 1) * 1024);
    const int tid = (int)threadIdx.x - team * (NW * 64);
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = sd.K;
    const int steps = K / 16;
    const int chunk = (steps + NW - 1) / NW;
    const int g0 = min(steps, wave * chunk), g1 = min(steps, g0 + chunk);

    // packed weights: row block rb starts at rb * K * 32 elements; step s, lane l at (s * 64 + l) * 16 bytes
    // (int8: steps come in pairs, 16 bytes per lane and pair, the even step first)
    const size_t block_bytes = (size_t)K * 32 * (I8 ? 1 : 2);
    const char* w0 = sd.w + (size_t)fb * block_bytes;
    const char* w1 = sd.w + (size_t)(sd.N / 32 + fb) * block_bytes;  // the matching up rows
    auto wfrag = [&](const char* base, int s) -> bf16x8 {
        if constexpr (I8) {
            const uint2 q = *reinterpret_cast<const uint2*>(base + ((size_t)(s >> 1) * 64 + lane) * 16 + (s & 1) * 8);
            return widen_i8(q);
        } else {
            const uint4 q = *reinterpret_cast<const uint4*>(base + ((size_t)s * 64 + lane) * 16);
            return __builtin_bit_cast(bf16x8, q);
        }
    };
    // token fragment: lane -> token lane % 32, columns 16 s + 8 (lane / 32) .. + 7
    int grow = 0;
    if constexpr (!LATE_ROWS) {
        const int trow = (lane & 31) < sd.rows ? (lane & 31) : 0;
        grow = (sd.row_index ? sd.row_index[sd.row0 + trow] : sd.row0 + trow) + sd.a_row0;  // awaited after the weight loads
    }

    floatx16 acc0, acc1;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.0f;

    // One batch of reduction steps.  The first batch stands in front of the loop over the others, as straight
    // code: at the head of a loop the compiler waits for every load still under way - the row index, what the
    // combine fetched early - before the first weight load could go out.  Returns true when the side has no rows.
    auto batch = [&](const int s0, auto first_tag) -> bool {
        constexpr bool kFirst = decltype(first_tag)::value;
        bf16x8 wa[BATCH], wb[BATCH], tf[BATCH];
        // the weights first: the address of a token row depends on a load of its own (the row index), and
        // loads are issued in order - nothing of the stream may queue up behind that wait
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const int s = min(s0 + u, g1 - 1);
            wa[u] = wfrag(w0, s);
            if constexpr (SWIGLU) wb[u] = wfrag(w1, s);
        }
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (LATE_ROWS && kFirst) {
            {
                // the three words, by scalar loads issued here and nowhere earlier (the compiler would fetch them
                // in front of the weights, or with vector loads that queue up behind them)
                unsigned int tokens;
                int first, with_rows;
                asm volatile(
                    "s_load_dword %0, %3, 0x0\n\t"
                    "s_load_dword %1, %4, 0x0\n\t"
                    "s_load_dword %2, %5, 0x0\n\t"
                    "s_waitcnt lgkmcnt(0)"
                    : "=&s"(tokens), "=&s"(first), "=&s"(with_rows)
                    : "s"(late->tokens), "s"(late->first), "s"(late->with_rows)
                    : "memory");
                late->with_rows_out = with_rows;
                if (late->routed) {
                    sd.rows = __popc(tokens);
                    sd.row0 = first;
                }
                if (sd.rows <= 0) return true;  // the whole workgroup
                const int trow = (lane & 31) < sd.rows ? (lane & 31) : 0;
                int token = sd.row0 + trow;
                if (late->routed) {  // row `trow` of the expert: the token of its set bit number `trow`
                    unsigned int rest = tokens;
                    for (int i = 0; i < trow; ++i) rest &= rest - 1u;
                    token = __ffs(rest) - 1;
                }
                grow = token + sd.a_row0;
            }
        }
        // (the empty statement pins the first use of the row index, and with it the wait for it, below the
        // weight loads; the barriers keep every load of the batch ahead of the first multiply)
        asm volatile("" : "+v"(grow));
        const bf16_t* arow = sd.a + (size_t)grow * K + 8 * (lane >> 5);
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const int s = min(s0 + u, g1 - 1);
            tf[u] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(arow + 16 * s));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            if (s0 + u < g1) {
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wa[u], tf[u], acc0, 0, 0, 0);
                if constexpr (SWIGLU) acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wb[u], tf[u], acc1, 0, 0, 0);
            }
        }
        return false;
    };
    // (LATE_ROWS: every wave takes the first batch, also one without a reduction step of its own, so that all of
    // them learn the rows and leave together when there are none)
    if (LATE_ROWS || g0 < g1) {
        if (batch(g0, std::true_type{})) return;
    }
    for (int s0 = g0 + BATCH; s0 < g1; s0 += BATCH) batch(s0, std::false_type{});
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        red[wave][0][v][lane] = acc0[v];
        if constexpr (SWIGLU) red[wave][1][v][lane] = acc1[v];
    }
    __syncthreads();
    // accumulator element v of lane l: feature 8 (v / 4) + 4 (l / 32) + v % 4, token l % 32;
    // the partial sums of the waves are added in wave order.  A thread takes four neighbouring features of one token
    // and eight neighbouring threads one token's 32 features of the block: a row segment of 64 bytes leaves as one
    // piece (rows that another workgroup of the launch reads go through to memory, where a write of a few bytes
    // costs what a whole segment does).
    if (tid < 256) {
        const int token = tid >> 3, q = tid & 7;
        const int v = 4 * (q >> 1), l = token + 32 * (q & 1), f = 4 * q;
        if (token < sd.rows) {
            float y4[4];
#pragma unroll
            for (int h = 0; h < 4; ++h) {
                float y = red[0][0][v + h][l];
#pragma unroll
                for (int w = 1; w < NW; ++w) y += red[w][0][v + h][l];
                if constexpr (I8) y *= sd.scales[fb * 32 + f + h];
                if constexpr (SWIGLU) {
                    float u = red[0][1][v + h][l];
#pragma unroll
                    for (int w = 1; w < NW; ++w) u += red[w][1][v + h][l];
                    if constexpr (I8) u *= sd.scales[sd.N + fb * 32 + f + h];
                    y = silu_bf16_grade(y) * u;
                }
                y4[h] = y;
            }
            bf16_t* const where = sd.out + (size_t)(sd.out_row0 + sd.row0 + token) * sd.N + fb * 32 + f;
            const unsigned long long four =
                (unsigned long long)((uint32_t)f32_to_bf16_bits(y4[0]) | ((uint32_t)f32_to_bf16_bits(y4[1]) << 16)) |
                ((unsigned long long)((uint32_t)f32_to_bf16_bits(y4[2]) | ((uint32_t)f32_to_bf16_bits(y4[3]) << 16)) << 32);
            if (sd.coherent_out)
                __hip_atomic_store(reinterpret_cast<unsigned long long*>(where), four, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else
                *reinterpret_cast<unsigned long long*>(where) = four;
        }
    }
}

// ---------------------------------------------------------------------------
// decode_front_kernel: the routing and the gate/up products in ONE launch, side by side.
// The routing is one workgroup walking a dependent chain for about ten microseconds; the gate/up
// product of a routed expert needs nothing of it but WHICH rows the expert takes.  With at most 32
// tokens an expert's rows are one tile whatever the routing says, so every expert's gate/up product
// is taken over ALL the call's rows - hidden rows [E][T, F] - without waiting for the routing: an
// expert that turns out unrouted costs its weights' bytes (the caller takes this launch only when
// most experts will be touched), the rows nobody routed to an expert cost nothing (the tile is 32
// rows either way).  Workgroup 0 routes; workgroup 1 + side * (N / 32) + fb takes feature block fb
// of side `side`: experts 0 .. E-1, then the shared expert's 32-row blocks.  The down product then
// picks the routed rows out of the per-expert hidden rows (DecodeGemmArgs::a_expert_rows).
// ---------------------------------------------------------------------------
template <bool I8>
__global__ __launch_bounds__(kSmallThreads, 2) void decode_front_kernel(SmallRouteArgs r, DecodeGemmArgs g, int E, int T) {
    __shared__ __align__(16) unsigned char smem[kFrontLdsBytes];
    if (blockIdx.x == 0) {
        route_small_body<bf16_t, kFrontStageBytes>(
            smem, static_cast<const bf16_t*>(r.x), r.wr, r.bias, r.valid, r.T, r.d, r.E, r.k, r.w_aux, r.w_z, r.tile_m, r.P,
            r.lse, r.expert_of, r.gate_of, r.counts, r.offsets, r.tile_expert, r.tile_row0, r.tile_rows, r.ntiles, r.losses,
            r.perm_slot, r.perm_token, r.inv_pos, nullptr, 0.0f, nullptr, nullptr, r.expert_tokens);
        return;
    }
    // a product workgroup is two teams of four waves, each with a block of 32 features of its own: the reduction is
    // split four ways as in the launch without the routing, and a compute unit has twice the weight bytes in flight
    const int widest = g.a_shared ? max(g.N, g.N_shared) : g.N;
    const int nfb = widest / 32, npair = (nfb + 1) / 2;
    const int idx = blockIdx.x - 1;
    const int fb = 2 * (idx % npair) + (int)threadIdx.x / (kSmallThreads / 2), side = idx / npair;
    DecodeSide sd;
    sd.row_index = nullptr;
    sd.row0 = 0;
    sd.a_row0 = 0;
    if (side < E) {
        sd.a = static_cast<const bf16_t*>(g.a);
        sd.w = static_cast<const char*>(g.w) + (size_t)side * g.w_expert_stride * (I8 ? 1 : 2);
        sd.scales = I8 ? g.scales + (size_t)side * g.s_expert_stride : nullptr;
        sd.out = static_cast<bf16_t*>(g.out);
        sd.N = g.N;
        sd.K = g.K;
        sd.rows = T;
        sd.out_row0 = side * T;
    } else {
        const int st = side - E;
        sd.a = static_cast<const bf16_t*>(g.a_shared);
        sd.w = static_cast<const char*>(g.w_shared);
        sd.scales = I8 ? g.scales_shared : nullptr;
        sd.out = static_cast<bf16_t*>(g.out_shared);
        sd.N = g.N_shared;
        sd.K = g.K_shared;
        sd.row0 = st * 32;
        sd.rows = min(32, g.T_shared - sd.row0);
        sd.out_row0 = 0;
    }
    if (fb * 32 >= sd.N) return;
    decode_gemm_body<true, I8, kSmallThreads / 128, kBatch, 2>(sd, fb, reinterpret_cast<float*>(smem));
}

bool decode_front_ok(const void* x, const float* wr, int T, int d, int E, int k) {
    // the routing workgroup of the fused launch has a smaller staging area; rows that do not fit it are read from
    // memory piecemeal, which takes longer than the products beside it: not worth it
    const size_t ds = (size_t)d + 8;
    const bool staged = d % 8 == 0 && (size_t)E * ds * 4 + (size_t)T * ds * 2 <= (size_t)kFrontStageBytes &&
                        reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(wr) % 16 == 0;
    // most experts must be about to be touched: an unrouted expert's gate/up weights are fetched for nothing
    return staged && T <= 32 && (long long)T * k >= 2LL * E;
}

hipError_t launch_decode_front(const SmallRouteArgs& r, const DecodeGemmArgs& g, WeightKind wk, hipStream_t s) {
    if (!small_route_ok(r.T, r.E, r.k) || r.norm_w || r.rows16 || !g.swiglu) return hipErrorInvalidValue;
    const int shared_tiles = g.a_shared ? (g.T_shared + 31) / 32 : 0;
    const int widest = g.a_shared ? (g.N > g.N_shared ? g.N : g.N_shared) : g.N;
    const int grid = 1 + (r.E + shared_tiles) * ((widest / 32 + 1) / 2);
    if (wk == WeightKind::BF16)
        RB_LAUNCH(decode_front_kernel<false>, dim3(grid), dim3(kSmallThreads), 0, s, r, g, r.E, r.T);
    else if (wk == WeightKind::I8)
        RB_LAUNCH(decode_front_kernel<true>, dim3(grid), dim3(kSmallThreads), 0, s, r, g, r.E, r.T);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

bool decode_down_by_expert_ok(const DecodeGemmArgs& g, int E, int T, int k) {
    return !g.swiglu && g.cmb_out != nullptr && g.cmb_counter != nullptr && g.cmb_inv_pos != nullptr &&
           g.cmb_gate_of != nullptr && g.a_expert_rows == T && T >= 1 && T <= 32 && k <= kCombineEarlySlots &&
           g.cmb_T == T && g.cmb_k == k && (!g.a_shared || g.N_shared == g.N) && g.N / 32 <= kDecodeCombineMaxBlocks &&
           g.N % 32 == 0 && E >= 1;
}

hipError_t launch_decode_down_by_expert(const DecodeGemmArgs& g, const unsigned int* expert_tokens, const int* offsets,
                                        int E, WeightKind wk, hipStream_t s) {
    if (!expert_tokens || !offsets || !decode_down_by_expert_ok(g, E, g.cmb_T, g.cmb_k)) return hipErrorInvalidValue;
    const int shared_tiles = g.a_shared ? (g.T_shared + 31) / 32 : 0;
    const dim3 grid(g.N / 32, E + shared_tiles);
    if (wk == WeightKind::BF16)
        RB_LAUNCH(decode_down_by_expert_kernel<false>, grid, dim3(512), 0, s, g, expert_tokens, offsets, E);
    else if (wk == WeightKind::I8)
        RB_LAUNCH(decode_down_by_expert_kernel<true>, grid, dim3(512), 0, s, g, expert_tokens, offsets, E);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

bool decode_shape_ok(int N, int K) { return K % 32 == 0 && K >= 32 && N % 32 == 0 && N >= 32; }

hipError_t launch_decode_gemm(const DecodeGemmArgs& g, WeightKind wk, hipStream_t s) {
    const int shared_tiles = g.a_shared ? (g.T_shared + 31) / 32 : 0;
    const int tiles = g.max_tiles + shared_tiles;
    if (tiles <= 0) return hipSuccess;
    const int widest = g.a_shared ? (g.N > g.N_shared ? g.N : g.N_shared) : g.N;
    if (g.cmb_out != nullptr) {  // the combine rides on a down-shaped launch whose two sides have the same width
        if (g.swiglu || !g.cmb_counter || !g.cmb_inv_pos || !g.cmb_gate_of || (g.a_shared && g.N_shared != g.N) ||
            g.N / 32 > kDecodeCombineMaxBlocks || g.N % 2 != 0)
            return hipErrorInvalidValue;
    }
    const dim3 grid(widest / 32, tiles);
    if (wk == WeightKind::BF16) {
        if (g.swiglu) RB_LAUNCH((decode_gemm_kernel<true, false, 4>), grid, dim3(256), 0, s, g);
        else RB_LAUNCH((decode_gemm_kernel<false, false, 8>), grid, dim3(512), 0, s, g);
    } else if (wk == WeightKind::I8) {
        if (g.swiglu) RB_LAUNCH((decode_gemm_kernel<true, true, 4>), grid, dim3(256), 0, s, g);
        else RB_LAUNCH((decode_gemm_kernel<false, true, 8>), grid, dim3(512), 0, s, g);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace rbmoe
