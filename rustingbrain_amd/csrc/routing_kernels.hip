// Router, dispatch and combine kernels of the mixture-of-experts forward pass
// for gfx950 (wave64).
//
//   logits_kernel   router logits in the reference's eight-lane `dot` order
//   router_kernel   softmax, log-sum-exp, deterministic top-k, per-block ranks
//                   and histogram, per-block partial sums for the auxiliary losses
//   scan_kernel     prefix scan over blocks and experts, tile table for the
//                   grouped products, the two auxiliary losses
//   dispatch_kernel stable permutation (slot -> position) and row gather
//   combine_kernel  gate-weighted sum in ascending expert order, then the
//                   shared expert, then the optional residual
//
// Nothing here uses floating-point atomics: every sum has a fixed order, so two
// runs give the same bits.
#include "rbmoe_kernels.h"

namespace rbmoe {

// Dynamic LDS layout of router_kernel (floats / ints, in this order):
//   prob   [TB][ES]   logits, then exp, then probabilities   (ES = E | 1)
//   lsev   [TB]       log-sum-exp per token
//   gates  [TB][k]    selected probabilities, then gates
//   lexp   [TB][k]    selected expert per local slot (-1 = unrouted)
//   wcount [4][E]     per-wave match counts of one ranking round
//   running[E]        slots already ranked per expert
//   taken  [TB][E]    bytes (padded to a multiple of 16)
__host__ __device__ static size_t router_fixed_bytes(int E, int k) {
    const int ES = E | 1;
    size_t n = (size_t)kRouterTokens * ES + kRouterTokens + 2 * (size_t)kRouterTokens * k + 4 * (size_t)E + E;
    size_t bytes = n * 4 + (size_t)kRouterTokens * E;
    return (bytes + 15) & ~(size_t)15;
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
// A workgroup owns 64 tokens x 8 experts.  Lane = token; each of the 4 waves owns 2 experts,
// so a router row is wave-uniform and is fetched with scalar loads (it costs neither vector
// memory bandwidth nor LDS), while the token rows are staged through LDS in slices of
// kLogitChunk columns (16-byte pieces, rows padded by 16 bytes so that a wave's 64 row reads
// spread over all banks).
// ---------------------------------------------------------------------------
constexpr int kLogitTokens = 64;
constexpr int kLogitExperts = 8;
constexpr int kLogitChunk = 256;

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

template <typename XT>
__global__ __launch_bounds__(256) void logits_kernel(const XT* __restrict__ x, const float* __restrict__ wr,
                                                     const float* __restrict__ bias, int T, int d, int E,
                                                     float* __restrict__ logits) {
    typedef typename XPiece<XT>::raw_t piece_t;
    constexpr int PIECES = kLogitChunk / 8;          // pieces per row per slice
    constexpr int STRIDE = PIECES + (sizeof(piece_t) == 16 ? 1 : 1);  // +1 piece of padding per row
    __shared__ piece_t xs[kLogitTokens * STRIDE];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t0 = blockIdx.x * kLogitTokens;
    const int nt = min(kLogitTokens, T - t0);
    const int e0 = blockIdx.y * kLogitExperts + wave * 2;  // this wave's experts e0, e0 + 1
    const bool has0 = e0 < E, has1 = e0 + 1 < E;
    const float* w0 = wr + (size_t)(has0 ? e0 : 0) * d;
    const float* w1 = wr + (size_t)(has1 ? e0 + 1 : 0) * d;
    const int tail = d - d % 8;
    float la[8], lb[8];
#pragma unroll
    for (int l = 0; l < 8; ++l) {
        la[l] = 0.0f;
        lb[l] = 0.0f;
    }
    const bool vec = d % 8 == 0;
    for (int c0 = 0; c0 < tail; c0 += kLogitChunk) {
        const int np = min(PIECES, (tail - c0) / 8);  // pieces in this slice
        __syncthreads();
        for (int idx = tid; idx < kLogitTokens * np; idx += 256) {
            const int r = idx / np, q = idx - r * np;
            piece_t v = {};
            if (r < nt) {
                const XT* src = x + (size_t)(t0 + r) * d + c0 + 8 * q;
                if (vec) {
                    v = *reinterpret_cast<const piece_t*>(src);
                } else {  // rows are not 16-byte aligned: gather the eight elements
                    XT tmp[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) tmp[j] = src[j];
                    v = *reinterpret_cast<const piece_t*>(tmp);
                }
            }
            xs[r * STRIDE + q] = v;
        }
        __syncthreads();
        if (has0) {
            const float* wa = w0 + c0;
            const float* wb = w1 + c0;
#pragma unroll 4
            for (int q = 0; q < np; ++q) {
                float xv[8];
                XPiece<XT>::widen(xs[lane * STRIDE + q], xv);
#pragma unroll
                for (int l = 0; l < 8; ++l) la[l] = __fadd_rn(la[l], __fmul_rn(xv[l], wa[8 * q + l]));
                if (has1) {
#pragma unroll
                    for (int l = 0; l < 8; ++l) lb[l] = __fadd_rn(lb[l], __fmul_rn(xv[l], wb[8 * q + l]));
                }
            }
        }
    }
    if (lane < nt && has0) {
        const XT* xr = x + (size_t)(t0 + lane) * d;
        float rest0 = 0.0f, rest1 = 0.0f;
        for (int c = tail; c < d; ++c) {
            const float xv = to_f32(xr[c]);
            rest0 = __fadd_rn(rest0, __fmul_rn(xv, w0[c]));
            rest1 = __fadd_rn(rest1, __fmul_rn(xv, w1[c]));
        }
        float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
        for (int l = 0; l < 8; ++l) {
            s0 = __fadd_rn(s0, la[l]);
            s1 = __fadd_rn(s1, lb[l]);
        }
        float v0 = __fadd_rn(s0, rest0), v1 = __fadd_rn(s1, rest1);
        if (bias) {
            v0 = __fadd_rn(v0, bias[e0]);
            if (has1) v1 = __fadd_rn(v1, bias[e0 + 1]);
        }
        logits[(size_t)(t0 + lane) * E + e0] = v0;
        if (has1) logits[(size_t)(t0 + lane) * E + e0 + 1] = v1;
    }
}

template <typename XT>
__global__ __launch_bounds__(256) void router_kernel(
    const XT* __restrict__ x, const float* __restrict__ wr, const float* __restrict__ bias,
    const uint8_t* __restrict__ valid, int T, int d, int E, int k, float* __restrict__ P,
    float* __restrict__ lse, int* __restrict__ expert_of, float* __restrict__ gate_of,
    int* __restrict__ rank_in_block, int* __restrict__ blockcnt, float* __restrict__ partial) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    constexpr int TB = kRouterTokens;
    const int ES = E | 1;
    float* prob = reinterpret_cast<float*>(lds_raw);
    float* lsev = prob + TB * ES;
    float* gates = lsev + TB;
    int* lexp = reinterpret_cast<int*>(gates + TB * k);
    int* wcount = lexp + TB * k;
    int* running = wcount + 4 * E;
    unsigned char* taken = reinterpret_cast<unsigned char*>(running + E);

    const int tid = threadIdx.x;
    const int blk = blockIdx.x;
    const int t0 = blk * TB;
    const int nt = min(TB, T - t0);

    // ---- logits were written to P by logits_kernel ------------------------------
    for (int idx = tid; idx < nt * E; idx += 256) {
        const int i = idx / E;
        prob[i * ES + (idx - i * E)] = P[(size_t)t0 * E + idx];
    }
    for (int idx = tid; idx < TB * E; idx += 256) taken[idx] = 0;
    for (int idx = tid; idx < E; idx += 256) running[idx] = 0;
    __syncthreads();

    // ---- softmax + top-k: one token per thread, sequential over experts ---
    if (tid < nt) {
        float* row = prob + tid * ES;
        float mx = __uint_as_float(0xff800000u);
        for (int e = 0; e < E; ++e) {
            const float v = row[e];
            if (v > mx) mx = v;
        }
        float sum = 0.0f;
        for (int e = 0; e < E; ++e) {
            const float ex = rb_expf(__fadd_rn(row[e], -mx));
            row[e] = ex;
            sum = __fadd_rn(sum, ex);
        }
        lsev[tid] = __fadd_rn(mx, rb_logf(sum));
        if (sum > 0.0f)
            for (int e = 0; e < E; ++e) row[e] = __fdiv_rn(row[e], sum);

        const bool ok = (valid == nullptr) || (valid[t0 + tid] != 0);
        float* g = gates + tid * k;
        int* le = lexp + tid * k;
        if (!ok) {
            for (int r = 0; r < k; ++r) {
                le[r] = -1;
                g[r] = 0.0f;
            }
        } else {
            unsigned char* tk = taken + tid * E;
            for (int r = 0; r < k; ++r) {
                int best = -1;
                float bestv = 0.0f;
                for (int e = 0; e < E; ++e) {
                    if (tk[e]) continue;
                    const float v = row[e];
                    if (best < 0 || v > bestv) {
                        best = e;
                        bestv = v;
                    }
                }
                tk[best] = 1;
                le[r] = best;
                g[r] = bestv;
            }
            float total = 0.0f;
            for (int r = 0; r < k; ++r) total = __fadd_rn(total, g[r]);
            if (total > 0.0f)
                for (int r = 0; r < k; ++r) g[r] = __fdiv_rn(g[r], total);
        }
    }
    __syncthreads();

    // ---- write probabilities, lse, assignments (coalesced) ----------------
    for (int idx = tid; idx < nt * E; idx += 256) {
        const int i = idx / E;
        const int e = idx - i * E;
        P[(size_t)t0 * E + idx] = prob[i * ES + e];
    }
    if (tid < nt) lse[t0 + tid] = lsev[tid];
    const int nls = nt * k;
    for (int ls = tid; ls < nls; ls += 256) {
        expert_of[(size_t)t0 * k + ls] = lexp[ls];
        gate_of[(size_t)t0 * k + ls] = gates[ls];
    }

    // ---- partial sums for the auxiliary losses (fixed order) --------------
    for (int e = tid; e <= E; e += 256) {
        float s = 0.0f;
        if (e < E) {
            for (int i = 0; i < nt; ++i)
                if (lexp[i * k] >= 0) s += prob[i * ES + e];
        } else {
            for (int i = 0; i < nt; ++i)
                if (lexp[i * k] >= 0) s += lsev[i] * lsev[i];
        }
        partial[(size_t)blk * (E + 1) + e] = s;
    }

    // ---- rank of every local slot among earlier slots of the same expert --
    const int lane = tid & 63;
    const int wave = tid >> 6;
    int ebits = 0;
    while ((1 << ebits) < E) ++ebits;
    const int rounds = (nls + 255) / 256;
    for (int rd = 0; rd < rounds; ++rd) {
        for (int idx = tid; idx < 4 * E; idx += 256) wcount[idx] = 0;
        __syncthreads();
        const int ls = rd * 256 + tid;
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
        for (int idx = tid; idx < E; idx += 256)
            running[idx] += wcount[idx] + wcount[E + idx] + wcount[2 * E + idx] + wcount[3 * E + idx];
        __syncthreads();
    }
    for (int idx = tid; idx < E; idx += 256) blockcnt[(size_t)blk * E + idx] = running[idx];
}

// ---------------------------------------------------------------------------
// scan_kernel: one block of 1024 threads.
//   blockbase[b][e] = number of slots of expert e in blocks before b
//   counts[e], offsets[e] (exclusive prefix, offsets[E] = routed slots)
//   tile table for the grouped products: tile i covers rows
//   [tile_row0[i], tile_row0[i] + tile_rows[i]) of expert tile_expert[i]
//   losses[0] = aux, losses[1] = z   (reference src/moe.rs:602-639)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void scan_kernel(
    const int* __restrict__ blockcnt, int* __restrict__ blockbase, const float* __restrict__ partial,
    int nb, int E, int k, float w_aux, float w_z, int tile_m0, int tile_m1, int* __restrict__ counts,
    int* __restrict__ offsets, int* __restrict__ tile_expert0, int* __restrict__ tile_row00,
    int* __restrict__ tile_rows0, int* __restrict__ tile_expert1, int* __restrict__ tile_row01,
    int* __restrict__ tile_rows1, int* __restrict__ ntiles, float* __restrict__ losses,
    float* __restrict__ mass_out) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    // LDS: partsum[parts][E] ints, partmass[parts][E+1] floats, cnt[E], off[E+1], toff[2][E+1], mass[E+1]
    const int parts = 1024 / E;  // E <= 256 -> parts >= 4
    int* partsum = reinterpret_cast<int*>(lds_raw);
    float* partmass = reinterpret_cast<float*>(partsum + parts * E);
    int* cnt = reinterpret_cast<int*>(partmass + parts * (E + 1));
    int* off = cnt + E;
    int* toff = off + (E + 1);
    float* mass = reinterpret_cast<float*>(toff + 2 * (E + 1));

    const int tid = threadIdx.x;
    const int len = (nb + parts - 1) / parts;
    const int p = tid / E;
    const int e = tid - p * E;
    const bool active = p < parts;
    const int b0 = active ? min(nb, p * len) : 0;
    const int b1 = active ? min(nb, b0 + len) : 0;

    if (active) {
        int s = 0;
        float m = 0.0f;
        for (int b = b0; b < b1; ++b) {
            s += blockcnt[(size_t)b * E + e];
            m += partial[(size_t)b * (E + 1) + e];
        }
        partsum[p * E + e] = s;
        partmass[p * (E + 1) + e] = m;
        if (e == 0) {
            float zs = 0.0f;
            for (int b = b0; b < b1; ++b) zs += partial[(size_t)b * (E + 1) + E];
            partmass[p * (E + 1) + E] = zs;
        }
    }
    __syncthreads();
    if (tid < E) {
        int run = 0;
        float m = 0.0f;
        for (int q = 0; q < parts; ++q) {
            const int s = partsum[q * E + tid];
            partsum[q * E + tid] = run;
            run += s;
            m += partmass[q * (E + 1) + tid];
        }
        cnt[tid] = run;
        mass[tid] = m;
    }
    if (tid == E) {
        float zs = 0.0f;
        for (int q = 0; q < parts; ++q) zs += partmass[q * (E + 1) + E];
        mass[E] = zs;
    }
    __syncthreads();
    if (tid == 0) {
        int run = 0, trun0 = 0, trun1 = 0;
        for (int q = 0; q < E; ++q) {
            off[q] = run;
            toff[q] = trun0;
            toff[E + 1 + q] = trun1;
            run += cnt[q];
            trun0 += (cnt[q] + tile_m0 - 1) / tile_m0;
            trun1 += (cnt[q] + tile_m1 - 1) / tile_m1;
        }
        off[E] = run;
        toff[E] = trun0;
        toff[2 * E + 1] = trun1;
        ntiles[0] = trun0;
        ntiles[1] = trun1;
        // auxiliary losses: every valid token routes exactly k slots, so the
        // number of valid tokens is routed / k.
        const int V = run / k;
        float aux = 0.0f, z = 0.0f;
        if (V > 0) {
            const float tokens = (float)V;
            const float slots = (float)V * (float)k;
            for (int q = 0; q < E; ++q) {
                const float load = (float)cnt[q] / slots;
                const float ms = mass[q] / tokens;
                aux = aux + load * ms;
            }
            aux = aux * ((float)E * w_aux);
            z = w_z * mass[E] / tokens;
        }
        losses[0] = aux;
        losses[1] = z;
    }
    __syncthreads();
    if (active) {
        int run = partsum[p * E + e];
        for (int b = b0; b < b1; ++b) {
            const int c = blockcnt[(size_t)b * E + e];
            blockbase[(size_t)b * E + e] = run;
            run += c;
        }
    }
    if (tid < E) {
        counts[tid] = cnt[tid];
        offsets[tid] = off[tid];
        if (mass_out) mass_out[tid] = mass[tid];
        const int nt0 = toff[tid + 1] - toff[tid];
        for (int i = 0; i < nt0; ++i) {
            const int ti = toff[tid] + i;
            tile_expert0[ti] = tid;
            tile_row00[ti] = off[tid] + i * tile_m0;
            tile_rows0[ti] = min(tile_m0, cnt[tid] - i * tile_m0);
        }
        const int nt1 = toff[E + 1 + tid + 1] - toff[E + 1 + tid];
        for (int i = 0; i < nt1; ++i) {
            const int ti = toff[E + 1 + tid] + i;
            tile_expert1[ti] = tid;
            tile_row01[ti] = off[tid] + i * tile_m1;
            tile_rows1[ti] = min(tile_m1, cnt[tid] - i * tile_m1);
        }
    }
    if (tid == 0) offsets[E] = off[E];
}

size_t scan_lds_bytes(int E) {
    const int parts = 1024 / E;
    return ((size_t)parts * E + (size_t)parts * (E + 1) + E + 3 * (E + 1) + (E + 1)) * 4;
}

// ---------------------------------------------------------------------------
// dispatch_kernel: block b owns the same tokens as router block b.  Position
// of a routed slot = offsets[e] + blockbase[b][e] + rank_in_block[slot]: slots
// are numbered token-major, so this is exactly the order in which the
// reference appends slots to an expert's list (src/moe.rs:266-274).  The row
// copy is `gather_rows` (src/moe.rs:658-664); the slot table of the block is
// staged in LDS, rows move as 16-byte pieces.
// ---------------------------------------------------------------------------
template <typename XT>
__global__ __launch_bounds__(256) void dispatch_kernel(
    const XT* __restrict__ x, const int* __restrict__ expert_of, const int* __restrict__ rank_in_block,
    const int* __restrict__ blockbase, const int* __restrict__ offsets, int T, int d, int E, int k,
    int* __restrict__ perm_slot, int* __restrict__ perm_token, int* __restrict__ inv_pos,
    XT* __restrict__ xg) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int* lpos = reinterpret_cast<int*>(lds_raw);  // [TB * k]
    constexpr int TB = kRouterTokens;
    const int tid = threadIdx.x;
    const int blk = blockIdx.x;
    const int t0 = blk * TB;
    const int nt = min(TB, T - t0);
    const int nls = nt * k;
    for (int ls = tid; ls < nls; ls += 256) {
        const int s = t0 * k + ls;
        const int e = expert_of[s];
        int pos = -1;
        if (e >= 0) {
            pos = offsets[e] + blockbase[(size_t)blk * E + e] + rank_in_block[s];
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
template <typename T>
struct Vec16;
template <>
struct Vec16<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const float4 a = *reinterpret_cast<const float4*>(p);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
};
template <>
struct Vec16<bf16_t> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
        const uint4 a = *reinterpret_cast<const uint4*>(p);
        v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
        v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
        v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xffff0000u);
        v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
        uint4 o;
        o.x = f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
        o.y = f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
        o.z = f32_to_bf16_bits(v[4]) | ((uint32_t)f32_to_bf16_bits(v[5]) << 16);
        o.w = f32_to_bf16_bits(v[6]) | ((uint32_t)f32_to_bf16_bits(v[7]) << 16);
        *reinterpret_cast<uint4*>(p) = o;
    }
};

template <typename XT, int KMAX>
__global__ __launch_bounds__(256) void combine_vec_kernel(
    const XT* __restrict__ y, const XT* __restrict__ yshared, const XT* __restrict__ residual,
    const int* __restrict__ inv_pos, const float* __restrict__ gate_of, int T, int d, int k,
    XT* __restrict__ out) {
    constexpr int VN = Vec16<XT>::N;
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
#pragma unroll
    for (int r = 0; r < KMAX; ++r) {
        if (r < k) {
            int p = inv_pos[(size_t)t * k + r];
            float g = gate_of[(size_t)t * k + r];
            if (p >= 0) {
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
    }
    float acc[VN];
#pragma unroll
    for (int i = 0; i < VN; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int r = 0; r < KMAX; ++r) {
        if (r < n) {
            float v[VN];
            Vec16<XT>::load(y + (size_t)pos[r] * d + c, v);
#pragma unroll
            for (int i = 0; i < VN; ++i) acc[i] = __fadd_rn(acc[i], __fmul_rn(gate[r], v[i]));
        }
    }
    if (yshared) {
        float v[VN];
        Vec16<XT>::load(yshared + (size_t)t * d + c, v);
#pragma unroll
        for (int i = 0; i < VN; ++i) acc[i] = __fadd_rn(acc[i], v[i]);
    }
    if (residual) {
        float v[VN];
        Vec16<XT>::load(residual + (size_t)t * d + c, v);
#pragma unroll
        for (int i = 0; i < VN; ++i) acc[i] = __fadd_rn(acc[i], v[i]);
    }
    Vec16<XT>::store(out + (size_t)t * d + c, acc);
}

// Any k, any d: one wave per token, one column per lane per step.
template <typename XT>
__global__ __launch_bounds__(256) void combine_any_kernel(
    const XT* __restrict__ y, const XT* __restrict__ yshared, const XT* __restrict__ residual,
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
template <typename XT>
static hipError_t launch_router_t(const RouterArgs& a, hipStream_t s) {
    const int nb = (a.T + kRouterTokens - 1) / kRouterTokens;
    static bool attr_set = false;
    if (!attr_set) {  // allow more than the default 64 KiB of dynamic LDS (gfx950 has 160 KiB per CU)
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(router_kernel<XT>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kMaxRouterLds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const dim3 lgrid((a.T + kLogitTokens - 1) / kLogitTokens, (a.E + kLogitExperts - 1) / kLogitExperts);
    hipLaunchKernelGGL((logits_kernel<XT>), lgrid, dim3(256), 0, s,
                       static_cast<const XT*>(a.x), a.wr, a.bias, a.T, a.d, a.E, a.P);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((router_kernel<XT>), dim3(nb), dim3(256), router_lds_bytes(a.E, a.k), s,
                       static_cast<const XT*>(a.x), a.wr, a.bias, a.valid, a.T, a.d, a.E, a.k, a.P, a.lse,
                       a.expert_of, a.gate_of, a.rank_in_block, a.blockcnt, a.partial);
    return hipGetLastError();
}

hipError_t launch_router(const RouterArgs& a, bool bf16, hipStream_t s) {
    if (a.T <= 0) return hipSuccess;
    return bf16 ? launch_router_t<bf16_t>(a, s) : launch_router_t<float>(a, s);
}

hipError_t launch_scan(const ScanArgs& a, hipStream_t s) {
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(1024), scan_lds_bytes(a.E), s, a.blockcnt,
                       a.blockbase, a.partial, a.nb, a.E, a.k, a.w_aux, a.w_z, a.tile_m[0], a.tile_m[1],
                       a.counts, a.offsets, a.tile_expert[0], a.tile_row0[0], a.tile_rows[0],
                       a.tile_expert[1], a.tile_row0[1], a.tile_rows[1], a.ntiles, a.losses, a.mass);
    return hipGetLastError();
}

template <typename XT>
static hipError_t launch_dispatch_t(const DispatchArgs& a, hipStream_t s) {
    const int nb = (a.T + kRouterTokens - 1) / kRouterTokens;
    hipLaunchKernelGGL(dispatch_kernel<XT>, dim3(nb), dim3(256),
                       (size_t)kRouterTokens * a.k * sizeof(int), s, static_cast<const XT*>(a.x),
                       a.expert_of, a.rank_in_block, a.blockbase, a.offsets, a.T, a.d, a.E, a.k,
                       a.perm_slot, a.perm_token, a.inv_pos, static_cast<XT*>(a.xg));
    return hipGetLastError();
}

hipError_t launch_dispatch(const DispatchArgs& a, bool bf16, hipStream_t s) {
    if (a.T <= 0) return hipSuccess;
    return bf16 ? launch_dispatch_t<bf16_t>(a, s) : launch_dispatch_t<float>(a, s);
}

template <typename XT>
static hipError_t launch_combine_t(const CombineArgs& a, hipStream_t s) {
    const XT* y = static_cast<const XT*>(a.y);
    const XT* ys = static_cast<const XT*>(a.yshared);
    const XT* res = static_cast<const XT*>(a.residual);
    XT* out = static_cast<XT*>(a.out);
    constexpr int VN = Vec16<XT>::N;
    if (a.d % VN == 0 && a.k <= 8) {
        const long long total = (long long)a.T * (a.d / VN);
        const dim3 grid((unsigned)((total + 255) / 256)), block(256);
        if (a.k <= 2)
            hipLaunchKernelGGL((combine_vec_kernel<XT, 2>), grid, block, 0, s, y, ys, res, a.inv_pos, a.gate_of, a.T, a.d, a.k, out);
        else if (a.k <= 4)
            hipLaunchKernelGGL((combine_vec_kernel<XT, 4>), grid, block, 0, s, y, ys, res, a.inv_pos, a.gate_of, a.T, a.d, a.k, out);
        else
            hipLaunchKernelGGL((combine_vec_kernel<XT, 8>), grid, block, 0, s, y, ys, res, a.inv_pos, a.gate_of, a.T, a.d, a.k, out);
    } else {
        hipLaunchKernelGGL((combine_any_kernel<XT>), dim3((a.T + 3) / 4), dim3(256), 0, s, y, ys, res, a.inv_pos,
                           a.gate_of, a.T, a.d, a.k, out);
    }
    return hipGetLastError();
}

hipError_t launch_combine(const CombineArgs& a, bool bf16, hipStream_t s) {
    if (a.T <= 0) return hipSuccess;
    return bf16 ? launch_combine_t<bf16_t>(a, s) : launch_combine_t<float>(a, s);
}

}  // namespace rbmoe
