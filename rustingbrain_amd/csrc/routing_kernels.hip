// Router, dispatch and combine kernels of the mixture-of-experts forward pass
// for gfx950 (wave64).
//
//   router_kernel   logits (the reference's eight-lane `dot` order), softmax,
//                   log-sum-exp, deterministic top-k, per-block ranks and
//                   histogram, per-block partial sums for the auxiliary losses
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
//   xs     [TB][kRouterChunk + 4]  f32 slice of the token rows
//   ws     [min(E, 64)][kRouterChunk + 4]  f32 slice of the router rows of one pass
constexpr int kRouterChunk = 128;              // columns staged per step (a multiple of 8)
constexpr int kRouterStride = kRouterChunk + 4; // +4 floats: rows start 4 banks apart
constexpr int kRouterPassExperts = 64;         // experts per pass (8 per thread)

__host__ __device__ static size_t router_fixed_bytes(int E, int k) {
    const int ES = E | 1;
    size_t n = (size_t)kRouterTokens * ES + kRouterTokens + 2 * (size_t)kRouterTokens * k + 4 * (size_t)E + E;
    size_t bytes = n * 4 + (size_t)kRouterTokens * E;
    return (bytes + 15) & ~(size_t)15;
}

size_t router_lds_bytes(int E, int k) {
    const int wrows = E < kRouterPassExperts ? E : kRouterPassExperts;
    return router_fixed_bytes(E, k) + (size_t)(kRouterTokens + wrows) * kRouterStride * 4;
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

    // ---- logits ----------------------------------------------------------------
    // Thread (t = tid % 32, eg = tid / 32) owns token t and experts eg, eg + 8, ... of the
    // current pass, eight lane accumulators each, exactly the reference `dot`: lanes[c % 8]
    // += x[c] * w[c] in increasing c, a rounded multiply then a rounded add.  Token and
    // router rows are staged in LDS slice by slice (coalesced loads, converted to f32).
    float* xs = reinterpret_cast<float*>(lds_raw + router_fixed_bytes(E, k));
    float* ws = xs + TB * kRouterStride;
    const int tl = tid & 31;
    const int eg = tid >> 5;
    const int tail = d - d % 8;
    for (int e0 = 0; e0 < E; e0 += kRouterPassExperts) {
        const int pe = min(kRouterPassExperts, E - e0);  // experts in this pass
        float lanes[8][8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int l = 0; l < 8; ++l) lanes[j][l] = 0.0f;
        for (int c0 = 0; c0 < tail; c0 += kRouterChunk) {
            const int clen = min(kRouterChunk, tail - c0);
            __syncthreads();
            for (int idx = tid; idx < TB * clen; idx += 256) {
                const int r = idx / clen, c = idx - r * clen;
                xs[r * kRouterStride + c] = r < nt ? to_f32(x[(size_t)(t0 + r) * d + c0 + c]) : 0.0f;
            }
            for (int idx = tid; idx < pe * clen; idx += 256) {
                const int r = idx / clen, c = idx - r * clen;
                ws[r * kRouterStride + c] = wr[(size_t)(e0 + r) * d + c0 + c];
            }
            __syncthreads();
            const float* xrow = xs + tl * kRouterStride;
            for (int c = 0; c < clen; c += 8) {
                const float4 xa = *reinterpret_cast<const float4*>(xrow + c);
                const float4 xb = *reinterpret_cast<const float4*>(xrow + c + 4);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int el = eg + 8 * j;
                    if (el < pe) {
                        const float* wrow = ws + el * kRouterStride + c;
                        const float4 wa = *reinterpret_cast<const float4*>(wrow);
                        const float4 wb = *reinterpret_cast<const float4*>(wrow + 4);
                        lanes[j][0] = __fadd_rn(lanes[j][0], __fmul_rn(xa.x, wa.x));
                        lanes[j][1] = __fadd_rn(lanes[j][1], __fmul_rn(xa.y, wa.y));
                        lanes[j][2] = __fadd_rn(lanes[j][2], __fmul_rn(xa.z, wa.z));
                        lanes[j][3] = __fadd_rn(lanes[j][3], __fmul_rn(xa.w, wa.w));
                        lanes[j][4] = __fadd_rn(lanes[j][4], __fmul_rn(xb.x, wb.x));
                        lanes[j][5] = __fadd_rn(lanes[j][5], __fmul_rn(xb.y, wb.y));
                        lanes[j][6] = __fadd_rn(lanes[j][6], __fmul_rn(xb.z, wb.z));
                        lanes[j][7] = __fadd_rn(lanes[j][7], __fmul_rn(xb.w, wb.w));
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int el = eg + 8 * j;
            if (el < pe && tl < nt) {
                const int e = e0 + el;
                float rest = 0.0f;
                for (int c = tail; c < d; ++c)
                    rest = __fadd_rn(rest, __fmul_rn(to_f32(x[(size_t)(t0 + tl) * d + c]), wr[(size_t)e * d + c]));
                float sum = 0.0f;
#pragma unroll
                for (int l = 0; l < 8; ++l) sum = __fadd_rn(sum, lanes[j][l]);
                float v = __fadd_rn(sum, rest);
                if (bias) v = __fadd_rn(v, bias[e]);
                prob[tl * ES + e] = v;
            }
        }
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
// One wave per token; eight columns per lane per step when d allows.
// ---------------------------------------------------------------------------
template <typename XT, typename YT>
__global__ __launch_bounds__(256) void combine_kernel(
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
            // next smallest position greater than `last`
            int best = 0x7fffffff, bi = -1;
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
    hipLaunchKernelGGL(router_kernel<XT>, dim3(nb), dim3(256), router_lds_bytes(a.E, a.k), s,
                       static_cast<const XT*>(a.x), a.wr, a.bias, a.valid, a.T, a.d, a.E, a.k, a.P,
                       a.lse, a.expert_of, a.gate_of, a.rank_in_block, a.blockcnt, a.partial);
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

hipError_t launch_combine(const CombineArgs& a, bool bf16, hipStream_t s) {
    if (a.T <= 0) return hipSuccess;
    const dim3 grid((a.T + 3) / 4), block(256);
    if (bf16)
        hipLaunchKernelGGL((combine_kernel<bf16_t, bf16_t>), grid, block, 0, s,
                           static_cast<const bf16_t*>(a.y), static_cast<const bf16_t*>(a.yshared),
                           static_cast<const bf16_t*>(a.residual), a.inv_pos, a.gate_of, a.T, a.d,
                           a.k, static_cast<bf16_t*>(a.out));
    else
        hipLaunchKernelGGL((combine_kernel<float, float>), grid, block, 0, s,
                           static_cast<const float*>(a.y), static_cast<const float*>(a.yshared),
                           static_cast<const float*>(a.residual), a.inv_pos, a.gate_of, a.T, a.d,
                           a.k, static_cast<float*>(a.out));
    return hipGetLastError();
}

}  // namespace rbmoe
