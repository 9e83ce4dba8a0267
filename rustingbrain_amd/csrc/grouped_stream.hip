// Grouped expert products on the bf16 matrix cores of gfx950.
//
//   out[row, n] = sum_c a[row, c] * w[expert][n, c]                 (down product)
//   out[row, n] = silu(a . wgate[n]) * (a . wup[n])                 (gate/up product)
//
// Data paths (nothing is staged through registers on its way to LDS):
//   weights      packed at upload into matrix-core operand order (see
//                pack_weight_bf16 / pack_weight_i8); every wave streams its own
//                fragments global -> VGPR through a 4-deep register ring, i.e.
//                the load for reduction step g + 3 is issued while step g runs.
//                int8 weights are widened to bf16 in registers right before the
//                multiply; the per-row scale multiplies the accumulator.
//   activations  128 token rows per workgroup (gathered through an index for
//                the gate/up product) go global -> LDS with the LDS-DMA load
//                (global_load_lds_dwordx4): lane l of a wave deposits its 16
//                bytes at LDS base + 16 l, so the XOR swizzle that keeps the
//                fragment reads free of bank conflicts is applied by choosing
//                which global piece each lane fetches.  Three LDS stages: the
//                DMA for slice k + 2 is issued in the last step of slice k, after
//                the barrier (behind step KS - 2) that proves its stage free, and
//                is awaited (vmcnt) just before the barrier of slice k + 1.
//   fragments    token fragments are read from LDS one step ahead of the
//                multiplies that use them, across slice boundaries too.
//   issue order  a wave that is alone on its SIMD must keep the matrix core fed
//                by itself: every memory instruction of the main loop sits
//                behind a multiply of its own (see pipe_loop).
// A workgroup is 4 waves side by side along the output features; a wave owns
// 128 tokens x 64 weight rows (32 gate + the matching 32 up rows, or 64 down
// rows).  The weight fragment is the matrix-core A operand and the token
// fragment the B operand, so a lane ends with 4 consecutive output features of
// one token and writes them with one 8-byte store.  Token blocks of 32 rows
// that lie beyond the end of a group are skipped, so a ragged group costs at
// most 31 rows of padding.
#include <algorithm>
#include <type_traits>

#include "rbmoe_kernels.h"

// Hook for timeline studies of the kernels: a harness that includes this file may define it to record a time
// stamp per tile (`slot` = the tile's number in launch order) at point i (0 tile taken up, 1 main loop entered,
// 2 main loop left, 3 tile written).  Expands to nothing in the library.
#ifndef RBMOE_TRACE_AT
#define RBMOE_TRACE_AT(slot, i)
#endif

namespace rbmoe {

namespace {

#ifndef RBMOE_STREAM_BM
#define RBMOE_STREAM_BM 128
#endif
#ifndef RBMOE_STREAM_OCC
#define RBMOE_STREAM_OCC 2
#endif
constexpr int BM = RBMOE_STREAM_BM;   // token rows per workgroup
constexpr int BK = 64;    // reduction slice held in one LDS stage
#ifndef RBMOE_STREAM_NW
#define RBMOE_STREAM_NW 4
#endif
constexpr int NW = RBMOE_STREAM_NW;     // waves per workgroup (4, or 8: one activation slice for twice the features)
constexpr int NT = NW * 64;
constexpr int CPR = BK / 8;            // 16-byte pieces per LDS row
constexpr int TT = BM / 32;            // token blocks per wave
constexpr int KS = BK / 16;            // matrix-core steps per slice
constexpr int DMA_PER_WAVE = BM * CPR / 64 / NW;  // LDS-DMA instructions per wave per slice
constexpr int RING = KS;    // weight-fragment steps in flight per wave (register ring depth)
constexpr int STAGES = 3;   // LDS stages of one activation slice each

// Token fragment read from LDS.
__device__ __forceinline__ bf16x8 lds_frag(const uint4* __restrict__ base, int idx) {
    return __builtin_bit_cast(bf16x8, base[idx]);
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Every vector-memory instruction of the main loop is issued from inline assembly and waited
// for by hand.  Left to the compiler, any wait that falls while an LDS-DMA is in flight
// becomes vmcnt(0), which drains the whole weight ring and the DMA just issued once per
// slice; and loads from read-only memory may be moved across the barriers the hand-written
// counts rely on.  Loads retire in order, so "at most N outstanding" proves that everything
// but the N youngest has landed; N is always the exact number of younger instructions.
__device__ __forceinline__ void issue_load(u32x4& d, uint32_t byte_off, const char* base) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(d) : "v"(byte_off), "s"(base));
}
__device__ __forceinline__ void issue_load(u32x2& d, uint32_t byte_off, const char* base) {
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(d) : "v"(byte_off), "s"(base));
}
// 64 lanes x 16 bytes from `src` (per lane) to LDS bytes [lds_addr, lds_addr + 1024).
__device__ __forceinline__ void issue_dma(uint32_t lds_addr, uint32_t byte_off, const char* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(byte_off), "s"(base) : "memory");
}
// Wait until at most N loads are outstanding; the two registers become usable only here.
template <int N, typename V>
__device__ __forceinline__ void wait_for(V& a, V& b) {
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N));
}
template <int N>
__device__ __forceinline__ void wait_outstanding() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>), in order
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// f(0), f(1), ... while f returns true: slice I + 1 of a loop's remainder is reached only through slice I
template <int I, int N, typename F>
__device__ __forceinline__ void static_while(F&& f) {
    if constexpr (I < N) {
        if (f(std::integral_constant<int, I>{})) static_while<I + 1, N>(f);
    }
}

// One ring slot: the wave's two weight fragments of one reduction step.
// bf16: 16 bytes per lane per fragment, step g at byte 1024 g + 16 lane of a row block.
// int8: 8 bytes per lane per fragment; the packed layout is [K/32][64 lanes][16 bytes] with
//       bytes 0..7 for the even step and 8..15 for the odd one.
template <bool I8>
struct Slot;
template <>
struct Slot<false> {
    u32x4 f0, f1;
    __device__ __forceinline__ void load(const char* p0, const char* p1, int g, uint32_t lane16) {
        const uint32_t off = lane16 + (uint32_t)g * 1024u;
        issue_load(f0, off, p0);
        issue_load(f1, off, p1);
    }
    static __device__ __forceinline__ uint32_t offset(int g, uint32_t lane16) { return lane16 + (uint32_t)g * 1024u; }
    __device__ __forceinline__ void load0(const char* p0, uint32_t off) { issue_load(f0, off, p0); }
    __device__ __forceinline__ void load1(const char* p1, uint32_t off) { issue_load(f1, off, p1); }
    __device__ __forceinline__ bf16x8 a0() const { return __builtin_bit_cast(bf16x8, f0); }
    __device__ __forceinline__ bf16x8 a1() const { return __builtin_bit_cast(bf16x8, f1); }
};
template <>
struct Slot<true> {
    u32x2 f0, f1;
    __device__ __forceinline__ void load(const char* p0, const char* p1, int g, uint32_t lane16) {
        const uint32_t off = lane16 + (uint32_t)(g >> 1) * 1024u + (uint32_t)(g & 1) * 8u;
        issue_load(f0, off, p0);
        issue_load(f1, off, p1);
    }
    static __device__ __forceinline__ uint32_t offset(int g, uint32_t lane16) {
        return lane16 + (uint32_t)(g >> 1) * 1024u + (uint32_t)(g & 1) * 8u;
    }
    __device__ __forceinline__ void load0(const char* p0, uint32_t off) { issue_load(f0, off, p0); }
    __device__ __forceinline__ void load1(const char* p1, uint32_t off) { issue_load(f1, off, p1); }
    __device__ __forceinline__ bf16x8 a0() const { return widen_i8(make_uint2(f0.x, f0.y)); }
    __device__ __forceinline__ bf16x8 a1() const { return widen_i8(make_uint2(f1.x, f1.y)); }
};

// ---- epilogue: the accumulators of one tile to memory -------------------------------------------------
struct TileOut {
    int rows, row0, tn_idx, N;
    bool act0, act1;      // whether the wave's two row blocks lie inside N
    int r0, r1;           // their first weight rows
    const float* sc;      // int8: the expert's scales, one per weight row
    bf16_t* out;
    bf16_t* gu_out;
    const bf16_t* bw_gu;
};

// `stage`: 32 KiB of LDS that no wave of the workgroup reads or writes any more (the caller has made sure of
// that with a barrier).  `before_stores()` is called once, when the first pass has been converted and staged and
// before its first store to memory is issued.
template <bool SWIGLU, bool I8, typename F>
__device__ __forceinline__ void write_tile(const TileOut& o, floatx16 (&acc)[2][TT], char* const stage,
                                           F&& before_stores) {
    constexpr int BN = SWIGLU ? NW * 32 : NW * 64;
    // The thread index is made opaque here: everything derived from it below (LDS and row offsets, two dozen
    // values per lane) is then worked out where it is used.  Otherwise a caller that writes tile after tile has
    // them computed once, in front of its tile loop, and carried through the main loop in registers that the
    // loop does not have.
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lrow = lane & 31;
    const int lhalf = lane >> 5;
    const int rows = o.rows, row0 = o.row0, tn_idx = o.tn_idx, N = o.N, r0 = o.r0, r1 = o.r1;
    const bool act0 = o.act0, act1 = o.act1;
    const float* const sc = o.sc;
    bf16_t* const out = o.out;
    bf16_t* const gu_out = o.gu_out;
    const bf16_t* const bw_gu = o.bw_gu;
    // Accumulator element v of block (b, t): feature 8*(v/4) + 4*(lane/32) + v%4 of the
    // wave's row block b, token t*32 + lane%32 - a lane holds 4 consecutive features of a
    // token, so a direct store would scatter 8-byte pieces over 32 rows per instruction.
    // Instead each block index goes through LDS as a 128-token x 128-feature tile (16-byte
    // pieces, piece p of row r kept at position p ^ (r % 16)), and is written out with
    // 16-byte stores, 16 consecutive lanes covering the 256 contiguous bytes of a row.
    // Passes through the staging tile: down product: the two blocks of 128 features; gate/up: the
    // hidden rows, then (only when the caller keeps them for a backward pass) the gate and the
    // up pre-activations, which go to `gu_out` [rows, 2N] with the gate half in columns [0, N).
    constexpr int PASSES = SWIGLU ? 3 : 2;
    constexpr int WH = NW < 4 ? NW : 4;  // waves that fill the staging tile at a time (32 features each)
    constexpr int SUB = NW / WH;         // ... in this many turns per block index
    constexpr int PW = WH * 4;           // 16-byte pieces of a staged row in use
#pragma unroll
    for (int bh = 0; bh < PASSES * SUB; ++bh) {
        const int b = bh / SUB, h = bh % SUB;
        if constexpr (SWIGLU) {
            if (b > 0 && gu_out == nullptr) break;  // uniform over the launch
        }
        if (bh) __syncthreads();  // the previous pass has been read out
        if ((wave / WH) == h && (SWIGLU ? act0 : (b ? act1 : act0))) {
            const int rb = b ? r1 : r0;
#pragma unroll
            for (int t = 0; t < TT; ++t) {
                if (t * 32 >= rows) continue;
                const int m = t * 32 + lrow;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int f = 8 * q + 4 * lhalf;  // first of 4 consecutive features inside the row block
                    float y[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if constexpr (SWIGLU) {
                            float gv = acc[0][t][4 * q + i], uv = acc[1][t][4 * q + i];
                            if constexpr (I8) {
                                gv *= sc[r0 + f + i];
                                uv *= sc[r1 + f + i];
                            }
                            y[i] = b == 0 ? silu_bf16_grade(gv) * uv : (b == 1 ? gv : uv);
                        } else {
                            y[i] = acc[b][t][4 * q + i];
                            if constexpr (I8) y[i] *= sc[rb + f + i];
                        }
                    }
                    const int piece = ((wave % WH) * 4 + q) ^ (m & 15);
                    *reinterpret_cast<uint2*>(stage + m * 256 + piece * 16 + lhalf * 8) =
                        make_uint2(pack2(y[0], y[1]), pack2(y[2], y[3]));
                }
            }
        }
        __syncthreads();
        if (bh == 0) before_stores();
        // where this pass goes: hidden rows and down rows into `out` (row stride N), the
        // pre-activations into `gu_out` (row stride 2 N)
        const int col0 = tn_idx * BN + (SWIGLU ? 0 : b * (NW * 32)) + h * (WH * 32);
        bf16_t* const dst = (SWIGLU && b > 0) ? gu_out + (b == 2 ? N : 0) : out;
        const size_t dstride = (SWIGLU && b > 0) ? (size_t)2 * N : (size_t)N;
#pragma unroll
        for (int i = 0; i < BM * PW / NT; ++i) {
            const int idx = i * NT + tid;
            const int r = idx / PW, p = idx % PW;
            if (r < rows && col0 + 8 * p < N) {
                const uint4 v = *reinterpret_cast<const uint4*>(stage + r * 256 + ((p ^ (r & 15)) * 16));
                if constexpr (!SWIGLU) {
                    if (bw_gu != nullptr) {  // uniform over the launch
                        // SwiGlu::backward (src/ffn.rs:87-120) on the way out: the product rows are the
                        // gradient of the hidden rows; with the gate and up pre-activations G | U of
                        // the forward pass, dG = dH * U * silu'(G) and dU = dH * silu(G) go to `gu_out`
                        // (both [rows, 2 N]) and the hidden gradient itself is never stored.
                        const size_t off = (size_t)(row0 + r) * 2 * N + col0 + 8 * p;
                        // (read once: fetched past the caches)
                        typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
                        const u32x4_t g8 = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(bw_gu + off));
                        const u32x4_t u8 = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(bw_gu + off + N));
                        const uint32_t hw[4] = {v.x, v.y, v.z, v.w}, gw[4] = {g8.x, g8.y, g8.z, g8.w},
                                       uw[4] = {u8.x, u8.y, u8.z, u8.w};
                        uint32_t dg[4], du[4];
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            float dgv[2], duv[2];
#pragma unroll
                            for (int h = 0; h < 2; ++h) {
                                const float dh = __uint_as_float(h ? hw[q] & 0xffff0000u : hw[q] << 16);
                                const float gv = __uint_as_float(h ? gw[q] & 0xffff0000u : gw[q] << 16);
                                const float uv = __uint_as_float(h ? uw[q] & 0xffff0000u : uw[q] << 16);
                                const float sg = __builtin_amdgcn_rcpf(
                                    1.0f + __builtin_amdgcn_exp2f(gv * -1.44269504088896340736f));
                                dgv[h] = dh * uv * (sg * (1.0f + gv * (1.0f - sg)));  // silu', src/ffn.rs:235-238
                                duv[h] = dh * (gv * sg);
                            }
                            dg[q] = pack2(dgv[0], dgv[1]);
                            du[q] = pack2(duv[0], duv[1]);
                        }
                        *reinterpret_cast<uint4*>(gu_out + off) = make_uint4(dg[0], dg[1], dg[2], dg[3]);
                        *reinterpret_cast<uint4*>(gu_out + off + N) = make_uint4(du[0], du[1], du[2], du[3]);
                        continue;
                    }
                }
                uint4* const where = reinterpret_cast<uint4*>(dst + (size_t)(row0 + r) * dstride + col0 + 8 * p);
                if (SWIGLU && b > 0) {
                    // the pre-activations are not read again before the backward pass: stored past the caches,
                    // so that they do not push the hidden rows out before the down product reads them
                    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
                    __builtin_nontemporal_store(u32x4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<u32x4_t*>(where));
                } else {
                    *where = v;
                }
            }
        }
    }
}

// ---- the pipelined main loop: one memory instruction behind each multiply -------------------------
// A wave issues in order, and while it issues a vector-memory or LDS instruction it issues no multiply: with
// the loads of a step in one cluster in front of its eight multiplies the matrix core runs dry for the
// length of the cluster unless another wave of the SIMD fills in - a wave that is alone on its SIMD (the
// last round of a launch, the partner in its prologue or epilogue) reaches 64 % of the multiply rate that
// way.  Here every multiply is followed by at most one or two of them, in an order pinned by scheduling
// barriers, and the slice boundary has no cluster either: three LDS stages, and the workgroup barrier sits
// behind step KS - 2 of a slice, so that the last step of a slice can already read the first fragments of
// the next slice and issue the DMA of the slice after that into the stage the barrier has just proven free.
//   steps 0 .. KS-2 of slice k:  ring loads of step g + D, fragments of step g + 1 (stage k % 3)
//   then: wait for this wave's DMA of slice k + 1 (issued a slice ago), barrier
//   step KS-1:                   ring loads, DMA of slice k + 2 (into stage (k + 2) % 3, last read in
//                                slice k - 1), fragments of step 0 of slice k + 1 (stage (k + 1) % 3)
// Vector-memory issue order inside a step: ring f0, ring f1, then the DMA instructions.  Younger than the
// ring loads of step g when step g waits for them (they were issued in step g - D, D = 3): the DMA of that
// step if it was a last step, then two ring loads per step in between and four DMA if one of them was a last
// step - 8 in all for the steps 0 .. KS-2 of a slice, 4 for the last one.
struct PipeCtx {
    const uint4* As;      // three LDS stages of one activation slice each
    uint32_t lds0;        // LDS byte address of this wave's rows in stage 0
    const char* a_base;   // activation rows (DMA source), byte offsets in a_src
    const char* wp0;      // this wave's two blocks of packed weight rows
    const char* wp1;
    uint32_t lane16;
    int lrow, lhalf, lxor;
    int KT;               // slices of the reduction
};

// Before the call: the DMA of slices 0 and 1 (stages 0 and 1) and the ring loads of steps 0 .. D-1 have been issued
// and have landed, and the workgroup has met at a barrier.  After it: nothing is outstanding; every wave may
// still be reading the stages until the next barrier.
template <bool I8, int NB>
__device__ __forceinline__ void pipe_loop(const PipeCtx& c, floatx16 (&acc)[2][TT], Slot<I8> (&ring)[KS],
                                          const uint32_t (&a_src)[DMA_PER_WAVE]) {
    constexpr int D = RING - 1;
    static_assert(KS == 4 && D == 3, "the wait counts below are derived for this configuration");
    const uint4* const As = c.As;
    const uint32_t lds0 = c.lds0, lane16 = c.lane16;
    const char* const a_base = c.a_base;
    const char* const wp0 = c.wp0;
    const char* const wp1 = c.wp1;
    const int lrow = c.lrow, lhalf = c.lhalf, lxor = c.lxor, KT = c.KT;
    const int GS = KT * KS;
    // The fragment of token block t for the step at position p of a slice sits at piece (2 p + lhalf) ^ lxor of
    // row t * 32 + lrow, i.e. at index t * 32 * CPR + (frag0 ^ 2 p): one register and an exclusive-or per step.
    // (Re-read through an empty statement per slice: four precomputed addresses would cost three registers.)
    static_assert(CPR == 8, "piece index = low three bits of the fragment index");
    int frag0 = lrow * CPR + (lhalf ^ lxor);
    bf16x8 tf[2][TT];
#pragma unroll
    for (int t = 0; t < NB; ++t) tf[0][t] = lds_frag(As, t * 32 * CPR + frag0);
    auto pslice = [&](int kt, auto idx_tag) {
        constexpr int IDX = decltype(idx_tag)::value;
        constexpr int BUF = IDX % 3, NEXT = (IDX + 1) % 3, FREE = (IDX + 2) % 3;
        const uint4* const Ab = As + BUF * (BM * CPR);
        const uint4* const An = As + NEXT * (BM * CPR);
        asm volatile("" : "+v"(frag0));
        static_for<0, KS>([&](auto s_tag) {
            constexpr int s = decltype(s_tag)::value;
            constexpr bool LAST = s == KS - 1;
            const int g = kt * KS + s;
            Slot<I8>& cur = ring[s % RING];
            Slot<I8>& nxt = ring[(s + D) % RING];
            wait_for<LAST ? 2 * (D - 1) : 2 * (D - 1) + DMA_PER_WAVE>(cur.f0, cur.f1);
            const bf16x8 w0 = cur.a0();
            const bf16x8 w1 = cur.a1();
            const uint32_t woff = Slot<I8>::offset(min(g + D, GS - 1), lane16);
            const uint32_t aoff = (uint32_t)min(kt + 2, KT - 1) * (BK * 2);
            const int frag = frag0 ^ (2 * ((s + 1) % KS));
            // memory instruction number i of the step
            constexpr int NOPS = 2 + ((LAST && DMA_PER_WAVE > NB) ? DMA_PER_WAVE : NB);
            auto op = [&](auto i_tag) {
                constexpr int i = decltype(i_tag)::value;
                if constexpr (i == 0) {
                    nxt.load0(wp0, woff);
                } else if constexpr (i == 1) {
                    nxt.load1(wp1, woff);
                } else {
                    constexpr int j = i - 2;
                    if constexpr (LAST && j < DMA_PER_WAVE)
                        issue_dma(lds0 + FREE * (BM * CPR * 16) + j * 8 * CPR * 16, a_src[j] + aoff, a_base);
                    if constexpr (j < NB)
                        tf[(s + 1) & 1][j] = lds_frag(LAST ? An : Ab, j * 32 * CPR + frag);
                }
            };
            static_for<0, 2 * NB>([&](auto m_tag) {
                constexpr int m = decltype(m_tag)::value;
                constexpr int b = m & 1, t = m >> 1;
                acc[b][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b ? w1 : w0, tf[s & 1][t], acc[b][t], 0, 0, 0);
                if constexpr (m < NOPS) op(m_tag);
                __builtin_amdgcn_sched_barrier(0);
            });
            static_for<2 * NB, NOPS>(op);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (s == KS - 2) {
                // this wave's DMA of the next slice (issued in the last step of the slice before this
                // one) is older than the 2 * (KS - 1) ring loads of this slice so far
                wait_outstanding<2 * (KS - 1)>();
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
        });
    };
    int kt = 0;
    for (; kt + 3 <= KT; kt += 3)
        static_for<0, 3>([&](auto i) { pslice(kt + decltype(i)::value, i); });
    static_while<0, 2>([&](auto i) {
        if (kt + decltype(i)::value >= KT) return false;
        pslice(kt + decltype(i)::value, i);
        return true;
    });
    wait_outstanding<0>();
    auto& ring_ref = ring;
#pragma unroll
    for (int i = 0; i < RING; ++i) asm volatile("" : : "v"(ring_ref[i].f0), "v"(ring_ref[i].f1));
}

template <bool SWIGLU, bool I8>
__global__ __launch_bounds__(NT, RBMOE_STREAM_OCC) void grouped_stream_kernel(
    const bf16_t* __restrict__ a, const int* __restrict__ row_index, const void* __restrict__ wpacked,
    size_t w_expert_stride_bytes, const float* __restrict__ scales, size_t s_expert_stride, int N, int K,
    const int* __restrict__ tile_expert, const int* __restrict__ tile_row0, const int* __restrict__ tile_rows,
    const int* __restrict__ ntiles, int dense_rows, bf16_t* __restrict__ out, bf16_t* __restrict__ gu_out,
    const bf16_t* __restrict__ bw_gu,
    int group_m) {
    constexpr int BN = SWIGLU ? NW * 32 : NW * 64;  // output features per workgroup
    // LDS stages of one activation slice each; the epilogue reuses the first two as one
    // 128 x 128 staging tile for the output.
    __shared__ uint4 As[STAGES * BM * CPR];

    // ---- which tile (each XCD walks a contiguous range, M fastest inside a group)
    const int tiles_n = (N + BN - 1) / BN;
    const int tiles_m = dense_rows >= 0 ? (dense_rows + BM - 1) / BM : *ntiles;
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int local = blockIdx.x >> 3;
    if (local >= per_xcd) return;
    const int pid = (blockIdx.x & 7) * per_xcd + local;
    if (pid >= total) return;
    const int per_group = group_m * tiles_n;
    const int grp = pid / per_group;
    const int first_m = grp * group_m;
    const int gsize = min(group_m, tiles_m - first_m);
    const int in_g = pid - grp * per_group;
    const int tm_idx = first_m + in_g % gsize;
    const int tn_idx = in_g / gsize;

    RBMOE_TRACE_AT(blockIdx.x, 0);
    int expert, row0, rows;
    if (dense_rows >= 0) {
        expert = 0;
        row0 = tm_idx * BM;
        rows = min(BM, dense_rows - row0);
    } else {
        expert = tile_expert[tm_idx];
        row0 = tile_row0[tm_idx];
        rows = tile_rows[tm_idx];
    }
    const int nblk = (rows + 31) >> 5;  // token blocks that hold at least one row

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- this wave's two blocks of 32 weight rows ---------------------------
    // A wave whose rows lie past N (ragged last feature tile) runs the same loop on row
    // block 0, so that every wave issues the same loads and meets the same barriers; it
    // stores nothing.
    // gate/up: gate rows nw .. nw + 31 and the matching up rows; down: rows nw .. nw + 31 and
    // the rows 128 further on, so that each block index covers 128 consecutive features of
    // the workgroup's tile.
    const int nw = tn_idx * BN + wave * 32;
    const int r0 = nw, r1 = SWIGLU ? N + nw : nw + NW * 32;
    const bool act0 = nw < N;
    const bool act1 = SWIGLU ? act0 : (nw + NW * 32 < N);
    const size_t block_bytes = (size_t)K * 32 * (I8 ? 1 : 2);  // one block of 32 weight rows over all of K
    const char* wexp = static_cast<const char*>(wpacked) + (size_t)expert * w_expert_stride_bytes;
    const char* wp0 = wexp + (size_t)(act0 ? r0 / 32 : 0) * block_bytes;
    const char* wp1 = wexp + (size_t)(act1 ? r1 / 32 : 0) * block_bytes;
    const uint32_t lane16 = (uint32_t)lane * 16u;

    // ---- LDS-DMA of the activation slice --------------------------------------
    // Wave w fills LDS rows [32 w, 32 w + 32): instruction j covers rows 32 w + 8 j .. + 7,
    // lane l lands in row 8 j + l / 8 (of the wave's 32), position l % 8, and therefore
    // fetches logical piece (l % 8) ^ ((row / 2) % 8): a 16-lane group of a fragment read
    // (16 consecutive rows, one logical piece) then touches 8 distinct pieces in the even rows
    // and 8 in the odd rows, i.e. all 64 banks once.  Rows past the end of the group are
    // clamped to the tile's first row: their products are never stored.
    // Byte offsets from `a` fit 32 bits (the launcher checks rows * K * 2 < 4 GiB).
    const char* const a_base = reinterpret_cast<const char*>(a);
    uint32_t a_src[DMA_PER_WAVE];
#pragma unroll
    for (int j = 0; j < DMA_PER_WAVE; ++j) {
        const int r = wave * (BM / NW) + j * 8 + (lane >> 3);
        const int rr = r < rows ? r : 0;
        const int grow = row_index ? row_index[row0 + rr] : row0 + rr;
        a_src[j] = ((uint32_t)grow * (uint32_t)K + 8u * ((lane & 7) ^ ((r >> 1) & 7))) * 2u;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)As + wave * (BM / NW) * CPR * 16;
    auto dma_a = [&](int kt, auto buf_tag) {
        constexpr int BUF = decltype(buf_tag)::value;
#pragma unroll
        for (int j = 0; j < DMA_PER_WAVE; ++j)
            issue_dma(lds0 + BUF * (BM * CPR * 16) + j * 8 * CPR * 16, a_src[j] + (uint32_t)kt * (BK * 2), a_base);
    };

    floatx16 acc[2][TT];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[b][t][v] = 0.0f;

    const int lrow = lane & 31;
    const int lhalf = lane >> 5;
    const int lxor = (lrow >> 1) & 7;

    const int KT = K / BK;
    const int GS = KT * KS;  // reduction steps in all
    constexpr int D = RING - 1;  // the load for step g + D is issued while step g runs

    // ---- prologue: the first STAGES - 1 activation slices, the first D weight steps; nothing is in flight
    // where the loop is entered (the compiler may copy registers there)
    Slot<I8> ring[RING];
    static_for<0, STAGES - 1>([&](auto st) { dma_a(min((int)decltype(st)::value, KT - 1), st); });
#pragma unroll
    for (int g = 0; g < D; ++g) ring[g].load(wp0, wp1, min(g, GS - 1), lane16);
    wait_outstanding<0>();
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    RBMOE_TRACE_AT(blockIdx.x, 1);

    // The loop is specialised at compile time for the number of token blocks that hold rows: a run-time branch per
    // block between the multiplies costs far more than the skipped multiplies save.
    {
        const PipeCtx pc{As, lds0, a_base, wp0, wp1, lane16, lrow, lhalf, lxor, KT};
        static_assert(TT >= 2 && TT <= 4, "one specialisation per possible block count");
        if (TT >= 4 && nblk >= 4) pipe_loop<I8, (TT >= 4 ? 4 : TT)>(pc, acc, ring, a_src);
        else if (TT >= 3 && nblk == 3) pipe_loop<I8, (TT >= 3 ? 3 : TT)>(pc, acc, ring, a_src);
        else if (nblk == 2) pipe_loop<I8, 2>(pc, acc, ring, a_src);
        else pipe_loop<I8, 1>(pc, acc, ring, a_src);
    }
    RBMOE_TRACE_AT(blockIdx.x, 2);
    // ---- epilogue -------------------------------------------------------------
    __syncthreads();  // every wave's last DMA has landed and its last fragment reads are done
    const TileOut to{rows, row0, tn_idx, N, act0, act1, r0, r1, I8 ? scales + (size_t)expert * s_expert_stride : nullptr,
                     out, gu_out, bw_gu};
    write_tile<SWIGLU, I8>(to, acc, reinterpret_cast<char*>(As), [] {});
    RBMOE_TRACE_AT(blockIdx.x, 3);
}

template <bool SWIGLU, bool I8>
hipError_t launch_t(const GroupedArgs& g, hipStream_t s) {
    constexpr int BN = SWIGLU ? NW * 32 : NW * 64;
    const int tiles_n = (g.N + BN - 1) / BN;
    const int tiles_m = g.dense_rows >= 0 ? (g.dense_rows + BM - 1) / BM : g.max_tiles;
    if (tiles_m <= 0) return hipSuccess;
    const int total = tiles_m * tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    RB_LAUNCH((grouped_stream_kernel<SWIGLU, I8>), dim3(grid), dim3(NT), 0, s,
                       static_cast<const bf16_t*>(g.a), g.row_index, g.w, g.w_expert_stride * (I8 ? 1 : 2), g.scales,
                       g.s_expert_stride, g.N, g.K, g.tile_expert, g.tile_row0, g.tile_rows, g.ntiles, g.dense_rows,
                       static_cast<bf16_t*>(g.out), static_cast<bf16_t*>(g.gu_out), static_cast<const bf16_t*>(g.swiglu_grad_gu),
                       g.group_m > 0 ? g.group_m : 8);
    return hipGetLastError();
}


}  // namespace

int stream_tile_m() { return BM; }

// K a multiple of 64 (one LDS slice), N a multiple of 32 (row blocks of the packed weights)
bool stream_shape_ok(int N, int K) { return K % 64 == 0 && K >= 64 && N % 32 == 0 && N >= 32; }

hipError_t launch_grouped_stream(const GroupedArgs& g, WeightKind wk, hipStream_t s) {
    if (!stream_shape_ok(g.N, g.K)) return hipErrorInvalidValue;
    if (wk == WeightKind::BF16) return g.swiglu ? launch_t<true, false>(g, s) : launch_t<false, false>(g, s);
    if (wk == WeightKind::I8) return g.swiglu ? launch_t<true, true>(g, s) : launch_t<false, true>(g, s);
    return hipErrorInvalidValue;
}

// Host-side repacking of one [rows, cols] weight matrix into fragment order.
// bf16: [rows/32][cols/16][64 lanes][8]; lane l holds row (l % 32), columns 16*s + 8*(l/32) + 0..7.
void pack_weight_bf16(const uint16_t* src, int rows, int cols, uint16_t* dst) {
    const int KS16 = cols / 16;
    for (int nb = 0; nb < rows / 32; ++nb)
        for (int s = 0; s < KS16; ++s)
            for (int l = 0; l < 64; ++l) {
                const uint16_t* p = src + (size_t)(nb * 32 + l % 32) * cols + 16 * s + 8 * (l / 32);
                uint16_t* q = dst + (((size_t)nb * KS16 + s) * 64 + l) * 8;
                for (int j = 0; j < 8; ++j) q[j] = p[j];
            }
}

// int8: [rows/32][cols/32][64 lanes][16]; bytes 0..7 are the lane's piece of step 2s, bytes 8..15 of step 2s+1.
void pack_weight_i8(const int8_t* src, int rows, int cols, int8_t* dst) {
    const int KS32 = cols / 32;
    for (int nb = 0; nb < rows / 32; ++nb)
        for (int s = 0; s < KS32; ++s)
            for (int l = 0; l < 64; ++l) {
                const int8_t* p = src + (size_t)(nb * 32 + l % 32) * cols + 32 * s + 8 * (l / 32);
                int8_t* q = dst + (((size_t)nb * KS32 + s) * 64 + l) * 16;
                for (int j = 0; j < 8; ++j) {
                    q[j] = p[j];
                    q[8 + j] = p[16 + j];
                }
            }
}

}  // namespace rbmoe
