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
//                which global piece each lane fetches.  Two LDS stages; the DMA
//                for slice k + 1 is issued when slice k starts and is awaited
//                (vmcnt) just before the barrier that ends slice k.
//   fragments    token fragments are read from LDS one step ahead of the
//                multiplies that use them.
// A workgroup is 4 waves side by side along the output features; a wave owns
// 128 tokens x 64 weight rows (32 gate + the matching 32 up rows, or 64 down
// rows).  The weight fragment is the matrix-core A operand and the token
// fragment the B operand, so a lane ends with 4 consecutive output features of
// one token and writes them with one 8-byte store.  Token blocks of 32 rows
// that lie beyond the end of a group are skipped, so a ragged group costs at
// most 31 rows of padding.
#include <type_traits>

#include "rbmoe_kernels.h"

namespace rbmoe {

namespace {

constexpr int BM = 128;   // token rows per workgroup
constexpr int BK = 64;    // reduction slice held in one LDS stage
constexpr int NW = 4;     // waves per workgroup
constexpr int NT = NW * 64;
constexpr int CPR = BK / 8;            // 16-byte pieces per LDS row
constexpr int TT = BM / 32;            // token blocks per wave
constexpr int KS = BK / 16;            // matrix-core steps per slice
constexpr int DMA_PER_WAVE = BM * CPR / 64 / NW;  // LDS-DMA instructions per wave per slice (4)

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
    __device__ __forceinline__ bf16x8 a0() const { return widen_i8(make_uint2(f0.x, f0.y)); }
    __device__ __forceinline__ bf16x8 a1() const { return widen_i8(make_uint2(f1.x, f1.y)); }
};

// RING = weight-fragment steps in flight per wave (register ring depth);
// TFBUF = 2: token fragments are read from LDS one step ahead, 1: just in time.
template <bool SWIGLU, bool I8, int RING, int TFBUF, bool AREG>
__global__ __launch_bounds__(NT, 2) void grouped_stream_kernel(
    const bf16_t* __restrict__ a, const int* __restrict__ row_index, const void* __restrict__ wpacked,
    size_t w_expert_stride_bytes, const float* __restrict__ scales, size_t s_expert_stride, int N, int K,
    const int* __restrict__ tile_expert, const int* __restrict__ tile_row0, const int* __restrict__ tile_rows,
    const int* __restrict__ ntiles, int dense_rows, bf16_t* __restrict__ out, bf16_t* __restrict__ gu_out,
    const bf16_t* __restrict__ bw_gu,
    int group_m) {
    constexpr int BN = SWIGLU ? NW * 32 : NW * 64;  // output features per workgroup
    // Two LDS stages of one activation slice each; the epilogue reuses both as one
    // 128 x 128 staging tile for the output.
    __shared__ uint4 As[2 * BM * CPR];
    uint4* const As0 = As;
    uint4* const As1 = As + BM * CPR;

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
        const int r = wave * 32 + j * 8 + (lane >> 3);
        const int rr = r < rows ? r : 0;
        const int grow = row_index ? row_index[row0 + rr] : row0 + rr;
        a_src[j] = ((uint32_t)grow * (uint32_t)K + 8u * ((lane & 7) ^ ((r >> 1) & 7))) * 2u;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)As0 + wave * 32 * CPR * 16;
    const uint32_t lds1 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)As1 + wave * 32 * CPR * 16;
    auto dma_a = [&](int kt, auto buf_tag) {
        constexpr int BUF = decltype(buf_tag)::value;
#pragma unroll
        for (int j = 0; j < DMA_PER_WAVE; ++j)
            issue_dma((BUF ? lds1 : lds0) + j * 8 * CPR * 16, a_src[j] + (uint32_t)kt * (BK * 2), a_base);
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

    // ---- prologue: first activation slice, first D weight steps -----------------
    // AREG: the activation slice travels global -> VGPR -> LDS instead of by LDS-DMA, one
    // 1 KB piece per wave per step: piece j of slice k + 2 is fetched in step j of slice k and
    // written to LDS in step j of slice k + 1 (into the stage slice k read).  Slices 0 and 1
    // are placed by the prologue, so that no load is in flight where the loop is entered
    // (the compiler may copy registers there); the first slice's writes go to a spare row.
    u32x4 areg[DMA_PER_WAVE];
    uint4* const a_dst0 = As0 + (wave * 32) * CPR + lane;
    uint4* const a_dst1 = As1 + (wave * 32) * CPR + lane;
    __shared__ uint4 spare[AREG ? NT : 1];
    Slot<I8> ring[RING];
    if constexpr (AREG) {
        u32x4 first[DMA_PER_WAVE];
#pragma unroll
        for (int j = 0; j < DMA_PER_WAVE; ++j) issue_load(first[j], a_src[j], a_base);
#pragma unroll
        for (int j = 0; j < DMA_PER_WAVE; ++j)
            issue_load(areg[j], a_src[j] + (uint32_t)min(1, KT - 1) * (BK * 2), a_base);
#pragma unroll
        for (int g = 0; g < D; ++g) ring[g].load(wp0, wp1, min(g, GS - 1), lane16);
        wait_outstanding<0>();
#pragma unroll
        for (int j = 0; j < DMA_PER_WAVE; ++j) {
            asm volatile("" : "+v"(first[j]), "+v"(areg[j]));
            a_dst0[j * 8 * CPR] = make_uint4(first[j].x, first[j].y, first[j].z, first[j].w);
            a_dst1[j * 8 * CPR] = make_uint4(areg[j].x, areg[j].y, areg[j].z, areg[j].w);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
    } else {
        dma_a(0, std::integral_constant<int, 0>{});
#pragma unroll
        for (int g = 0; g < D; ++g) ring[g].load(wp0, wp1, min(g, GS - 1), lane16);
        wait_outstanding<0>();
    }
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);

    // One slice = KS steps.  BUF is the LDS stage the slice reads (its parity); the ring
    // position of the slice's first step is 0, or BUF * KS when the ring holds two slices.
    // NB = token blocks of this tile that hold rows, a compile-time constant inside the
    // loop: a run-time branch per block between the multiplies costs far more than the
    // skipped multiplies save, so the whole loop is specialised instead.
    // The loop is straight-line and every wave issues, per slice, exactly: 4 DMA
    // instructions, then 2 weight loads in each of the KS steps.  Past the end the last
    // slice / step is fetched again, so that the counts below hold everywhere.
    auto slice = [&](int kt, auto buf_tag, auto nb_tag) {
        constexpr int BUF = decltype(buf_tag)::value;
        constexpr int G0 = RING == 2 * KS ? BUF * KS : 0;
        constexpr int NB = decltype(nb_tag)::value;
        if constexpr (!AREG) dma_a(min(kt + 1, KT - 1), std::integral_constant<int, BUF ^ 1>{});
        const uint4* Ab = BUF ? As1 : As0;
        bf16x8 tf[TFBUF][TT];
#pragma unroll
        for (int t = 0; t < NB; ++t) tf[0][t] = lds_frag(Ab, (t * 32 + lrow) * CPR + (lhalf ^ lxor));
        static_for<0, KS>([&](auto s_tag) {
            constexpr int s = decltype(s_tag)::value;
            const int g = kt * KS + s;
            Slot<I8>& cur = ring[(G0 + s) % RING];
            // weight fragments for step g + D go into the slot step g - 1 released
            ring[(G0 + s + D) % RING].load(wp0, wp1, min(g + D, GS - 1), lane16);
            if constexpr (TFBUF == 2) {
                if (s + 1 < KS) {
                    const int piece = (2 * (s + 1) + lhalf) ^ lxor;
#pragma unroll
                    for (int t = 0; t < NB; ++t) tf[(s + 1) & 1][t] = lds_frag(Ab, (t * 32 + lrow) * CPR + piece);
                }
            } else if (s > 0) {
                const int piece = (2 * s + lhalf) ^ lxor;
#pragma unroll
                for (int t = 0; t < NB; ++t) tf[0][t] = lds_frag(Ab, (t * 32 + lrow) * CPR + piece);
            }
            if constexpr (AREG) {
                // Per step: 2 weight loads, then 1 activation load.  Younger than the weight loads
                // of step g: 3 per step for D steps.  The activation piece this step writes to LDS
                // was fetched a whole slice ago, i.e. is older still.
                static_assert(KS == DMA_PER_WAVE && D <= KS, "one activation piece per step, fetched KS steps before use");
                wait_for<3 * D>(cur.f0, cur.f1);
                asm volatile("" : "+v"(areg[s]));
                uint4* const dst = kt > 0 ? (BUF ? a_dst0 : a_dst1) + s * 8 * CPR : spare + tid;
                *dst = make_uint4(areg[s].x, areg[s].y, areg[s].z, areg[s].w);
                issue_load(areg[s], a_src[s] + (uint32_t)min(kt + 2, KT - 1) * (BK * 2), a_base);
            } else {
                // Younger than the loads of step g: the weight loads of steps g+1 .. g+D (2 each)
                // and the DMA (4) of every slice that started after they were issued.
                wait_for<2 * D + DMA_PER_WAVE * ((D - s + KS - 1) / KS)>(cur.f0, cur.f1);
            }
            const bf16x8 w0 = cur.a0();
            const bf16x8 w1 = cur.a1();
#pragma unroll
            for (int t = 0; t < NB; ++t) {
                acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w0, tf[s % TFBUF][t], acc[0][t], 0, 0, 0);
                acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w1, tf[s % TFBUF][t], acc[1][t], 0, 0, 0);
            }
        });
        // Every LDS read of this slice has been consumed by a multiply issued above this
        // point.  The DMA of the next slice is older than this slice's 2 * KS weight loads.
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (AREG)
            asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");  // this wave's pieces of the next slice are in LDS
        else
            wait_outstanding<2 * KS>();
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };

    static_assert(RING == KS || RING == 2 * KS, "ring depth is one or two slices");
    static_assert(DMA_PER_WAVE == 4, "the wait counts assume 4 DMA instructions per wave per slice");
    auto run = [&](auto nb_tag) {
        int kt = 0;
        for (; kt + 1 < KT; kt += 2) {
            slice(kt, std::integral_constant<int, 0>{}, nb_tag);
            slice(kt + 1, std::integral_constant<int, 1>{}, nb_tag);
        }
        if (kt < KT) slice(kt, std::integral_constant<int, 0>{}, nb_tag);
        // The loads fetched again past the end still target ring registers and LDS.  Naming
        // the registers after the wait keeps them allocated until their data has arrived: a
        // loaded value the compiler sees no use for would otherwise hand its register to
        // something live while the load is still in flight.  (Done here, inside each
        // specialisation, so that no path leaves it with loads outstanding.)
        wait_outstanding<0>();
        auto& ring_ref = ring;
        auto& areg_ref = areg;
#pragma unroll
        for (int i = 0; i < RING; ++i) asm volatile("" : : "v"(ring_ref[i].f0), "v"(ring_ref[i].f1));
#pragma unroll
        for (int j = 0; j < DMA_PER_WAVE; ++j) asm volatile("" : : "v"(areg_ref[j]));
    };
    static_assert(TT == 4, "one specialisation per possible block count");
    if (nblk == 4) run(std::integral_constant<int, 4>{});
    else if (nblk == 3) run(std::integral_constant<int, 3>{});
    else if (nblk == 2) run(std::integral_constant<int, 2>{});
    else run(std::integral_constant<int, 1>{});
    // ---- epilogue -------------------------------------------------------------
    // Accumulator element v of block (b, t): feature 8*(v/4) + 4*(lane/32) + v%4 of the
    // wave's row block b, token t*32 + lane%32 - a lane holds 4 consecutive features of a
    // token, so a direct store would scatter 8-byte pieces over 32 rows per instruction.
    // Instead each block index goes through LDS as a 128-token x 128-feature tile (16-byte
    // pieces, piece p of row r kept at position p ^ (r % 16)), and is written out with
    // 16-byte stores, 16 consecutive lanes covering the 256 contiguous bytes of a row.
    const float* sc = I8 ? scales + (size_t)expert * s_expert_stride : nullptr;
    char* const stage = reinterpret_cast<char*>(As);
    // Passes through the staging tile: down product: the two blocks of 128 features; gate/up: the
    // hidden rows, then (only when the caller keeps them for a backward pass) the gate and the
    // up pre-activations, which go to `gu_out` [rows, 2N] with the gate half in columns [0, N).
    constexpr int PASSES = SWIGLU ? 3 : 2;
    __syncthreads();  // every wave's last DMA has landed and its last fragment reads are done
#pragma unroll
    for (int b = 0; b < PASSES; ++b) {
        if constexpr (SWIGLU) {
            if (b > 0 && gu_out == nullptr) break;  // uniform over the launch
        }
        if (b) __syncthreads();  // the previous pass has been read out
        if (SWIGLU ? act0 : (b ? act1 : act0)) {
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
                    const int piece = (wave * 4 + q) ^ (m & 15);
                    *reinterpret_cast<uint2*>(stage + m * 256 + piece * 16 + lhalf * 8) =
                        make_uint2(pack2(y[0], y[1]), pack2(y[2], y[3]));
                }
            }
        }
        __syncthreads();
        // where this pass goes: hidden rows and down rows into `out` (row stride N), the
        // pre-activations into `gu_out` (row stride 2 N)
        const int col0 = tn_idx * BN + (SWIGLU ? 0 : b * (NW * 32));
        bf16_t* const dst = (SWIGLU && b > 0) ? gu_out + (b == 2 ? N : 0) : out;
        const size_t dstride = (SWIGLU && b > 0) ? (size_t)2 * N : (size_t)N;
#pragma unroll
        for (int i = 0; i < BM * 16 / NT; ++i) {
            const int idx = i * NT + tid;
            const int r = idx >> 4, p = idx & 15;
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

template <bool SWIGLU, bool I8, int RING, int TFBUF, bool AREG>
hipError_t launch_t(const GroupedArgs& g, hipStream_t s) {
    constexpr int BN = SWIGLU ? NW * 32 : NW * 64;
    const int tiles_n = (g.N + BN - 1) / BN;
    const int tiles_m = g.dense_rows >= 0 ? (g.dense_rows + BM - 1) / BM : g.max_tiles;
    if (tiles_m <= 0) return hipSuccess;
    const int total = tiles_m * tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL((grouped_stream_kernel<SWIGLU, I8, RING, TFBUF, AREG>), dim3(grid), dim3(NT), 0, s,
                       static_cast<const bf16_t*>(g.a), g.row_index, g.w, g.w_expert_stride * (I8 ? 1 : 2), g.scales,
                       g.s_expert_stride, g.N, g.K, g.tile_expert, g.tile_row0, g.tile_rows, g.ntiles, g.dense_rows,
                       static_cast<bf16_t*>(g.out), static_cast<bf16_t*>(g.gu_out), static_cast<const bf16_t*>(g.swiglu_grad_gu),
                       g.group_m > 0 ? g.group_m : 4);
    return hipGetLastError();
}

}  // namespace

template <int RING, int TFBUF, bool AREG>
static hipError_t launch_ring(const GroupedArgs& g, WeightKind wk, hipStream_t s) {
    if (wk == WeightKind::BF16)
        return g.swiglu ? launch_t<true, false, RING, TFBUF, AREG>(g, s) : launch_t<false, false, RING, TFBUF, AREG>(g, s);
    if (wk == WeightKind::I8)
        return g.swiglu ? launch_t<true, true, RING, TFBUF, AREG>(g, s) : launch_t<false, true, RING, TFBUF, AREG>(g, s);
    return hipErrorInvalidValue;
}

// variant 0: ring of 4 steps, token fragments read one step ahead, activation slices by LDS-DMA
// variant 1: ring of 4 steps, token fragments read just in time, activation slices global -> VGPR -> LDS
int stream_tile_m() { return BM; }

// K a multiple of 64 (one LDS slice), N a multiple of 32 (row blocks of the packed weights)
bool stream_shape_ok(int N, int K) { return K % 64 == 0 && K >= 64 && N % 32 == 0 && N >= 32; }

hipError_t launch_grouped_stream(const GroupedArgs& g, WeightKind wk, int variant, hipStream_t s) {
    if (!stream_shape_ok(g.N, g.K)) return hipErrorInvalidValue;
    switch (variant) {
        case 0: return launch_ring<4, 2, false>(g, wk, s);
        case 1: return launch_ring<4, 1, true>(g, wk, s);
    }
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
