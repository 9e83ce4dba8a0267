// Grouped expert products on the bf16 matrix cores of gfx950.
//
//   out[row, n] = sum_c a[row, c] * w[expert][n, c]                 (down product)
//   out[row, n] = silu(a . wgate[n]) * (a . wup[n])                 (gate/up product)
//
// `a` rows and weight rows are both contiguous along the reduction dimension,
// which is exactly the operand layout of v_mfma_f32_32x32x16_bf16 (each lane
// feeds 8 consecutive bf16 of one row), so neither operand is transposed.
//
// One workgroup computes a BM x BN output tile of ONE expert (a tile never
// spans two experts; the tile table comes from the scan kernel), walking the
// reduction dimension in BK-wide slices that are double-buffered in LDS:
//   global -> registers (next slice) | LDS (current slice) -> MFMA | registers -> LDS
// LDS rows are stored with their 16-byte pieces XOR-swizzled by the row number,
// so both the 16-byte stores and the 16-byte fragment reads are bank-conflict
// free without padding.  For the gate/up product the B slice holds BN gate rows
// followed by the BN matching up rows; the two accumulators of one output
// element live in the same lane, so SwiGLU is applied in registers and only the
// hidden activations are written.  Rows of `a` may be fetched through an index
// (the token gather folded into the operand load).
// int8 weights are widened to bf16 (exactly) on their way into LDS and the
// per-row scale is applied to the accumulator, i.e. (sum a*q) * scale.
//
// Workgroup ids are remapped so that each XCD (ids congruent mod 8 share an
// XCD and its L2) walks a contiguous range of tiles, M-tiles innermost in
// groups, which keeps the weight slices of an expert resident in that L2.
#include "rbmoe_kernels.h"

namespace rbmoe {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

// One 16-byte LDS piece (8 bf16) from global memory.
template <typename WT>
struct Piece;
template <>
struct Piece<bf16_t> {
    typedef uint4 raw_t;  // 8 bf16
    static __device__ __forceinline__ uint4 widen(const raw_t& r) { return r; }
};
template <>
struct Piece<int8_t> {
    typedef uint2 raw_t;  // 8 int8
    static __device__ __forceinline__ uint32_t two(uint32_t word, int shift) {
        const float lo = (float)(int)(int8_t)(word >> shift);
        const float hi = (float)(int)(int8_t)(word >> (shift + 8));
        // small integers are exact in bf16: keep the upper halves
        return (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
    }
    static __device__ __forceinline__ uint4 widen(const raw_t& r) {
        return make_uint4(two(r.x, 0), two(r.x, 16), two(r.y, 0), two(r.y, 16));
    }
};

template <int BM, int BN, int BK, int WM, int WN, int OCC, bool SWIGLU, typename WT>
__global__ __launch_bounds__(WM* WN * 64, OCC) void grouped_mfma_kernel(
    const bf16_t* __restrict__ a, const int* __restrict__ row_index, const WT* __restrict__ w,
    size_t w_expert_stride, const float* __restrict__ scales, size_t s_expert_stride, int N, int K,
    const int* __restrict__ tile_expert, const int* __restrict__ tile_row0,
    const int* __restrict__ tile_rows, const int* __restrict__ ntiles, int dense_rows,
    bf16_t* __restrict__ out, int group_m) {
    constexpr int NT = WM * WN * 64;
    constexpr int NB = SWIGLU ? 2 * BN : BN;   // weight rows staged per slice
    constexpr int CPR = BK / 8;                // 16-byte pieces per LDS row
    constexpr int RP = CPR >= 8 ? 1 : 8 / CPR; // LDS rows per 128 bytes
    constexpr int A_CH = BM * CPR / NT;        // pieces per thread per slice
    constexpr int B_CH = NB * CPR / NT;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(BM * CPR % NT == 0 && NB * CPR % NT == 0, "slice must divide over the threads");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of 32x32");
    typedef typename Piece<WT>::raw_t braw_t;
    constexpr int WPP = 16 / (int)sizeof(braw_t);  // 1 for bf16, 2 for int8: raw pieces per 16 bytes of weights

    extern __shared__ uint4 lds[];
    uint4* As = lds;                     // [2][BM * CPR]
    uint4* Bs = lds + 2 * BM * CPR;      // [2][NB * CPR]

    // ---- which tile --------------------------------------------------------
    const int tiles_n = (N + BN - 1) / BN;
    const int tiles_m = dense_rows >= 0 ? (dense_rows + BM - 1) / BM : *ntiles;
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    const int local = blockIdx.x >> 3;
    if (local >= per_xcd) return;
    const int pid = (blockIdx.x & 7) * per_xcd + local;
    if (pid >= total) return;
    // groups of `group_m` M-tiles; inside a group the M index runs fastest
    const int per_group = group_m * tiles_n;
    const int g = pid / per_group;
    const int first_m = g * group_m;
    const int gsize = min(group_m, tiles_m - first_m);
    const int in_g = pid - g * per_group;
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
    const int n0 = tn_idx * BN;
    const WT* wbase = w + (size_t)expert * w_expert_stride;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    // ---- global offsets (in pieces) of this thread's pieces -----------------
    const uint4* a_pieces = reinterpret_cast<const uint4*>(a);
    const braw_t* b_pieces = reinterpret_cast<const braw_t*>(wbase);
    const int kp = K / 8;  // pieces per global row
    uint32_t a_off[A_CH];
    int a_lds[A_CH];
    uint32_t a_mask = 0;
#pragma unroll
    for (int j = 0; j < A_CH; ++j) {
        const int q = tid + j * NT;
        const int r = q / CPR, c = q % CPR;
        const bool ok = r < rows;
        int grow = 0;
        if (ok) grow = row_index ? row_index[row0 + r] : row0 + r;
        a_off[j] = (uint32_t)grow * (uint32_t)kp + c;
        a_lds[j] = r * CPR + (c ^ ((r / RP) % CPR));
        a_mask |= ok ? (1u << j) : 0u;
    }
    uint32_t b_off[B_CH];
    int b_lds[B_CH];
    uint32_t b_mask = 0;
#pragma unroll
    for (int j = 0; j < B_CH; ++j) {
        const int q = tid + j * NT;
        const int r = q / CPR, c = q % CPR;
        int n;  // weight row of the expert
        bool ok;
        if (SWIGLU) {
            const int h = r < BN ? r : r - BN;
            ok = n0 + h < N;
            n = (r < BN ? 0 : N) + n0 + h;
        } else {
            ok = n0 + r < N;
            n = n0 + r;
        }
        if (!ok) n = 0;
        b_off[j] = (uint32_t)n * (uint32_t)kp + c;
        b_lds[j] = r * CPR + (c ^ ((r / RP) % CPR));
        b_mask |= ok ? (1u << j) : 0u;
    }

    uint4 ra[A_CH];
    braw_t rb[B_CH];
    auto fetch = [&](int kt) {
#pragma unroll
        for (int j = 0; j < A_CH; ++j) {
            ra[j] = make_uint4(0, 0, 0, 0);
            if (a_mask & (1u << j)) ra[j] = a_pieces[a_off[j] + kt * CPR];
        }
#pragma unroll
        for (int j = 0; j < B_CH; ++j) {
            braw_t z = {};
            rb[j] = z;
            if (b_mask & (1u << j)) rb[j] = b_pieces[b_off[j] + kt * CPR];
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int j = 0; j < A_CH; ++j) As[buf * BM * CPR + a_lds[j]] = ra[j];
#pragma unroll
        for (int j = 0; j < B_CH; ++j) Bs[buf * NB * CPR + b_lds[j]] = Piece<WT>::widen(rb[j]);
    };
    (void)WPP;

    floatx16 accg[TM][TN];
    floatx16 accu[SWIGLU ? TM : 1][SWIGLU ? TN : 1];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                accg[i][j][v] = 0.0f;
                if constexpr (SWIGLU) accu[i][j][v] = 0.0f;
            }

    // fragment addressing: row = base + (lane & 31), piece = 2 * kk + (lane >> 5)
    const int lrow = lane & 31;
    const int lhalf = lane >> 5;
    const int lxor = (lrow / RP) % CPR;  // every base is a multiple of 32, so the swizzle term is per lane
    const int a_frag0 = (wm * WTM + lrow) * CPR;
    const int b_frag0 = (wn * WTN + lrow) * CPR;

    const int KT = K / BK;
    fetch(0);
    stage(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < KT) fetch(kt + 1);
        const uint4* Ab = As + buf * BM * CPR;
        const uint4* Bb = Bs + buf * NB * CPR;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            const int piece = (2 * kk + lhalf) ^ lxor;
            bf16x8 af[TM], bg[TN], bu[SWIGLU ? TN : 1];
#pragma unroll
            for (int i = 0; i < TM; ++i) af[i] = __builtin_bit_cast(bf16x8, Ab[a_frag0 + i * 32 * CPR + piece]);
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                bg[j] = __builtin_bit_cast(bf16x8, Bb[b_frag0 + j * 32 * CPR + piece]);
                if constexpr (SWIGLU) bu[j] = __builtin_bit_cast(bf16x8, Bb[b_frag0 + (BN + j * 32) * CPR + piece]);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    accg[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bg[j], accg[i][j], 0, 0, 0);
                    if constexpr (SWIGLU)
                        accu[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bu[j], accu[i][j], 0, 0, 0);
                }
        }
        if (kt + 1 < KT) stage(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue ----------------------------------------------------------
    // accumulator element v of a 32x32 block: row 8*(v/4) + 4*(lane/32) + v%4, column lane%32
    const float* sc = scales ? scales + (size_t)expert * s_expert_stride : nullptr;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn * WTN + j * 32 + lrow;
        const bool n_ok = n < N;
        float sg = 1.0f, su = 1.0f;
        if (sc && n_ok) {
            sg = sc[n];
            if (SWIGLU) su = sc[N + n];
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = wm * WTM + i * 32 + 8 * (v / 4) + 4 * lhalf + (v % 4);
                if (m < rows && n_ok) {
                    float val = accg[i][j][v] * sg;
                    if constexpr (SWIGLU) val = silu_f32(val) * (accu[i][j][v] * su);
                    out[(size_t)(row0 + m) * N + n] = bf16_t{f32_to_bf16_bits(val)};
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// configurations
// ---------------------------------------------------------------------------
template <int BM, int BN, int BK, int WM, int WN, int OCC, bool SWIGLU, typename WT>
static hipError_t launch_cfg(const GroupedArgs& g, hipStream_t s) {
    constexpr int NB = SWIGLU ? 2 * BN : BN;
    constexpr size_t lds_bytes = (size_t)2 * (BM + NB) * BK * 2;
    auto kern = grouped_mfma_kernel<BM, BN, BK, WM, WN, OCC, SWIGLU, WT>;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles_n = (g.N + BN - 1) / BN;
    const int tiles_m = g.dense_rows >= 0 ? (g.dense_rows + BM - 1) / BM : g.max_tiles;
    if (tiles_m <= 0) return hipSuccess;
    const int total = tiles_m * tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WM * WN * 64), lds_bytes, s, static_cast<const bf16_t*>(g.a),
                       g.row_index, static_cast<const WT*>(g.w), g.w_expert_stride, g.scales, g.s_expert_stride,
                       g.N, g.K, g.tile_expert, g.tile_row0, g.tile_rows, g.ntiles, g.dense_rows,
                       static_cast<bf16_t*>(g.out), g.group_m > 0 ? g.group_m : 4);
    return hipGetLastError();
}

template <typename WT>
static hipError_t launch_wt(const GroupedArgs& g, int cfg, hipStream_t s) {
    if (g.swiglu) {
        switch (cfg) {
            case 0: return launch_cfg<128, 128, 32, 2, 2, 2, true, WT>(g, s);
            case 1: return launch_cfg<128, 128, 64, 2, 2, 1, true, WT>(g, s);
            case 2: return launch_cfg<128, 64, 64, 2, 2, 2, true, WT>(g, s);
            case 3: return launch_cfg<64, 128, 64, 2, 2, 2, true, WT>(g, s);
            case 4: return launch_cfg<256, 128, 32, 2, 2, 1, true, WT>(g, s);
            case 5: return launch_cfg<128, 256, 32, 1, 4, 1, true, WT>(g, s);
            case 6: return launch_cfg<64, 64, 64, 2, 2, 2, true, WT>(g, s);
        }
    } else {
        switch (cfg) {
            case 0: return launch_cfg<128, 128, 32, 2, 2, 2, false, WT>(g, s);
            case 1: return launch_cfg<128, 128, 64, 2, 2, 1, false, WT>(g, s);
            case 2: return launch_cfg<128, 256, 64, 2, 2, 1, false, WT>(g, s);
            case 3: return launch_cfg<64, 128, 64, 2, 2, 2, false, WT>(g, s);
            case 4: return launch_cfg<256, 256, 32, 2, 2, 1, false, WT>(g, s);
            case 5: return launch_cfg<128, 256, 32, 2, 2, 2, false, WT>(g, s);
            case 6: return launch_cfg<64, 64, 64, 2, 2, 2, false, WT>(g, s);
        }
    }
    return hipErrorInvalidValue;
}

int mfma_tile_m(bool swiglu, int cfg) {
    static const int gu[] = {128, 128, 128, 64, 256, 128, 64};
    static const int dn[] = {128, 128, 128, 64, 256, 128, 64};
    if (cfg < 0 || cfg >= kNumMfmaConfigs) return -1;
    return swiglu ? gu[cfg] : dn[cfg];
}

bool mfma_shape_ok(int K) { return K % 64 == 0 && K >= 64; }

hipError_t launch_grouped_mfma(const GroupedArgs& g, WeightKind wk, int cfg, hipStream_t s) {
    if (!mfma_shape_ok(g.K)) return hipErrorInvalidValue;
    switch (wk) {
        case WeightKind::BF16: return launch_wt<bf16_t>(g, cfg, s);
        case WeightKind::I8: return launch_wt<int8_t>(g, cfg, s);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace rbmoe
