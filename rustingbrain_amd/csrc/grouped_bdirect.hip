// Grouped expert products on the bf16 matrix cores of gfx950, weights streamed
// straight from HBM/L2 into the matrix-core operand registers.
//
//   out[row, n] = sum_c a[row, c] * w[expert][n, c]                 (down product)
//   out[row, n] = silu(a . wgate[n]) * (a . wup[n])                 (gate/up product)
//
// Weights are repacked once, at upload, into the operand order of
// v_mfma_f32_32x32x16_bf16: for every block of 32 weight rows and every 16-wide
// step of the reduction dimension, the 64 lanes' 8-element pieces are stored
// back to back (1 KiB per fragment).  A wave then fetches a whole fragment with
// one fully coalesced 16-byte-per-lane load and never touches LDS for weights;
// int8 weights are widened to bf16 in registers right before the multiply
// ("dequantisation in the operand load") and the per-row scale is applied to the
// accumulator, i.e. (sum a*q) * scale as the reference does.
//
// Activations (128 token rows per workgroup, gathered through an index for the
// gate/up product) go through LDS, XOR-swizzled in 16-byte pieces so that the
// stores and the fragment reads are free of bank conflicts, double-buffered along
// the reduction dimension.  A workgroup is 4 waves side by side along the output
// features; each wave owns 128 tokens x 64 weight rows (32 gate + the matching
// 32 up rows, or 64 down rows), so the two accumulators of one hidden element
// sit in the same lane and SwiGLU is applied in registers.
//
// The weight fragment is the matrix-core A operand and the token fragment the B
// operand, so a lane ends up with 4 consecutive output features of one token and
// writes them with one 8-byte store.
#include "rbmoe_kernels.h"

namespace rbmoe {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

namespace {

constexpr int BM = 128;   // token rows per workgroup
constexpr int BK = 64;    // reduction slice staged in LDS
constexpr int NW = 4;     // waves per workgroup
constexpr int NT = NW * 64;
constexpr int CPR = BK / 8;            // 16-byte pieces per LDS row
constexpr int A_CH = BM * CPR / NT;    // pieces per thread per slice
constexpr int TT = BM / 32;            // token blocks per wave
constexpr int KS = BK / 16;            // matrix-core steps per slice

__device__ __forceinline__ uint32_t widen2(uint32_t word, int shift) {
    const float lo = (float)(int)(int8_t)(word >> shift);
    const float hi = (float)(int)(int8_t)(word >> (shift + 8));
    return (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);  // small integers are exact in bf16
}

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

// Weight fragments of one wave for one LDS slice: 2 row blocks x KS steps.
template <bool I8>
struct WFrag;
template <>
struct WFrag<false> {
    uint4 v[2][KS];
    __device__ __forceinline__ void load(const uint4* p0, const uint4* p1, int kt, int lane) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            v[0][s] = p0[(size_t)(kt * KS + s) * 64 + lane];
            v[1][s] = p1[(size_t)(kt * KS + s) * 64 + lane];
        }
    }
    __device__ __forceinline__ bf16x8 get(int b, int s) const { return __builtin_bit_cast(bf16x8, v[b][s]); }
};
template <>
struct WFrag<true> {
    uint4 v[2][KS / 2];  // 16 int8 per lane cover two steps
    __device__ __forceinline__ void load(const uint4* p0, const uint4* p1, int kt, int lane) {
#pragma unroll
        for (int s = 0; s < KS / 2; ++s) {
            v[0][s] = p0[(size_t)(kt * (KS / 2) + s) * 64 + lane];
            v[1][s] = p1[(size_t)(kt * (KS / 2) + s) * 64 + lane];
        }
    }
    __device__ __forceinline__ bf16x8 get(int b, int s) const {
        const uint4 q = v[b][s >> 1];
        const uint32_t lo = (s & 1) ? q.z : q.x, hi = (s & 1) ? q.w : q.y;
        const uint4 w = make_uint4(widen2(lo, 0), widen2(lo, 16), widen2(hi, 0), widen2(hi, 16));
        return __builtin_bit_cast(bf16x8, w);
    }
};

template <bool SWIGLU, bool I8>
__global__ __launch_bounds__(NT, 2) void grouped_bdirect_kernel(
    const bf16_t* __restrict__ a, const int* __restrict__ row_index, const void* __restrict__ wpacked,
    size_t w_expert_stride_bytes, const float* __restrict__ scales, size_t s_expert_stride, int N, int K,
    const int* __restrict__ tile_expert, const int* __restrict__ tile_row0, const int* __restrict__ tile_rows,
    const int* __restrict__ ntiles, int dense_rows, bf16_t* __restrict__ out, int group_m) {
    // output features per workgroup: 4 waves x 32 hidden (gate/up) or 4 x 64 (down)
    constexpr int BN = SWIGLU ? NW * 32 : NW * 64;
    __shared__ uint4 As[2][BM * CPR];

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

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    // ---- this wave's two blocks of 32 weight rows ---------------------------
    // gate/up: hidden columns [nw, nw + 32): gate rows nw.., up rows N + nw..
    // down   : output columns [nw, nw + 64): rows nw.. and nw + 32..
    const int nw = tn_idx * BN + wave * (SWIGLU ? 32 : 64);
    const int r0 = nw, r1 = SWIGLU ? N + nw : nw + 32;
    const bool act0 = nw < N;
    const bool act1 = SWIGLU ? act0 : (nw + 32 < N);
    const size_t frag_bytes_per_block = (size_t)K * 32 * (I8 ? 1 : 2);  // one block of 32 rows, all of K
    const char* wexp = static_cast<const char*>(wpacked) + (size_t)expert * w_expert_stride_bytes;
    const uint4* wp0 = reinterpret_cast<const uint4*>(wexp + (size_t)(act0 ? r0 / 32 : 0) * frag_bytes_per_block);
    const uint4* wp1 = reinterpret_cast<const uint4*>(wexp + (size_t)(act1 ? r1 / 32 : 0) * frag_bytes_per_block);

    // ---- activation pieces of this thread -----------------------------------
    const uint4* a_pieces = reinterpret_cast<const uint4*>(a);
    const int kp = K / 8;
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
        a_lds[j] = r * CPR + (c ^ (r % CPR));
        a_mask |= ok ? (1u << j) : 0u;
    }
    uint4 ra[A_CH];
    auto fetch_a = [&](int kt) {
#pragma unroll
        for (int j = 0; j < A_CH; ++j) {
            ra[j] = make_uint4(0, 0, 0, 0);
            if (a_mask & (1u << j)) ra[j] = a_pieces[a_off[j] + kt * CPR];
        }
    };
    auto stage_a = [&](int buf) {
#pragma unroll
        for (int j = 0; j < A_CH; ++j) As[buf][a_lds[j]] = ra[j];
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
    const int lxor = lrow % CPR;  // token block bases are multiples of 32

    const int KT = K / BK;
    WFrag<I8> wcur, wnext;
    fetch_a(0);
    if (act0) wcur.load(wp0, wp1, 0, lane);
    stage_a(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < KT) {
            fetch_a(kt + 1);
            if (act0) wnext.load(wp0, wp1, kt + 1, lane);
        }
        if (act0) {
            const uint4* Ab = As[buf];
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const int piece = (2 * s + lhalf) ^ lxor;
                bf16x8 tf[TT];
#pragma unroll
                for (int t = 0; t < TT; ++t) tf[t] = __builtin_bit_cast(bf16x8, Ab[(t * 32 + lrow) * CPR + piece]);
                const bf16x8 w0 = wcur.get(0, s);
                const bf16x8 w1 = wcur.get(1, s);
#pragma unroll
                for (int t = 0; t < TT; ++t) {
                    acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w0, tf[t], acc[0][t], 0, 0, 0);
                    acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(w1, tf[t], acc[1][t], 0, 0, 0);
                }
            }
        }
        if (kt + 1 < KT) {
            stage_a(buf ^ 1);
            wcur = wnext;
        }
        __syncthreads();
    }
    if (!act0) return;

    // ---- epilogue -------------------------------------------------------------
    // accumulator element v of block (b, t): feature 8*(v/4) + 4*(lane/32) + v%4 of the
    // wave's row block b, token t*32 + lane%32.
    const float* sc = scales ? scales + (size_t)expert * s_expert_stride : nullptr;
#pragma unroll
    for (int t = 0; t < TT; ++t) {
        const int m = t * 32 + lrow;
        if (m >= rows) continue;
        bf16_t* orow = out + (size_t)(row0 + m) * N;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int f = 8 * q + 4 * lhalf;  // first of 4 consecutive features inside a row block
            if (SWIGLU) {
                float h[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float gv = acc[0][t][4 * q + i], uv = acc[1][t][4 * q + i];
                    if (sc) {
                        gv *= sc[r0 + f + i];
                        uv *= sc[r1 + f + i];
                    }
                    h[i] = silu_f32(gv) * uv;
                }
                *reinterpret_cast<uint2*>(orow + nw + f) = make_uint2(pack2(h[0], h[1]), pack2(h[2], h[3]));
            } else {
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    if (b == 1 && !act1) continue;
                    const int rb = b ? r1 : r0;
                    float y[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        y[i] = acc[b][t][4 * q + i];
                        if (sc) y[i] *= sc[rb + f + i];
                    }
                    *reinterpret_cast<uint2*>(orow + rb + f) = make_uint2(pack2(y[0], y[1]), pack2(y[2], y[3]));
                }
            }
        }
    }
}

template <bool SWIGLU, bool I8>
hipError_t launch_t(const GroupedArgs& g, hipStream_t s) {
    constexpr int BN = SWIGLU ? NW * 32 : NW * 64;
    const int tiles_n = (g.N + BN - 1) / BN;
    const int tiles_m = g.dense_rows >= 0 ? (g.dense_rows + BM - 1) / BM : g.max_tiles;
    if (tiles_m <= 0) return hipSuccess;
    const int total = tiles_m * tiles_n;
    const int grid = ((total + 7) / 8) * 8;
    hipLaunchKernelGGL((grouped_bdirect_kernel<SWIGLU, I8>), dim3(grid), dim3(NT), 0, s,
                       static_cast<const bf16_t*>(g.a), g.row_index, g.w, g.w_expert_stride * (I8 ? 1 : 2), g.scales,
                       g.s_expert_stride, g.N, g.K, g.tile_expert, g.tile_row0, g.tile_rows, g.ntiles, g.dense_rows,
                       static_cast<bf16_t*>(g.out), g.group_m > 0 ? g.group_m : 4);
    return hipGetLastError();
}

}  // namespace

int bdirect_tile_m() { return BM; }

// K a multiple of 64 (LDS slice), N a multiple of 32 (row blocks of the packed weights)
bool bdirect_shape_ok(int N, int K) { return K % 64 == 0 && K >= 64 && N % 32 == 0 && N >= 32; }

hipError_t launch_grouped_bdirect(const GroupedArgs& g, WeightKind wk, hipStream_t s) {
    if (!bdirect_shape_ok(g.N, g.K)) return hipErrorInvalidValue;
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
