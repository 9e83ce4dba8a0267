// Grouped expert products for all-f32 layers on the f32 matrix cores of gfx950
// (v_mfma_f32_32x32x2_f32: f32 products, f32 accumulation).
//
//   out[row, n] = sum_c a[row, c] * w[expert][n, c]                 (down product)
//   out[row, n] = silu(a . wgate[n]) * (a . wup[n])                 (gate/up product)
//
// A workgroup owns 64 token rows x 64 output features; a wave owns 32 x 32 of them (gate/up: two
// accumulators, the gate rows and the matching up rows).  Both operands go global -> registers -> LDS
// in slices of 32 reduction columns per wave group; the loads of the next slice are in flight while a
// slice is multiplied.  With SPLIT = 2 the workgroup has two groups of 4 waves that take alternate
// slices of the reduction and add their accumulators through LDS at the end (group 1 first, then group 0
// on top: a fixed order): twice the waves for the same tiles, which is what a launch with few tiles needs -
// a wave's multiplies depend on one another through its accumulator, and a SIMD with one such wave idles
// between them, so 320 tiles on 256 compute units (the down product of a 2048-row batch) leave most of
// the matrix cores' time unused.  Rows are fetched through `row_index`, so the gather of
// the routed rows (gather_rows, src/moe.rs:658-664) never materialises.  The weight fragment
// is the matrix-core A operand and the token fragment B, so a lane ends with 4 consecutive
// features of one token (one 16-byte store).  SiLU uses the exact division: this path is held
// to 1e-5.  For a backward pass the gate/up launch can also keep the pre-activations (`gu_out`),
// and a plain launch can apply SwiGLU's backward where it stores its rows (`swiglu_grad_gu`).
#include <type_traits>

#include "rbmoe_kernels.h"

namespace rbmoe {

namespace {

constexpr int FN = 64;   // output features per workgroup (two waves side by side)
constexpr int FK = 32;   // reduction columns per slice

// FM = token rows per workgroup, 64 or 32 (FM / 32 x 2 waves per group); SPLIT = wave groups
template <bool SWIGLU, int FM, int SPLIT>
__global__ __launch_bounds__(FM * 4 * SPLIT) void grouped_f32_kernel(
    const float* __restrict__ a, const int* __restrict__ row_index, const float* __restrict__ w,
    size_t w_expert_stride, int N, int K, const int* __restrict__ tile_expert, const int* __restrict__ tile_row0,
    const int* __restrict__ tile_rows, const int* __restrict__ ntiles, int dense_rows, float* __restrict__ out,
    float* __restrict__ gu_out, const float* __restrict__ bw_gu) {
    constexpr int WR = SWIGLU ? 2 * FN : FN;  // weight rows staged per slice
    constexpr int WPG = FM / 32 * 2;          // waves per group
    constexpr int NTH = 64 * WPG * SPLIT;     // threads
    constexpr int SK = FK * SPLIT;            // reduction columns staged at once: one slice per wave group
    constexpr int LSS = SK + 2;               // LDS row stride: the 64 lanes of a fragment read (32 rows x 2 columns) fall into 64 distinct banks
    __shared__ float As[FM * LSS];
    __shared__ float Ws[WR * LSS];

    int expert, row0, rows;
    if (dense_rows >= 0) {
        expert = 0;
        row0 = blockIdx.y * FM;
        rows = min(FM, dense_rows - row0);
        if (rows <= 0) return;
    } else {
        if ((int)blockIdx.y >= *ntiles) return;
        expert = tile_expert[blockIdx.y];
        row0 = tile_row0[blockIdx.y];
        rows = tile_rows[blockIdx.y];
    }
    const int n0 = blockIdx.x * FN;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = (tid >> 6) % WPG;
    const int grp = tid / (64 * WPG);         // wave group: which slice of each staged pair it multiplies
    const int wy = wave >> 1, wx = wave & 1;  // token half, feature half
    const float* wbase = w + (size_t)expert * w_expert_stride;

    // ---- staging: 16-byte pieces; thread -> (row, piece) ----------------------
    // activations: 64 rows x SK / 4 pieces, 2 per thread; weights: WR rows x SK / 4 pieces, 2 or 4 per thread
    constexpr int PPR = SK / 4;               // pieces per staged row
    constexpr int AP = FM * PPR / NTH;
    constexpr int WP = WR * PPR / NTH;
    static_assert(AP * NTH == FM * PPR && WP * NTH == WR * PPR, "every thread moves the same number of pieces");
    const float* a_src[AP];
    int a_dst[AP];
#pragma unroll
    for (int i = 0; i < AP; ++i) {
        const int p = i * NTH + tid;
        const int r = p / PPR, c = p % PPR;
        const int rr = r < rows ? r : 0;  // rows past the end of the group: products never stored
        const int grow = row_index ? row_index[row0 + rr] : row0 + rr;
        a_src[i] = a + (size_t)grow * K + 4 * c;
        a_dst[i] = r * LSS + 4 * c;
    }
    const float* w_src[WP];
    int w_dst[WP];
#pragma unroll
    for (int i = 0; i < WP; ++i) {
        const int p = i * NTH + tid;
        const int r = p / PPR, c = p % PPR;
        // staged row r < FN: gate (or plain) feature n0 + r; r >= FN: the matching up row
        const int feat = n0 + (r % FN);
        const int fr = feat < N ? feat : 0;
        const int wrow = (SWIGLU && r >= FN) ? N + fr : fr;
        w_src[i] = wbase + (size_t)wrow * K + 4 * c;
        w_dst[i] = r * LSS + 4 * c;
    }
    float4 areg[AP], wreg[WP];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < AP; ++i) areg[i] = *reinterpret_cast<const float4*>(a_src[i] + k0);
#pragma unroll
        for (int i = 0; i < WP; ++i) wreg[i] = *reinterpret_cast<const float4*>(w_src[i] + k0);
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < AP; ++i) {
            float* d = As + a_dst[i];
            d[0] = areg[i].x; d[1] = areg[i].y; d[2] = areg[i].z; d[3] = areg[i].w;
        }
#pragma unroll
        for (int i = 0; i < WP; ++i) {
            float* d = Ws + w_dst[i];
            d[0] = wreg[i].x; d[1] = wreg[i].y; d[2] = wreg[i].z; d[3] = wreg[i].w;
        }
    };

    floatx16 acc0, acc1;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.0f;

    // fragment addresses: lane l -> row l % 32 of the wave's block, reduction column 2 s + l / 32 of the group's slice
    const float* a_frag = As + (wy * 32 + (lane & 31)) * LSS + grp * FK + (lane >> 5);
    const float* w_frag = Ws + (wx * 32 + (lane & 31)) * LSS + grp * FK + (lane >> 5);

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += SK) {
        stage();
        __syncthreads();
        if (k0 + SK < K) fetch(k0 + SK);
#pragma unroll
        for (int s = 0; s < FK / 2; ++s) {
            const float tv = a_frag[2 * s];
            const float gv = w_frag[2 * s];
            acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(gv, tv, acc0, 0, 0, 0);
            if constexpr (SWIGLU) {
                const float uv = w_frag[FN * LSS + 2 * s];
                acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(uv, tv, acc1, 0, 0, 0);
            }
        }
        __syncthreads();
    }

    if constexpr (SPLIT > 1) {
        // the two groups' sums meet in LDS (the staging tiles are free: the loop's last barrier is behind us)
        static_assert(FM * LSS >= WPG * 16 * 64 && WR * LSS >= (SWIGLU ? WPG * 16 * 64 : 0), "room for the accumulators");
        float* const r0 = As + wave * (16 * 64) + lane;
        float* const r1 = Ws + wave * (16 * 64) + lane;
        // groups SPLIT - 1 ... 1 hand their sums down one after the other; group 0 adds the last and stores
#pragma unroll
        for (int gsrc = SPLIT - 1; gsrc >= 1; --gsrc) {
            if (grp == gsrc) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    r0[v * 64] = acc0[v];
                    if constexpr (SWIGLU) r1[v * 64] = acc1[v];
                }
            }
            __syncthreads();
            if (grp == gsrc - 1) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    acc0[v] += r0[v * 64];
                    if constexpr (SWIGLU) acc1[v] += r1[v * 64];
                }
            }
            if (gsrc > 1) __syncthreads();
        }
        if (grp != 0) return;
    }

    // accumulator element v of lane l: feature 8 (v / 4) + 4 (l / 32) + v % 4 of the wave's
    // block, token l % 32
    const int tok = wy * 32 + (lane & 31);
    if (tok >= rows) return;
    float* orow = out + (size_t)(row0 + tok) * N + n0 + wx * 32;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int f = 8 * q + 4 * (lane >> 5);
        if (n0 + wx * 32 + f >= N) continue;  // N is a multiple of 4: a group of 4 is in or out as a whole
        float4 y;
        if constexpr (SWIGLU) {
            y.x = silu_f32(acc0[4 * q + 0]) * acc1[4 * q + 0];
            y.y = silu_f32(acc0[4 * q + 1]) * acc1[4 * q + 1];
            y.z = silu_f32(acc0[4 * q + 2]) * acc1[4 * q + 2];
            y.w = silu_f32(acc0[4 * q + 3]) * acc1[4 * q + 3];
            if (gu_out != nullptr) {  // uniform: the pre-activations G | U [rows, 2 N] kept for a backward pass
                float* const grow = gu_out + (size_t)(row0 + tok) * 2 * N + n0 + wx * 32 + f;
                *reinterpret_cast<float4*>(grow) =
                    make_float4(acc0[4 * q + 0], acc0[4 * q + 1], acc0[4 * q + 2], acc0[4 * q + 3]);
                *reinterpret_cast<float4*>(grow + N) =
                    make_float4(acc1[4 * q + 0], acc1[4 * q + 1], acc1[4 * q + 2], acc1[4 * q + 3]);
            }
        } else {
            y = make_float4(acc0[4 * q + 0], acc0[4 * q + 1], acc0[4 * q + 2], acc0[4 * q + 3]);
            if (bw_gu != nullptr) {  // uniform
                // SwiGlu::backward (src/ffn.rs:87-120) on the way out: the product row is the gradient of the
                // hidden row; dG = dH * U * silu'(G), dU = dH * silu(G) go to `gu_out`, `out` is not written.
                const size_t off = (size_t)(row0 + tok) * 2 * N + n0 + wx * 32 + f;
                const float4 g4 = *reinterpret_cast<const float4*>(bw_gu + off);
                const float4 u4 = *reinterpret_cast<const float4*>(bw_gu + off + N);
                const float dh[4] = {y.x, y.y, y.z, y.w}, gv[4] = {g4.x, g4.y, g4.z, g4.w}, uv[4] = {u4.x, u4.y, u4.z, u4.w};
                float dg[4], du[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float sg = 1.0f / (1.0f + __expf(-gv[i]));
                    dg[i] = dh[i] * uv[i] * (sg * (1.0f + gv[i] * (1.0f - sg)));  // silu', src/ffn.rs:235-238
                    du[i] = dh[i] * (gv[i] * sg);
                }
                *reinterpret_cast<float4*>(gu_out + off) = make_float4(dg[0], dg[1], dg[2], dg[3]);
                *reinterpret_cast<float4*>(gu_out + off + N) = make_float4(du[0], du[1], du[2], du[3]);
                continue;
            }
        }
        *reinterpret_cast<float4*>(orow + f) = y;
    }
}

}  // namespace

// 64-row tiles; 32-row tiles when the launches of such a batch would have few tiles for the chip (their workgroups
// cannot be spread evenly over 256 compute units: 320 tiles leave a quarter of them with twice the work)
int f32_tile_m(int rows, int groups, int n_min) {
    const long long tiles64 = (long long)(rows / 64 + groups) * ((n_min + FN - 1) / FN);
    return tiles64 < 4 * 256 ? 32 : 64;
}

// reduction width a multiple of the slice, output width a multiple of 4 (16-byte stores)
bool f32_shape_ok(int N, int K) { return K % FK == 0 && K >= FK && N % 4 == 0 && N >= 4; }

hipError_t launch_grouped_f32(const GroupedArgs& g, hipStream_t s) {
    // the tile table's tile height (a dense launch makes its own tiles: 64 rows, or 32 when that leaves few)
    int fm = g.tile_m;
    if (g.dense_rows >= 0) fm = f32_tile_m(g.dense_rows, 0, g.N);
    if (fm != 32 && fm != 64) return hipErrorInvalidValue;
    const int tiles_m = g.dense_rows >= 0 ? (g.dense_rows + fm - 1) / fm : g.max_tiles;
    if (tiles_m <= 0) return hipSuccess;
    const dim3 grid((g.N + FN - 1) / FN, tiles_m);
    // 32-row tiles have two waves per group; a second group taking alternate slices of the reduction brings the
    // workgroup back to four (the reduction must split into pairs of slices)
    const bool split = fm == 32 && g.K % (2 * FK) == 0;

    auto go = [&](auto swiglu_tag, auto fm_tag, auto split_tag) {
        constexpr bool SW = decltype(swiglu_tag)::value;
        constexpr int FMv = decltype(fm_tag)::value, SP = decltype(split_tag)::value;
        RB_LAUNCH((grouped_f32_kernel<SW, FMv, SP>), grid, dim3(FMv * 4 * SP), 0, s, static_cast<const float*>(g.a),
                  g.row_index, static_cast<const float*>(g.w), g.w_expert_stride, g.N, g.K, g.tile_expert, g.tile_row0,
                  g.tile_rows, g.ntiles, g.dense_rows, static_cast<float*>(g.out), static_cast<float*>(g.gu_out),
                  static_cast<const float*>(g.swiglu_grad_gu));
    };
    typedef std::integral_constant<int, 1> One;
    typedef std::integral_constant<int, 2> Two;
    typedef std::integral_constant<int, 32> M32;
    typedef std::integral_constant<int, 64> M64;
    auto pick = [&](auto swiglu_tag) {
        if (fm == 64) go(swiglu_tag, M64{}, One{});
        else if (split) go(swiglu_tag, M32{}, Two{});
        else go(swiglu_tag, M32{}, One{});
    };
    if (g.swiglu) pick(std::true_type{});
    else pick(std::false_type{});
    return hipGetLastError();
}

}  // namespace rbmoe
