// Grouped expert products for any shape and dtype: the fallback when a shape
// does not fit the MFMA kernels (tiny widths, odd sizes) and the path for f32
// and f32-activation layers.  A 16x16 thread block computes a 16x16 output tile
// from 16-wide K slices staged in LDS; accumulation is f32 in index order.  Like the matrix-core
// kernels, the gate/up launch can keep the pre-activations for a backward pass (`gu_out`), and a
// down-shaped launch can apply SwiGLU's backward to its rows on the way out (`bw_gu`).
#include "rbmoe_kernels.h"

namespace rbmoe {

__device__ __forceinline__ float w_to_f32(float v) { return v; }
__device__ __forceinline__ float w_to_f32(bf16_t v) { return to_f32(v); }
__device__ __forceinline__ float w_to_f32(int8_t v) { return (float)v; }

template <typename AT, typename WT, bool SWIGLU>
__global__ __launch_bounds__(256) void grouped_generic_kernel(
    const AT* __restrict__ a, const int* __restrict__ row_index, const WT* __restrict__ w,
    size_t w_expert_stride, const float* __restrict__ scales, size_t s_expert_stride, int N, int K,
    const int* __restrict__ tile_expert, const int* __restrict__ tile_row0,
    const int* __restrict__ tile_rows, const int* __restrict__ ntiles, int dense_rows,
    AT* __restrict__ out, AT* __restrict__ gu_out, const AT* __restrict__ bw_gu) {
    constexpr int TM = kGenericTileM, TN = 16, TK = 16;
    __shared__ float As[TM][TK + 1];
    __shared__ float Wg[TN][TK + 1];
    __shared__ float Wu[TN][TK + 1];

    int expert, row0, rows;
    if (dense_rows >= 0) {
        expert = 0;
        row0 = blockIdx.x * TM;
        rows = min(TM, dense_rows - row0);
        if (rows <= 0) return;
    } else {
        if ((int)blockIdx.x >= *ntiles) return;
        expert = tile_expert[blockIdx.x];
        row0 = tile_row0[blockIdx.x];
        rows = tile_rows[blockIdx.x];
    }
    const int n0 = blockIdx.y * TN;
    const int tx = threadIdx.x & 15;  // column within the tile
    const int ty = threadIdx.x >> 4;  // row within the tile
    const WT* wbase = w + (size_t)expert * w_expert_stride;

    // row of `a` this thread stages
    int arow = -1;
    if (ty < rows) arow = row_index ? row_index[row0 + ty] : row0 + ty;

    float accg = 0.0f, accu = 0.0f;
    for (int k0 = 0; k0 < K; k0 += TK) {
        const int c = k0 + tx;
        As[ty][tx] = (arow >= 0 && c < K) ? to_f32(a[(size_t)arow * K + c]) : 0.0f;
        const int n = n0 + ty;
        Wg[ty][tx] = (n < N && c < K) ? w_to_f32(wbase[(size_t)n * K + c]) : 0.0f;
        if (SWIGLU) Wu[ty][tx] = (n < N && c < K) ? w_to_f32(wbase[(size_t)(N + n) * K + c]) : 0.0f;
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; ++kk) {
            const float av = As[ty][kk];
            accg = fmaf(av, Wg[tx][kk], accg);
            if (SWIGLU) accu = fmaf(av, Wu[tx][kk], accu);
        }
        __syncthreads();
    }
    const int n = n0 + tx;
    if (ty < rows && n < N) {
        if (scales) {
            const float* sc = scales + (size_t)expert * s_expert_stride;
            accg *= sc[n];
            if (SWIGLU) accu *= sc[N + n];
        }
        const size_t row = (size_t)(row0 + ty);
        if (SWIGLU) {
            if (gu_out != nullptr) {  // pre-activations G | U [rows, 2 N]
                gu_out[row * 2 * N + n] = from_f32<AT>(accg);
                gu_out[row * 2 * N + N + n] = from_f32<AT>(accu);
            }
            out[row * N + n] = from_f32<AT>(silu_f32(accg) * accu);
        } else if (bw_gu != nullptr) {
            // SwiGlu::backward (src/ffn.rs:87-120): the product row is the gradient of the hidden row;
            // dG = dH * U * silu'(G), dU = dH * silu(G) go to `gu_out`, `out` is not written.
            const float gv = to_f32(bw_gu[row * 2 * N + n]), uv = to_f32(bw_gu[row * 2 * N + N + n]);
            const float sg = 1.0f / (1.0f + __expf(-gv));
            gu_out[row * 2 * N + n] = from_f32<AT>(accg * uv * (sg * (1.0f + gv * (1.0f - sg))));  // silu', src/ffn.rs:235-238
            gu_out[row * 2 * N + N + n] = from_f32<AT>(accg * (gv * sg));
        } else {
            out[row * N + n] = from_f32<AT>(accg);
        }
    }
}

template <typename AT, typename WT>
static hipError_t launch_t(const GroupedArgs& g, hipStream_t s) {
    const int tiles = g.dense_rows >= 0 ? (g.dense_rows + kGenericTileM - 1) / kGenericTileM : g.max_tiles;
    if (tiles <= 0) return hipSuccess;
    const dim3 grid(tiles, (g.N + 15) / 16), block(256);
    if (g.swiglu)
        RB_LAUNCH((grouped_generic_kernel<AT, WT, true>), grid, block, 0, s,
                           static_cast<const AT*>(g.a), g.row_index, static_cast<const WT*>(g.w),
                           g.w_expert_stride, g.scales, g.s_expert_stride, g.N, g.K, g.tile_expert,
                           g.tile_row0, g.tile_rows, g.ntiles, g.dense_rows, static_cast<AT*>(g.out),
                           static_cast<AT*>(g.gu_out), static_cast<const AT*>(g.swiglu_grad_gu));
    else
        RB_LAUNCH((grouped_generic_kernel<AT, WT, false>), grid, block, 0, s,
                           static_cast<const AT*>(g.a), g.row_index, static_cast<const WT*>(g.w),
                           g.w_expert_stride, g.scales, g.s_expert_stride, g.N, g.K, g.tile_expert,
                           g.tile_row0, g.tile_rows, g.ntiles, g.dense_rows, static_cast<AT*>(g.out),
                           static_cast<AT*>(g.gu_out), static_cast<const AT*>(g.swiglu_grad_gu));
    return hipGetLastError();
}

hipError_t launch_grouped_generic(const GroupedArgs& g, bool act_bf16, WeightKind wk, int tile_m,
                                  hipStream_t s) {
    if (tile_m != kGenericTileM) return hipErrorInvalidValue;
    if (act_bf16) {
        switch (wk) {
            case WeightKind::F32: return launch_t<bf16_t, float>(g, s);
            case WeightKind::BF16: return launch_t<bf16_t, bf16_t>(g, s);
            case WeightKind::I8: return launch_t<bf16_t, int8_t>(g, s);
        }
    } else {
        switch (wk) {
            case WeightKind::F32: return launch_t<float, float>(g, s);
            case WeightKind::BF16: return launch_t<float, bf16_t>(g, s);
            case WeightKind::I8: return launch_t<float, int8_t>(g, s);
        }
    }
    return hipErrorInvalidValue;
}

}  // namespace rbmoe
