// Backward pass of the layer (MoeLayer::backward, src/moe.rs:348-489; SwiGlu::backward,
// src/ffn.rs:87-120): the small kernels around the matrix products.
//
//   scale_rows_kernel      dY[pos] = gate * dOut[token]; dgate[slot] = dOut[token] . Y[pos]
//   swiglu_grad_kernel     dG = dH * U * silu'(G),  dU = dH * silu(G)
//   grouped_tn_kernel      dW[e] += A_e^T . B_e   (weight.grad += grad_output^T . input)
//   route_backward_kernel  dgate -> dP (renormalisation, balancing loss) -> dlogits (softmax, z loss)
//   router_grad_*          dWr += dlogits^T . X (two stages, fixed order), dX_router = dlogits . Wr
//
// The row products (dH = dY . Wd, dX = dG . Wg + dU . Wu) run on the forward pass's streaming
// kernel with transposed packed copies of the weights.  No floating-point atomics anywhere:
// every sum has one fixed order.
#include "rbmoe_kernels.h"

namespace rbmoe {

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + __expf(-x)); }

// ---------------------------------------------------------------------------
// One wave per routed row (src/moe.rs:374-385 and :404-416).
// ---------------------------------------------------------------------------
template <typename XT>
__global__ __launch_bounds__(256) void scale_rows_kernel(const XT* __restrict__ gout, const XT* __restrict__ y,
                                                         const int* __restrict__ perm_slot,
                                                         const int* __restrict__ perm_token,
                                                         const float* __restrict__ gate_of,
                                                         const int* __restrict__ offsets, int E, int d,
                                                         XT* __restrict__ dy, float* __restrict__ grad_gates) {
    const int lane = threadIdx.x & 63;
    const int pos = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (pos >= offsets[E]) return;
    const int slot = perm_slot[pos];
    const float g = gate_of[slot];
    const XT* go = gout + (size_t)perm_token[pos] * d;
    const XT* yr = y + (size_t)pos * d;
    XT* dr = dy + (size_t)pos * d;
    float dot = 0.0f;
    for (int c = lane; c < d; c += 64) {
        const float v = to_f32(go[c]);
        dr[c] = from_f32<XT>(g * v);
        dot += v * to_f32(yr[c]);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
    if (lane == 0) grad_gates[slot] = dot;
}

// gu, dgu: [rows, 2F] with the gate half in columns [0, F) and the up half in [F, 2F)
template <typename XT>
__global__ __launch_bounds__(256) void swiglu_grad_kernel(const XT* __restrict__ dh, const XT* __restrict__ gu,
                                                          const int* __restrict__ row_limit, int limit_index,
                                                          int rows, int F, XT* __restrict__ dgu) {
    const int nrows = row_limit ? row_limit[limit_index] : rows;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)nrows * F) return;
    const int r = (int)(idx / F), f = (int)(idx - (long long)r * F);
    const float g = to_f32(gu[(size_t)r * 2 * F + f]);
    const float u = to_f32(gu[(size_t)r * 2 * F + F + f]);
    const float up = to_f32(dh[(size_t)r * F + f]);
    const float s = sigmoid_f32(g);
    dgu[(size_t)r * 2 * F + f] = from_f32<XT>(up * u * (s * (1.0f + g * (1.0f - s))));  // silu'(g), src/ffn.rs:235-238
    dgu[(size_t)r * 2 * F + F + f] = from_f32<XT>(up * (g * s));
}

// ---------------------------------------------------------------------------
// out[e][m][n] += sum over the rows r of group e of A[r][m] * B[row(r)][n].
// 64 x 64 outputs per workgroup, 16 x 16 threads with 4 x 4 outputs each, rows in chunks of
// 16 through LDS; f32 accumulation in row order.  dense_rows >= 0: one group of that many rows.
// ---------------------------------------------------------------------------
template <typename XT>
__global__ __launch_bounds__(256) void grouped_tn_kernel(const XT* __restrict__ a, int M, const XT* __restrict__ b,
                                                         const int* __restrict__ b_row_index, int N,
                                                         const int* __restrict__ counts,
                                                         const int* __restrict__ offsets, int dense_rows,
                                                         float* __restrict__ out, size_t out_expert_stride) {
    __shared__ float As[16][64 + 1];
    __shared__ float Bs[16][64 + 1];
    const int e = blockIdx.z;
    const int row0 = dense_rows >= 0 ? 0 : offsets[e];
    const int rows = dense_rows >= 0 ? dense_rows : counts[e];
    if (rows == 0) return;
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
    for (int r0 = 0; r0 < rows; r0 += 16) {
        // stage 16 rows x 64 columns of each operand: thread -> (row = tid / 16, 4 columns at 4 * (tid % 16))
        const int r = r0 + ty;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int cm = m0 + 4 * tx + j, cn = n0 + 4 * tx + j;
            float av = 0.0f, bv = 0.0f;
            if (r < rows) {
                if (cm < M) av = to_f32(a[(size_t)(row0 + r) * M + cm]);
                if (cn < N) {
                    const int br = b_row_index ? b_row_index[row0 + r] : row0 + r;
                    bv = to_f32(b[(size_t)br * N + cn]);
                }
            }
            As[ty][4 * tx + j] = av;
            Bs[ty][4 * tx + j] = bv;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[kk][4 * ty + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) bv[j] = Bs[kk][4 * tx + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
        }
        __syncthreads();
    }
    float* o = out + (size_t)e * out_expert_stride;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + 4 * ty + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + 4 * tx + j;
            if (n < N) o[(size_t)m * N + n] += acc[i][j];
        }
    }
}

// ---------------------------------------------------------------------------
// One token per thread (src/moe.rs:421-478).  V = routed slots / k.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void route_backward_kernel(const float* __restrict__ P, const float* __restrict__ lse,
                                                             const int* __restrict__ expert_of,
                                                             const float* __restrict__ grad_gates,
                                                             const int* __restrict__ counts,
                                                             const int* __restrict__ offsets, int T, int E, int k,
                                                             float w_aux, float w_z, float* __restrict__ dlogits) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= T) return;
    float* row = dlogits + (size_t)t * E;
    const int* sel = expert_of + (size_t)t * k;
    if (sel[0] < 0) {  // padding row: nothing flows
        for (int e = 0; e < E; ++e) row[e] = 0.0f;
        return;
    }
    const float* p = P + (size_t)t * E;
    const int V = offsets[E] / k;
    // dL/dP: renormalised gates, then the balancing loss (a constant per expert)
    float total = 0.0f;
    for (int r = 0; r < k; ++r) total += p[sel[r]];
    float weighted = 0.0f;
    for (int r = 0; r < k; ++r) weighted += grad_gates[(size_t)t * k + r] * p[sel[r]];
    const float aux_scale = (w_aux != 0.0f && V > 0) ? w_aux * (float)E / (float)V : 0.0f;
    const float slots = (float)(V * k);
    // first pass: dot = sum_e p_e * dP_e, with dP assembled on the fly
    float dot = 0.0f;
    for (int e = 0; e < E; ++e) {
        float gp = 0.0f;
        if (total > 0.0f)
            for (int r = 0; r < k; ++r)
                if (sel[r] == e) gp += grad_gates[(size_t)t * k + r] / total - weighted / (total * total);
        if (aux_scale != 0.0f) gp += aux_scale * ((float)counts[e] / slots);
        row[e] = gp;
        dot += p[e] * gp;
    }
    const float zf = (w_z != 0.0f) ? 2.0f * w_z * lse[t] / (float)(V > 0 ? V : 1) : 0.0f;
    for (int e = 0; e < E; ++e) row[e] = p[e] * (row[e] - dot) + zf * p[e];
}

// ---------------------------------------------------------------------------
// dWr[e][c] += sum_t dlogits[t][e] * x[t][c]: stage 1 sums chunks of 128 tokens into
// partial[chunk][e][c] (one thread per column, experts in batches of 8); stage 2 adds the
// chunks in order.  dxr[t][c] = sum_e dlogits[t][e] * wr[e][c].
// ---------------------------------------------------------------------------
constexpr int kRouterGradChunk = 128;

template <typename XT>
__global__ __launch_bounds__(256) void router_grad_partial_kernel(const float* __restrict__ dlogits,
                                                                  const XT* __restrict__ x, int T, int d, int E,
                                                                  float* __restrict__ partial) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    const int chunk = blockIdx.y;
    const int t0 = chunk * kRouterGradChunk, t1 = min(T, t0 + kRouterGradChunk);
    __shared__ float dl[kRouterGradChunk][8];
    for (int e0 = 0; e0 < E; e0 += 8) {
        __syncthreads();
        for (int i = threadIdx.x; i < (t1 - t0) * 8; i += 256) {
            const int tt = i >> 3, j = i & 7;
            dl[tt][j] = e0 + j < E ? dlogits[(size_t)(t0 + tt) * E + e0 + j] : 0.0f;
        }
        __syncthreads();
        if (c < d) {
            float acc[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
            for (int t = t0; t < t1; ++t) {
                const float xv = to_f32(x[(size_t)t * d + c]);
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] = fmaf(dl[t - t0][j], xv, acc[j]);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (e0 + j < E) partial[((size_t)chunk * E + e0 + j) * d + c] = acc[j];
        }
    }
}

__global__ __launch_bounds__(256) void router_grad_reduce_kernel(const float* __restrict__ partial, int chunks, int n,
                                                                 float* __restrict__ grad) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float s = 0.0f;
    for (int ch = 0; ch < chunks; ++ch) s += partial[(size_t)ch * n + i];
    grad[i] += s;
}

template <typename XT>
__global__ __launch_bounds__(256) void router_dx_kernel(const float* __restrict__ dlogits, const float* __restrict__ wr,
                                                        int T, int d, int E, XT* __restrict__ dxr) {
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)T * d) return;
    const int t = (int)(idx / d), c = (int)(idx - (long long)t * d);
    float s = 0.0f;
    for (int e = 0; e < E; ++e) s = fmaf(dlogits[(size_t)t * E + e], wr[(size_t)e * d + c], s);
    dxr[idx] = from_f32<XT>(s);
}

__global__ __launch_bounds__(256) void fill_f32_kernel(float* p, float v, long long n) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = v;
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
hipError_t launch_scale_rows(const void* gout, const void* y, const int* perm_slot, const int* perm_token,
                             const float* gate_of, const int* offsets, int E, int d, int max_rows, void* dy,
                             float* grad_gates, bool bf16, hipStream_t s) {
    if (max_rows <= 0) return hipSuccess;
    const dim3 grid((max_rows + 3) / 4), block(256);
    if (bf16)
        hipLaunchKernelGGL(scale_rows_kernel<bf16_t>, grid, block, 0, s, static_cast<const bf16_t*>(gout),
                           static_cast<const bf16_t*>(y), perm_slot, perm_token, gate_of, offsets, E, d,
                           static_cast<bf16_t*>(dy), grad_gates);
    else
        hipLaunchKernelGGL(scale_rows_kernel<float>, grid, block, 0, s, static_cast<const float*>(gout),
                           static_cast<const float*>(y), perm_slot, perm_token, gate_of, offsets, E, d,
                           static_cast<float*>(dy), grad_gates);
    return hipGetLastError();
}

hipError_t launch_swiglu_grad(const void* dh, const void* gu, const int* row_limit, int limit_index, int rows, int F,
                              void* dgu, bool bf16, hipStream_t s) {
    if (rows <= 0) return hipSuccess;
    const long long total = (long long)rows * F;
    const dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (bf16)
        hipLaunchKernelGGL(swiglu_grad_kernel<bf16_t>, grid, block, 0, s, static_cast<const bf16_t*>(dh),
                           static_cast<const bf16_t*>(gu), row_limit, limit_index, rows, F, static_cast<bf16_t*>(dgu));
    else
        hipLaunchKernelGGL(swiglu_grad_kernel<float>, grid, block, 0, s, static_cast<const float*>(dh),
                           static_cast<const float*>(gu), row_limit, limit_index, rows, F, static_cast<float*>(dgu));
    return hipGetLastError();
}

hipError_t launch_grouped_tn(const void* a, int M, const void* b, const int* b_row_index, int N, const int* counts,
                             const int* offsets, int groups, int dense_rows, float* out, size_t out_expert_stride,
                             bool bf16, hipStream_t s) {
    if (groups <= 0 || M <= 0 || N <= 0) return hipSuccess;
    const dim3 grid((N + 63) / 64, (M + 63) / 64, groups), block(256);
    if (bf16)
        hipLaunchKernelGGL(grouped_tn_kernel<bf16_t>, grid, block, 0, s, static_cast<const bf16_t*>(a), M,
                           static_cast<const bf16_t*>(b), b_row_index, N, counts, offsets, dense_rows, out,
                           out_expert_stride);
    else
        hipLaunchKernelGGL(grouped_tn_kernel<float>, grid, block, 0, s, static_cast<const float*>(a), M,
                           static_cast<const float*>(b), b_row_index, N, counts, offsets, dense_rows, out,
                           out_expert_stride);
    return hipGetLastError();
}

hipError_t launch_route_backward(const float* P, const float* lse, const int* expert_of, const float* grad_gates,
                                 const int* counts, const int* offsets, int T, int E, int k, float w_aux, float w_z,
                                 float* dlogits, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    hipLaunchKernelGGL(route_backward_kernel, dim3((T + 255) / 256), dim3(256), 0, s, P, lse, expert_of, grad_gates,
                       counts, offsets, T, E, k, w_aux, w_z, dlogits);
    return hipGetLastError();
}

int router_grad_chunks(int T) { return (T + kRouterGradChunk - 1) / kRouterGradChunk; }

hipError_t launch_router_grad(const float* dlogits, const void* x, const float* wr, int T, int d, int E,
                              float* partial, float* grad_router, void* dxr, bool bf16, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    const int chunks = router_grad_chunks(T);
    const dim3 g1((d + 255) / 256, chunks), block(256);
    const long long td = (long long)T * d;
    if (bf16) {
        hipLaunchKernelGGL(router_grad_partial_kernel<bf16_t>, g1, block, 0, s, dlogits,
                           static_cast<const bf16_t*>(x), T, d, E, partial);
        hipLaunchKernelGGL(router_dx_kernel<bf16_t>, dim3((unsigned)((td + 255) / 256)), block, 0, s, dlogits, wr, T, d,
                           E, static_cast<bf16_t*>(dxr));
    } else {
        hipLaunchKernelGGL(router_grad_partial_kernel<float>, g1, block, 0, s, dlogits, static_cast<const float*>(x),
                           T, d, E, partial);
        hipLaunchKernelGGL(router_dx_kernel<float>, dim3((unsigned)((td + 255) / 256)), block, 0, s, dlogits, wr, T, d,
                           E, static_cast<float*>(dxr));
    }
    hipLaunchKernelGGL(router_grad_reduce_kernel, dim3((E * d + 255) / 256), block, 0, s, partial, chunks, E * d,
                       grad_router);
    return hipGetLastError();
}

hipError_t launch_fill_f32(float* p, float v, long long n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, v, n);
    return hipGetLastError();
}

}  // namespace rbmoe
