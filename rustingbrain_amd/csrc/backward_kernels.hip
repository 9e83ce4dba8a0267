// Backward pass of the layer (MoeLayer::backward, src/moe.rs:348-489; SwiGlu::backward,
// src/ffn.rs:87-120): the small kernels around the matrix products.
//
//   scale_rows_kernel      dY[pos] = gate * dOut[token]; dgate[slot] = dOut[token] . Y[pos]
//   grouped_tn_kernel      dW[e] += A_e^T . B_e   (weight.grad += grad_output^T . input), plain f32
//                          arithmetic: the path for shapes the matrix-core kernel does not take
//   route_backward_kernel  dgate -> dP (renormalisation, balancing loss) -> dlogits (softmax, z loss)
//   router_grad_*          dWr += dlogits^T . X (two stages, fixed order), dX_router = dlogits . Wr
//
// The row products (dH = dY . Wd, dX = dG . Wg + dU . Wu) run on the forward pass's streaming
// kernel with transposed packed copies of the weights (SwiGLU's backward is applied where the
// first of them stores its rows); the weight gradients have a matrix-core kernel of their own.
// Every sum in this file has one fixed order.  Rows are moved in 16-byte pieces when the row
// width is a multiple of 8 (bf16) or 4 (f32) elements; any other width takes the same kernels
// one element at a time (`Vec1`) or the plain `*_any_kernel` versions further down.
#include "rbmoe_kernels.h"

namespace rbmoe {

// ---------------------------------------------------------------------------
// One wave per routed row (src/moe.rs:374-385 and :404-416).
// ---------------------------------------------------------------------------
// One element of a row, with the interface of Vec16: rows of any width.
template <typename XT>
struct Vec1 {
    static constexpr int N = 1;
    static __device__ __forceinline__ void load(const XT* p, float (&v)[1]) { v[0] = to_f32(*p); }
    static __device__ __forceinline__ void store(XT* p, const float (&v)[1]) { *p = from_f32<XT>(v[0]); }
};

template <typename XT, typename V>
__global__ __launch_bounds__(256) void scale_rows_kernel(const XT* __restrict__ gout, const XT* __restrict__ y,
                                                         const int* __restrict__ perm_slot,
                                                         const int* __restrict__ perm_token,
                                                         const float* __restrict__ gate_of,
                                                         const int* __restrict__ offsets, int E, int d,
                                                         XT* __restrict__ dy, float* __restrict__ grad_gates) {
    constexpr int VN = V::N;
    const int lane = threadIdx.x & 63;
    const int pos = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (pos >= offsets[E]) return;
    const int slot = perm_slot[pos];
    const float g = gate_of[slot];
    const XT* go = gout + (size_t)perm_token[pos] * d;
    const XT* yr = y + (size_t)pos * d;
    XT* dr = dy + (size_t)pos * d;
    float dot = 0.0f;
    for (int c = lane * VN; c < d; c += 64 * VN) {
        float v[VN], w[VN], o[VN];
        V::load(go + c, v);
        V::load(yr + c, w);
#pragma unroll
        for (int i = 0; i < VN; ++i) {
            o[i] = g * v[i];
            dot = fmaf(v[i], w[i], dot);
        }
        V::store(dr + c, o);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
    if (lane == 0) grad_gates[slot] = dot;
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
// Gates -> probabilities -> logits (src/moe.rs:421-478).  V = routed slots / k.  A group of G
// lanes (16, 32 or 64: the smallest that covers E, or 64) owns one token; lane j owns experts
// j, j + G, ...: a token's row of probabilities is read and its row of logit gradients written
// by neighbouring lanes.  The sum over the experts (the softmax's dot product) is a butterfly
// inside the group, so every lane of the group holds the same value in the same order.
// ---------------------------------------------------------------------------
template <int G>
__global__ __launch_bounds__(256) void route_backward_kernel(
    const float* __restrict__ P, const float* __restrict__ lse, const int* __restrict__ expert_of,
    const float* __restrict__ grad_gates, const int* __restrict__ counts, const int* __restrict__ offsets, int T, int E,
    int k, float w_aux, float w_z, float* __restrict__ dlogits) {
    const int t = (blockIdx.x * 256 + threadIdx.x) / G;
    const int j = threadIdx.x % G;
    // a whole group leaves together: the shuffles below stay inside groups that are all there
    if (t >= T) return;
    float* row = dlogits + (size_t)t * E;
    const int* sel = expert_of + (size_t)t * k;
    if (sel[0] < 0) {  // padding row: nothing flows
        for (int e = j; e < E; e += G) row[e] = 0.0f;
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
    // the reference's own two quotients (src/moe.rs:438-441): with one expert per token they cancel to rounding
    // noise, and the noise should at least be the same kind of noise
    const float renorm = total > 0.0f ? __fdiv_rn(weighted, __fmul_rn(total, total)) : 0.0f;
    // dP of expert e, assembled on the fly (twice: once for the softmax's dot product, once for
    // the result - cheaper than a trip through memory)
    auto grad_p = [&](int e) {
        float gp = 0.0f;
        if (total > 0.0f)
            for (int r = 0; r < k; ++r)
                if (sel[r] == e) gp += __fdiv_rn(grad_gates[(size_t)t * k + r], total) - renorm;
        if (aux_scale != 0.0f) gp += aux_scale * ((float)counts[e] / slots);
        return gp;
    };
    float dot = 0.0f;
    for (int e = j; e < E; e += G) dot += p[e] * grad_p(e);
#pragma unroll
    for (int o = G / 2; o > 0; o >>= 1) dot += __shfl_xor(dot, o);
    const float zf = (w_z != 0.0f) ? 2.0f * w_z * lse[t] / (float)(V > 0 ? V : 1) : 0.0f;
    for (int e = j; e < E; e += G) row[e] = p[e] * (grad_p(e) - dot) + zf * p[e];
}

// ---------------------------------------------------------------------------
// Router weight gradient dWr[e][c] += sum_t dlogits[t][e] * x[t][c] in two stages with one
// fixed order of additions.  Stage 1: a block of 128 threads owns 256 columns (a thread: two
// neighbours, one 4-byte or 8-byte load per token), one chunk of tokens and a batch of 16
// experts, with the chunk's dlogits in LDS; it writes partial[chunk][e][c].  Stage 2 adds the
// chunks in order.  At most kRouterGradMaxChunks chunks, of a multiple of 32 tokens each.
// ---------------------------------------------------------------------------
constexpr int kRouterGradMaxChunks = 256;
constexpr int kRouterGradExperts = 16;

__host__ __device__ inline int router_grad_chunk_tokens(int T) {
    const int per = (T + kRouterGradMaxChunks - 1) / kRouterGradMaxChunks;
    return ((per > 0 ? per : 1) + 31) & ~31;
}

__device__ __forceinline__ float2 load_pair(const float* p) { return *reinterpret_cast<const float2*>(p); }
__device__ __forceinline__ float2 load_pair(const bf16_t* p) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
    return make_float2(__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u));
}

template <typename XT>
__global__ __launch_bounds__(128) void router_grad_partial_kernel(const float* __restrict__ dlogits,
                                                                  const XT* __restrict__ x, int T, int d, int E,
                                                                  int chunk_tokens, float* __restrict__ partial) {
    extern __shared__ float dl[];  // [chunk_tokens][16]
    const int c = (blockIdx.x * 128 + threadIdx.x) * 2;
    const int chunk = blockIdx.y;
    const int e0 = blockIdx.z * kRouterGradExperts;
    const int t0 = chunk * chunk_tokens, t1 = min(T, t0 + chunk_tokens);
    for (int i = threadIdx.x; i < (t1 - t0) * kRouterGradExperts; i += 128) {
        const int tt = i / kRouterGradExperts, j = i % kRouterGradExperts;
        dl[i] = e0 + j < E ? dlogits[(size_t)(t0 + tt) * E + e0 + j] : 0.0f;
    }
    __syncthreads();
    if (c >= d) return;  // d is even
    float acc0[kRouterGradExperts], acc1[kRouterGradExperts];
#pragma unroll
    for (int j = 0; j < kRouterGradExperts; ++j) acc0[j] = acc1[j] = 0.0f;
#pragma unroll 4
    for (int t = t0; t < t1; ++t) {
        const float2 xp = load_pair(x + (size_t)t * d + c);
        const float x0 = xp.x, x1 = xp.y;
        const float4* row = reinterpret_cast<const float4*>(dl + (t - t0) * kRouterGradExperts);
#pragma unroll
        for (int q = 0; q < kRouterGradExperts / 4; ++q) {
            const float4 v = row[q];
            acc0[4 * q + 0] = fmaf(v.x, x0, acc0[4 * q + 0]); acc1[4 * q + 0] = fmaf(v.x, x1, acc1[4 * q + 0]);
            acc0[4 * q + 1] = fmaf(v.y, x0, acc0[4 * q + 1]); acc1[4 * q + 1] = fmaf(v.y, x1, acc1[4 * q + 1]);
            acc0[4 * q + 2] = fmaf(v.z, x0, acc0[4 * q + 2]); acc1[4 * q + 2] = fmaf(v.z, x1, acc1[4 * q + 2]);
            acc0[4 * q + 3] = fmaf(v.w, x0, acc0[4 * q + 3]); acc1[4 * q + 3] = fmaf(v.w, x1, acc1[4 * q + 3]);
        }
    }
#pragma unroll
    for (int j = 0; j < kRouterGradExperts; ++j)
        if (e0 + j < E)
            *reinterpret_cast<float2*>(partial + ((size_t)chunk * E + e0 + j) * d + c) = make_float2(acc0[j], acc1[j]);
}

// 64 outputs per block of 256 threads; thread (q, i) adds every fourth chunk starting at q for
// output i, then the four sums are added in order.
__global__ __launch_bounds__(256) void router_grad_reduce_kernel(const float* __restrict__ partial, int chunks, int n,
                                                                 float* __restrict__ grad) {
    __shared__ float part[4][64];
    const int i = blockIdx.x * 64 + (threadIdx.x & 63);
    const int q = threadIdx.x >> 6;
    float s = 0.0f;
    if (i < n) {
#pragma unroll 8
        for (int ch = q; ch < chunks; ch += 4) s += partial[(size_t)ch * n + i];
    }
    part[q][threadIdx.x & 63] = s;
    __syncthreads();
    if (q == 0 && i < n) grad[i] += ((part[0][threadIdx.x] + part[1][threadIdx.x]) + part[2][threadIdx.x]) + part[3][threadIdx.x];
}

// dxr[t][c] = sum_e dlogits[t][e] * wr[e][c].  A thread owns one 16-byte piece of the output
// rows of kDxTokens consecutive tokens, so a piece of a router row fetched once serves them all.
constexpr int kDxTokens = 4;

template <typename XT>
__global__ __launch_bounds__(256) void router_dx_kernel(const float* __restrict__ dlogits, const float* __restrict__ wr,
                                                        int T, int d, int E, XT* __restrict__ dxr) {
    constexpr int VN = Vec16<XT>::N;
    const int pieces = d / VN;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    const int groups = (T + kDxTokens - 1) / kDxTokens;
    if (idx >= (long long)groups * pieces) return;
    const int tg = (int)(idx / pieces), c = (int)(idx - (long long)tg * pieces) * VN;
    const int t0 = tg * kDxTokens;
    float s[kDxTokens][VN];
#pragma unroll
    for (int u = 0; u < kDxTokens; ++u)
#pragma unroll
        for (int i = 0; i < VN; ++i) s[u][i] = 0.0f;
    for (int e0 = 0; e0 < E; e0 += 4) {
        // a batch of 4 experts: every load is issued before the first product (experts past E and
        // tokens past T re-read the last one; the former with a zero factor, the latter unstored)
        float g[kDxTokens][4];
        float4 w[4][VN / 4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = min(e0 + j, E - 1);
#pragma unroll
            for (int q = 0; q < VN / 4; ++q) w[j][q] = *reinterpret_cast<const float4*>(wr + (size_t)e * d + c + 4 * q);
#pragma unroll
            for (int u = 0; u < kDxTokens; ++u) {
                const float v = dlogits[(size_t)min(t0 + u, T - 1) * E + e];
                g[u][j] = e0 + j < E ? v : 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int u = 0; u < kDxTokens; ++u)
#pragma unroll
                for (int q = 0; q < VN / 4; ++q) {
                    s[u][4 * q + 0] = fmaf(g[u][j], w[j][q].x, s[u][4 * q + 0]);
                    s[u][4 * q + 1] = fmaf(g[u][j], w[j][q].y, s[u][4 * q + 1]);
                    s[u][4 * q + 2] = fmaf(g[u][j], w[j][q].z, s[u][4 * q + 2]);
                    s[u][4 * q + 3] = fmaf(g[u][j], w[j][q].w, s[u][4 * q + 3]);
                }
    }
#pragma unroll
    for (int u = 0; u < kDxTokens; ++u)
        if (t0 + u < T) Vec16<XT>::store(dxr + (size_t)(t0 + u) * d + c, s[u]);
}

// ---------------------------------------------------------------------------
// RmsNorm::backward (src/norm.rs:63-121) behind the layer's own backward pass, with the block's residual
// gradient added on the way out (src/transformer_block.rs:258-263): one wave per row,
//   inverse_rms = 1 / sqrt(mean(x^2) + eps),  projection = sum_j up_j w_j x_j,
//   dx_j = up_j w_j inverse_rms - x_j projection inverse_rms^3 / d  (+ residual_grad_j).
// The inverse rms of every row is kept for the scale gradient, which is summed in the reference's tiles of 32
// rows: partial[tile][c] = sum over the tile's rows of up * x * inverse_rms, tiles added in order afterwards.
// ---------------------------------------------------------------------------
template <typename XT, typename V>
__global__ __launch_bounds__(256) void rmsnorm_backward_kernel(const XT* __restrict__ x, const XT* __restrict__ up,
                                                               const float* __restrict__ weight, float eps,
                                                               const XT* residual_grad, int T, int d,
                                                               XT* grad_input, float* __restrict__ inv_rms) {
    constexpr int VN = V::N;
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const XT* xr = x + (size_t)t * d;
    const XT* ur = up + (size_t)t * d;
    float sumsq = 0.0f, proj = 0.0f;
    for (int c = lane * VN; c < d; c += 64 * VN) {
        float xv[VN], uv[VN];
        V::load(xr + c, xv);
        V::load(ur + c, uv);
#pragma unroll
        for (int i = 0; i < VN; ++i) {
            sumsq = fmaf(xv[i], xv[i], sumsq);
            proj = fmaf(uv[i] * weight[c + i], xv[i], proj);
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        sumsq += __shfl_xor(sumsq, o);
        proj += __shfl_xor(proj, o);
    }
    const float inv = 1.0f / sqrtf(sumsq / (float)d + eps);
    const float shared = proj * (inv * inv * inv) / (float)d;
    if (lane == 0) inv_rms[t] = inv;
    for (int c = lane * VN; c < d; c += 64 * VN) {
        float xv[VN], uv[VN], o[VN];
        V::load(xr + c, xv);
        V::load(ur + c, uv);
#pragma unroll
        for (int i = 0; i < VN; ++i) o[i] = uv[i] * weight[c + i] * inv - xv[i] * shared;
        if (residual_grad) {  // uniform
            float rv[VN];
            V::load(residual_grad + (size_t)t * d + c, rv);
#pragma unroll
            for (int i = 0; i < VN; ++i) o[i] += rv[i];
        }
        V::store(grad_input + (size_t)t * d + c, o);
    }
}

constexpr int kNormTileRows = 32;  // ROWS_PER_TILE, src/norm.rs:14

template <typename XT>
__global__ __launch_bounds__(128) void rmsnorm_wgrad_partial_kernel(const XT* __restrict__ x, const XT* __restrict__ up,
                                                                    const float* __restrict__ inv_rms, int T, int d,
                                                                    float* __restrict__ partial) {
    const int c = (blockIdx.x * 128 + threadIdx.x) * 2;
    if (c >= d) return;  // d is even
    const int tile = blockIdx.y;
    const int t0 = tile * kNormTileRows, t1 = min(T, t0 + kNormTileRows);
    float a0 = 0.0f, a1 = 0.0f;
#pragma unroll 4
    for (int t = t0; t < t1; ++t) {
        const float2 xp = load_pair(x + (size_t)t * d + c);
        const float2 upv = load_pair(up + (size_t)t * d + c);
        const float s = inv_rms[t];
        a0 += upv.x * xp.x * s;
        a1 += upv.y * xp.y * s;
    }
    *reinterpret_cast<float2*>(partial + (size_t)tile * d + c) = make_float2(a0, a1);
}

// ---------------------------------------------------------------------------
// The same three sums for rows of any width, one output element per thread (the order of the
// additions inside an element is the one of the kernels above: tokens, experts, rows in sequence).
// ---------------------------------------------------------------------------
template <typename XT>
__global__ __launch_bounds__(256) void router_grad_partial_any_kernel(const float* __restrict__ dlogits,
                                                                      const XT* __restrict__ x, int T, int d, int E,
                                                                      int chunk_tokens, float* __restrict__ partial) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= d) return;
    const int chunk = blockIdx.y, e = blockIdx.z;
    const int t0 = chunk * chunk_tokens, t1 = min(T, t0 + chunk_tokens);
    float acc = 0.0f;
    for (int t = t0; t < t1; ++t) acc = fmaf(dlogits[(size_t)t * E + e], to_f32(x[(size_t)t * d + c]), acc);
    partial[((size_t)chunk * E + e) * d + c] = acc;
}

template <typename XT>
__global__ __launch_bounds__(256) void router_dx_any_kernel(const float* __restrict__ dlogits,
                                                            const float* __restrict__ wr, int T, int d, int E,
                                                            XT* __restrict__ dxr) {
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)T * d) return;
    const int t = (int)(idx / d), c = (int)(idx - (long long)t * d);
    float acc = 0.0f;
    for (int e = 0; e < E; ++e) acc = fmaf(dlogits[(size_t)t * E + e], wr[(size_t)e * d + c], acc);
    dxr[idx] = from_f32<XT>(acc);
}

template <typename XT>
__global__ __launch_bounds__(256) void rmsnorm_wgrad_partial_any_kernel(const XT* __restrict__ x,
                                                                        const XT* __restrict__ up,
                                                                        const float* __restrict__ inv_rms, int T, int d,
                                                                        float* __restrict__ partial) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= d) return;
    const int tile = blockIdx.y;
    const int t0 = tile * kNormTileRows, t1 = min(T, t0 + kNormTileRows);
    float a = 0.0f;
    for (int t = t0; t < t1; ++t) a += to_f32(up[(size_t)t * d + c]) * to_f32(x[(size_t)t * d + c]) * inv_rms[t];
    partial[(size_t)tile * d + c] = a;
}

__global__ __launch_bounds__(256) void fill_f32_kernel(float* p, float v, long long n) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = v;
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
bool backward_width_ok(int d, bool bf16) { return d > 0 && d % (bf16 ? 8 : 4) == 0; }

hipError_t launch_scale_rows(const void* gout, const void* y, const int* perm_slot, const int* perm_token,
                             const float* gate_of, const int* offsets, int E, int d, int max_rows, void* dy,
                             float* grad_gates, bool bf16, hipStream_t s) {
    if (max_rows <= 0) return hipSuccess;
    const dim3 grid((max_rows + 3) / 4), block(256);
    auto go = [&](auto tag, auto piece) {
        using XT = decltype(tag);
        using V = decltype(piece);
        hipLaunchKernelGGL((scale_rows_kernel<XT, V>), grid, block, 0, s, static_cast<const XT*>(gout),
                           static_cast<const XT*>(y), perm_slot, perm_token, gate_of, offsets, E, d,
                           static_cast<XT*>(dy), grad_gates);
    };
    const bool wide = backward_width_ok(d, bf16);
    if (bf16) { if (wide) go(bf16_t{}, Vec16<bf16_t>{}); else go(bf16_t{}, Vec1<bf16_t>{}); }
    else { if (wide) go(float{}, Vec16<float>{}); else go(float{}, Vec1<float>{}); }
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
    const float* const cP = P;
    auto go = [&](auto gc) {
        constexpr int G = decltype(gc)::value;
        const long long threads = (long long)T * G;
        hipLaunchKernelGGL(route_backward_kernel<G>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, cP, lse,
                           expert_of, grad_gates, counts, offsets, T, E, k, w_aux, w_z, dlogits);
    };
    if (E <= 16) go(std::integral_constant<int, 16>{});
    else if (E <= 32) go(std::integral_constant<int, 32>{});
    else go(std::integral_constant<int, 64>{});
    return hipGetLastError();
}

// Rows up to which the router's weight gradient runs in one launch: at most kRouterGradMaxChunks chunks, a chunk's
// logit gradients (tokens x kRouterGradExperts floats) held in 48 KiB of LDS.
int router_grad_max_tokens() {
    return kRouterGradMaxChunks * (int)((48 * 1024 / sizeof(float) / kRouterGradExperts) / 32 * 32);
}

// chunks of partial sums a layer of up to `max_tokens` rows needs room for
int router_grad_chunks(int max_tokens) { return std::min(kRouterGradMaxChunks, (std::max(max_tokens, 1) + 31) / 32); }

hipError_t launch_router_grad(const float* dlogits, const void* x, const float* wr, int T, int d, int E,
                              float* partial, float* grad_router, void* dxr, bool bf16, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    const int ct = router_grad_chunk_tokens(T);
    const int chunks = (T + ct - 1) / ct;
    if (!backward_width_ok(d, bf16)) {
        const dim3 ga((d + 255) / 256, chunks, E), gd((unsigned)(((long long)T * d + 255) / 256));
        if (bf16) {
            hipLaunchKernelGGL(router_grad_partial_any_kernel<bf16_t>, ga, dim3(256), 0, s, dlogits,
                               static_cast<const bf16_t*>(x), T, d, E, ct, partial);
            hipLaunchKernelGGL(router_dx_any_kernel<bf16_t>, gd, dim3(256), 0, s, dlogits, wr, T, d, E,
                               static_cast<bf16_t*>(dxr));
        } else {
            hipLaunchKernelGGL(router_grad_partial_any_kernel<float>, ga, dim3(256), 0, s, dlogits,
                               static_cast<const float*>(x), T, d, E, ct, partial);
            hipLaunchKernelGGL(router_dx_any_kernel<float>, gd, dim3(256), 0, s, dlogits, wr, T, d, E,
                               static_cast<float*>(dxr));
        }
        hipLaunchKernelGGL(router_grad_reduce_kernel, dim3((E * d + 63) / 64), dim3(256), 0, s, partial, chunks, E * d,
                           grad_router);
        return hipGetLastError();
    }
    const dim3 g1((d / 2 + 127) / 128, chunks, (E + kRouterGradExperts - 1) / kRouterGradExperts), b1(128);
    const size_t lds = (size_t)ct * kRouterGradExperts * sizeof(float);
    if (lds > 48 * 1024) return hipErrorInvalidValue;  // 768 tokens a chunk: beyond 196608 tokens a launch
    const long long pieces = (long long)((T + kDxTokens - 1) / kDxTokens) * (d / (bf16 ? 8 : 4));
    if (bf16) {
        hipLaunchKernelGGL(router_grad_partial_kernel<bf16_t>, g1, b1, lds, s, dlogits,
                           static_cast<const bf16_t*>(x), T, d, E, ct, partial);
        hipLaunchKernelGGL(router_dx_kernel<bf16_t>, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, s, dlogits,
                           wr, T, d, E, static_cast<bf16_t*>(dxr));
    } else {
        hipLaunchKernelGGL(router_grad_partial_kernel<float>, g1, b1, lds, s, dlogits, static_cast<const float*>(x),
                           T, d, E, ct, partial);
        hipLaunchKernelGGL(router_dx_kernel<float>, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, s, dlogits,
                           wr, T, d, E, static_cast<float*>(dxr));
    }
    hipLaunchKernelGGL(router_grad_reduce_kernel, dim3((E * d + 63) / 64), dim3(256), 0, s, partial, chunks, E * d,
                       grad_router);
    return hipGetLastError();
}

int rmsnorm_grad_tiles(int T) { return (std::max(T, 1) + kNormTileRows - 1) / kNormTileRows; }

hipError_t launch_rmsnorm_backward(const void* x, const void* up, const float* weight, float eps,
                                   const void* residual_grad, int T, int d, void* grad_input, float* inv_rms,
                                   float* partial, float* grad_weight, bool bf16, hipStream_t s) {
    if (T <= 0) return hipSuccess;
    const dim3 g1((T + 3) / 4), b1(256);
    const int tiles = rmsnorm_grad_tiles(T);
    const bool wide = backward_width_ok(d, bf16);
    auto go = [&](auto tag, auto piece) {
        using XT = decltype(tag);
        using V = decltype(piece);
        hipLaunchKernelGGL((rmsnorm_backward_kernel<XT, V>), g1, b1, 0, s, static_cast<const XT*>(x),
                           static_cast<const XT*>(up), weight, eps, static_cast<const XT*>(residual_grad), T, d,
                           static_cast<XT*>(grad_input), inv_rms);
        if (V::N > 1)
            hipLaunchKernelGGL(rmsnorm_wgrad_partial_kernel<XT>, dim3((d / 2 + 127) / 128, tiles), dim3(128), 0, s,
                               static_cast<const XT*>(x), static_cast<const XT*>(up), inv_rms, T, d, partial);
        else
            hipLaunchKernelGGL(rmsnorm_wgrad_partial_any_kernel<XT>, dim3((d + 255) / 256, tiles), dim3(256), 0, s,
                               static_cast<const XT*>(x), static_cast<const XT*>(up), inv_rms, T, d, partial);
    };
    if (bf16) { if (wide) go(bf16_t{}, Vec16<bf16_t>{}); else go(bf16_t{}, Vec1<bf16_t>{}); }
    else { if (wide) go(float{}, Vec16<float>{}); else go(float{}, Vec1<float>{}); }
    hipLaunchKernelGGL(router_grad_reduce_kernel, dim3((d + 63) / 64), dim3(256), 0, s, partial, tiles, d, grad_weight);
    return hipGetLastError();
}

// out[i] = bf16(in[i]) (nearest even), 8 elements per thread; n a multiple of 8
__global__ __launch_bounds__(256) void cast_rows_bf16_kernel(const float* __restrict__ in, bf16_t* __restrict__ out,
                                                             long long n8) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    const float4 a = reinterpret_cast<const float4*>(in)[2 * i], b = reinterpret_cast<const float4*>(in)[2 * i + 1];
    uint4 o;
    o.x = f32_to_bf16_bits(a.x) | ((uint32_t)f32_to_bf16_bits(a.y) << 16);
    o.y = f32_to_bf16_bits(a.z) | ((uint32_t)f32_to_bf16_bits(a.w) << 16);
    o.z = f32_to_bf16_bits(b.x) | ((uint32_t)f32_to_bf16_bits(b.y) << 16);
    o.w = f32_to_bf16_bits(b.z) | ((uint32_t)f32_to_bf16_bits(b.w) << 16);
    reinterpret_cast<uint4*>(out)[i] = o;
}

hipError_t launch_cast_rows_bf16(const float* in, void* out, long long n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    if (n % 8 != 0) return hipErrorInvalidValue;
    const long long n8 = n / 8;
    hipLaunchKernelGGL(cast_rows_bf16_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, s, in,
                       static_cast<bf16_t*>(out), n8);
    return hipGetLastError();
}

hipError_t launch_fill_f32(float* p, float v, long long n, hipStream_t s) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(fill_f32_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, p, v, n);
    return hipGetLastError();
}

}  // namespace rbmoe
