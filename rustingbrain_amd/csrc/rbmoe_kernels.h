// Launch interfaces between the C ABI (rbmoe_api.hip) and the kernel files.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <stddef.h>
#include <stdint.h>

#include "rbmoe_device.h"

namespace rbmoe {

// A kernel attribute is set once per device.  `done` has one bit per device; setting an attribute twice is
// harmless, so two threads that race here only repeat the call.  Devices past the 64th set it on every launch.
template <typename F>
inline hipError_t once_per_device(std::atomic<unsigned long long>& done, F&& set) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned long long bit = dev < 64 ? 1ull << dev : 0ull;
    if (bit && (done.load(std::memory_order_acquire) & bit)) return hipSuccess;
    e = set();
    if (e == hipSuccess && bit) done.fetch_or(bit, std::memory_order_release);
    return e;
}


// Kernel durations the way a kernel trace reports them: while a KernelTimer is installed on the calling thread,
// every forward-path launch below carries its own start and stop events (hipExtLaunchKernelGGL), which receive the
// begin and end time stamps of that dispatch itself - no launch gap, no event-pair overhead.  Up to kMaxTimedLaunches
// launches per timer; further ones are plain launches.
constexpr int kMaxTimedLaunches = 4;
struct KernelTimer {
    hipEvent_t ev[2 * kMaxTimedLaunches] = {};
    int used = 0;
};
extern thread_local KernelTimer* g_kernel_timer;  // null (the default): plain launches
#define RB_LAUNCH(kernel, grid, block, lds, stream, ...)                                                        \
    do {                                                                                                        \
        ::rbmoe::KernelTimer* const kt_ = ::rbmoe::g_kernel_timer;                                              \
        if (kt_ != nullptr && kt_->used < ::rbmoe::kMaxTimedLaunches) {                                         \
            hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, kt_->ev[2 * kt_->used],                     \
                                  kt_->ev[2 * kt_->used + 1], 0, __VA_ARGS__);                                  \
            ++kt_->used;                                                                                        \
        } else {                                                                                                \
            hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                                  \
        }                                                                                                       \
    } while (0)

// Tokens owned by one router / dispatch block.  Slots are numbered
// token * k + rank, so a block owns a contiguous slot range.
constexpr int kRouterTokens = 32;
constexpr int kRouterThreads = 512;     // router_kernel workgroup
constexpr int kRouterWaves = kRouterThreads / 64;

// Largest expert count and top-k the routing kernels are laid out for.
constexpr int kMaxExperts = 256;
constexpr int kMaxTopK = 32;

size_t router_lds_bytes(int E, int k);
constexpr int kMaxRouterLds = 160 * 1024;  // LDS per workgroup on gfx950
size_t dispatch_lds_bytes(int E, int k);

struct RouterArgs {
    const void* x;       // [T, d] f32 or bf16
    const float* wr;     // [E, d] f32
    const float* bias;   // [E] or null
    const uint8_t* valid;  // [T] or null
    int T, d, E, k;
    float* P;            // [T, E]
    float* lse;          // [T]
    int* expert_of;      // [T*k]
    float* gate_of;      // [T*k]
    int* rank_in_block;  // [T*k]
    int* blockcnt;       // [nb, E]
    float* partial;      // [nb, E+1]
    void* rows16 = nullptr;  // f32 rows only: [T, d] bf16 copy of x written on the way (d a multiple of 8), or null
    bool allow_fused = true; // logits and everything behind them in one launch where the shapes allow
    // a quantized router (Quantized::matmul_rhs_transposed, src/quantized.rs:55-62): int8 rows and one scale per row;
    // `wr` is then not read and the logits are (sum_c x[c] * f32(q[c]), in the reference's 32 lanes) * scale
    const int8_t* wq = nullptr;      // [E, d]
    const float* wscale = nullptr;   // [E]
};
hipError_t launch_router(const RouterArgs& a, bool bf16, hipStream_t s);

struct DispatchArgs {
    const void* x;
    const int* expert_of;
    const int* rank_in_block;
    const int* blockcnt;   // [nb, E]    per-block histogram from the router kernel
    const float* partial;  // [nb, E+1]  per-block sums of probabilities and of lse^2
    int T, d, E, k;
    float w_aux, w_z;
    int tile_m;            // rows per tile of the grouped products
    int* counts;           // [E]
    int* offsets;          // [E+1]
    int* tile_expert;      // [max_tiles]
    int* tile_row0;
    int* tile_rows;
    int* ntiles;           // [1]
    float* losses;         // [2]
    int* blockbase;        // [nb, E]  scratch: slots of expert e routed by the blocks before block b
    int* perm_slot;
    int* perm_token;
    int* inv_pos;
    void* xg;  // [T*k, d] or null (rows are then gathered by the consumer)
};
hipError_t launch_dispatch(const DispatchArgs& a, bool bf16, hipStream_t s);

struct CombineArgs {
    const void* y;        // [R, d] expert output rows, activation dtype
    const void* yshared;  // [T, d] or null
    const void* residual; // [T, d] or null
    const int* inv_pos;   // [T*k]
    const float* gate_of; // [T*k]
    int T, d, k;
    void* out;            // [T, d]
    bool rows_bf16 = false;  // under f32 activations: y and yshared are bf16 (matrix-core products of a bf16 / int8 layer)
};
hipError_t launch_combine(const CombineArgs& a, bool bf16, hipStream_t s);

// RmsNorm::forward (src/norm.rs:41-61) over rows: out = (x * inverse_rms(row)) * weight, the sum of squares in
// index order
hipError_t launch_rmsnorm(const void* x, const float* weight, float eps, int T, int d, void* out, bool bf16,
                          hipStream_t s);

// ---------------------------------------------------------------------------
// Grouped expert products.  Rows of `a` are grouped by expert through the tile
// table written by the scan kernel; a tile never spans two experts.
//   out[row, n] = sum_c a[row, c] * w[expert][n, c]        (SWIGLU = false)
//   out[row, n] = silu(a . wg[n]) * (a . wu[n])            (SWIGLU = true; the
//       expert's weight block holds the F gate rows, then the F up rows)
// int8 weights carry one f32 scale per weight row; the product is
// (sum_c a*q) * scale as in the reference (src/quantized.rs:55-62).
// ---------------------------------------------------------------------------
enum class WeightKind : int { F32 = 0, BF16 = 1, I8 = 2 };

struct GroupedArgs {
    const void* a;          // [rows, K] activation dtype
    const int* row_index;   // null: row r of a tile is a[row0 + r]; else a[row_index[row0 + r]]
    const void* w;          // expert 0's weight block
    size_t w_expert_stride; // elements between experts
    const float* scales;    // int8: expert 0's scales, one per weight row
    size_t s_expert_stride;
    int N;                  // output columns (F for SWIGLU, d for the down product)
    int K;
    const int* tile_expert;
    const int* tile_row0;
    const int* tile_rows;
    const int* ntiles;
    int max_tiles;
    int dense_rows;         // >= 0: one group of this many rows, no tile table (shared expert)
    void* out;              // [rows, N] activation dtype
    void* gu_out = nullptr; // gate/up launches: [rows, 2N] pre-activations (gate | up) kept for a backward pass
    // down-shaped launches: [rows, 2N] pre-activations of the forward pass.  The product rows are
    // then taken as the gradient of the hidden rows and SwiGLU's backward is applied on the way out: the
    // gradients of the pre-activations go to `gu_out` [rows, 2N] and `out` is not written.
    const void* swiglu_grad_gu = nullptr;
    bool swiglu;
    int group_m;            // MFMA path: M-tiles per scheduling group (0 = default)
    int tile_m = 0;         // f32 matrix-core path: rows per tile of the tile table (64 or 32)
};
hipError_t launch_grouped_generic(const GroupedArgs& a, bool act_bf16, WeightKind wk, int tile_m,
                                  hipStream_t s);
constexpr int kGenericTileM = 16;

// bf16 matrix-core path (bf16 activations; bf16 or int8 weights): weights repacked into
// matrix-core operand order (pack_weight_*) and streamed global -> registers, activations
// global -> LDS by DMA.  `w` must have been packed matrix by matrix.
int stream_tile_m();
bool stream_shape_ok(int N, int K);
hipError_t launch_grouped_stream(const GroupedArgs& a, WeightKind wk, hipStream_t s);
void pack_weight_bf16(const uint16_t* src, int rows, int cols, uint16_t* dst);
void pack_weight_i8(const int8_t* src, int rows, int cols, int8_t* dst);

// f32 matrix cores (all-f32 layers): 64-row tiles, plain row-major weights.
int f32_tile_m(int rows, int groups, int n_min);  // tile height (64 or 32) for a batch of `rows` routed rows in `groups` groups; n_min: the narrower product's width
bool f32_shape_ok(int N, int K);
hipError_t launch_grouped_f32(const GroupedArgs& a, hipStream_t s);

// ---- backward pass: the kernels around the matrix products (backward_kernels.hip) --------
// dy[pos] = gate * gout[token(pos)], grad_gates[slot] = gout[token] . y[pos]; row widths: multiples of 16 bytes
hipError_t launch_scale_rows(const void* gout, const void* y, const int* perm_slot, const int* perm_token,
                             const float* gate_of, const int* offsets, int E, int d, int max_rows, void* dy,
                             float* grad_gates, bool bf16, hipStream_t s);
// out[e][M][N] += A_e^T . B_e over the rows of group e (counts/offsets), or over dense_rows rows when >= 0
hipError_t launch_grouped_tn(const void* a, int M, const void* b, const int* b_row_index, int N, const int* counts,
                             const int* offsets, int groups, int dense_rows, float* out, size_t out_expert_stride,
                             bool bf16, hipStream_t s);

// Weight gradients on the matrix cores (bf16 or f32 operands): out[e] += A_e^T . B_e with the rows of a group cut into
// chunks.  How an expert far above the average share is handled:
//   None     one chunk per expert (a skewed load then serialises the launch)
//   Ordered  cut into several chunks; the first adds in place, the others store partial matrices (`partial`) that
//            a second kernel adds in chunk order: identical bits run to run
//   Atomic   cut into several chunks that all add with f32 atomics, in whatever order they arrive
// `overwrite`: out is known to hold zeros, whatever its bytes are, and is written instead of added to.
// `chunks` is scratch of weight_grad_table_ints(...) ints, `partial` of weight_grad_partial_bytes(...) bytes
// (a smaller buffer is legal: the launch then cuts less).
enum class WgradSplit : int { None = 0, Ordered = 1, Atomic = 2 };
bool weight_grad_shape_ok(int M, int N, bool bf16);
int weight_grad_max_chunks(int groups, int total_rows);
int weight_grad_table_ints(int groups, int total_rows);
size_t weight_grad_partial_bytes(int M, int N, int groups, int dense_rows, int total_rows, bool bf16);
// ... for a buffer that serves every launch of 1 .. max_tokens tokens (rows_per_token rows each; dense: rows = tokens)
size_t weight_grad_partial_bytes_upto(int M, int N, int groups, bool dense, int max_tokens, int rows_per_token,
                                      bool bf16);
// `part`: the chunk table is a launch of its own in front of the product and depends on nothing but counts and
// offsets - a caller may have it computed early, on another stream (TableOnly), and later issue the product with
// the same arguments (ProductOnly) once that launch has completed.
enum class WgradPart : int { Both = 0, TableOnly = 1, ProductOnly = 2 };
hipError_t launch_weight_grad(const void* a, int M, const void* b, int N, const int* counts, const int* offsets,
                              int groups, int dense_rows, int total_rows, WgradSplit split_mode, bool overwrite,
                              int* chunks, float* partial, size_t partial_bytes, float* out, size_t out_expert_stride,
                              bool bf16, hipStream_t s, WgradPart part = WgradPart::Both);

// gates -> probabilities -> logits, with the gradients of the two auxiliary losses
hipError_t launch_route_backward(const float* P, const float* lse, const int* expert_of, const float* grad_gates,
                                 const int* counts, const int* offsets, int T, int E, int k, float w_aux, float w_z,
                                 float* dlogits, hipStream_t s);
// grad_router += dlogits^T . x (through `partial`, router_grad_chunks(max_tokens) * E * d floats) and
// dxr = dlogits . wr
int router_grad_chunks(int max_tokens);
int router_grad_max_tokens();  // launch_router_grad refuses more rows than this
hipError_t launch_router_grad(const float* dlogits, const void* x, const float* wr, int T, int d, int E,
                              float* partial, float* grad_router, void* dxr, bool bf16, hipStream_t s);
// RmsNorm::backward (src/norm.rs:63-121): grad_input = d(norm)/dx applied to `up` (+ residual_grad when given),
// grad_weight += scale gradient (through `partial`, rmsnorm_grad_tiles(max_tokens) * d floats); `inv_rms` [T] scratch
int rmsnorm_grad_tiles(int max_tokens);
hipError_t launch_rmsnorm_backward(const void* x, const void* up, const float* weight, float eps,
                                   const void* residual_grad, int T, int d, void* grad_input, float* inv_rms,
                                   float* partial, float* grad_weight, bool bf16, hipStream_t s);
// out[i] = bf16(in[i]), nearest even; n a multiple of 8
hipError_t launch_cast_rows_bf16(const float* in, void* out, long long n, hipStream_t s);
hipError_t launch_fill_f32(float* p, float v, long long n, hipStream_t s);

// ---- decode-shaped path (a few tokens) -------------------------------------------
constexpr int kSmallRouteMaxTokens = 32;
constexpr int kSmallRouteMaxPairs = 2048;  // T * E
constexpr int kDecodeTileM = 32;

struct SmallRouteArgs {
    const void* x;
    const float* wr;
    const float* bias;
    const uint8_t* valid;
    int T, d, E, k;
    float w_aux, w_z;
    int tile_m;
    float* P;
    float* lse;
    int* expert_of;
    float* gate_of;
    int* counts;
    int* offsets;
    int* tile_expert;
    int* tile_row0;
    int* tile_rows;
    int* ntiles;
    float* losses;
    int* perm_slot;
    int* perm_token;
    int* inv_pos;
    // Optional norm in front of the layer (RmsNorm::forward, src/norm.rs:41-61): `x` holds the raw rows, the
    // kernel normalises them in LDS, routes on the normed rows and writes them to `xn_out` [T, d].  Only for
    // calls whose rows are staged in LDS (small_route_stages_rows).
    const float* norm_w = nullptr;
    float norm_eps = 0.0f;
    void* xn_out = nullptr;
    // f32 rows only: a bf16 copy [T, d] of the rows the routing is decided on (after the norm, if any), for the
    // matrix-core products; only for calls whose rows are staged in LDS (small_route_stages_rows)
    void* rows16 = nullptr;
    // launch_decode_front only, or null: [E] the tokens every expert takes, one bit a token (at most 32 tokens); the
    // expert's rows are these tokens in ascending order
    unsigned int* expert_tokens = nullptr;
};
bool small_route_stages_rows(const void* x, const float* wr, int T, int d, int E, bool bf16);
bool small_route_ok(int T, int E, int k);
hipError_t launch_route_small(const SmallRouteArgs& a, bool bf16, hipStream_t s);

// One launch covers the routed tiles (<= 32 rows each) and, when a_shared is set, the shared
// expert over rows [0, T_shared).  Weights are in the packed layout of pack_weight_*.
struct DecodeGemmArgs {
    const void* a;
    const int* row_index;
    const void* w;
    size_t w_expert_stride;  // elements
    const float* scales;
    size_t s_expert_stride;
    int N, K;
    const int* tile_expert;
    const int* tile_row0;
    const int* tile_rows;
    const int* ntiles;
    int max_tiles;
    void* out;
    int a_expert_rows = 0;  // rows of `a` per expert: a routed row r of expert e is a[e * a_expert_rows + row]
    const void* a_shared;
    const void* w_shared;
    const float* scales_shared;
    int N_shared, K_shared, T_shared;
    void* out_shared;
    int swiglu;
    // Down-shaped launches only, all null / zero otherwise: the combine folded into the launch.  The last workgroup
    // of a feature block to finish (one counter per block of 32 output features: zero before the launch, zero
    // again after it) sums that block's columns for every token - the token's expert rows in ascending expert order,
    // a rounded multiply by the gate and a rounded add each, then the shared expert's row, then the residual - and
    // writes them to cmb_out.  Nobody waits for anybody: whoever arrives last does the work.
    int* cmb_counter = nullptr;           // block b's counter at [b * kDecodeCombineCounterStride]
    const int* cmb_inv_pos = nullptr;     // [T * k]
    const float* cmb_gate_of = nullptr;   // [T * k]
    const void* cmb_residual = nullptr;   // [T, N] bf16, or f32 when cmb_f32, or null
    void* cmb_out = nullptr;              // [T, N] bf16, or f32 when cmb_f32; null: no combine in this launch
    int cmb_T = 0, cmb_k = 0;
    int cmb_f32 = 0;
};
constexpr int kDecodeCombineMaxBlocks = 1024;  // feature blocks a folded combine has counters for
// ints between two blocks' counters: every block's arrivals go to a cache line - and an L2 channel - of their own
// (side by side in one line, the atomics of a launch's two hundred workgroups queue up behind one another)
constexpr int kDecodeCombineCounterStride = 64;
constexpr size_t kDecodeCombineCounterBytes = (size_t)kDecodeCombineMaxBlocks * kDecodeCombineCounterStride * 4;
bool decode_shape_ok(int N, int K);
hipError_t launch_decode_gemm(const DecodeGemmArgs& g, WeightKind wk, hipStream_t s);
// Routing and gate/up products in one launch (bf16 rows, no norm): every expert's gate/up product over all T rows,
// hidden rows to g.out as [E][T, N]; the shared expert as in launch_decode_gemm.  g.a / g.a_shared: the T rows.
bool decode_front_ok(const void* x, const float* wr, int T, int d, int E, int k);
hipError_t launch_decode_front(const SmallRouteArgs& r, const DecodeGemmArgs& g, WeightKind wk, hipStream_t s);
// The down product behind launch_decode_front with the combine folded in (g as for launch_decode_gemm: cmb_* set,
// a_expert_rows = tokens of the call), one row of workgroups per EXPERT instead of per entry of the tile table: a
// workgroup knows its weights from its place in the grid and requests them at once, and learns its rows from
// expert_tokens / offsets / g.ntiles behind them.  An expert without rows costs its weights' bytes.
bool decode_down_by_expert_ok(const DecodeGemmArgs& g, int E, int T, int k);
hipError_t launch_decode_down_by_expert(const DecodeGemmArgs& g, const unsigned int* expert_tokens, const int* offsets,
                                        int E, WeightKind wk, hipStream_t s);

}  // namespace rbmoe
