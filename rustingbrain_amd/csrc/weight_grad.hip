// Weight gradients of the expert matrices on the bf16 matrix cores of gfx950
// (Linear::backward, src/param.rs:819-821: weight.grad += grad_output^T . input):
//
//   out[e][m][n] += sum over the rows r of expert e of  A[r][m] * B[r][n]
//
// Both operands are stored row by row (m and n contiguous), while the matrix cores want, per
// lane, consecutive elements of the reduction dimension, here the ROW index.  The tiles go to
// LDS as they are (16-byte pieces, rows padded so that the eight rows a wave reads at once
// fall in distinct bank groups), and the fragment reads use the transposing LDS read
// (ds_read_b64_tr_b16): in a group of 16 lanes, lane 4 j + q supplies the address of four
// consecutive 16-bit elements and lane 4 q + e receives element e of the pieces of lanes
// q, 4 + q, 8 + q, 12 + q - so pointing lane 4 j + q at (row r0 + j, columns c0 + 4 q ..) hands
// lane i column c0 + i of rows r0 .. r0 + 3, four consecutive reduction elements.
//
// A workgroup of 8 waves (4 x 2) owns 256 (m) x 256 (n) outputs of one CHUNK of one expert's rows;
// a wave owns 64 x 128 (2 x 4 accumulator blocks of 32 x 32).  Rows go through LDS 32 at a
// time, double buffered; the global loads run three stages ahead in three register sets, so a
// load has two full stages of products to arrive in.  An expert with many more rows than the
// others is cut into several chunks so that the launch stays balanced.  The sums of a cut expert's
// chunks meet in a fixed order (the reference's convention for reductions, src/norm.rs:8-14): the first
// chunk adds in place like an expert's only chunk, every further chunk stores its tile sums into a
// partial matrix of its own, and a second kernel adds the partial matrices to the gradient in chunk
// order - two runs give identical bits.  (Opt-in alternative: the chunks add into the gradient with
// hardware f32 atomics, in whatever order they arrive.)  When the caller knows that the gradient is
// zero (first backward pass after it was cleared), a first chunk stores instead of adding, and only
// the experts without rows are cleared beforehand.
#include "rbmoe_kernels.h"

namespace rbmoe {

namespace {

constexpr int GM = 256;            // outputs along m per workgroup
constexpr int GN = 256;            // outputs along n per workgroup
constexpr int GR = 32;             // rows per LDS stage
constexpr int GT = 512;            // threads per workgroup
constexpr int GAS = GM * 2 + 64;   // LDS row pitch of the A tile in bytes: 64 mod 256
constexpr int GBS = GN * 2 + 64;   // same for the B tile
constexpr int GSTAGE = GR * (GAS + GBS);
constexpr int GDEPTH = 3;          // register sets of loads in flight

typedef short v4i16 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4i16 lds_v4i16;

__device__ __forceinline__ bf16x8 tr_fragment(const char* p, int pitch) {
    union {
        v4i16 h[2];
        bf16x8 v;
    } u;
    u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16*)(p));
    u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16*)(p + 4 * pitch));
    return u.v;
}

// A wave's NI x NJ accumulator blocks of 32 x 32 go into the gradient.  Accumulator element v of lane
// l: m = 8 (v / 4) + 4 (l / 32) + v % 4, n = l % 32 of the block.  The only chunk of an expert owns its
// elements: it reads the 16 values of a block, adds, and stores (M is a multiple of 4, so a group of 4
// rows is inside or outside as a whole) - or just stores when the gradient is known to be zero.  The chunks
// of a cut expert meet on the same elements and add with no-return f32 atomics.
// mode: 0 = add in place (or store when `overwrite`), 1 = atomic add, 2 = plain store (`o` is then the chunk's
// partial matrix).
template <int NI, int NJ>
__device__ __forceinline__ void add_tiles(const floatx16 (&acc)[NI][NJ], float* __restrict__ o, int M, int N, int mw,
                                          int nw, int lane, int mode, bool overwrite) {
    const bool split = mode == 1;
    overwrite = overwrite || mode == 2;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const int mb = mw + i * 32 + 4 * (lane >> 5);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int n = nw + j * 32 + (lane & 31);
            if (n >= N) continue;
            float* const base = o + (size_t)mb * N + n;
            if (split) {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (mb + 8 * (v >> 2) < M) unsafeAtomicAdd(base + (size_t)(8 * (v >> 2) + (v & 3)) * N, acc[i][j][v]);
            } else if (overwrite) {
                // (the gradient is read again only by the optimiser: stored past the caches, which hold the
                // operand rows that other workgroups are still reading)
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (mb + 8 * (v >> 2) < M)
                        __builtin_nontemporal_store(acc[i][j][v], base + (size_t)(8 * (v >> 2) + (v & 3)) * N);
            } else {
                float old[16];
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (mb + 8 * (v >> 2) < M)
                        old[v] = __builtin_nontemporal_load(base + (size_t)(8 * (v >> 2) + (v & 3)) * N);
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (mb + 8 * (v >> 2) < M)
                        __builtin_nontemporal_store(old[v] + acc[i][j][v], base + (size_t)(8 * (v >> 2) + (v & 3)) * N);
            }
        }
    }
}

// The tile [m0, m0 + tm) x [n0, n0 + tn) of an expert without rows, in a launch that overwrites: zeros.
__device__ __forceinline__ void zero_tile(float* __restrict__ o, int M, int N, int m0, int n0, int tm, int tn, int tid,
                                          int threads) {
    const int w4 = tn / 4;  // N is a multiple of 4
    for (int i = tid; i < tm * w4; i += threads) {
        const int m = m0 + i / w4, n = n0 + 4 * (i % w4);
        if (m < M && n < N) *reinterpret_cast<float4*>(o + (size_t)m * N + n) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
}

// chunk table: expert e with c rows gets ceil(c / limit) chunks of equal size (a multiple of 32)
// chunk_split[c]: 0 = the expert's only or first chunk (adds in place), 1 = adds with atomics (`ordered` off),
// 2 + s = stores into partial matrix s; slot_first[e] / slot_count[e]: the partial matrices of expert e, in chunk order
__global__ __launch_bounds__(256) void chunk_table_kernel(const int* __restrict__ counts,
                                                          const int* __restrict__ offsets, int groups,
                                                          int dense_rows, int limit, int max_chunks, int ordered,
                                                          int max_slots, int zero_empty,
                                                          int* __restrict__ chunk_expert, int* __restrict__ chunk_row0,
                                                          int* __restrict__ chunk_rows, int* __restrict__ chunk_split,
                                                          int* __restrict__ nchunks, int* __restrict__ slot_first,
                                                          int* __restrict__ slot_count) {
    __shared__ int scan[256];
    __shared__ int scan_x[256];
    __shared__ int base, base_x;
    const int tid = threadIdx.x;
    if (tid == 0) base = base_x = 0;
    __syncthreads();
    for (int e0 = 0; e0 < groups; e0 += 256) {
        const int e = e0 + tid;
        int rows = 0, row0 = 0;
        if (e < groups) {
            rows = dense_rows >= 0 ? dense_rows : counts[e];
            row0 = dense_rows >= 0 ? 0 : offsets[e];
        }
        // zero_empty: an expert without rows gets one chunk without rows, marked -1: its tiles store zeros
        const bool empty = zero_empty && e < groups && rows <= 0;
        const int n = rows > 0 ? (rows + limit - 1) / limit : (empty ? 1 : 0);
        const int nx = n > 1 ? n - 1 : 0;  // chunks beyond the first
        scan[tid] = n;
        scan_x[tid] = nx;
        __syncthreads();
        for (int o = 1; o < 256; o <<= 1) {
            const int v = tid >= o ? scan[tid - o] : 0;
            const int vx = tid >= o ? scan_x[tid - o] : 0;
            __syncthreads();
            scan[tid] += v;
            scan_x[tid] += vx;
            __syncthreads();
        }
        const int first = base + scan[tid] - n;
        const int first_x = base_x + scan_x[tid] - nx;
        // An ordered cut needs a partial matrix per further chunk.  The launcher sizes the limit so that there is
        // always room; should there not be, the expert is not cut at all (one chunk over all its rows: slower,
        // never wrong), and its unused table entries are empty chunks.
        const bool cut = n > 1 && (!ordered || first_x + nx <= max_slots);
        if (e < groups) {
            slot_first[e] = first_x;
            slot_count[e] = (ordered && cut) ? nx : 0;
        }
        if (n > 0) {
            const int per = cut ? (((rows + n - 1) / n) + 31) & ~31 : rows;
            for (int c = 0; c < n; ++c) {
                if (first + c >= max_chunks) break;
                const int r0 = c * per;
                const int r = max(0, min(per, rows - r0));
                chunk_expert[first + c] = e;
                chunk_row0[first + c] = r > 0 ? row0 + r0 : row0;
                chunk_rows[first + c] = r;
                chunk_split[first + c] = empty ? -1 : !cut ? 0 : (!ordered ? 1 : (c == 0 ? 0 : 2 + first_x + c - 1));
            }
        }
        __syncthreads();
        if (tid == 255) {
            base += scan[255];
            base_x += scan_x[255];
        }
        __syncthreads();
    }
    if (tid == 0) *nchunks = min(base, max_chunks);
}

// out[e] += partial[slot_first[e]] + partial[slot_first[e] + 1] + ... in that order, element by element
__global__ __launch_bounds__(256) void add_partials_kernel(const int* __restrict__ slot_first,
                                                           const int* __restrict__ slot_count,
                                                           const float* __restrict__ partial, size_t elems,
                                                           float* __restrict__ out, size_t out_expert_stride) {
    const int e = blockIdx.y;
    const int ns = slot_count[e];
    if (ns <= 0) return;
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4* const p = reinterpret_cast<const f32x4*>(partial + (size_t)slot_first[e] * elems);
    f32x4* const o = reinterpret_cast<f32x4*>(out + (size_t)e * out_expert_stride);
    const size_t n4 = elems / 4;  // M and N are multiples of 4
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256) {
        f32x4 v = o[i];
        for (int s = 0; s < ns; ++s) v += __builtin_nontemporal_load(p + (size_t)s * n4 + i);  // read once
        o[i] = v;
    }
}

__global__ __launch_bounds__(GT) void weight_grad_kernel(
    const bf16_t* __restrict__ a, int M, const bf16_t* __restrict__ b, int N, int tiles_m, int tiles_n,
    const int* __restrict__ chunk_expert, const int* __restrict__ chunk_row0, const int* __restrict__ chunk_rows,
    const int* __restrict__ chunk_split, const int* __restrict__ nchunks, float* __restrict__ out,
    size_t out_expert_stride, int overwrite, float* __restrict__ partial) {
    extern __shared__ __attribute__((aligned(16))) char lds[];  // 2 * GSTAGE

    // Workgroup i runs on XCD i % 8.  A unit is one chunk's row of tiles (same m, every n): its
    // workgroups share the A columns, so they go to one XCD and its L2; units go to the XCDs in
    // turn, which spreads the long chunks of a cut expert (neighbours in the table) evenly.
    const int idx = (int)(blockIdx.x >> 3);
    const int unit = (int)(blockIdx.x & 7) + 8 * (idx / tiles_n);
    const int ch = unit / tiles_m;
    if (ch >= *nchunks) return;
    const int tile = (unit - ch * tiles_m) * tiles_n + idx % tiles_n;
    const int m0 = (tile / tiles_n) * GM, n0 = (tile % tiles_n) * GN;
    const int rows = chunk_rows[ch];
    const int cs = chunk_split[ch];
    if (rows <= 0) {
        if (cs == -1 && overwrite)
            zero_tile(out + (size_t)chunk_expert[ch] * out_expert_stride, M, N, m0, n0, GM, GN, threadIdx.x, GT);
        return;
    }
    const int row0 = chunk_row0[ch];
    const int mode = cs >= 2 ? 2 : cs;
    float* const o = cs >= 2 ? partial + (size_t)(cs - 2) * M * N : out + (size_t)chunk_expert[ch] * out_expert_stride;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- global -> register -> LDS staging: 16-byte pieces ---------------------
    // each tile: 32 rows x 32 pieces; a thread moves piece tid % 32 of rows tid / 32 and tid / 32 + 16
    const int pc = tid & 31, tr = tid >> 5;
    // columns past the edge: loaded from a valid place, never stored
    const bf16_t* const a_src = a + (size_t)row0 * M + (m0 + 8 * pc < M ? m0 + 8 * pc : 0);
    const bf16_t* const b_src = b + (size_t)row0 * N + (n0 + 8 * pc < N ? n0 + 8 * pc : 0);
    struct Set {
        uint4 a[2], b[2];
    } sets[GDEPTH];
    auto fetch = [&](auto kc, int r0) {
        constexpr int k = decltype(kc)::value;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int r = min(r0 + tr + 16 * i, rows - 1);  // past the end: a valid row, zeroed when staged
            sets[k].a[i] = *reinterpret_cast<const uint4*>(a_src + (size_t)r * M);
            sets[k].b[i] = *reinterpret_cast<const uint4*>(b_src + (size_t)r * N);
        }
    };
    auto stage = [&](auto kc, int buf, int r0) {
        constexpr int k = decltype(kc)::value;
        char* const A = lds + buf * GSTAGE;
        char* const B = A + GR * GAS;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const bool in = r0 + tr + 16 * i < rows;  // rows past the end of the chunk contribute nothing
            *reinterpret_cast<uint4*>(A + (tr + 16 * i) * GAS + pc * 16) = in ? sets[k].a[i] : make_uint4(0, 0, 0, 0);
            *reinterpret_cast<uint4*>(B + (tr + 16 * i) * GBS + pc * 16) = in ? sets[k].b[i] : make_uint4(0, 0, 0, 0);
        }
    };

    floatx16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // lane's share of a fragment read: group of 16 lanes gi covers columns 16 (gi % 2) .. and rows
    // 8 (gi / 2) ..; inside the group lane s points at row s / 4, columns 4 (s % 4) ..
    const int gi = lane >> 4, sl = lane & 15;
    const int frow = 8 * (gi >> 1) + (sl >> 2);
    const int fcol = 16 * (gi & 1) + 4 * (sl & 3);
    const int a_lane = frow * GAS + (wm * 64 + fcol) * 2;
    const int b_lane = frow * GBS + (wn * 128 + fcol) * 2;

    const int nstages = (rows + GR - 1) / GR;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    fetch(I0{}, 0);
    fetch(I1{}, GR);
    fetch(I2{}, 2 * GR);
    stage(I0{}, 0, 0);
    __syncthreads();
    // stage s: its rows are in LDS buffer s % 2; register set s % 3 is free and takes stage s + 3;
    // set (s + 1) % 3 holds stage s + 1, which goes to the other LDS buffer after the products
    auto step = [&](auto kc, int s) {
        constexpr int k = decltype(kc)::value;
        const int buf = s & 1;
        fetch(kc, (s + GDEPTH) * GR);
        const char* const A = lds + buf * GSTAGE;
        const char* const B = A + GR * GAS;
        // both 16-row steps' fragments are requested before the first product: the second step's reads
        // are in flight during the first step's products
        bf16x8 af[GR / 16][2], bf[GR / 16][4];
#pragma unroll
        for (int ks = 0; ks < GR / 16; ++ks) {
#pragma unroll
            for (int i = 0; i < 2; ++i) af[ks][i] = tr_fragment(A + a_lane + ks * 16 * GAS + i * 64, GAS);
#pragma unroll
            for (int j = 0; j < 4; ++j) bf[ks][j] = tr_fragment(B + b_lane + ks * 16 * GBS + j * 64, GBS);
        }
#pragma unroll
        for (int ks = 0; ks < GR / 16; ++ks)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks][i], bf[ks][j], acc[i][j], 0, 0, 0);
        stage(std::integral_constant<int, (k + 1) % GDEPTH>{}, buf ^ 1, (s + 1) * GR);
        __syncthreads();
    };
    // The stage count is rounded up to the number of register sets, so that every trip runs the
    // same straight-line code (a stage past the end holds zeros: staged rows past the chunk are
    // zeroed, and its loads re-read the last row).
    for (int s = 0; s < nstages; s += GDEPTH) {
        step(I0{}, s);
        step(I1{}, s + 1);
        step(I2{}, s + 2);
    }

    add_tiles<2, 4>(acc, o, M, N, m0 + wm * 64, n0 + wn * 128, lane, mode, overwrite != 0);
}

// ---------------------------------------------------------------------------
// The same product with the tiles brought in by LDS-DMA (global_load_lds_dwordx4): no registers, no LDS store
// instructions and no wait between a load and its store.  A wave instruction deposits its 64 pieces of 16 bytes at
// consecutive LDS addresses - two whole tile rows of 512 bytes - so rows cannot be padded apart; instead the lane
// that fills position q of row r fetches piece q ^ 4 (r % 4) of that row, which spreads the four rows a half-wave
// reads at once (the same pieces of rows r0 .. r0 + 3) over all banks.  A fragment read finds column piece p of row r
// at position p ^ 4 (r % 4); r % 4 is the same for every read of a lane.
// Four LDS stages.  A stage is two 16-row steps; the fragments of the step after the current one are requested
// before the current step's products, into a second set of registers.  The one barrier per stage sits between the
// two steps of stage s: in front of it a wave waits for its own (in-order) DMA of stage s + 1, behind it stage
// s + 1 is complete and nobody reads stage s - 1 any more, whose LDS the DMA of stage s + 3 then takes.  The rows of
// the last stage past the chunk's end are fetched from the chunk's last row and then zeroed in LDS by the wave that
// fetched them.  Byte offsets are 32 bits (the launcher checks; larger operands take the kernel above).
// On C3 this is 7 % faster than the kernel above (110 against 119 us for the gate/up gradient with its side
// launches, ordered chunks, overwriting).  Taking out of the kernel above, one at a time, the LDS stores, the load
// latency (a deeper pipeline), the re-reads from L2 (every workgroup reading the same rows) or the wait for the
// fragment reads moves the time by a few percent only: the product's time is the matrix cores' (38 us alone), the
// final stores' (26 us, 138 MB of f32) and the rounds' (594 workgroups of 24 or 52 stages on 256 compute units,
// one at a time) side by side.
constexpr int DSTAGE = GR * (GM + GN) * 2;  // 32 KB
constexpr int DSTAGES = 4;

__device__ __forceinline__ void wg_issue_dma(uint32_t lds_addr, uint32_t byte_off, const void* base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(byte_off), "s"(base) : "memory");
}
template <int N>
__device__ __forceinline__ void wg_wait_outstanding() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

__global__ __launch_bounds__(GT) void weight_grad_dma_kernel(
    const bf16_t* __restrict__ a, int M, const bf16_t* __restrict__ b, int N, int tiles_m, int tiles_n,
    const int* __restrict__ chunk_expert, const int* __restrict__ chunk_row0, const int* __restrict__ chunk_rows,
    const int* __restrict__ chunk_split, const int* __restrict__ nchunks, float* __restrict__ out,
    size_t out_expert_stride, int overwrite, float* __restrict__ partial) {
    extern __shared__ __attribute__((aligned(16))) char lds[];  // DSTAGES * DSTAGE

    const int idx = (int)(blockIdx.x >> 3);
    const int unit = (int)(blockIdx.x & 7) + 8 * (idx / tiles_n);
    const int ch = unit / tiles_m;
    if (ch >= *nchunks) return;
    const int tile = (unit - ch * tiles_m) * tiles_n + idx % tiles_n;
    const int m0 = (tile / tiles_n) * GM, n0 = (tile % tiles_n) * GN;
    const int rows = chunk_rows[ch];
    const int cs = chunk_split[ch];
    if (rows <= 0) {
        if (cs == -1 && overwrite)
            zero_tile(out + (size_t)chunk_expert[ch] * out_expert_stride, M, N, m0, n0, GM, GN, threadIdx.x, GT);
        return;
    }
    const int row0 = chunk_row0[ch];
    const int mode = cs >= 2 ? 2 : cs;
    float* const o = cs >= 2 ? partial + (size_t)(cs - 2) * M * N : out + (size_t)chunk_expert[ch] * out_expert_stride;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- DMA: wave w fills rows 4 w .. 4 w + 3 of both tiles, two rows an instruction ------------
    const int q = lane & 31;
    uint32_t a_col[2], b_col[2];  // byte offset of this lane's piece inside a row, per instruction
    int d_row[2];                 // its row inside the stage
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        d_row[j] = 4 * wave + 2 * j + (lane >> 5);
        const int piece = q ^ ((d_row[j] & 3) << 2);
        // columns past the edge: fetched from a valid place, never stored
        a_col[j] = (uint32_t)(m0 + 8 * piece < M ? m0 + 8 * piece : 0) * 2u;
        b_col[j] = (uint32_t)(n0 + 8 * piece < N ? n0 + 8 * piece : 0) * 2u;
    }
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds;
    auto dma = [&](int st) {  // stage st -> LDS stage st % 3
        const uint32_t dst = lds0 + (uint32_t)(st % DSTAGES) * DSTAGE + (uint32_t)wave * (4 * GM * 2);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t r = (uint32_t)(row0 + min(st * GR + d_row[j], rows - 1));  // past the end: a valid row, zeroed below
            wg_issue_dma(dst + j * (2 * GM * 2), r * (uint32_t)(M * 2) + a_col[j], a);
            wg_issue_dma(dst + GR * GM * 2 + j * (2 * GN * 2), r * (uint32_t)(N * 2) + b_col[j], b);
        }
    };
    // rows of stage st past the end of the chunk contribute nothing: zeroed by the wave whose DMA has just landed
    auto zero_tail = [&](int st) {
        if ((st + 1) * GR <= rows) return;
        char* const A = lds + (st % DSTAGES) * DSTAGE;
        char* const B = A + GR * GM * 2;
#pragma unroll
        for (int j = 0; j < 2; ++j)
            if (st * GR + d_row[j] >= rows) {
                *reinterpret_cast<uint4*>(A + d_row[j] * (GM * 2) + q * 16) = make_uint4(0, 0, 0, 0);
                *reinterpret_cast<uint4*>(B + d_row[j] * (GN * 2) + q * 16) = make_uint4(0, 0, 0, 0);
            }
    };

    floatx16 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // lane's share of a fragment read: group of 16 lanes gi covers columns 16 (gi % 2) .. and rows
    // 8 (gi / 2) ..; inside the group lane s points at row s / 4, columns 4 (s % 4) ..
    const int gi = lane >> 4, sl = lane & 15;
    const int frow = 8 * (gi >> 1) + (sl >> 2);
    const int fcol = 16 * (gi & 1) + 4 * (sl & 3);
    const int sw = ((sl >> 2) & 3) << 2;  // frow % 4, and of every row this lane reads
    int a_frag[2], b_frag[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int col = wm * 64 + i * 32 + fcol;
        a_frag[i] = frow * (GM * 2) + (((col >> 3) ^ sw) << 4) + (col & 7) * 2;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = wn * 128 + j * 32 + fcol;
        b_frag[j] = frow * (GN * 2) + (((col >> 3) ^ sw) << 4) + (col & 7) * 2;
    }

    const int nstages = (rows + GR - 1) / GR;
    // Fragments of the 16-row step after the current one are requested before the current step's products, into
    // a second set of registers; the barrier sits between the two steps of a stage.
    auto read_frags = [&](int st, int ks, bf16x8 (&af)[2], bf16x8 (&bf)[4]) {
        const char* const A = lds + (st % DSTAGES) * DSTAGE + ks * 16 * (GM * 2);
        const char* const B = lds + (st % DSTAGES) * DSTAGE + GR * GM * 2 + ks * 16 * (GN * 2);
#pragma unroll
        for (int i = 0; i < 2; ++i) af[i] = tr_fragment(A + a_frag[i], GM * 2);
#pragma unroll
        for (int j = 0; j < 4; ++j) bf[j] = tr_fragment(B + b_frag[j], GN * 2);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto products = [&](const bf16x8 (&af)[2], const bf16x8 (&bf)[4]) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    for (int st = 0; st < DSTAGES - 1; ++st) dma(st);
    wg_wait_outstanding<4 * (DSTAGES - 2)>();  // stage 0 (this wave's four instructions) has landed
    zero_tail(0);
    __syncthreads();
    bf16x8 af0[2], bf0[4], af1[2], bf1[4];
    read_frags(0, 0, af0, bf0);
    for (int s = 0; s < nstages; ++s) {
        read_frags(s, 1, af1, bf1);
        products(af0, bf0);
        wg_wait_outstanding<4 * (DSTAGES - 3)>();  // stage s + 1 has landed (the later ones may be in flight)
        zero_tail(s + 1);
        __syncthreads();  // stage s + 1 is complete; nobody reads stage s - 1 any more
        dma(s + DSTAGES - 1);
        read_frags(s + 1, 0, af0, bf0);
        products(af1, bf1);
    }
    wg_wait_outstanding<0>();  // nothing may arrive in LDS once the workgroup has gone

    add_tiles<2, 4>(acc, o, M, N, m0 + wm * 64, n0 + wn * 128, lane, mode, overwrite != 0);
}

// ---------------------------------------------------------------------------
// The same product for all-f32 layers on the f32 matrix cores (v_mfma_f32_32x32x2_f32: one
// reduction element per lane, so a fragment is read from the row-major LDS tile as it lies,
// 32 neighbouring columns of two neighbouring rows).  4 waves (2 x 2) own 128 x 128 outputs, a
// wave 64 x 64; 16 rows per LDS stage, double buffered, loads three stages ahead.  LDS rows are
// padded to 160 floats: the two rows of a fragment read fall into different halves of the banks.
// ---------------------------------------------------------------------------
constexpr int FM = 128, FN = 128, FR = 16, FT = 256;
constexpr int FP = FM + 32;                 // LDS row pitch in floats (FM == FN)
constexpr int FSTAGE = FR * 2 * FP;         // floats per stage (A tile, then B tile)

__global__ __launch_bounds__(FT, 2) void weight_grad_f32_kernel(
    const float* __restrict__ a, int M, const float* __restrict__ b, int N, int tiles_m, int tiles_n,
    const int* __restrict__ chunk_expert, const int* __restrict__ chunk_row0, const int* __restrict__ chunk_rows,
    const int* __restrict__ chunk_split, const int* __restrict__ nchunks, float* __restrict__ out,
    size_t out_expert_stride, int overwrite, float* __restrict__ partial) {
    __shared__ __attribute__((aligned(16))) float lds[2 * FSTAGE];  // 40 KB

    const int idx = (int)(blockIdx.x >> 3);
    const int unit = (int)(blockIdx.x & 7) + 8 * (idx / tiles_n);
    const int ch = unit / tiles_m;
    if (ch >= *nchunks) return;
    const int m0 = (unit - ch * tiles_m) * FM, n0 = (idx % tiles_n) * FN;
    const int rows = chunk_rows[ch];
    const int cs = chunk_split[ch];
    if (rows <= 0) {
        if (cs == -1 && overwrite)
            zero_tile(out + (size_t)chunk_expert[ch] * out_expert_stride, M, N, m0, n0, FM, FN, threadIdx.x, FT);
        return;
    }
    const int row0 = chunk_row0[ch];
    const int mode = cs >= 2 ? 2 : cs;
    float* const o = cs >= 2 ? partial + (size_t)(cs - 2) * M * N : out + (size_t)chunk_expert[ch] * out_expert_stride;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // each tile: 16 rows x 32 pieces of 4 floats; a thread moves piece tid % 32 of rows tid / 32 and tid / 32 + 8
    const int pc = tid & 31, tr = tid >> 5;
    const float* const a_src = a + (size_t)row0 * M + (m0 + 4 * pc < M ? m0 + 4 * pc : 0);
    const float* const b_src = b + (size_t)row0 * N + (n0 + 4 * pc < N ? n0 + 4 * pc : 0);
    // (three sets of registers by name: an array of sets is placed in scratch memory)
    struct Set {
        float4 a0, a1, b0, b1;
    } set0, set1, set2;
    static_assert(GDEPTH == 3, "one named set per stage in flight");
    auto fetch = [&](auto kc, int r0) {
        constexpr int k = decltype(kc)::value;
        Set& st = k == 0 ? set0 : k == 1 ? set1 : set2;
        const int ra = min(r0 + tr, rows - 1), rb = min(r0 + tr + 8, rows - 1);
        st.a0 = *reinterpret_cast<const float4*>(a_src + (size_t)ra * M);
        st.b0 = *reinterpret_cast<const float4*>(b_src + (size_t)ra * N);
        st.a1 = *reinterpret_cast<const float4*>(a_src + (size_t)rb * M);
        st.b1 = *reinterpret_cast<const float4*>(b_src + (size_t)rb * N);
    };
    auto stage = [&](auto kc, int buf, int r0) {
        constexpr int k = decltype(kc)::value;
        const Set& st = k == 0 ? set0 : k == 1 ? set1 : set2;
        float* const A = lds + buf * FSTAGE;
        float* const B = A + FR * FP;
        // (rows past the chunk's end are zeros; a choice between two named float4 would be a choice between their
        // addresses, and the sets would live in scratch memory)
        const float in0 = r0 + tr < rows ? 1.0f : 0.0f, in1 = r0 + tr + 8 < rows ? 1.0f : 0.0f;
        auto keep = [](const float4& v, float on) {
            return make_float4(on != 0.0f ? v.x : 0.0f, on != 0.0f ? v.y : 0.0f, on != 0.0f ? v.z : 0.0f, on != 0.0f ? v.w : 0.0f);
        };
        *reinterpret_cast<float4*>(A + tr * FP + pc * 4) = keep(st.a0, in0);
        *reinterpret_cast<float4*>(B + tr * FP + pc * 4) = keep(st.b0, in0);
        *reinterpret_cast<float4*>(A + (tr + 8) * FP + pc * 4) = keep(st.a1, in1);
        *reinterpret_cast<float4*>(B + (tr + 8) * FP + pc * 4) = keep(st.b1, in1);
    };

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    const int a_lane = (lane >> 5) * FP + wm * 64 + (lane & 31);
    const int b_lane = (lane >> 5) * FP + wn * 64 + (lane & 31);

    const int nstages = (rows + FR - 1) / FR;
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    fetch(I0{}, 0);
    fetch(I1{}, FR);
    fetch(I2{}, 2 * FR);
    stage(I0{}, 0, 0);
    __syncthreads();
    auto step = [&](auto kc, int s) {
        constexpr int k = decltype(kc)::value;
        const int buf = s & 1;
        fetch(kc, (s + GDEPTH) * FR);
        const float* const A = lds + buf * FSTAGE;
        const float* const B = A + FR * FP;
#pragma unroll
        for (int kk = 0; kk < FR / 2; ++kk) {
            float af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) af[i] = A[a_lane + 2 * kk * FP + i * 32];
#pragma unroll
            for (int j = 0; j < 2; ++j) bf[j] = B[b_lane + 2 * kk * FP + j * 32];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        stage(std::integral_constant<int, (k + 1) % GDEPTH>{}, buf ^ 1, (s + 1) * FR);
        __syncthreads();
    };
    for (int s = 0; s < nstages; s += GDEPTH) {
        step(I0{}, s);
        step(I1{}, s + 1);
        step(I2{}, s + 2);
    }
    add_tiles<2, 2>(acc, o, M, N, m0 + wm * 64, n0 + wn * 64, lane, mode, overwrite != 0);
}

// Overwrite mode: an expert with exactly one chunk is written in full by that chunk's tiles; every
// other expert (no rows, or cut into chunks that add atomically) is cleared here first.
__global__ __launch_bounds__(256) void clear_other_experts_kernel(const int* __restrict__ counts, int dense_rows,
                                                                  int limit, int ordered, float* __restrict__ out,
                                                                  size_t out_expert_stride, size_t elems) {
    const int e = blockIdx.y;
    const int rows = dense_rows >= 0 ? dense_rows : counts[e];
    if (rows > 0 && (rows <= limit || ordered)) return;  // a chunk that stores: the only one, or the first of an ordered cut
    float4* const o = reinterpret_cast<float4*>(out + (size_t)e * out_expert_stride);
    const size_t n4 = elems / 4;  // M and N are multiples of 4
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256)
        o[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
}

}  // namespace

bool weight_grad_shape_ok(int M, int N, bool bf16) {
    const int q = bf16 ? 8 : 4;  // 16-byte pieces
    return M % q == 0 && N % q == 0 && M >= q && N >= q;
}

// Upper bound of the number of chunks of one launch; `chunks` needs weight_grad_table_ints(...) ints.
int weight_grad_max_chunks(int groups, int total_rows) { return groups + total_rows / 256 + 1; }
int weight_grad_table_ints(int groups, int total_rows) { return 4 * weight_grad_max_chunks(groups, total_rows) + 1 + 2 * groups; }

namespace {
// rows above which an expert is cut: enough (chunk, tile) pairs to fill the chip twice, and no chunk longer than
// twice the average expert's share (a cut costs a partial matrix per further chunk)
int cut_limit(int M, int N, int groups, int dense_rows, int total_rows, bool bf16) {
    const int tile_m = bf16 ? GM : FM, tile_n = bf16 ? GN : FN;
    const int tiles = ((M + tile_m - 1) / tile_m) * ((N + tile_n - 1) / tile_n);
    const int want = std::max(groups, (512 + tiles - 1) / tiles);
    const int share = (total_rows + want - 1) / want;
    return std::max(256, ((dense_rows >= 0 ? share : 2 * share) + 31) & ~31);
}
}  // namespace

// Partial matrices an ordered launch of `total_rows` rows needs: every further chunk of a cut expert has one, and
// there are at most total_rows / limit of them.
size_t weight_grad_partial_bytes(int M, int N, int groups, int dense_rows, int total_rows, bool bf16) {
    if (groups <= 0 || total_rows <= 0) return 0;
    const int limit = cut_limit(M, N, groups, dense_rows, total_rows, bf16);
    return (size_t)(total_rows / limit + 1) * M * N * sizeof(float);
}

// The same for a buffer that has to serve every launch of 1 .. max_tokens tokens (rows_per_token rows each; for
// a dense launch the rows are the tokens).  The cut limit follows the row count with a floor and a rounding, so
// the number of partial matrices is not monotone in the row count: a smaller batch can need more of them.
size_t weight_grad_partial_bytes_upto(int M, int N, int groups, bool dense, int max_tokens, int rows_per_token,
                                      bool bf16) {
    size_t need = 0;
    for (int t = 1; t <= max_tokens; ++t) {
        const int rows = dense ? t : t * rows_per_token;
        need = std::max(need, weight_grad_partial_bytes(M, N, groups, dense ? rows : -1, rows, bf16));
    }
    return need;
}

hipError_t launch_weight_grad(const void* a, int M, const void* b, int N, const int* counts, const int* offsets,
                              int groups, int dense_rows, int total_rows, WgradSplit split_mode, bool overwrite,
                              int* chunks, float* partial, size_t partial_bytes, float* out, size_t out_expert_stride,
                              bool bf16, hipStream_t s, WgradPart part) {
    if (groups <= 0 || total_rows <= 0) return hipSuccess;
    if (!weight_grad_shape_ok(M, N, bf16)) return hipErrorInvalidValue;
    if (bf16) {
        static std::atomic<unsigned long long> attr_set{0};
        const hipError_t attr = once_per_device(attr_set, [] {
            return hipFuncSetAttribute(reinterpret_cast<const void*>(weight_grad_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 2 * GSTAGE);
        });
        if (attr != hipSuccess) return attr;
    }
    const int tile_m = bf16 ? GM : FM, tile_n = bf16 ? GN : FN;
    const int tiles_m = (M + tile_m - 1) / tile_m, tiles_n = (N + tile_n - 1) / tile_n;
    int limit = 1 << 30;  // WgradSplit::None: an expert is one chunk, whatever its share
    int max_slots = 0;
    bool ordered = false;
    if (split_mode != WgradSplit::None) {
        limit = cut_limit(M, N, groups, dense_rows, total_rows, bf16);
        if (split_mode == WgradSplit::Ordered) {
            ordered = true;
            max_slots = partial ? (int)std::min<size_t>(partial_bytes / ((size_t)M * N * sizeof(float)), 1 << 20) : 0;
            // A buffer with fewer partial matrices than this row count would cut out (total_rows / limit at most)
            // gets longer chunks, down to no cut at all, instead of a refusal.
            if (max_slots == 0) limit = 1 << 30;
            else if (total_rows / limit > max_slots) limit = ((total_rows / max_slots + 1) + 31) & ~31;
        }
    }
    const int max_chunks = weight_grad_max_chunks(groups, total_rows);
    int* const chunk_expert = chunks;
    int* const chunk_row0 = chunks + max_chunks;
    int* const chunk_rows = chunks + 2 * max_chunks;
    int* const chunk_split = chunks + 3 * max_chunks;
    int* const nchunks = chunks + 4 * max_chunks;
    int* const slot_first = nchunks + 1;
    int* const slot_count = slot_first + groups;
    // Overwriting: with atomic chunks the cut experts and those without rows are cleared by a launch in front; in
    // the other modes every expert with rows has a chunk that stores, and one without rows gets a chunk that
    // stores zeros.
    const bool clear_first = overwrite && split_mode == WgradSplit::Atomic;
    if (part != WgradPart::ProductOnly)
        hipLaunchKernelGGL(chunk_table_kernel, dim3(1), dim3(256), 0, s, counts, offsets, groups, dense_rows, limit,
                           max_chunks, ordered ? 1 : 0, max_slots, (overwrite && !clear_first) ? 1 : 0, chunk_expert,
                           chunk_row0, chunk_rows, chunk_split, nchunks, slot_first, slot_count);
    if (part == WgradPart::TableOnly) return hipGetLastError();
    if (clear_first)
        hipLaunchKernelGGL(clear_other_experts_kernel, dim3(64, groups), dim3(256), 0, s, counts, dense_rows, limit,
                           ordered ? 1 : 0, out, out_expert_stride, (size_t)M * N);
    const int grid = ((max_chunks * tiles_m + 7) / 8) * 8 * tiles_n;
    // byte offsets inside the operands fit 32 bits: tiles by LDS-DMA
    const bool dma = bf16 && (size_t)total_rows * (size_t)std::max(M, N) * 2 < ((size_t)1 << 32) && GM == GN;
    if (dma) {
        static std::atomic<unsigned long long> attr2_set{0};
        const hipError_t attr2 = once_per_device(attr2_set, [] {
            return hipFuncSetAttribute(reinterpret_cast<const void*>(weight_grad_dma_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, DSTAGES * DSTAGE);
        });
        if (attr2 != hipSuccess) return attr2;
        hipLaunchKernelGGL(weight_grad_dma_kernel, dim3(grid), dim3(GT), DSTAGES * DSTAGE, s, static_cast<const bf16_t*>(a), M,
                           static_cast<const bf16_t*>(b), N, tiles_m, tiles_n, chunk_expert, chunk_row0, chunk_rows,
                           chunk_split, nchunks, out, out_expert_stride, overwrite ? 1 : 0, partial);
    } else if (bf16)
        hipLaunchKernelGGL(weight_grad_kernel, dim3(grid), dim3(GT), 2 * GSTAGE, s, static_cast<const bf16_t*>(a), M,
                           static_cast<const bf16_t*>(b), N, tiles_m, tiles_n, chunk_expert, chunk_row0, chunk_rows,
                           chunk_split, nchunks, out, out_expert_stride, overwrite ? 1 : 0, partial);
    else
        hipLaunchKernelGGL(weight_grad_f32_kernel, dim3(grid), dim3(FT), 0, s, static_cast<const float*>(a), M,
                           static_cast<const float*>(b), N, tiles_m, tiles_n, chunk_expert, chunk_row0, chunk_rows,
                           chunk_split, nchunks, out, out_expert_stride, overwrite ? 1 : 0, partial);
    if (ordered)
        // (most experts have nothing to add and leave at once: enough workgroups per expert for one cut expert to
        // fill the chip by itself)
        hipLaunchKernelGGL(add_partials_kernel, dim3(1024, groups), dim3(256), 0, s, slot_first, slot_count, partial,
                           (size_t)M * N, out, out_expert_stride);
    return hipGetLastError();
}

}  // namespace rbmoe
