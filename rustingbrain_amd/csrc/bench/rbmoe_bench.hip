// Measurement helpers of the benchmark (include/rbmoe_bench.h), built into a library of their own
// (librbmoe_bench.so): nothing here is part of the layer, and librbmoe.so does not contain it.
//   a loop of nothing but bf16 matrix-core multiplies (what the matrix cores sustain at the clock they settle at),
//   a plain read of a buffer (what a launch of that size gets out of HBM, with cold or warm caches),
//   a read-only sweep of a large buffer that evicts L2 and the Infinity Cache without leaving dirty lines behind,
//   a stream and an event timer for hosts without a HIP binding of their own.
#include "../../../include/rbmoe_bench.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// One wave per SIMD-slot, eight independent accumulators, operands held in registers.
__global__ __launch_bounds__(256, 2) void mfma_only_kernel(float* out, int steps) {
    floatx16 acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const uint32_t one = 0x3f803f80u;  // two bf16 ones
    u32x4 raw = {one, one, one, one ^ (threadIdx.x & 1u)};
    const bf16x8 a = __builtin_bit_cast(bf16x8, raw);
    for (int s = 0; s < steps; ++s) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, a, acc[i], 0, 0, 0);
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) sum += acc[i][v];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = sum;
}

// Every workgroup reads a contiguous share of the buffer with 16-byte loads, eight in flight per lane.
__global__ __launch_bounds__(256) void read_only_kernel(const uint4* __restrict__ src, size_t pieces, uint32_t* out) {
    const size_t per = (pieces + gridDim.x - 1) / gridDim.x;
    const size_t lo = (size_t)blockIdx.x * per, hi = lo + per < pieces ? lo + per : pieces;
    uint32_t x = 0;
    for (size_t i = lo + threadIdx.x; i < hi; i += 8 * 256) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const size_t j = i + (size_t)u * 256;
            v[u] = src[j < hi ? j : lo];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) x ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    if (x == 0x9e3779b9u) out[0] = x;  // keeps the loads alive; practically never true
}

hipError_t launch_read_only(const void* src, size_t bytes, int workgroups, uint32_t* out, hipStream_t s) {
    hipLaunchKernelGGL(read_only_kernel, dim3(workgroups), dim3(256), 0, s, static_cast<const uint4*>(src), bytes / 16, out);
    return hipGetLastError();
}

struct Flush {
    void* buf = nullptr;
    uint32_t* sink = nullptr;
    size_t bytes = 0;
};

struct Timer {
    hipEvent_t e0 = nullptr, e1 = nullptr;
};

int rc(hipError_t e) { return e == hipSuccess ? 0 : (int)e; }

}  // namespace

extern "C" {

int rbbench_stream_create(void** stream) {
    if (!stream) return -1;
    hipStream_t s = nullptr;
    const hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    *stream = s;
    return rc(e);
}

int rbbench_stream_destroy(void* stream) {
    if (!stream) return 0;
    (void)hipStreamSynchronize(static_cast<hipStream_t>(stream));
    return rc(hipStreamDestroy(static_cast<hipStream_t>(stream)));
}

int rbbench_timer_create(void** timer) {
    if (!timer) return -1;
    Timer* t = new Timer();
    hipError_t e = hipEventCreate(&t->e0);
    if (e == hipSuccess) e = hipEventCreate(&t->e1);
    if (e != hipSuccess) {
        if (t->e0) (void)hipEventDestroy(t->e0);
        delete t;
        *timer = nullptr;
        return rc(e);
    }
    *timer = t;
    return 0;
}

int rbbench_timer_start(void* timer, void* stream) {
    if (!timer) return -1;
    return rc(hipEventRecord(static_cast<Timer*>(timer)->e0, static_cast<hipStream_t>(stream)));
}

int rbbench_timer_stop(void* timer, void* stream, float* ms) {
    if (!timer || !ms) return -1;
    Timer* t = static_cast<Timer*>(timer);
    hipError_t e = hipEventRecord(t->e1, static_cast<hipStream_t>(stream));
    if (e == hipSuccess) e = hipEventSynchronize(t->e1);
    if (e == hipSuccess) e = hipEventElapsedTime(ms, t->e0, t->e1);
    return rc(e);
}

void rbbench_timer_destroy(void* timer) {
    if (!timer) return;
    Timer* t = static_cast<Timer*>(timer);
    (void)hipEventDestroy(t->e0);
    (void)hipEventDestroy(t->e1);
    delete t;
}

int rbbench_flush_create(size_t bytes, void** flush) {
    if (!flush || bytes < 4096) return -1;
    Flush* f = new Flush();
    f->bytes = bytes & ~(size_t)4095;
    hipError_t e = hipMalloc(&f->buf, f->bytes);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&f->sink), 256);
    if (e == hipSuccess) e = hipMemset(f->buf, 1, f->bytes);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        if (f->buf) (void)hipFree(f->buf);
        if (f->sink) (void)hipFree(f->sink);
        delete f;
        *flush = nullptr;
        return rc(e);
    }
    *flush = f;
    return 0;
}

int rbbench_flush(void* flush, void* stream) {
    if (!flush) return -1;
    Flush* f = static_cast<Flush*>(flush);
    return rc(launch_read_only(f->buf, f->bytes, 2048, f->sink, static_cast<hipStream_t>(stream)));
}

void rbbench_flush_destroy(void* flush) {
    if (!flush) return;
    Flush* f = static_cast<Flush*>(flush);
    (void)hipDeviceSynchronize();
    (void)hipFree(f->buf);
    (void)hipFree(f->sink);
    delete f;
}

int rbbench_mfma_only(void* stream, int32_t launches, double* tflops, double* avg_launch_ms) {
    if (!tflops || launches <= 0) return -1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return rc(e);
    const int workgroups = 2 * cus, steps = 2048;  // two waves on every SIMD
    float* out = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    e = hipMalloc(reinterpret_cast<void**>(&out), (size_t)workgroups * 256 * sizeof(float));
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    auto launch = [&]() -> hipError_t {
        hipLaunchKernelGGL(mfma_only_kernel, dim3(workgroups), dim3(256), 0, s, out, steps);
        return hipGetLastError();
    };
    if (e == hipSuccess) e = launch();  // warm-up
    if (e == hipSuccess) e = hipEventRecord(e0, s);
    for (int i = 0; i < launches && e == hipSuccess; ++i) e = launch();
    if (e == hipSuccess) e = hipEventRecord(e1, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (out) (void)hipFree(out);
    if (e != hipSuccess) return rc(e);
    const double flops = (double)workgroups * 4 * steps * 8 * 32768.0;  // 2 * 32 * 32 * 16 per multiply
    const double avg = (double)ms / launches;
    *tflops = flops / (avg * 1e-3) / 1e12;
    if (avg_launch_ms) *avg_launch_ms = avg;
    return 0;
}

int rbbench_read(void* stream, size_t bytes, int32_t launches, void* flush, double* gbs, double* avg_launch_ms) {
    if (!gbs || launches <= 0 || bytes < 16 || bytes % 16 != 0) return -1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    void* buf = nullptr;
    uint32_t* sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t e = hipMalloc(&buf, bytes);
    if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void**>(&sink), 256);
    if (e == hipSuccess) e = hipMemsetAsync(buf, 1, bytes, s);
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    // the split over workgroups that reads fastest is the one reported
    double best = 1e30;
    const int splits[3] = {512, 1024, 2048};
    for (int sp = 0; sp < 3 && e == hipSuccess; ++sp) {
        const int workgroups = splits[sp];
        e = launch_read_only(buf, bytes, workgroups, sink, s);  // warm-up
        double total = 0.0;
        if (flush) {  // every launch by itself, behind a sweep of the flush buffer: the raw event interval
            for (int i = 0; i < launches && e == hipSuccess; ++i) {
                e = (hipError_t)rbbench_flush(flush, stream);
                if (e == hipSuccess) e = hipEventRecord(e0, s);
                if (e == hipSuccess) e = launch_read_only(buf, bytes, workgroups, sink, s);
                if (e == hipSuccess) e = hipEventRecord(e1, s);
                if (e == hipSuccess) e = hipStreamSynchronize(s);
                float ms = 0.0f;
                if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
                total += ms;
            }
        } else {  // back to back between one pair of events
            if (e == hipSuccess) e = hipEventRecord(e0, s);
            for (int i = 0; i < launches && e == hipSuccess; ++i) e = launch_read_only(buf, bytes, workgroups, sink, s);
            if (e == hipSuccess) e = hipEventRecord(e1, s);
            if (e == hipSuccess) e = hipStreamSynchronize(s);
            float ms = 0.0f;
            if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
            total = ms;
        }
        best = std::min(best, total / launches);
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (buf) (void)hipFree(buf);
    if (sink) (void)hipFree(sink);
    if (e != hipSuccess) return rc(e);
    *gbs = (double)bytes / (best * 1e-3) / 1e9;
    if (avg_launch_ms) *avg_launch_ms = best;
    return 0;
}

}  // extern "C"
