// Device-side helpers shared by the gfx950 kernels: element types, bf16
// conversion and the fixed-sequence exp/log the router uses.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rbmoe {

constexpr int kWave = 64;

// Raw bf16 storage.  Values are converted explicitly so that the rounding rule
// (nearest even on the bit pattern) is visible and identical everywhere.
struct bf16_t {
    uint16_t bits;
};

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return __uint_as_float((uint32_t)v.bits << 16); }
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t b = __float_as_uint(f);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x0040u);
    b += 0x7fffu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) {
    return v;
}
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) {
    return bf16_t{f32_to_bf16_bits(v)};
}

// ---------------------------------------------------------------------------
// exp and log as fixed sequences of binary32 operations (Cephes expf/logf).
// Every step is either one fused multiply-add (__fmaf_rn) or one correctly
// rounded multiply/add (__fmul_rn/__fadd_rn), so the compiler cannot reorder
// or contract them and the result is the same on any IEEE-754 machine that
// runs the same sequence.  Softmax probabilities and the log-sum-exp depend on
// these bit for bit, and routing depends on the probabilities.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float rb_expf(float x) {
    if (x != x) return x;
    if (x > 88.72283935546875f) return __uint_as_float(0x7f800000u);
    if (x < -103.97208404541015625f) return 0.0f;
    const float t = __fmul_rn(x, 1.44269502162933349609375f);
    const float kf = rintf(t);
    float r = __fmaf_rn(kf, -0.693145751953125f, x);
    r = __fmaf_rn(kf, -1.428606765330187045037746429443359375e-6f, r);
    float p = 1.9875691500e-4f;
    p = __fmaf_rn(p, r, 1.3981999507e-3f);
    p = __fmaf_rn(p, r, 8.3334519073e-3f);
    p = __fmaf_rn(p, r, 4.1665795894e-2f);
    p = __fmaf_rn(p, r, 1.6666665459e-1f);
    p = __fmaf_rn(p, r, 5.0000001201e-1f);
    const float r2 = __fmul_rn(r, r);
    p = __fmaf_rn(p, r2, r);
    p = __fadd_rn(p, 1.0f);
    const int k = (int)kf;
    const int k1 = k / 2;
    const int k2 = k - k1;
    const float s1 = __uint_as_float((uint32_t)(k1 + 127) << 23);
    const float s2 = __uint_as_float((uint32_t)(k2 + 127) << 23);
    return __fmul_rn(__fmul_rn(p, s1), s2);
}

__device__ __forceinline__ float rb_logf(float x) {
    if (x != x) return x;
    if (x < 0.0f) return __uint_as_float(0x7fc00000u);
    if (x == 0.0f) return __uint_as_float(0xff800000u);
    if (__float_as_uint(x) == 0x7f800000u) return x;
    int e = 0;
    uint32_t b = __float_as_uint(x);
    if (b < 0x00800000u) {
        x = __fmul_rn(x, 8388608.0f);
        b = __float_as_uint(x);
        e = -23;
    }
    e += (int)(b >> 23) - 126;
    float m = __uint_as_float((b & 0x007fffffu) | 0x3f000000u);
    if (m < 0.707106769084930419921875f) {
        e -= 1;
        m = __fadd_rn(__fadd_rn(m, m), -1.0f);
    } else {
        m = __fadd_rn(m, -1.0f);
    }
    const float z = __fmul_rn(m, m);
    float y = 7.0376836292e-2f;
    y = __fmaf_rn(y, m, -1.1514610310e-1f);
    y = __fmaf_rn(y, m, 1.1676998740e-1f);
    y = __fmaf_rn(y, m, -1.2420140846e-1f);
    y = __fmaf_rn(y, m, 1.4249322787e-1f);
    y = __fmaf_rn(y, m, -1.6668057665e-1f);
    y = __fmaf_rn(y, m, 2.0000714765e-1f);
    y = __fmaf_rn(y, m, -2.4999993993e-1f);
    y = __fmaf_rn(y, m, 3.3333331174e-1f);
    y = __fmul_rn(__fmul_rn(y, m), z);
    const float fe = (float)e;
    y = __fmaf_rn(-2.12194440e-4f, fe, y);
    y = __fmaf_rn(-0.5f, z, y);
    float r = __fadd_rn(m, y);
    r = __fmaf_rn(0.693359375f, fe, r);
    return r;
}

// silu(x) = x * (1 / (1 + exp(-x))), the reference's operation order
// (src/ffn.rs:223-229).  Tolerance-checked, so the fast exponential is used.
__device__ __forceinline__ float silu_f32(float x) { return x * (1.0f / (1.0f + __expf(-x))); }

// The same with the hardware's 1-ulp reciprocal and base-2 exponential, for results that are
// rounded to bf16 anyway: 2 transcendental and 4 plain operations per value instead of a
// full IEEE division.
__device__ __forceinline__ float silu_bf16_grade(float x) {
    const float e = __builtin_amdgcn_exp2f(x * -1.44269504088896340736f);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// ---- matrix-core operand helpers ------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

// two int8 values of `word` (bytes shift/8 and shift/8 + 1) as a pair of bf16
__device__ __forceinline__ uint32_t widen2(uint32_t word, int shift) {
    const float lo = (float)(int)(int8_t)(word >> shift);
    const float hi = (float)(int)(int8_t)(word >> (shift + 8));
    return pack2(lo, hi);  // small integers are exact in bf16; one packed conversion instead of shift + and-or
}

__device__ __forceinline__ bf16x8 widen_i8(uint2 q) {
    const uint4 w = make_uint4(widen2(q.x, 0), widen2(q.x, 16), widen2(q.y, 0), widen2(q.y, 16));
    return __builtin_bit_cast(bf16x8, w);
}

// ---- 16-byte pieces of an activation row: 4 f32 or 8 bf16 --------------------------
template <typename T>
struct Vec16;
template <>
struct Vec16<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ uint4 load_raw(const float* p) { return *reinterpret_cast<const uint4*>(p); }
    static __device__ __forceinline__ void widen(const uint4& a, float (&v)[4]) {
        v[0] = __uint_as_float(a.x); v[1] = __uint_as_float(a.y); v[2] = __uint_as_float(a.z); v[3] = __uint_as_float(a.w);
    }
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const float4 a = *reinterpret_cast<const float4*>(p);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
};
template <>
struct Vec16<bf16_t> {
    static constexpr int N = 8;
    static __device__ __forceinline__ uint4 load_raw(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
    static __device__ __forceinline__ void widen(const uint4& a, float (&v)[8]) {
        v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
        v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
        v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xffff0000u);
        v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xffff0000u);
    }
    static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
        const uint4 a = *reinterpret_cast<const uint4*>(p);
        v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xffff0000u);
        v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xffff0000u);
        v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xffff0000u);
        v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xffff0000u);
    }
    static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
        uint4 o;
        o.x = f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
        o.y = f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
        o.z = f32_to_bf16_bits(v[4]) | ((uint32_t)f32_to_bf16_bits(v[5]) << 16);
        o.w = f32_to_bf16_bits(v[6]) | ((uint32_t)f32_to_bf16_bits(v[7]) << 16);
        *reinterpret_cast<uint4*>(p) = o;
    }
};

// Reductions over the G neighbouring lanes of a group (G a power of two up to 64, the same for the whole wave)
// without LDS: inside a row of 16 lanes through the lane-permuting operand of the instruction itself (every lane of
// the row ends with the result), across rows through four scalar reads.
template <int CTRL>
__device__ __forceinline__ uint32_t lanes_from(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);
}
template <typename Op>
__device__ __forceinline__ uint32_t group_reduce(uint32_t v, int G, Op op) {
    if (G >= 2) v = op(v, lanes_from<0xB1>(v));   // quad_perm [1,0,3,2]
    if (G >= 4) v = op(v, lanes_from<0x4E>(v));   // quad_perm [2,3,0,1]
    if (G >= 8) v = op(v, lanes_from<0x141>(v));  // row_half_mirror
    if (G >= 16) v = op(v, lanes_from<0x140>(v)); // row_mirror
    if (G >= 32) {
        const uint32_t r0 = __builtin_amdgcn_readlane(v, 0), r1 = __builtin_amdgcn_readlane(v, 16);
        const uint32_t r2 = __builtin_amdgcn_readlane(v, 32), r3 = __builtin_amdgcn_readlane(v, 48);
        const uint32_t lo = op(r0, r1), hi = op(r2, r3);
        v = G == 64 ? op(lo, hi) : ((threadIdx.x & 32) ? hi : lo);
    }
    return v;
}
__device__ __forceinline__ uint32_t group_umax(uint32_t v, int G) {
    return group_reduce(v, G, [](uint32_t a, uint32_t b) { return a > b ? a : b; });
}
__device__ __forceinline__ uint32_t group_umin(uint32_t v, int G) {
    return group_reduce(v, G, [](uint32_t a, uint32_t b) { return a < b ? a : b; });
}
// (no NaN among the operands; which zero wins among zeros of both signs does not matter to the callers)
__device__ __forceinline__ float group_fmax(float v, int G) {
    return __uint_as_float(group_reduce(__float_as_uint(v), G, [](uint32_t a, uint32_t b) {
        return __float_as_uint(fmaxf(__uint_as_float(a), __uint_as_float(b)));
    }));
}

}  // namespace rbmoe
