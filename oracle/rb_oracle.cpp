// TEST INFRASTRUCTURE — CPU oracle for the mixture-of-experts layer.
//
// This file restates, on the CPU and in plain C++, the algorithm of
// RustingBrain's `MoeLayer::forward_train` (reference src/moe.rs:243-341), of
// `MoeLayer::backward` (src/moe.rs:348-489), of the helpers under them, and of the block's
// steps either side of the layer (RmsNorm::forward, src/norm.rs:41-61; the residual add,
// src/transformer_block.rs:221-222).  It is NOT the Rust binary: no Rust toolchain exists
// where this is built, so every function below follows the reference source
// text line by line and cites the lines it follows.  Nothing in the shipped
// library links, loads or calls this file; only tests, the smoke check and
// the benchmark's CPU-baseline leg do.
//
// Arithmetic that the reference delegates to code outside its repository:
//   * matrixmultiply 0.3.11 `sgemm` (reference Cargo.lock:551, call site
//     src/matrix.rs:155-172).  Its blocking and summation order are not
//     visible, so f32 bit patterns of products versus the Rust binary are
//     PARITY UNPINNED; products here are compared by tolerance only.
//   * libm `expf`/`logf` behind `f32::exp`/`f32::ln` (platform dependent in the
//     last ulp).  The router path here uses the fixed operation sequences
//     `rbo_expf`/`rbo_logf` below so that an accelerator can reproduce the
//     probabilities bit for bit; they are pinned against libm to <= 2 ulp.
//   * the router logits use one fixed summation order (`rbo_router_logits`):
//     the reference's own eight-lane `dot` (src/matrix.rs:26-40), which the
//     reference takes for a single input row; for more rows it calls sgemm.  Routing decisions on
//     tokens whose k-th and (k+1)-th probabilities differ by a few ulp are
//     therefore PARITY UNPINNED against the Rust binary; `rbo_near_ties`
//     counts them.
//
// Pinned by: tests/test_oracle_*.py (hand vectors and known answers from the
// reference's own unit tests, closed forms, brute force on small inputs; the
// backward pass by the reference's four gradient tests and by finite
// differences of an independent float64 evaluation of the layer).
//
// Build: see oracle/Makefile (g++ -O2 -ffp-contract=off -mavx2 -mfma).

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <thread>
#include <vector>

#include <immintrin.h>

namespace {

inline float bits_to_f32(uint32_t b) {
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}
inline uint32_t f32_to_bits(float f) {
    uint32_t b;
    std::memcpy(&b, &f, 4);
    return b;
}

}  // namespace

extern "C" {

// ---------------------------------------------------------------------------
// Fixed-sequence exp and log (f32).  Published Cephes single-precision
// algorithms (expf.c / logf.c, S. Moshier), written as an explicit sequence of
// IEEE-754 binary32 operations: every `__builtin_fmaf` is one fused
// multiply-add, every other operator is one correctly rounded operation, and
// the file is compiled with -ffp-contract=off so nothing else is fused.
// ---------------------------------------------------------------------------

float rbo_expf(float x) {
    if (x != x) return x;
    if (x > 88.72283935546875f) return std::numeric_limits<float>::infinity();
    if (x < -103.97208404541015625f) return 0.0f;
    const float t = x * 1.44269502162933349609375f;  // log2(e)
    const float kf = __builtin_rintf(t);             // round half to even
    float r = __builtin_fmaf(kf, -0.693145751953125f, x);
    r = __builtin_fmaf(kf, -1.428606765330187045037746429443359375e-6f, r);
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    const float r2 = r * r;
    p = __builtin_fmaf(p, r2, r);
    p = p + 1.0f;
    const int k = (int)kf;
    const int k1 = k / 2;  // truncates toward zero
    const int k2 = k - k1;
    const float s1 = bits_to_f32((uint32_t)(k1 + 127) << 23);
    const float s2 = bits_to_f32((uint32_t)(k2 + 127) << 23);
    return (p * s1) * s2;
}

float rbo_logf(float x) {
    if (x != x) return x;
    if (x < 0.0f) return std::numeric_limits<float>::quiet_NaN();
    if (x == 0.0f) return -std::numeric_limits<float>::infinity();
    if (x == std::numeric_limits<float>::infinity()) return x;
    int e = 0;
    uint32_t b = f32_to_bits(x);
    if (b < 0x00800000u) {  // subnormal: scale by 2^23 (exact)
        x = x * 8388608.0f;
        b = f32_to_bits(x);
        e = -23;
    }
    // x = m * 2^e with m in [0.5, 1)
    e += (int)(b >> 23) - 126;
    float m = bits_to_f32((b & 0x007fffffu) | 0x3f000000u);
    if (m < 0.707106769084930419921875f) {
        e -= 1;
        m = (m + m) - 1.0f;
    } else {
        m = m - 1.0f;
    }
    const float z = m * m;
    float y = 7.0376836292e-2f;
    y = __builtin_fmaf(y, m, -1.1514610310e-1f);
    y = __builtin_fmaf(y, m, 1.1676998740e-1f);
    y = __builtin_fmaf(y, m, -1.2420140846e-1f);
    y = __builtin_fmaf(y, m, 1.4249322787e-1f);
    y = __builtin_fmaf(y, m, -1.6668057665e-1f);
    y = __builtin_fmaf(y, m, 2.0000714765e-1f);
    y = __builtin_fmaf(y, m, -2.4999993993e-1f);
    y = __builtin_fmaf(y, m, 3.3333331174e-1f);
    y = (y * m) * z;
    const float fe = (float)e;
    y = __builtin_fmaf(-2.12194440e-4f, fe, y);
    y = __builtin_fmaf(-0.5f, z, y);
    float r = m + y;
    r = __builtin_fmaf(0.693359375f, fe, r);
    return r;
}

void rbo_expf_array(const float* x, int64_t n, float* y) {
    for (int64_t i = 0; i < n; ++i) y[i] = rbo_expf(x[i]);
}
void rbo_logf_array(const float* x, int64_t n, float* y) {
    for (int64_t i = 0; i < n; ++i) y[i] = rbo_logf(x[i]);
}

// bf16 <-> f32, round to nearest even on the raw bit pattern (the same rule the
// reference's device casts use, src/cuda_training.rs:32-39).
uint16_t rbo_f32_to_bf16(float f) {
    uint32_t b = f32_to_bits(f);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x0040u);
    b += 0x7fffu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}
float rbo_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

void rbo_round_to_bf16(float* data, int64_t n) {
    for (int64_t i = 0; i < n; ++i) data[i] = rbo_bf16_to_f32(rbo_f32_to_bf16(data[i]));
}

// ---------------------------------------------------------------------------
// Router logits: logits[t,e] = sum_c x[t,c] * w[e,c] (+ bias[e]).
// Follows Router::forward (src/moe.rs:107-110) -> Linear::forward
// (src/param.rs:762-796, bias-free, weight [out,in] row-major) ->
// Matrix::dot_rhs_transposed (src/matrix.rs:121-173).
//
// Summation order.  For one input row the reference computes each logit with
// its eight-lane `dot` (src/matrix.rs:26-40, taken at src/matrix.rs:131-153):
//   lanes[c % 8] += x[c] * w[c]      for c below tail = d - d % 8
//   rest         += x[c] * w[c]      for the remaining columns
//   result = ((((((((0 + lanes[0]) + lanes[1]) + ...) + lanes[7]) + rest
// each `+=` being a rounded multiply followed by a rounded add (Rust never
// contracts them).  For more than one row the reference calls sgemm, whose
// order is not visible; this build uses the `dot` order for every row count,
// so the single-row path follows the reference text exactly and the multi-row
// path is this build's fixed contract.  bias[e], when given, is added last.
// `bias` is not part of the reference router (bias-free); it exists so that a
// benchmark can skew the load (NULL = reference semantics).
// ---------------------------------------------------------------------------
float rbo_dot8(const float* a, const float* b, int n) {
    float lanes[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const int tail = n - n % 8;
    for (int c = 0; c < tail; c += 8)
        for (int l = 0; l < 8; ++l) {
            const float prod = a[c + l] * b[c + l];
            lanes[l] = lanes[l] + prod;
        }
    float rest = 0.0f;
    for (int c = tail; c < n; ++c) {
        const float prod = a[c] * b[c];
        rest = rest + prod;
    }
    float sum = 0.0f;
    for (int l = 0; l < 8; ++l) sum = sum + lanes[l];
    return sum + rest;
}

void rbo_router_logits(const float* x, const float* w, const float* bias, int T, int d, int E,
                       float* logits) {
    for (int t = 0; t < T; ++t)
        for (int e = 0; e < E; ++e) {
            float v = rbo_dot8(x + (int64_t)t * d, w + (int64_t)e * d, d);
            if (bias) v = v + bias[e];
            logits[(int64_t)t * E + e] = v;
        }
}

// The router after `TransformerLm::quantize()` (src/transformer.rs:899-910 reaches it through
// MoeLayer::linears_mut, src/moe.rs:491-500): Linear::forward takes Quantized::matmul_rhs_transposed
// (src/param.rs:778-780, src/quantized.rs:55-99), i.e. per (token, row)
//     dot(activations, weights) * scale                       (:61)
// with `dot` = dot_lanes::<32> on every x86-64 machine with AVX2 and FMA (:179-196; the target feature
// only widens the vectors: Rust never contracts `x * w` and `+=` into one operation), and dot_lanes
// (:154-177): lanes[c % 32] += x[c] * f32(q[c]) over the whole chunks of 32, a scalar `rest` over the
// tail, then lanes.iter().sum() - a fold from 0.0 in lane order - plus rest.  (The 8-lane fallback of
// machines without AVX2 is a different summation order; this restatement follows the 32-lane one.)
float rbo_dot_q8(const float* x, const int8_t* q, int n) {
    float lanes[32];
    for (int l = 0; l < 32; ++l) lanes[l] = 0.0f;
    const int tail = n - n % 32;
    for (int c = 0; c < tail; c += 32)
        for (int l = 0; l < 32; ++l) {
            const float prod = x[c + l] * (float)q[c + l];
            lanes[l] = lanes[l] + prod;
        }
    float rest = 0.0f;
    for (int c = tail; c < n; ++c) {
        const float prod = x[c] * (float)q[c];
        rest = rest + prod;
    }
    float sum = 0.0f;
    for (int l = 0; l < 32; ++l) sum = sum + lanes[l];
    return sum + rest;
}

void rbo_router_logits_q8(const float* x, const int8_t* q, const float* scales, const float* bias, int T, int d,
                          int E, float* logits) {
    for (int t = 0; t < T; ++t)
        for (int e = 0; e < E; ++e) {
            float v = rbo_dot_q8(x + (int64_t)t * d, q + (int64_t)e * d, d) * scales[e];
            if (bias) v = v + bias[e];
            logits[(int64_t)t * E + e] = v;
        }
}

// Same product accumulated in f64 in plain index order; used only to count
// tokens whose routing is sensitive to the f32 summation order.
void rbo_router_logits_f64(const float* x, const float* w, const float* bias, int T, int d, int E,
                           double* logits) {
    for (int t = 0; t < T; ++t)
        for (int e = 0; e < E; ++e) {
            double acc = 0.0;
            for (int c = 0; c < d; ++c)
                acc += (double)x[(int64_t)t * d + c] * (double)w[(int64_t)e * d + c];
            if (bias) acc += (double)bias[e];
            logits[(int64_t)t * E + e] = acc;
        }
}

// ---------------------------------------------------------------------------
// softmax_rows (src/moe.rs:643-656) with softmax (src/activations.rs:56-70):
//   max  = fold(-inf, f32::max)            (NaN-ignoring)
//   sum  = sequential sum of exp(v - max)  in index order
//   lse  = max + ln(sum)
//   p    = exp(v - max) / sum              only if sum > 0
// exp/ln are rbo_expf/rbo_logf.
// ---------------------------------------------------------------------------
void rbo_softmax_rows(const float* logits, int T, int E, float* P, float* lse) {
    for (int t = 0; t < T; ++t) {
        const float* src = logits + (int64_t)t * E;
        float* dst = P + (int64_t)t * E;
        float mx = -std::numeric_limits<float>::infinity();
        for (int e = 0; e < E; ++e)
            if (src[e] > mx) mx = src[e];  // f32::max: a NaN operand never replaces the accumulator
        float sum = 0.0f;
        for (int e = 0; e < E; ++e) {
            dst[e] = rbo_expf(src[e] - mx);
            sum = sum + dst[e];
        }
        lse[t] = mx + rbo_logf(sum);
        if (sum > 0.0f)
            for (int e = 0; e < E; ++e) dst[e] = dst[e] / sum;
    }
}

// ---------------------------------------------------------------------------
// MoeLayer::route (src/moe.rs:553-593).  k rounds; in each, the first expert
// not yet taken is the initial best and is replaced only by a strictly greater
// probability, so ties go to the lower index.  Gates are the chosen
// probabilities divided by their sum (summed in rank order) when that sum is
// positive.  A padding row gets expert -1 (the reference's UNROUTED,
// src/moe.rs:190-191) and gate 0 in all k slots.
// ---------------------------------------------------------------------------
void rbo_route(const float* P, const uint8_t* valid, int T, int E, int k, int32_t* expert_of,
               float* gate_of) {
    for (int t = 0; t < T; ++t) {
        int32_t* eo = expert_of + (int64_t)t * k;
        float* go = gate_of + (int64_t)t * k;
        if (valid && !valid[t]) {
            for (int r = 0; r < k; ++r) {
                eo[r] = -1;
                go[r] = 0.0f;
            }
            continue;
        }
        const float* row = P + (int64_t)t * E;
        for (int r = 0; r < k; ++r) {
            int best = -1;
            for (int e = 0; e < E; ++e) {
                bool taken = false;
                for (int q = 0; q < r; ++q) taken = taken || (eo[q] == e);
                if (taken) continue;
                if (best < 0 || row[e] > row[best]) best = e;
            }
            eo[r] = best;
            go[r] = row[best];
        }
        float total = 0.0f;
        for (int r = 0; r < k; ++r) total = total + go[r];
        if (total > 0.0f)
            for (int r = 0; r < k; ++r) go[r] = go[r] / total;
    }
}

// ---------------------------------------------------------------------------
// Bucket loop (src/moe.rs:266-274): walking the slots in increasing order and
// appending each routed slot to its expert's list is a stable counting sort.
// counts[e]  = length of expert e's list
// offsets[e] = exclusive prefix sum (offsets[E] = total routed slots)
// perm_slot[offsets[e] + i]  = i-th slot of expert e (expert_slots)
// perm_token[offsets[e] + i] = its token = slot / k (expert_tokens)
// ---------------------------------------------------------------------------
void rbo_bucket(const int32_t* expert_of, int S, int E, int k, int32_t* counts, int32_t* offsets,
                int32_t* perm_slot, int32_t* perm_token) {
    std::vector<std::vector<int32_t>> slots(E);
    for (int s = 0; s < S; ++s) {
        const int32_t e = expert_of[s];
        if (e < 0) continue;
        slots[e].push_back(s);
    }
    int32_t run = 0;
    for (int e = 0; e < E; ++e) {
        counts[e] = (int32_t)slots[e].size();
        offsets[e] = run;
        for (size_t i = 0; i < slots[e].size(); ++i) {
            perm_slot[run + (int32_t)i] = slots[e][i];
            perm_token[run + (int32_t)i] = slots[e][i] / k;
        }
        run += counts[e];
    }
    offsets[E] = run;
}

// ---------------------------------------------------------------------------
// Dense product y[M,N] = x[M,K] * w[N,K]^T in f32 — the shape of
// Matrix::dot_rhs_transposed (src/matrix.rs:121-173).  `rbo_linear_plain` is the
// textbook triple loop with one accumulator in index order; `rbo_linear` is a
// blocked AVX2 version (8 partial sums per output, folded at the end) used where
// speed matters.  Both are f32 and agree to rounding; neither claims sgemm's
// bit pattern.
// ---------------------------------------------------------------------------
void rbo_linear_plain(const float* x, int M, int K, const float* w, int N, float* y) {
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float acc = 0.0f;
            for (int c = 0; c < K; ++c) acc = acc + x[(int64_t)m * K + c] * w[(int64_t)n * K + c];
            y[(int64_t)m * N + n] = acc;
        }
}

static inline float hsum8(__m256 v) {
    __m128 lo = _mm256_castps256_ps128(v);
    __m128 hi = _mm256_extractf128_ps(v, 1);
    lo = _mm_add_ps(lo, hi);
    lo = _mm_add_ps(lo, _mm_movehl_ps(lo, lo));
    lo = _mm_add_ss(lo, _mm_shuffle_ps(lo, lo, 1));
    return _mm_cvtss_f32(lo);
}

// rows [m0, m1) of y
static void linear_rows(const float* x, int m0, int m1, int K, const float* w, int N, float* y) {
    const int K8 = K & ~7;
    int m = m0;
    for (; m + 4 <= m1; m += 4) {
        const float* x0 = x + (int64_t)m * K;
        const float* x1 = x0 + K;
        const float* x2 = x1 + K;
        const float* x3 = x2 + K;
        int n = 0;
        for (; n + 2 <= N; n += 2) {
            const float* w0 = w + (int64_t)n * K;
            const float* w1 = w0 + K;
            __m256 a00 = _mm256_setzero_ps(), a01 = a00, a10 = a00, a11 = a00, a20 = a00, a21 = a00,
                   a30 = a00, a31 = a00;
            for (int c = 0; c < K8; c += 8) {
                const __m256 b0 = _mm256_loadu_ps(w0 + c), b1 = _mm256_loadu_ps(w1 + c);
                __m256 a = _mm256_loadu_ps(x0 + c);
                a00 = _mm256_fmadd_ps(a, b0, a00);
                a01 = _mm256_fmadd_ps(a, b1, a01);
                a = _mm256_loadu_ps(x1 + c);
                a10 = _mm256_fmadd_ps(a, b0, a10);
                a11 = _mm256_fmadd_ps(a, b1, a11);
                a = _mm256_loadu_ps(x2 + c);
                a20 = _mm256_fmadd_ps(a, b0, a20);
                a21 = _mm256_fmadd_ps(a, b1, a21);
                a = _mm256_loadu_ps(x3 + c);
                a30 = _mm256_fmadd_ps(a, b0, a30);
                a31 = _mm256_fmadd_ps(a, b1, a31);
            }
            float r[4][2] = {{hsum8(a00), hsum8(a01)},
                             {hsum8(a10), hsum8(a11)},
                             {hsum8(a20), hsum8(a21)},
                             {hsum8(a30), hsum8(a31)}};
            const float* xs[4] = {x0, x1, x2, x3};
            for (int c = K8; c < K; ++c)
                for (int i = 0; i < 4; ++i) {
                    r[i][0] += xs[i][c] * w0[c];
                    r[i][1] += xs[i][c] * w1[c];
                }
            for (int i = 0; i < 4; ++i) {
                y[(int64_t)(m + i) * N + n] = r[i][0];
                y[(int64_t)(m + i) * N + n + 1] = r[i][1];
            }
        }
        for (; n < N; ++n) {
            const float* w0 = w + (int64_t)n * K;
            const float* xs[4] = {x0, x1, x2, x3};
            for (int i = 0; i < 4; ++i) {
                __m256 a = _mm256_setzero_ps();
                for (int c = 0; c < K8; c += 8)
                    a = _mm256_fmadd_ps(_mm256_loadu_ps(xs[i] + c), _mm256_loadu_ps(w0 + c), a);
                float r = hsum8(a);
                for (int c = K8; c < K; ++c) r += xs[i][c] * w0[c];
                y[(int64_t)(m + i) * N + n] = r;
            }
        }
    }
    for (; m < m1; ++m) {
        const float* x0 = x + (int64_t)m * K;
        for (int n = 0; n < N; ++n) {
            const float* w0 = w + (int64_t)n * K;
            __m256 a = _mm256_setzero_ps();
            for (int c = 0; c < K8; c += 8)
                a = _mm256_fmadd_ps(_mm256_loadu_ps(x0 + c), _mm256_loadu_ps(w0 + c), a);
            float r = hsum8(a);
            for (int c = K8; c < K; ++c) r += x0[c] * w0[c];
            y[(int64_t)m * N + n] = r;
        }
    }
}

void rbo_linear(const float* x, int M, int K, const float* w, int N, float* y) {
    linear_rows(x, 0, M, K, w, N, y);
}

// ---------------------------------------------------------------------------
// int8 weights.  mode 0 = the checkpoint writer's rule (src/transformer.rs:
// 512-519 with :1839-1847): scale = absmax/127, q = clamp(round(w / scale)),
// scale 0 -> q 0.  mode 1 = the in-memory rule (src/quantized.rs:29-51):
// q = clamp(round(w * (1/scale))).  `round` is Rust's f32::round: half away
// from zero.  Product (src/quantized.rs:55-62): y[t,r] = (sum_c x[t,c]*f32(q[r,c]))
// * scale[r]; the reference sums in 8 or 32 lanes (src/quantized.rs:154-177),
// here in plain index order — tolerance only.
// ---------------------------------------------------------------------------
static inline float round_half_away(float v) { return std::round(v); }  // C round(): half away from zero

void rbo_q8_quantize(const float* w, int rows, int cols, int mode, int8_t* q, float* scales) {
    for (int r = 0; r < rows; ++r) {
        const float* row = w + (int64_t)r * cols;
        float absmax = 0.0f;
        for (int c = 0; c < cols; ++c) absmax = std::max(absmax, std::fabs(row[c]));
        const float scale = absmax / 127.0f;
        scales[r] = scale;
        const float inverse = scale > 0.0f ? 1.0f / scale : 0.0f;
        for (int c = 0; c < cols; ++c) {
            float v;
            if (mode == 0)
                v = (scale == 0.0f) ? 0.0f : round_half_away(row[c] / scale);
            else
                v = round_half_away(row[c] * inverse);
            v = std::min(127.0f, std::max(-127.0f, v));
            q[(int64_t)r * cols + c] = (int8_t)v;
        }
    }
}

void rbo_q8_linear(const float* x, int M, int K, const int8_t* q, const float* scales, int N,
                   float* y) {
    std::vector<float> wide((size_t)K);
    for (int n = 0; n < N; ++n) {
        for (int c = 0; c < K; ++c) wide[c] = (float)q[(int64_t)n * K + c];
        for (int m = 0; m < M; ++m) {
            const float* xr = x + (int64_t)m * K;
            __m256 a = _mm256_setzero_ps();
            const int K8 = K & ~7;
            for (int c = 0; c < K8; c += 8)
                a = _mm256_fmadd_ps(_mm256_loadu_ps(xr + c), _mm256_loadu_ps(wide.data() + c), a);
            float r = hsum8(a);
            for (int c = K8; c < K; ++c) r += xr[c] * wide[c];
            y[(int64_t)m * N + n] = r * scales[n];
        }
    }
}

// ---------------------------------------------------------------------------
// SwiGLU (src/ffn.rs:56-85, silu src/ffn.rs:223-229):
//   gate = x Wg^T, up = x Wu^T, hidden = silu(gate) * up, out = hidden Wd^T
//   silu(x) = x * (1 / (1 + exp(-x)))
// Weights are either f32 (q == NULL) or int8 with per-row scales.
// ---------------------------------------------------------------------------
struct rbo_expert_weights {
    const float* gate;  // [F, d]
    const float* up;    // [F, d]
    const float* down;  // [d, F]
    const int8_t* gate_q;
    const int8_t* up_q;
    const int8_t* down_q;
    const float* gate_s;
    const float* up_s;
    const float* down_s;
};

static inline float silu_ref(float x) { return x * (1.0f / (1.0f + std::exp(-x))); }

float rbo_silu(float x) { return silu_ref(x); }

static void swiglu_rows(const rbo_expert_weights* w, const float* x, int m0, int m1, int d, int F,
                        float* gate, float* up, float* hidden, float* out) {
    const int rows = m1 - m0;
    if (rows <= 0) return;
    const float* xs = x + (int64_t)m0 * d;
    float* g = gate + (int64_t)m0 * F;
    float* u = up + (int64_t)m0 * F;
    float* h = hidden + (int64_t)m0 * F;
    float* o = out + (int64_t)m0 * d;
    if (w->gate_q) {
        rbo_q8_linear(xs, rows, d, w->gate_q, w->gate_s, F, g);
        rbo_q8_linear(xs, rows, d, w->up_q, w->up_s, F, u);
    } else {
        linear_rows(xs, 0, rows, d, w->gate, F, g);
        linear_rows(xs, 0, rows, d, w->up, F, u);
    }
    for (int64_t i = 0; i < (int64_t)rows * F; ++i) h[i] = silu_ref(g[i]) * u[i];
    if (w->down_q)
        rbo_q8_linear(h, rows, F, w->down_q, w->down_s, d, o);
    else
        linear_rows(h, 0, rows, F, w->down, d, o);
}

void rbo_swiglu_forward(const rbo_expert_weights* w, const float* x, int M, int d, int F,
                        float* gate, float* up, float* hidden, float* out) {
    swiglu_rows(w, x, 0, M, d, F, gate, up, hidden, out);
}

// ---------------------------------------------------------------------------
// auxiliary_losses (src/moe.rs:602-639).  All sums sequential in f32 over the
// valid tokens in increasing order.
//   load_e = count_e / (V*k); mass_e = (sum_t p[t,e]) / V
//   aux = (sum_e load_e*mass_e) * (E as f32 * w_aux)
//   z   = w_z * (sum_t lse_t^2) / V
// ---------------------------------------------------------------------------
void rbo_aux_losses(const float* P, const float* lse, const int32_t* counts, const uint8_t* valid,
                    int T, int E, int k, float w_aux, float w_z, float* aux_out, float* z_out) {
    int V = 0;
    for (int t = 0; t < T; ++t) V += (!valid || valid[t]) ? 1 : 0;
    if (V == 0) {
        *aux_out = 0.0f;
        *z_out = 0.0f;
        return;
    }
    const float tokens = (float)V;
    const float slots = (float)V * (float)k;
    float aux = 0.0f;
    for (int e = 0; e < E; ++e) {
        const float load = (float)counts[e] / slots;
        float mass = 0.0f;
        for (int t = 0; t < T; ++t)
            if (!valid || valid[t]) mass = mass + P[(int64_t)t * E + e];
        mass = mass / tokens;
        aux = aux + load * mass;
    }
    aux = aux * ((float)E * w_aux);
    float zsum = 0.0f;
    for (int t = 0; t < T; ++t)
        if (!valid || valid[t]) zsum = zsum + lse[t] * lse[t];
    *aux_out = aux;
    *z_out = w_z * zsum / tokens;
}

// ---------------------------------------------------------------------------
// Whole layer: MoeLayer::forward_train (src/moe.rs:243-341).
// ---------------------------------------------------------------------------
struct rbo_layer {
    int32_t d_model, num_experts, experts_per_token, d_ff;
    int32_t shared_expert, shared_d_ff;
    float aux_loss_weight, router_z_loss_weight;
    const float* router;                // [E, d]
    const rbo_expert_weights* experts;  // [E]
    const rbo_expert_weights* shared;   // or NULL
    const int8_t* router_q;             // [E, d] quantized router (then `router` is not read by the forward), or NULL
    const float* router_s;              // [E] its scales
};

struct rbo_outputs {
    float* out;           // [T, d]
    float* logits;        // [T, E] or NULL
    float* probabilities; // [T, E] or NULL
    float* lse;           // [T] or NULL
    int32_t* expert_of;   // [T*k] or NULL
    float* gate_of;       // [T*k] or NULL
    int32_t* counts;      // [E] or NULL
    int32_t* offsets;     // [E+1] or NULL
    int32_t* perm_slot;   // [T*k] or NULL
    int32_t* perm_token;  // [T*k] or NULL
    float* hidden;        // [T*k, F] expert hidden rows in permuted order, or NULL
    float* expert_out;    // [T*k, d] expert output rows in permuted order, or NULL
    float aux_loss, z_loss;
};

// Returns 0, or 1 when `cols` is not d_model (InvalidInput, src/moe.rs:248-253).
// `threads` workers split the (expert, 64-row block) tasks, standing in for
// rayon over experts (src/moe.rs:283-288) nested with threaded sgemm.
int rbo_moe_forward(const rbo_layer* L, const float* x, int T, int cols, const uint8_t* valid,
                    const float* router_bias, int threads, rbo_outputs* O) {
    const int d = L->d_model, E = L->num_experts, k = L->experts_per_token, F = L->d_ff;
    if (cols != d) return 1;
    const int S = T * k;

    std::vector<float> logits((size_t)T * E), P((size_t)T * E), lse((size_t)T);
    if (L->router_q) rbo_router_logits_q8(x, L->router_q, L->router_s, router_bias, T, d, E, logits.data());
    else rbo_router_logits(x, L->router, router_bias, T, d, E, logits.data());
    rbo_softmax_rows(logits.data(), T, E, P.data(), lse.data());

    std::vector<int32_t> expert_of((size_t)S), counts((size_t)E), offsets((size_t)E + 1),
        perm_slot((size_t)S), perm_token((size_t)S);
    std::vector<float> gate_of((size_t)S);
    rbo_route(P.data(), valid, T, E, k, expert_of.data(), gate_of.data());
    rbo_bucket(expert_of.data(), S, E, k, counts.data(), offsets.data(), perm_slot.data(),
               perm_token.data());
    const int R = offsets[E];

    // gather_rows (src/moe.rs:658-664)
    std::vector<float> xg((size_t)std::max(R, 1) * d);
    for (int i = 0; i < R; ++i)
        std::memcpy(xg.data() + (int64_t)i * d, x + (int64_t)perm_token[i] * d, sizeof(float) * d);

    std::vector<float> gate((size_t)std::max(R, 1) * F), up((size_t)std::max(R, 1) * F),
        hidden((size_t)std::max(R, 1) * F), eout((size_t)std::max(R, 1) * d);

    const int Fs = L->shared_d_ff > 0 ? L->shared_d_ff : F;
    std::vector<float> sg, su, sh, so;
    if (L->shared) {
        sg.resize((size_t)T * Fs);
        su.resize((size_t)T * Fs);
        sh.resize((size_t)T * Fs);
        so.resize((size_t)T * d);
    }

    struct Task {
        int expert, m0, m1;
    };
    std::vector<Task> tasks;
    const int BLK = 64;
    for (int e = 0; e < E; ++e)
        for (int m = 0; m < counts[e]; m += BLK) tasks.push_back({e, m, std::min(counts[e], m + BLK)});
    if (L->shared)
        for (int m = 0; m < T; m += BLK) tasks.push_back({E, m, std::min(T, m + BLK)});

    std::atomic<size_t> next{0};
    auto worker = [&]() {
        for (;;) {
            const size_t i = next.fetch_add(1);
            if (i >= tasks.size()) break;
            const Task& tk = tasks[i];
            if (tk.expert < E) {
                const int64_t base = offsets[tk.expert];
                swiglu_rows(&L->experts[tk.expert], xg.data() + base * d, tk.m0, tk.m1, d, F,
                            gate.data() + base * F, up.data() + base * F, hidden.data() + base * F,
                            eout.data() + base * d);
            } else {
                swiglu_rows(L->shared, x, tk.m0, tk.m1, d, Fs, sg.data(), su.data(), sh.data(),
                            so.data());
            }
        }
    };
    const int nthreads = std::max(1, threads);
    if (nthreads == 1) {
        worker();
    } else {
        std::vector<std::thread> pool;
        for (int i = 0; i < nthreads; ++i) pool.emplace_back(worker);
        for (auto& th : pool) th.join();
    }

    // combine (src/moe.rs:290-311): experts ascending, rows ascending,
    // `*target += gate * value` as a separate multiply and add.
    float* out = O->out;
    std::memset(out, 0, sizeof(float) * (size_t)T * d);
    for (int e = 0; e < E; ++e)
        for (int i = 0; i < counts[e]; ++i) {
            const int pos = offsets[e] + i;
            const float g = gate_of[perm_slot[pos]];
            float* dst = out + (int64_t)perm_token[pos] * d;
            const float* src = eout.data() + (int64_t)pos * d;
            for (int c = 0; c < d; ++c) {
                const float prod = g * src[c];
                dst[c] = dst[c] + prod;
            }
        }
    // shared expert over every row, padding included (src/moe.rs:313-319)
    if (L->shared)
        for (int64_t i = 0; i < (int64_t)T * d; ++i) out[i] = out[i] + so[i];

    rbo_aux_losses(P.data(), lse.data(), counts.data(), valid, T, E, k, L->aux_loss_weight,
                   L->router_z_loss_weight, &O->aux_loss, &O->z_loss);

    auto copy_f = [](float* dst, const std::vector<float>& src, size_t n) {
        if (dst && n) std::memcpy(dst, src.data(), n * sizeof(float));
    };
    auto copy_i = [](int32_t* dst, const std::vector<int32_t>& src, size_t n) {
        if (dst && n) std::memcpy(dst, src.data(), n * sizeof(int32_t));
    };
    copy_f(O->logits, logits, (size_t)T * E);
    copy_f(O->probabilities, P, (size_t)T * E);
    copy_f(O->lse, lse, (size_t)T);
    copy_i(O->expert_of, expert_of, (size_t)S);
    copy_f(O->gate_of, gate_of, (size_t)S);
    copy_i(O->counts, counts, (size_t)E);
    copy_i(O->offsets, offsets, (size_t)E + 1);
    copy_i(O->perm_slot, perm_slot, (size_t)R);
    copy_i(O->perm_token, perm_token, (size_t)R);
    copy_f(O->hidden, hidden, (size_t)R * F);
    copy_f(O->expert_out, eout, (size_t)R * d);
    return 0;
}

// ---------------------------------------------------------------------------
// Census of routing decisions that hinge on the last bits of a probability:
// tokens whose k-th and (k+1)-th largest probabilities differ by fewer than
// `ulps` units in the last place.  Such tokens may route differently under
// another summation order or libm; every other token cannot.
// ---------------------------------------------------------------------------
// RmsNorm::forward (reference src/norm.rs:41-61 with inverse_rms, :128-131), the step in front of
// the layer in a decoder block (feed_forward_norm, src/transformer_block.rs:216): per row
// mean_square = (sum of value * value, in index order) / cols; inverse_rms = 1 / sqrt(mean_square + eps);
// out = (value * inverse_rms) * weight.  Pinned by the reference's three forward tests
// (src/norm.rs:138-170) and a float64 closed form (tests/test_oracle_norm.py).
void rbo_rmsnorm_rows(const float* x, int T, int d, const float* weight, float eps, float* out) {
    for (int t = 0; t < T; ++t) {
        const float* row = x + (size_t)t * d;
        float sum = 0.0f;
        for (int c = 0; c < d; ++c) sum = sum + row[c] * row[c];
        const float mean_square = sum / (float)d;
        const float inverse_rms = 1.0f / std::sqrt(mean_square + eps);
        for (int c = 0; c < d; ++c) out[(size_t)t * d + c] = (row[c] * inverse_rms) * weight[c];
    }
}

// RmsNorm::backward (reference src/norm.rs:63-121): returns dL/dinput and ACCUMULATES the scale gradient into
// grad_weight (tiles of 32 rows, per-tile partials added in tile order, src/norm.rs:8-14, :111-118).  The inverse
// rms is recomputed per row.  Pinned by the reference's two finite-difference tests (src/norm.rs:172-216) and a
// float64 differentiation (tests/test_oracle_norm.py).
void rbo_rmsnorm_backward(const float* x, const float* grad_output, int T, int d, const float* weight, float eps,
                          float* grad_input, float* grad_weight) {
    const int ROWS_PER_TILE = 32;
    std::vector<float> partial(d);
    for (int tile0 = 0; tile0 < T; tile0 += ROWS_PER_TILE) {
        std::fill(partial.begin(), partial.end(), 0.0f);
        for (int t = tile0; t < std::min(T, tile0 + ROWS_PER_TILE); ++t) {
            const float* source = x + (size_t)t * d;
            const float* upstream = grad_output + (size_t)t * d;
            float sum = 0.0f;
            for (int c = 0; c < d; ++c) sum = sum + source[c] * source[c];
            const float inverse_rms = 1.0f / std::sqrt(sum / (float)d + eps);
            float projection = 0.0f;
            for (int c = 0; c < d; ++c) projection += upstream[c] * weight[c] * source[c];
            const float shared = projection * (inverse_rms * inverse_rms * inverse_rms) / (float)d;  // powi(3)
            for (int c = 0; c < d; ++c)
                grad_input[(size_t)t * d + c] = upstream[c] * weight[c] * inverse_rms - source[c] * shared;
            for (int c = 0; c < d; ++c) partial[c] += upstream[c] * source[c] * inverse_rms;
        }
        for (int c = 0; c < d; ++c) grad_weight[c] += partial[c];
    }
}

int rbo_near_ties(const float* P, int T, int E, int k, int ulps) {
    if (k >= E) return 0;
    int n = 0;
    std::vector<float> row((size_t)E);
    for (int t = 0; t < T; ++t) {
        std::copy(P + (int64_t)t * E, P + (int64_t)(t + 1) * E, row.begin());
        std::sort(row.begin(), row.end(), [](float a, float b) { return a > b; });
        const int32_t a = (int32_t)f32_to_bits(row[k - 1]);
        const int32_t b = (int32_t)f32_to_bits(row[k]);
        if (a - b < ulps) ++n;
    }
    return n;
}


// ---------------------------------------------------------------------------
// Backward pass: MoeLayer::backward (src/moe.rs:348-489) with SwiGlu::backward
// (src/ffn.rs:87-120), Linear::backward (src/param.rs:799-825: weight.grad +=
// grad_output^T . input, grad_input = grad_output . weight) and
// silu_derivative (src/ffn.rs:235-238).  f32 expert weights only (the
// reference's quantized experts have no backward).  The forward pass is
// recomputed here to obtain what MoeCache holds.  Gradients are ACCUMULATED
// into the weight-gradient buffers, as the reference accumulates into
// Param.grad; grad_input is overwritten.
// Order of the contributions to grad_input, as in the reference: shared expert,
// then the routed experts in ascending expert index (rows ascending), then the
// router.  The auxiliary losses' gradients reach the router here (the load
// fractions are constants, as in the reference).
// ---------------------------------------------------------------------------
struct rbo_grads {
    float* grad_input;    // [T, d]
    float* grad_router;   // [E, d]
    float* grad_gate;     // [E, F, d]
    float* grad_up;       // [E, F, d]
    float* grad_down;     // [E, d, F]
    float* grad_sgate;    // [Fs, d] or NULL
    float* grad_sup;      // [Fs, d] or NULL
    float* grad_sdown;    // [d, Fs] or NULL
    float* grad_gates;    // [T*k] dL/dgate per slot, or NULL (diagnostic)
    float* grad_logits;   // [T, E] or NULL (diagnostic)
};

static float silu_derivative_ref(float x) {
    const float s = 1.0f / (1.0f + std::exp(-x));
    return s * (1.0f + x * (1.0f - s));
}

// y[M, K] = g[M, N] . w[N, K]      (grad_input = grad_output . weight)
static void matmul_nn(const float* g, const float* w, int M, int N, int K, float* y) {
    for (int m = 0; m < M; ++m) {
        float* yr = y + (int64_t)m * K;
        for (int c = 0; c < K; ++c) yr[c] = 0.0f;
        for (int n = 0; n < N; ++n) {
            const float gv = g[(int64_t)m * N + n];
            const float* wr = w + (int64_t)n * K;
            for (int c = 0; c < K; ++c) yr[c] = yr[c] + gv * wr[c];
        }
    }
}

// dw[N, K] += g[M, N]^T . x[M, K]  (weight.grad += grad_output^T . input)
static void matmul_tn_acc(const float* g, const float* x, int M, int N, int K, float* dw) {
    for (int m = 0; m < M; ++m) {
        const float* xr = x + (int64_t)m * K;
        for (int n = 0; n < N; ++n) {
            const float gv = g[(int64_t)m * N + n];
            float* dr = dw + (int64_t)n * K;
            for (int c = 0; c < K; ++c) dr[c] = dr[c] + gv * xr[c];
        }
    }
}

// SwiGlu::backward for `rows` rows; returns grad_input in gx [rows, d]
static void swiglu_backward(const rbo_expert_weights* w, const float* x, const float* gate, const float* up,
                            const float* hidden, const float* gy, int rows, int d, int F, float* dgate_w,
                            float* dup_w, float* ddown_w, float* gx) {
    std::vector<float> gh((size_t)rows * F), gg((size_t)rows * F), gu((size_t)rows * F), tmp((size_t)rows * d);
    matmul_tn_acc(gy, hidden, rows, d, F, ddown_w);       // down.weight.grad += gy^T . hidden
    matmul_nn(gy, w->down, rows, d, F, gh.data());        // grad_hidden = gy . Wdown
    for (int64_t i = 0; i < (int64_t)rows * F; ++i) {
        const float g = gate[i];
        gg[i] = gh[i] * up[i] * silu_derivative_ref(g);
        gu[i] = gh[i] * silu_ref(g);
    }
    matmul_tn_acc(gg.data(), x, rows, F, d, dgate_w);
    matmul_nn(gg.data(), w->gate, rows, F, d, gx);
    matmul_tn_acc(gu.data(), x, rows, F, d, dup_w);
    matmul_nn(gu.data(), w->up, rows, F, d, tmp.data());
    for (int64_t i = 0; i < (int64_t)rows * d; ++i) gx[i] = gx[i] + tmp[i];
}

// Returns 0; 1 when cols != d_model; 2 when an expert is quantized.
// `threads` > 1: experts are independent tasks (their forward rows, then their backward); everything that adds
// into rows shared between experts runs afterwards on one thread, in the same order as with one thread, so the
// results do not depend on the thread count.
int rbo_moe_backward_mt(const rbo_layer* L, const float* x, int T, int cols, const uint8_t* valid,
                        const float* router_bias, const float* grad_output, rbo_grads* G, int threads) {
    const int d = L->d_model, E = L->num_experts, k = L->experts_per_token, F = L->d_ff;
    if (cols != d) return 1;
    for (int e = 0; e < E; ++e)
        if (L->experts[e].gate_q) return 2;
    if (L->shared && L->shared->gate_q) return 2;
    const int S = T * k;
    const int Fs = L->shared_d_ff > 0 ? L->shared_d_ff : F;

    // ---- what the forward pass cached ------------------------------------------
    std::vector<float> logits((size_t)T * E), P((size_t)T * E), lse((size_t)T), gate_of((size_t)S);
    std::vector<int32_t> expert_of((size_t)S), counts((size_t)E), offsets((size_t)E + 1), perm_slot((size_t)S),
        perm_token((size_t)S);
    rbo_router_logits(x, L->router, router_bias, T, d, E, logits.data());
    rbo_softmax_rows(logits.data(), T, E, P.data(), lse.data());
    rbo_route(P.data(), valid, T, E, k, expert_of.data(), gate_of.data());
    rbo_bucket(expert_of.data(), S, E, k, counts.data(), offsets.data(), perm_slot.data(), perm_token.data());
    const int R = offsets[E];
    int V = 0;
    for (int t = 0; t < T; ++t) V += (!valid || valid[t]) ? 1 : 0;
    const size_t Rn = (size_t)std::max(R, 1);
    std::vector<float> xg(Rn * d), gate(Rn * F), up(Rn * F), hidden(Rn * F), eout(Rn * d);
    for (int i = 0; i < R; ++i)
        std::memcpy(xg.data() + (int64_t)i * d, x + (int64_t)perm_token[i] * d, sizeof(float) * d);
    auto for_each_expert = [&](auto&& body) {
        std::atomic<int> next{0};
        auto worker = [&]() {
            for (;;) {
                const int e = next.fetch_add(1);
                if (e >= E) break;
                body(e);
            }
        };
        const int nthreads = std::max(1, std::min(threads, E));
        if (nthreads == 1) {
            worker();
        } else {
            std::vector<std::thread> pool;
            for (int i = 0; i < nthreads; ++i) pool.emplace_back(worker);
            for (auto& th : pool) th.join();
        }
    };
    for_each_expert([&](int e) {
        swiglu_rows(&L->experts[e], xg.data() + (int64_t)offsets[e] * d, 0, counts[e], d, F,
                    gate.data() + (int64_t)offsets[e] * F, up.data() + (int64_t)offsets[e] * F,
                    hidden.data() + (int64_t)offsets[e] * F, eout.data() + (int64_t)offsets[e] * d);
    });

    float* gin = G->grad_input;
    std::memset(gin, 0, sizeof(float) * (size_t)T * d);

    // ---- shared expert (src/moe.rs:356-361) ----------------------------------------
    if (L->shared) {
        std::vector<float> sg((size_t)T * Fs), su((size_t)T * Fs), sh((size_t)T * Fs), so((size_t)T * d),
            sgx((size_t)T * d);
        swiglu_rows(L->shared, x, 0, T, d, Fs, sg.data(), su.data(), sh.data(), so.data());
        swiglu_backward(L->shared, x, sg.data(), su.data(), sh.data(), grad_output, T, d, Fs, G->grad_sgate,
                        G->grad_sup, G->grad_sdown, sgx.data());
        for (int64_t i = 0; i < (int64_t)T * d; ++i) gin[i] = gin[i] + sgx[i];
    }

    // ---- routed experts (src/moe.rs:366-399) -----------------------------------------
    std::vector<float> grad_gates((size_t)std::max(S, 1), 0.0f);
    std::vector<float> gx_rows(Rn * d);  // every expert's input-gradient rows, permuted order
    for_each_expert([&](int e) {
        const int rows = counts[e];
        if (rows == 0) return;
        const int64_t base = offsets[e];
        std::vector<float> scaled((size_t)rows * d);
        for (int i = 0; i < rows; ++i) {
            const float g = gate_of[perm_slot[base + i]];
            const float* upstream = grad_output + (int64_t)perm_token[base + i] * d;
            for (int c = 0; c < d; ++c) scaled[(int64_t)i * d + c] = g * upstream[c];
        }
        swiglu_backward(&L->experts[e], xg.data() + base * d, gate.data() + base * F, up.data() + base * F,
                        hidden.data() + base * F, scaled.data(), rows, d, F, G->grad_gate + (int64_t)e * F * d,
                        G->grad_up + (int64_t)e * F * d, G->grad_down + (int64_t)e * d * F, gx_rows.data() + base * d);
    });
    for (int e = 0; e < E; ++e) {  // scatter-add in expert order, rows ascending (src/moe.rs:392-398)
        const int64_t base = offsets[e];
        for (int i = 0; i < counts[e]; ++i) {
            float* dst = gin + (int64_t)perm_token[base + i] * d;
            const float* src = gx_rows.data() + (base + i) * d;
            for (int c = 0; c < d; ++c) dst[c] = dst[c] + src[c];
        }
    }
    // gate gradients: one dot product per routed slot (src/moe.rs:404-416)
    for (int e = 0; e < E; ++e)
        for (int i = 0; i < counts[e]; ++i) {
            const int64_t pos = offsets[e] + i;
            const float* go = grad_output + (int64_t)perm_token[pos] * d;
            const float* eo = eout.data() + pos * d;
            float sum = 0.0f;
            for (int c = 0; c < d; ++c) sum = sum + go[c] * eo[c];
            grad_gates[perm_slot[pos]] = sum;
        }

    // ---- through the renormalisation, the softmax and the two losses (src/moe.rs:421-478) ----
    std::vector<float> gp((size_t)T * E, 0.0f), gl((size_t)T * E, 0.0f);
    for (int t = 0; t < T; ++t) {
        const int32_t* sel = expert_of.data() + (int64_t)t * k;
        if (sel[0] < 0) continue;
        const float* p = P.data() + (int64_t)t * E;
        float total = 0.0f;
        for (int r = 0; r < k; ++r) total = total + p[sel[r]];
        if (total <= 0.0f) continue;
        float weighted = 0.0f;
        for (int r = 0; r < k; ++r) weighted = weighted + grad_gates[(int64_t)t * k + r] * p[sel[r]];
        float* row = gp.data() + (int64_t)t * E;
        for (int r = 0; r < k; ++r)
            row[sel[r]] = row[sel[r]] + (grad_gates[(int64_t)t * k + r] / total - weighted / (total * total));
    }
    if (L->aux_loss_weight != 0.0f && V > 0) {
        const float scale = L->aux_loss_weight * (float)E / (float)V;
        const float slots = (float)(V * k);
        for (int e = 0; e < E; ++e) {
            const float load = (float)counts[e] / slots;
            for (int t = 0; t < T; ++t) {
                if (expert_of[(int64_t)t * k] < 0) continue;
                gp[(int64_t)t * E + e] = gp[(int64_t)t * E + e] + scale * load;
            }
        }
    }
    for (int t = 0; t < T; ++t) {
        if (expert_of[(int64_t)t * k] < 0) continue;
        const float* p = P.data() + (int64_t)t * E;
        const float* upstream = gp.data() + (int64_t)t * E;
        float dot = 0.0f;
        for (int e = 0; e < E; ++e) dot = dot + p[e] * upstream[e];
        float* row = gl.data() + (int64_t)t * E;
        for (int e = 0; e < E; ++e) row[e] = p[e] * (upstream[e] - dot);
        if (L->router_z_loss_weight != 0.0f) {
            const float factor = 2.0f * L->router_z_loss_weight * lse[t] / (float)std::max(V, 1);
            for (int e = 0; e < E; ++e) row[e] = row[e] + factor * p[e];
        }
    }
    // ---- router (src/moe.rs:480-484) ------------------------------------------------
    matmul_tn_acc(gl.data(), x, T, E, d, G->grad_router);
    std::vector<float> from_router((size_t)T * d);
    matmul_nn(gl.data(), L->router, T, E, d, from_router.data());
    for (int64_t i = 0; i < (int64_t)T * d; ++i) gin[i] = gin[i] + from_router[i];

    if (G->grad_gates && S > 0) std::memcpy(G->grad_gates, grad_gates.data(), sizeof(float) * (size_t)S);
    if (G->grad_logits) std::memcpy(G->grad_logits, gl.data(), sizeof(float) * (size_t)T * E);
    return 0;
}

int rbo_moe_backward(const rbo_layer* L, const float* x, int T, int cols, const uint8_t* valid,
                     const float* router_bias, const float* grad_output, rbo_grads* G) {
    return rbo_moe_backward_mt(L, x, T, cols, valid, router_bias, grad_output, G, 1);
}

}  // extern "C"
