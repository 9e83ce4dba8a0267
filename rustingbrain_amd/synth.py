"""Seeded synthetic tensors for the mixture-of-experts layer workloads.

The reference draws its weights from Rust's ``StdRng`` (``Param::he_uniform``,
reference src/param.rs:240-246), a stream that cannot be reproduced without the
Rust toolchain.  The benchmark workloads specify distributions, not streams, so
this module defines its own counter-based generator: value ``i`` of tensor
``stream`` under ``seed`` depends only on ``(seed, stream, i)``.

    key   = mix(seed * GOLDEN + stream)
    r(i)  = mix(key + (i + 1) * GOLDEN)                    (splitmix64 finaliser)
    U(i)  = (r(i) >> 11) * 2**-53                          in [0, 1)
    uniform(+-a) : f32((2 U(i) - 1) * a)
    normal(std)  : Box-Muller on (1 - U(2i), U(2i + 1)) in f64, f32(z * std)
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z: np.ndarray) -> np.ndarray:
    z = np.asarray(z, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        z = z ^ (z >> np.uint64(31))
    return z


def _raw(seed: int, stream: int, start: int, n: int) -> np.ndarray:
    with np.errstate(over="ignore"):
        key = _mix(np.uint64(seed) * _GOLDEN + np.uint64(stream))
        idx = np.arange(start + 1, start + n + 1, dtype=np.uint64)
        return _mix(key + idx * _GOLDEN)


def _unit(seed: int, stream: int, start: int, n: int) -> np.ndarray:
    return (_raw(seed, stream, start, n) >> np.uint64(11)).astype(np.float64) * (2.0 ** -53)


def uniform(shape, bound: float, seed: int, stream: int) -> np.ndarray:
    n = int(np.prod(shape))
    u = _unit(seed, stream, 0, n)
    return ((2.0 * u - 1.0) * float(bound)).astype(np.float32).reshape(shape)


def normal(shape, std: float, seed: int, stream: int) -> np.ndarray:
    n = int(np.prod(shape))
    u = _unit(seed, stream, 0, 2 * n)
    u1 = 1.0 - u[0::2]
    u2 = u[1::2]
    z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return (z * float(std)).astype(np.float32).reshape(shape)


def xavier_uniform(rows: int, cols: int, seed: int, stream: int) -> np.ndarray:
    """U(+-sqrt(6 / (fan_in + fan_out))) for a ``[out, in]`` weight."""
    bound = float(np.sqrt(6.0 / (rows + cols)))
    return uniform((rows, cols), bound, seed, stream)


# --------------------------------------------------------------------------- bf16
def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round to nearest even on the raw bit pattern; returns uint16."""
    b = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    nan = (b & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    r = b + np.uint32(0x7FFF) + ((b >> np.uint32(16)) & np.uint32(1))
    out = (r >> np.uint32(16)).astype(np.uint16)
    out[nan] = ((b[nan] >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16)
    return out


def bf16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_bf16(a: np.ndarray) -> np.ndarray:
    """f32 array whose values are exactly representable in bf16."""
    return bf16_bits_to_f32(f32_to_bf16_bits(a)).reshape(np.shape(a))


# --------------------------------------------------------------------------- int8
def quantize_rows(w: np.ndarray):
    """Per-output-row symmetric int8, the checkpoint writer's rule.

    ``scale = absmax / 127``; ``q = clamp(round(w / scale), -127, 127)`` with
    rounding half away from zero; a zero row keeps scale 0 and q 0
    (reference src/transformer.rs:512-519 and :1839-1847).
    """
    w = np.ascontiguousarray(w, dtype=np.float32)
    absmax = np.max(np.abs(w), axis=1).astype(np.float32)
    scale = (absmax / np.float32(127.0)).astype(np.float32)
    safe = np.where(scale > 0, scale, np.float32(1.0)).astype(np.float32)
    v = (w / safe[:, None]).astype(np.float32)
    a = np.abs(v)
    fl = np.floor(a)
    frac = a - fl  # exact in f32
    r = np.sign(v) * (fl + (frac >= np.float32(0.5)))
    q = np.clip(r, -127, 127).astype(np.int8)
    q[scale == 0] = 0
    return q, scale


# --------------------------------------------------------------------------- workloads
@dataclass
class Workload:
    name: str
    d_model: int
    num_experts: int
    experts_per_token: int
    d_ff: int
    tokens: int
    seed: int
    act_dtype: str            # "f32" | "bf16"
    weight_dtype: str         # "f32" | "bf16" | "int8"
    shared_expert: bool = False
    shared_d_ff: int = 0
    skew_share: float = 0.0   # >0: router bias on expert 0 sized for this share of assignments
    description: str = ""


WORKLOADS: Dict[str, Workload] = {
    "c1_f32_d512_e8": Workload("c1_f32_d512_e8", 512, 8, 2, 1408, 1024, 42, "f32", "f32",
                               description="README layer, all f32, 2x512 tokens"),
    "c2_decode_d768_e8": Workload("c2_decode_d768_e8", 768, 8, 2, 1408, 8, 1, "bf16", "bf16",
                                  shared_expert=True, shared_d_ff=1408,
                                  description="decode-shaped, 8 tokens, shared expert"),
    "c3_prefill_d768_e16": Workload("c3_prefill_d768_e16", 768, 16, 2, 1408, 8192, 7, "bf16", "bf16",
                                    skew_share=0.30,
                                    description="headline: 8192 tokens, one expert takes ~30%"),
    "c4_finegrained_d1024_e64": Workload("c4_finegrained_d1024_e64", 1024, 64, 6, 704, 16384, 11, "bf16", "bf16",
                                         shared_expert=True, shared_d_ff=1408,
                                         description="64 experts top-6 + shared expert"),
    "c5_int8_d768_e8": Workload("c5_int8_d768_e8", 768, 8, 2, 1408, 4096, 3, "bf16", "int8",
                                description="int8 weight-only experts"),
}

# tensor stream ids
_S_X, _S_ROUTER, _S_EXPERT0, _S_SHARED = 1, 2, 1000, 900


@dataclass
class Tensors:
    """All host tensors of one workload, as f32 arrays holding the stored values.

    For bf16 workloads every value is exactly representable in bf16; for int8
    workloads ``experts[e]`` holds (q, scales) triples instead of f32 matrices.
    """
    workload: Workload
    x: np.ndarray
    router: np.ndarray
    experts: List[dict]
    shared: Optional[dict]
    router_bias: Optional[np.ndarray]


def _expert(w: Workload, d_ff: int, stream: int, quantized: bool, bf16: bool) -> dict:
    gate = xavier_uniform(d_ff, w.d_model, w.seed, stream)
    up = xavier_uniform(d_ff, w.d_model, w.seed, stream + 1)
    down = xavier_uniform(w.d_model, d_ff, w.seed, stream + 2)
    if quantized:
        out = {}
        for name, m in (("gate", gate), ("up", up), ("down", down)):
            q, s = quantize_rows(m)
            out[name + "_q"] = q
            out[name + "_s"] = s
        return out
    if bf16:
        gate, up, down = round_bf16(gate), round_bf16(up), round_bf16(down)
    return {"gate": gate, "up": up, "down": down}


def skew_bias(x: np.ndarray, router: np.ndarray, k: int, share: float) -> float:
    """Bias for expert 0's logit so that it takes ``share`` (+-0.01) of the
    assignments: bisection on top-k of the f64 logits.  The share is a
    statistic of thousands of tokens, so the summation order is immaterial."""
    logits = x.astype(np.float64) @ router.astype(np.float64).T
    lo, hi, b = 0.0, 8.0, 0.0
    for _ in range(60):
        b = 0.5 * (lo + hi)
        shifted = logits.copy()
        shifted[:, 0] += np.float64(np.float32(b))
        top = np.argsort(-shifted, axis=1, kind="stable")[:, :k]
        frac = float(np.mean(top == 0))
        if abs(frac - share) <= 0.002:
            break
        if frac < share:
            lo = b
        else:
            hi = b
    return float(np.float32(b))


def make(name_or_workload, tokens: Optional[int] = None) -> Tensors:
    w = WORKLOADS[name_or_workload] if isinstance(name_or_workload, str) else name_or_workload
    T = w.tokens if tokens is None else tokens
    bf16 = w.act_dtype == "bf16"
    x = normal((T, w.d_model), 1.0, w.seed, _S_X)
    router = normal((w.num_experts, w.d_model), 0.02, w.seed, _S_ROUTER)
    if bf16:
        x = round_bf16(x)
    if w.weight_dtype in ("bf16", "int8"):
        router = round_bf16(router)
    quantized = w.weight_dtype == "int8"
    wbf16 = w.weight_dtype == "bf16"
    experts = [_expert(w, w.d_ff, _S_EXPERT0 + 3 * e, quantized, wbf16) for e in range(w.num_experts)]
    shared = None
    if w.shared_expert:
        shared = _expert(w, w.shared_d_ff or w.d_ff, _S_SHARED, quantized, wbf16)
    bias = None
    if w.skew_share > 0.0:
        bias = np.zeros((w.num_experts,), np.float32)
        bias[0] = skew_bias(x, router, w.experts_per_token, w.skew_share)
    return Tensors(w, x, router, experts, shared, bias)
