"""ctypes binding of the CPU oracle (oracle/rb_oracle.cpp).

TEST INFRASTRUCTURE: imported only by tests/, by ``__graft_entry__.smoke()`` and
by the CPU-baseline leg of ``bench.py``.  Nothing in ``rustingbrain_amd`` imports
it.  Every function is a thin call into the C++ restatement of the reference
algorithm; arrays are numpy, f32/int32/uint8, C-contiguous.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "librb_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with g++ (see oracle/Makefile)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "librb_oracle.so"], check=True, capture_output=True)
    return _SO


def _load() -> C.CDLL:
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


_lib = _load()

_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)
_i32p = C.POINTER(C.c_int32)
_u8p = C.POINTER(C.c_uint8)
_i8p = C.POINTER(C.c_int8)


def _fp(a: Optional[np.ndarray]):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(_f32p)


def _ip(a: Optional[np.ndarray]):
    if a is None:
        return None
    assert a.dtype == np.int32 and a.flags.c_contiguous
    return a.ctypes.data_as(_i32p)


def _up(a: Optional[np.ndarray]):
    if a is None:
        return None
    assert a.dtype == np.uint8 and a.flags.c_contiguous
    return a.ctypes.data_as(_u8p)


def _qp(a: Optional[np.ndarray]):
    if a is None:
        return None
    assert a.dtype == np.int8 and a.flags.c_contiguous
    return a.ctypes.data_as(_i8p)


_lib.rbo_expf.restype = C.c_float
_lib.rbo_expf.argtypes = [C.c_float]
_lib.rbo_logf.restype = C.c_float
_lib.rbo_logf.argtypes = [C.c_float]
_lib.rbo_expf_array.restype = None
_lib.rbo_expf_array.argtypes = [_f32p, C.c_int64, _f32p]
_lib.rbo_logf_array.restype = None
_lib.rbo_logf_array.argtypes = [_f32p, C.c_int64, _f32p]
_lib.rbo_silu.restype = C.c_float
_lib.rbo_silu.argtypes = [C.c_float]
_lib.rbo_f32_to_bf16.restype = C.c_uint16
_lib.rbo_f32_to_bf16.argtypes = [C.c_float]
_lib.rbo_round_to_bf16.restype = None
_lib.rbo_round_to_bf16.argtypes = [_f32p, C.c_int64]
_lib.rbo_near_ties.restype = C.c_int
_lib.rbo_near_ties.argtypes = [_f32p, C.c_int, C.c_int, C.c_int, C.c_int]


def expf(x: float) -> float:
    return float(_lib.rbo_expf(C.c_float(x)))


def logf(x: float) -> float:
    return float(_lib.rbo_logf(C.c_float(x)))


def silu(x: float) -> float:
    return float(_lib.rbo_silu(C.c_float(x)))


def expf_array(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    _lib.rbo_expf_array(_fp(x), x.size, _fp(y))
    return y


def logf_array(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty_like(x)
    _lib.rbo_logf_array(_fp(x), x.size, _fp(y))
    return y


def round_to_bf16(a: np.ndarray) -> np.ndarray:
    out = np.ascontiguousarray(a, dtype=np.float32).copy()
    _lib.rbo_round_to_bf16(_fp(out), out.size)
    return out


_lib.rbo_dot8.restype = C.c_float
_lib.rbo_dot8.argtypes = [_f32p, _f32p, C.c_int]


def dot8(a: np.ndarray, b: np.ndarray) -> float:
    return float(_lib.rbo_dot8(_fp(a), _fp(b), a.size))


def router_logits(x: np.ndarray, w: np.ndarray, bias: Optional[np.ndarray] = None) -> np.ndarray:
    T, d = x.shape
    E = w.shape[0]
    assert w.shape[1] == d
    out = np.empty((T, E), dtype=np.float32)
    _lib.rbo_router_logits(_fp(x), _fp(w), _fp(bias), T, d, E, _fp(out))
    return out


def dot_q8(x: np.ndarray, q: np.ndarray) -> float:
    """f32 activations against int8 weights in the reference's 32-lane order (src/quantized.rs:154-177)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    q = np.ascontiguousarray(q, dtype=np.int8)
    assert x.shape == q.shape and x.ndim == 1
    _lib.rbo_dot_q8.restype = C.c_float
    return float(_lib.rbo_dot_q8(_fp(x), _qp(q), x.shape[0]))


def router_logits_q8(x: np.ndarray, q: np.ndarray, scales: np.ndarray, bias: Optional[np.ndarray] = None) -> np.ndarray:
    """Logits of a quantized router: dot_q8(x[t], q[e]) * scales[e] (+ bias[e])."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    q = np.ascontiguousarray(q, dtype=np.int8)
    scales = np.ascontiguousarray(scales, dtype=np.float32)
    T, d = x.shape
    E = q.shape[0]
    out = np.empty((T, E), np.float32)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32)
    _lib.rbo_router_logits_q8(_fp(x), _qp(q), _fp(scales), _fp(bias), T, d, E, _fp(out))
    return out


def router_logits_f64(x: np.ndarray, w: np.ndarray, bias: Optional[np.ndarray] = None) -> np.ndarray:
    T, d = x.shape
    E = w.shape[0]
    out = np.empty((T, E), dtype=np.float64)
    _lib.rbo_router_logits_f64(_fp(x), _fp(w), _fp(bias), T, d, E, out.ctypes.data_as(_f64p))
    return out


def softmax_rows(logits: np.ndarray):
    T, E = logits.shape
    P = np.empty((T, E), dtype=np.float32)
    lse = np.empty((T,), dtype=np.float32)
    _lib.rbo_softmax_rows(_fp(logits), T, E, _fp(P), _fp(lse))
    return P, lse


def route(P: np.ndarray, k: int, valid: Optional[np.ndarray] = None):
    T, E = P.shape
    expert_of = np.empty((T * k,), dtype=np.int32)
    gate_of = np.empty((T * k,), dtype=np.float32)
    _lib.rbo_route(_fp(P), _up(valid), T, E, k, _ip(expert_of), _fp(gate_of))
    return expert_of, gate_of


def bucket(expert_of: np.ndarray, E: int, k: int):
    S = expert_of.size
    counts = np.zeros((E,), dtype=np.int32)
    offsets = np.zeros((E + 1,), dtype=np.int32)
    perm_slot = np.full((S,), -1, dtype=np.int32)
    perm_token = np.full((S,), -1, dtype=np.int32)
    _lib.rbo_bucket(_ip(expert_of), S, E, k, _ip(counts), _ip(offsets), _ip(perm_slot), _ip(perm_token))
    R = int(offsets[E])
    return counts, offsets, perm_slot[:R].copy(), perm_token[:R].copy()


def linear(x: np.ndarray, w: np.ndarray, plain: bool = False) -> np.ndarray:
    M, K = x.shape
    N = w.shape[0]
    assert w.shape[1] == K
    y = np.empty((M, N), dtype=np.float32)
    fn = _lib.rbo_linear_plain if plain else _lib.rbo_linear
    fn(_fp(x), M, K, _fp(w), N, _fp(y))
    return y


def q8_quantize(w: np.ndarray, mode: int = 0):
    rows, cols = w.shape
    q = np.empty((rows, cols), dtype=np.int8)
    s = np.empty((rows,), dtype=np.float32)
    _lib.rbo_q8_quantize(_fp(w), rows, cols, mode, _qp(q), _fp(s))
    return q, s


def q8_linear(x: np.ndarray, q: np.ndarray, scales: np.ndarray) -> np.ndarray:
    M, K = x.shape
    N = q.shape[0]
    y = np.empty((M, N), dtype=np.float32)
    _lib.rbo_q8_linear(_fp(x), M, K, _qp(q), _fp(scales), N, _fp(y))
    return y


def aux_losses(P, lse, counts, k, w_aux, w_z, valid=None):
    T, E = P.shape
    aux = C.c_float(0)
    z = C.c_float(0)
    _lib.rbo_aux_losses(_fp(P), _fp(lse), _ip(counts), _up(valid), T, E, k, C.c_float(w_aux), C.c_float(w_z),
                        C.byref(aux), C.byref(z))
    return float(aux.value), float(z.value)


def near_ties(P: np.ndarray, k: int, ulps: int = 4) -> int:
    T, E = P.shape
    return int(_lib.rbo_near_ties(_fp(P), T, E, k, ulps))


class _ExpertWeights(C.Structure):
    _fields_ = [("gate", _f32p), ("up", _f32p), ("down", _f32p),
                ("gate_q", _i8p), ("up_q", _i8p), ("down_q", _i8p),
                ("gate_s", _f32p), ("up_s", _f32p), ("down_s", _f32p)]


class _Layer(C.Structure):
    _fields_ = [("d_model", C.c_int32), ("num_experts", C.c_int32), ("experts_per_token", C.c_int32),
                ("d_ff", C.c_int32), ("shared_expert", C.c_int32), ("shared_d_ff", C.c_int32),
                ("aux_loss_weight", C.c_float), ("router_z_loss_weight", C.c_float),
                ("router", _f32p), ("experts", C.POINTER(_ExpertWeights)), ("shared", C.POINTER(_ExpertWeights)),
                ("router_q", C.POINTER(C.c_int8)), ("router_s", _f32p)]


class _Outputs(C.Structure):
    _fields_ = [("out", _f32p), ("logits", _f32p), ("probabilities", _f32p), ("lse", _f32p),
                ("expert_of", _i32p), ("gate_of", _f32p), ("counts", _i32p), ("offsets", _i32p),
                ("perm_slot", _i32p), ("perm_token", _i32p), ("hidden", _f32p), ("expert_out", _f32p),
                ("aux_loss", C.c_float), ("z_loss", C.c_float)]


_lib.rbo_moe_forward.restype = C.c_int
_lib.rbo_moe_forward.argtypes = [C.POINTER(_Layer), _f32p, C.c_int, C.c_int, _u8p, _f32p, C.c_int,
                                 C.POINTER(_Outputs)]
_lib.rbo_swiglu_forward.restype = None
_lib.rbo_swiglu_forward.argtypes = [C.POINTER(_ExpertWeights), _f32p, C.c_int, C.c_int, C.c_int,
                                    _f32p, _f32p, _f32p, _f32p]


@dataclass
class ExpertWeights:
    """One SwiGLU expert: f32 matrices, or int8 matrices with per-row f32 scales."""
    gate: Optional[np.ndarray] = None   # [F, d]
    up: Optional[np.ndarray] = None     # [F, d]
    down: Optional[np.ndarray] = None   # [d, F]
    gate_q: Optional[np.ndarray] = None
    up_q: Optional[np.ndarray] = None
    down_q: Optional[np.ndarray] = None
    gate_s: Optional[np.ndarray] = None
    up_s: Optional[np.ndarray] = None
    down_s: Optional[np.ndarray] = None

    def _c(self) -> _ExpertWeights:
        return _ExpertWeights(_fp(self.gate), _fp(self.up), _fp(self.down),
                              _qp(self.gate_q), _qp(self.up_q), _qp(self.down_q),
                              _fp(self.gate_s), _fp(self.up_s), _fp(self.down_s))


@dataclass
class ForwardResult:
    out: np.ndarray
    logits: np.ndarray
    probabilities: np.ndarray
    lse: np.ndarray
    expert_of: np.ndarray
    gate_of: np.ndarray
    counts: np.ndarray
    offsets: np.ndarray
    perm_slot: np.ndarray
    perm_token: np.ndarray
    hidden: np.ndarray
    expert_out: np.ndarray
    aux_loss: float
    z_loss: float

    def load_fractions(self) -> np.ndarray:
        """MoeCache::load_fractions (reference src/moe.rs:176-182)."""
        slots = max(int(self.counts.sum()), 1)
        return self.counts.astype(np.float32) / np.float32(slots)


class _Grads(C.Structure):
    _fields_ = [("grad_input", _f32p), ("grad_router", _f32p), ("grad_gate", _f32p), ("grad_up", _f32p),
                ("grad_down", _f32p), ("grad_sgate", _f32p), ("grad_sup", _f32p), ("grad_sdown", _f32p),
                ("grad_gates", _f32p), ("grad_logits", _f32p)]


_lib.rbo_moe_backward_mt.restype = C.c_int
_lib.rbo_moe_backward_mt.argtypes = [C.POINTER(_Layer), _f32p, C.c_int, C.c_int, _u8p, _f32p, _f32p, C.POINTER(_Grads), C.c_int]
_lib.rbo_moe_backward.restype = C.c_int
_lib.rbo_moe_backward.argtypes = [C.POINTER(_Layer), _f32p, C.c_int, C.c_int, _u8p, _f32p, _f32p, C.POINTER(_Grads)]


_lib.rbo_rmsnorm_rows.restype = None
_lib.rbo_rmsnorm_rows.argtypes = [_f32p, C.c_int, C.c_int, _f32p, C.c_float, _f32p]


def rmsnorm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """RmsNorm::forward (src/norm.rs:41-61): rows of ``x`` times ``1 / sqrt(mean(x^2) + eps)`` times ``weight``."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    weight = np.ascontiguousarray(weight, dtype=np.float32)
    T, d = x.shape
    assert weight.shape == (d,)
    out = np.empty_like(x)
    _lib.rbo_rmsnorm_rows(_fp(x), T, d, _fp(weight), C.c_float(eps), _fp(out))
    return out


_lib.rbo_rmsnorm_backward.restype = None
_lib.rbo_rmsnorm_backward.argtypes = [_f32p, _f32p, C.c_int, C.c_int, _f32p, C.c_float, _f32p, _f32p]


def rmsnorm_backward(x: np.ndarray, grad_output: np.ndarray, weight: np.ndarray, eps: float):
    """RmsNorm::backward (src/norm.rs:63-121): (dL/dinput, dL/dweight); the weight gradient starts from zero."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    grad_output = np.ascontiguousarray(grad_output, dtype=np.float32)
    weight = np.ascontiguousarray(weight, dtype=np.float32)
    T, d = x.shape
    gi = np.zeros_like(x)
    gw = np.zeros(d, np.float32)
    _lib.rbo_rmsnorm_backward(_fp(x), _fp(grad_output), T, d, _fp(weight), C.c_float(eps), _fp(gi), _fp(gw))
    return gi, gw


@dataclass
class BackwardResult:
    """Gradients of MoeLayer::backward (src/moe.rs:348-489); the weight gradients start from zero here."""
    grad_input: np.ndarray     # [T, d]
    grad_router: np.ndarray    # [E, d]
    grad_gate: np.ndarray      # [E, F, d]
    grad_up: np.ndarray        # [E, F, d]
    grad_down: np.ndarray      # [E, d, F]
    grad_shared: Optional[tuple]  # (gate [Fs, d], up [Fs, d], down [d, Fs]) or None
    grad_gates: np.ndarray     # [T*k]
    grad_logits: np.ndarray    # [T, E]


@dataclass
class OracleLayer:
    d_model: int
    num_experts: int
    experts_per_token: int
    d_ff: int
    router: np.ndarray
    experts: List[ExpertWeights]
    shared: Optional[ExpertWeights] = None
    shared_d_ff: int = 0
    aux_loss_weight: float = 0.01
    router_z_loss_weight: float = 1e-3
    _keep: list = field(default_factory=list, repr=False)
    # the router after TransformerLm::quantize(): int8 rows [E, d] and one scale per row; the forward then routes
    # with the quantized product (src/quantized.rs:55-62) and does not read `router`
    router_q: Optional[np.ndarray] = None
    router_s: Optional[np.ndarray] = None

    def swiglu(self, w: ExpertWeights, x: np.ndarray, d_ff: int):
        M, d = x.shape
        g = np.empty((M, d_ff), np.float32)
        u = np.empty((M, d_ff), np.float32)
        h = np.empty((M, d_ff), np.float32)
        o = np.empty((M, d), np.float32)
        cw = w._c()
        _lib.rbo_swiglu_forward(C.byref(cw), _fp(x), M, d, d_ff, _fp(g), _fp(u), _fp(h), _fp(o))
        return o, g, u, h

    def forward(self, x: np.ndarray, valid: Optional[np.ndarray] = None,
                router_bias: Optional[np.ndarray] = None, threads: int = 1) -> ForwardResult:
        x = np.ascontiguousarray(x, dtype=np.float32)
        T, cols = x.shape
        E, k, F, d = self.num_experts, self.experts_per_token, self.d_ff, self.d_model
        S = T * k
        arr = (_ExpertWeights * E)(*[w._c() for w in self.experts])
        shared_c = self.shared._c() if self.shared is not None else None
        rq = rs = None
        if self.router_q is not None:
            rq = np.ascontiguousarray(self.router_q, dtype=np.int8)
            rs = np.ascontiguousarray(self.router_s, dtype=np.float32)
        layer = _Layer(d, E, k, F, 1 if self.shared is not None else 0, self.shared_d_ff,
                       self.aux_loss_weight, self.router_z_loss_weight, _fp(self.router),
                       C.cast(arr, C.POINTER(_ExpertWeights)),
                       C.pointer(shared_c) if shared_c is not None else None,
                       _qp(rq) if rq is not None else None, _fp(rs))
        res = dict(out=np.zeros((T, max(cols, 1)), np.float32), logits=np.zeros((T, E), np.float32),
                   probabilities=np.zeros((T, E), np.float32), lse=np.zeros((T,), np.float32),
                   expert_of=np.zeros((S,), np.int32), gate_of=np.zeros((S,), np.float32),
                   counts=np.zeros((E,), np.int32), offsets=np.zeros((E + 1,), np.int32),
                   perm_slot=np.full((S,), -1, np.int32), perm_token=np.full((S,), -1, np.int32),
                   hidden=np.zeros((max(S, 1), F), np.float32), expert_out=np.zeros((max(S, 1), d), np.float32))
        outs = _Outputs(_fp(res["out"]), _fp(res["logits"]), _fp(res["probabilities"]), _fp(res["lse"]),
                        _ip(res["expert_of"]), _fp(res["gate_of"]), _ip(res["counts"]), _ip(res["offsets"]),
                        _ip(res["perm_slot"]), _ip(res["perm_token"]), _fp(res["hidden"]),
                        _fp(res["expert_out"]), 0.0, 0.0)
        if valid is not None:
            valid = np.ascontiguousarray(valid, dtype=np.uint8)
        if router_bias is not None:
            router_bias = np.ascontiguousarray(router_bias, dtype=np.float32)
        rc = _lib.rbo_moe_forward(C.byref(layer), _fp(x), T, cols, _up(valid), _fp(router_bias), threads,
                                  C.byref(outs))
        if rc != 0:
            raise ValueError(f"InvalidInput: expected {d} columns, got {cols}")
        R = int(res["offsets"][E])
        res["perm_slot"] = res["perm_slot"][:R]
        res["perm_token"] = res["perm_token"][:R]
        res["hidden"] = res["hidden"][:R]
        res["expert_out"] = res["expert_out"][:R]
        return ForwardResult(aux_loss=float(outs.aux_loss), z_loss=float(outs.z_loss), **res)

    def forward_block(self, residual: np.ndarray, norm_weight: np.ndarray, eps: float,
                      valid: Optional[np.ndarray] = None, router_bias: Optional[np.ndarray] = None,
                      threads: int = 1, round_normed=None):
        """The feed-forward half of TransformerBlock::forward_train (src/transformer_block.rs:216-222):
        ``normed = feed_forward_norm.forward(residual)``, ``projected = moe.forward_train(normed)``,
        ``output = projected + residual``.  ``round_normed`` (e.g. rounding to bf16) is applied to the normed rows
        when the layer's activations are narrower than f32.  Returns (output, normed, ForwardResult)."""
        residual = np.ascontiguousarray(residual, dtype=np.float32)
        normed = rmsnorm(residual, norm_weight, eps)
        if round_normed is not None:
            normed = np.ascontiguousarray(round_normed(normed), dtype=np.float32)
        res = self.forward(normed, valid=valid, router_bias=router_bias, threads=threads)
        return res.out + residual, normed, res

    def backward_block(self, residual: np.ndarray, norm_weight: np.ndarray, eps: float, grad_output: np.ndarray,
                       valid: Optional[np.ndarray] = None, router_bias: Optional[np.ndarray] = None,
                       round_normed=None, threads: int = 1):
        """The feed-forward half of TransformerBlock::backward (src/transformer_block.rs:257-263):
        ``grad_projected = moe.backward(cache, grad_output)``, ``grad_residual = feed_forward_norm.backward(residual,
        grad_projected) + grad_output``.  Returns (grad_residual, grad_norm_weight, BackwardResult of the layer)."""
        residual = np.ascontiguousarray(residual, dtype=np.float32)
        normed = rmsnorm(residual, norm_weight, eps)
        if round_normed is not None:
            normed = np.ascontiguousarray(round_normed(normed), dtype=np.float32)
        inner = self.backward(normed, grad_output, valid=valid, router_bias=router_bias, threads=threads)
        gi, gw = rmsnorm_backward(residual, inner.grad_input, norm_weight, eps)
        return gi + np.ascontiguousarray(grad_output, dtype=np.float32), gw, inner

    def backward(self, x: np.ndarray, grad_output: np.ndarray, valid: Optional[np.ndarray] = None,
                 router_bias: Optional[np.ndarray] = None, threads: int = 1) -> BackwardResult:
        x = np.ascontiguousarray(x, dtype=np.float32)
        grad_output = np.ascontiguousarray(grad_output, dtype=np.float32)
        T, cols = x.shape
        E, k, F, d = self.num_experts, self.experts_per_token, self.d_ff, self.d_model
        Fs = self.shared_d_ff or F
        arr = (_ExpertWeights * E)(*[w._c() for w in self.experts])
        shared_c = self.shared._c() if self.shared is not None else None
        layer = _Layer(d, E, k, F, 1 if self.shared is not None else 0, self.shared_d_ff,
                       self.aux_loss_weight, self.router_z_loss_weight, _fp(self.router),
                       C.cast(arr, C.POINTER(_ExpertWeights)),
                       C.pointer(shared_c) if shared_c is not None else None, None, None)
        gi = np.zeros((T, d), np.float32)
        gr = np.zeros((E, d), np.float32)
        gg = np.zeros((E, F, d), np.float32)
        gu = np.zeros((E, F, d), np.float32)
        gd = np.zeros((E, d, F), np.float32)
        sh = (np.zeros((Fs, d), np.float32), np.zeros((Fs, d), np.float32), np.zeros((d, Fs), np.float32)) \
            if self.shared is not None else None
        ggates = np.zeros((max(T * k, 1),), np.float32)
        gl = np.zeros((T, E), np.float32)
        grads = _Grads(_fp(gi), _fp(gr), _fp(gg), _fp(gu), _fp(gd), _fp(sh[0]) if sh else None,
                       _fp(sh[1]) if sh else None, _fp(sh[2]) if sh else None, _fp(ggates), _fp(gl))
        if valid is not None:
            valid = np.ascontiguousarray(valid, dtype=np.uint8)
        if router_bias is not None:
            router_bias = np.ascontiguousarray(router_bias, dtype=np.float32)
        rc = _lib.rbo_moe_backward_mt(C.byref(layer), _fp(x), T, cols, _up(valid), _fp(router_bias),
                                      _fp(grad_output), C.byref(grads), threads)
        if rc == 1:
            raise ValueError(f"InvalidInput: expected {d} columns, got {cols}")
        if rc == 2:
            raise ValueError("quantized experts have no backward pass")
        return BackwardResult(gi, gr, gg, gu, gd, sh, ggates[:T * k], gl)
