"""Host-side mirror of RustingBrain's mixture-of-experts interface over librbmoe.

Names, argument meaning and error behaviour follow the reference:

* ``MoeConfig``      — reference src/moe.rs:25-87
* ``Layout``         — reference src/batch.rs:224-269
* ``MoeLayer``       — reference src/moe.rs:203-341 (``forward``, ``forward_train``)
* ``MoeCache``       — reference src/moe.rs:131-188 (``aux_loss``, ``z_loss``,
  ``auxiliary_loss``, ``load_fractions`` and the routing tables)
* ``NetworkError``   — reference src/network.rs:19-83 (the variants this path raises)

All arithmetic happens in the HIP library; this module only marshals numpy
arrays (or raw device pointers) across the C ABI.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, replace
from typing import List, Optional, Sequence, Tuple

import numpy as np

from . import _lib as L
from .synth import bf16_bits_to_f32, f32_to_bf16_bits

DEFAULT_AUX_LOSS_WEIGHT = 0.01       # reference src/moe.rs:20
DEFAULT_ROUTER_Z_LOSS_WEIGHT = 1e-3  # reference src/moe.rs:23
UNROUTED = -1                        # reference src/moe.rs:190-191 (usize::MAX there)


# --------------------------------------------------------------------------- errors
class NetworkError(Exception):
    """Base of the error variants this path can raise."""


class InvalidInput(NetworkError):
    def __init__(self, message: str, expected: Optional[int] = None, actual: Optional[int] = None):
        super().__init__(message)
        self.expected, self.actual = expected, actual


class InvalidConfig(NetworkError):
    pass


class DeviceError(NetworkError):          # NetworkError::Cuda(String)
    pass


class BackendUnavailable(NetworkError):   # NetworkError::CudaFeatureDisabled
    pass


class MemoryBudget(NetworkError):         # NetworkError::CudaMemoryBudget
    pass


class OutOfMemory(NetworkError):          # NetworkError::CudaOutOfMemory
    pass


class Unsupported(NetworkError):          # NetworkError::UnsupportedCuda(String)
    pass


_ERRORS = {L.INVALID_INPUT: InvalidInput, L.INVALID_CONFIG: InvalidConfig, L.DEVICE_ERROR: DeviceError,
           L.BACKEND_UNAVAILABLE: BackendUnavailable, L.MEMORY_BUDGET: MemoryBudget,
           L.OUT_OF_MEMORY: OutOfMemory, L.UNSUPPORTED: Unsupported, L.NULL_POINTER: InvalidInput}


def _check(rc: int, ctx=None) -> None:
    if rc == L.OK:
        return
    lib = L.load()
    msg = lib.rbmoe_last_error(ctx) if ctx else lib.rbmoe_last_global_error()
    raise _ERRORS.get(rc, NetworkError)((msg or b"").decode() or f"rbmoe status {rc}")


# --------------------------------------------------------------------------- switches
# The library reads no environment variable; this host layer does, for A/B runs of the benchmark and the tests:
# variable -> (option, value it sets when the variable is "1"), RBMOE_GROUP_M carries its value.
_ENV_SWITCHES = {
    "RBMOE_FORCE_GENERIC": (L.OPT_FORCE_GENERIC, 1), "RBMOE_EXPLICIT_GATHER": (L.OPT_EXPLICIT_GATHER, 1),
    "RBMOE_NO_DECODE_PATH": (L.OPT_DECODE_PATH, 0), "RBMOE_NO_DECODE_FRONT": (L.OPT_DECODE_FRONT, 0),
    "RBMOE_NO_FUSED_ROUTER": (L.OPT_FUSED_ROUTER, 0), "RBMOE_NO_SIDE_STREAM": (L.OPT_SIDE_STREAM, 0),
    "RBMOE_ATOMIC_WGRAD": (L.OPT_WGRAD_MODE, 1), "RBMOE_DETERMINISTIC": (L.OPT_WGRAD_MODE, 2),
    "RBMOE_WGRAD_GENERIC": (L.OPT_WGRAD_GENERIC, 1), "RBMOE_NO_DECODE_COMBINE_FOLD": (L.OPT_DECODE_COMBINE_FOLD, 0),
    "RBMOE_NO_DECODE_DOWN_BY_EXPERT": (L.OPT_DECODE_DOWN_BY_EXPERT, 0),
}


def options_from_environment() -> dict:
    import os
    out = {}
    for name, (option, value) in _ENV_SWITCHES.items():
        if os.environ.get(name, "") == "1":
            out[option] = value
    if os.environ.get("RBMOE_GROUP_M", ""):
        out[L.OPT_GROUP_M] = max(0, int(os.environ["RBMOE_GROUP_M"]))
    return out


# --------------------------------------------------------------------------- config
@dataclass(frozen=True)
class MoeConfig:
    num_experts: int
    experts_per_token: int
    d_ff: int
    shared_expert: bool = False
    aux_loss_weight: float = DEFAULT_AUX_LOSS_WEIGHT
    router_z_loss_weight: float = DEFAULT_ROUTER_Z_LOSS_WEIGHT

    @staticmethod
    def new(num_experts: int, experts_per_token: int, d_ff: int) -> "MoeConfig":
        return MoeConfig(num_experts, experts_per_token, d_ff)

    def with_shared_expert(self, shared_expert: bool) -> "MoeConfig":
        return replace(self, shared_expert=shared_expert)

    def with_aux_loss_weight(self, weight: float) -> "MoeConfig":
        return replace(self, aux_loss_weight=weight)

    def with_router_z_loss_weight(self, weight: float) -> "MoeConfig":
        return replace(self, router_z_loss_weight=weight)

    def _c(self, d_model: int, act_dtype: str = "f32", weight_dtype: str = "f32", max_tokens: int = 0,
           shared_d_ff: int = 0) -> L.Config:
        return L.Config(d_model, self.num_experts, self.experts_per_token, self.d_ff,
                        1 if self.shared_expert else 0, shared_d_ff, self.aux_loss_weight,
                        self.router_z_loss_weight, L.DTYPES[weight_dtype], L.DTYPES[act_dtype], max_tokens)

    def validate(self) -> None:
        """Raises ``InvalidConfig`` exactly where the reference's validate errs."""
        cfg = self._c(1)
        buf = C.create_string_buffer(256)
        rc = L.load().rbmoe_validate(C.byref(cfg), buf, 256)
        if rc != L.OK:
            raise _ERRORS.get(rc, NetworkError)(buf.value.decode())


@dataclass(frozen=True)
class Layout:
    """How the rows of a packed matrix map onto sequences; ``valid`` marks padding."""
    seq_len: Optional[int] = None
    valid: Optional[Sequence[bool]] = None

    @staticmethod
    def single(rows: int) -> "Layout":
        return Layout(seq_len=rows)

    def resolved_seq_len(self, rows: int) -> int:
        return max(self.seq_len if self.seq_len is not None else rows, 1)

    def is_valid(self, row: int) -> bool:
        return True if self.valid is None else bool(self.valid[row])

    def check(self, rows: int) -> None:
        seq_len = self.resolved_seq_len(rows)
        if rows % seq_len != 0:
            raise InvalidConfig(f"{rows} rows do not divide into sequences of {seq_len}")
        if self.valid is not None and len(self.valid) != rows:
            raise InvalidConfig(f"padding mask covers {len(self.valid)} rows, not {rows}")


# --------------------------------------------------------------------------- device
class Device:
    """One GPU with a memory budget: the role of the reference's ``CudaDevice``
    handle (src/param.rs:86-190).  Fails closed when no GPU is usable."""

    def __init__(self, index: int = 0, budget_mib: int = 0):
        self._lib = L.load()
        h = C.c_void_p()
        _check(self._lib.rbmoe_ctx_create(index, budget_mib, C.byref(h)))
        self.handle = h

    @staticmethod
    def open(index: int = 0, budget_mib: int = 0) -> "Device":
        return Device(index, budget_mib)

    def set_stream(self, hip_stream: Optional[int]) -> None:
        _check(self._lib.rbmoe_ctx_set_stream(self.handle, C.c_void_p(hip_stream or 0)), self.handle)

    def synchronize(self) -> None:
        _check(self._lib.rbmoe_synchronize(self.handle), self.handle)

    def close(self) -> None:
        if self.handle:
            self._lib.rbmoe_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# --------------------------------------------------------------------------- cache
@dataclass
class MoeCache:
    """What ``forward_train`` hands back besides the output."""
    assignments: List[Tuple[int, float]]
    expert_of: np.ndarray
    gate_of: np.ndarray
    counts: np.ndarray
    offsets: np.ndarray
    perm_slot: np.ndarray
    perm_token: np.ndarray
    probabilities: np.ndarray
    log_sum_exp: np.ndarray
    valid_tokens: int
    _aux: float
    _z: float

    def aux_loss(self) -> float:
        return self._aux

    def z_loss(self) -> float:
        return self._z

    def auxiliary_loss(self) -> float:
        return float(np.float32(self._aux) + np.float32(self._z))

    def load_fractions(self) -> List[float]:
        slots = np.float32(max(int(self.counts.sum()), 1))
        return [float(np.float32(c) / slots) for c in self.counts]

    @property
    def expert_tokens(self) -> List[np.ndarray]:
        return [self.perm_token[self.offsets[e]:self.offsets[e + 1]] for e in range(len(self.counts))]

    @property
    def expert_slots(self) -> List[np.ndarray]:
        return [self.perm_slot[self.offsets[e]:self.offsets[e + 1]] for e in range(len(self.counts))]


# --------------------------------------------------------------------------- layer
class MoeLayer:
    """``num_experts`` SwiGLU experts, a router and an optional shared expert on
    the GPU.  Weights start at zero; fill them with ``set_router`` /
    ``set_expert`` / ``set_shared`` (``[out_features, in_features]`` matrices,
    as the reference's ``Linear``)."""

    def __init__(self, d_model: int, config: MoeConfig, device: Device, *, act_dtype: str = "f32",
                 weight_dtype: str = "f32", max_tokens: int = 1024, shared_d_ff: int = 0):
        config.validate()
        self.config = config
        self._d_model = d_model
        self.device = device
        self.act_dtype = act_dtype
        self.weight_dtype = weight_dtype
        self.shared_d_ff = shared_d_ff or config.d_ff
        self.max_tokens = max_tokens
        self._lib = L.load()
        cfg = config._c(d_model, act_dtype, weight_dtype, max_tokens, shared_d_ff)
        h = C.c_void_p()
        _check(self._lib.rbmoe_layer_create(device.handle, C.byref(cfg), C.byref(h)), device.handle)
        self.handle = h
        for option, value in options_from_environment().items():
            self.set_option(option, value)

    def set_option(self, option: int, value: int) -> None:
        """A behaviour switch of the layer (``_lib.OPT_*``); every default is the fast path."""
        _check(self._lib.rbmoe_layer_set_option(self.handle, option, value), self.device.handle)

    @staticmethod
    def new(d_model: int, config: MoeConfig, device: Device, **kw) -> "MoeLayer":
        return MoeLayer(d_model, config, device, **kw)

    # ---- shape / accounting (reference src/moe.rs:233-235, :527-545)
    def d_model(self) -> int:
        return self._d_model

    def _counts(self) -> Tuple[int, int]:
        cfg = self.config._c(self._d_model, shared_d_ff=self.shared_d_ff)
        total, active = C.c_uint64(), C.c_uint64()
        _check(self._lib.rbmoe_parameter_counts(C.byref(cfg), C.byref(total), C.byref(active)))
        return int(total.value), int(active.value)

    def num_parameters(self) -> int:
        return self._counts()[0]

    def active_parameters(self) -> int:
        return self._counts()[1]

    # ---- weights
    def _set(self, which: int, expert: int, a: np.ndarray, scales: Optional[np.ndarray] = None) -> None:
        dt = L.I8 if a.dtype == np.int8 else L.F32
        a = np.ascontiguousarray(a)
        sp = None
        if scales is not None:
            scales = np.ascontiguousarray(scales, dtype=np.float32)
            sp = scales.ctypes.data_as(C.POINTER(C.c_float))
        rows, cols = a.shape
        _check(self._lib.rbmoe_set_weight(self.handle, which, expert, a.ctypes.data_as(C.c_void_p), dt, sp,
                                          rows, cols), self.device.handle)

    def set_router(self, weight: np.ndarray) -> None:
        self._set(L.W_ROUTER, 0, np.asarray(weight, dtype=np.float32))

    def set_router_q8(self, q: np.ndarray, scales: np.ndarray) -> None:
        """A quantized router as it is: int8 rows ``[num_experts, d_model]`` and one scale per row.  The layer then
        routes with the quantized product (reference src/quantized.rs:55-62)."""
        self._set(L.W_ROUTER, 0, np.asarray(q, dtype=np.int8), scales)

    def quantize_on_upload(self, rule: str = "in_memory", router: bool = True) -> None:
        """What ``TransformerLm::quantize()`` (reference src/transformer.rs:899-910) does to this layer's Linears,
        applied to f32 weights as they are set from here on: ``rule`` "in_memory" is ``Quantized::from_matrix``
        (src/quantized.rs:29-51), "checkpoint" the .rbw writer's (src/transformer.rs:512-519); ``router``: the router
        is quantized too (src/moe.rs:491-500).  The layer's weight dtype must be int8 for the experts to follow."""
        self.set_option(L.OPT_QUANT_RULE, {"checkpoint": 0, "in_memory": 1}[rule])
        self.set_option(L.OPT_QUANTIZE_ROUTER, 1 if router else 0)

    def set_expert(self, expert: int, gate: np.ndarray, up: np.ndarray, down: np.ndarray) -> None:
        for which, m in ((L.W_GATE, gate), (L.W_UP, up), (L.W_DOWN, down)):
            self._set(which, expert, np.asarray(m, dtype=np.float32))

    def set_expert_q8(self, expert: int, gate_q, gate_s, up_q, up_s, down_q, down_s) -> None:
        for which, q, s in ((L.W_GATE, gate_q, gate_s), (L.W_UP, up_q, up_s), (L.W_DOWN, down_q, down_s)):
            self._set(which, expert, np.asarray(q, dtype=np.int8), s)

    def set_shared(self, gate: np.ndarray, up: np.ndarray, down: np.ndarray) -> None:
        for which, m in ((L.W_SHARED_GATE, gate), (L.W_SHARED_UP, up), (L.W_SHARED_DOWN, down)):
            self._set(which, 0, np.asarray(m, dtype=np.float32))

    def set_shared_q8(self, gate_q, gate_s, up_q, up_s, down_q, down_s) -> None:
        for which, q, s in ((L.W_SHARED_GATE, gate_q, gate_s), (L.W_SHARED_UP, up_q, up_s),
                            (L.W_SHARED_DOWN, down_q, down_s)):
            self._set(which, 0, np.asarray(q, dtype=np.int8), s)

    def load_tensors(self, tensors) -> None:
        """Upload a ``synth.Tensors`` bundle."""
        self.set_router(tensors.router)
        for e, w in enumerate(tensors.experts):
            if "gate_q" in w:
                self.set_expert_q8(e, w["gate_q"], w["gate_s"], w["up_q"], w["up_s"], w["down_q"], w["down_s"])
            else:
                self.set_expert(e, w["gate"], w["up"], w["down"])
        if tensors.shared is not None:
            w = tensors.shared
            if "gate_q" in w:
                self.set_shared_q8(w["gate_q"], w["gate_s"], w["up_q"], w["up_s"], w["down_q"], w["down_s"])
            else:
                self.set_shared(w["gate"], w["up"], w["down"])

    # ---- forward
    def _to_act(self, a: np.ndarray) -> np.ndarray:
        a = np.ascontiguousarray(a, dtype=np.float32)
        return f32_to_bf16_bits(a).reshape(a.shape) if self.act_dtype == "bf16" else a

    def forward(self, input: np.ndarray) -> np.ndarray:
        return self.forward_train(input, Layout())[0]

    def forward_train(self, input: np.ndarray, layout: Layout = Layout(),
                      router_bias: Optional[np.ndarray] = None,
                      residual: Optional[np.ndarray] = None) -> Tuple[np.ndarray, MoeCache]:
        input = np.asarray(input)
        if input.ndim != 2:
            raise InvalidInput("input must be a [tokens, d_model] matrix")
        rows, cols = input.shape
        if cols != self._d_model:
            # the library makes the same check; raising here keeps expected/actual typed
            raise InvalidInput(f"input length {cols} does not match expected length {self._d_model}",
                               expected=self._d_model, actual=cols)
        layout.check(rows)
        x = self._to_act(input)
        out = np.empty_like(x)
        vp = bp = rp = None
        valid = None
        if layout.valid is not None:
            valid = np.ascontiguousarray(np.asarray(layout.valid, dtype=bool).astype(np.uint8))
            vp = valid.ctypes.data_as(C.c_void_p)
        if router_bias is not None:
            router_bias = np.ascontiguousarray(router_bias, dtype=np.float32)
            bp = router_bias.ctypes.data_as(C.c_void_p)
        if residual is not None:
            residual = self._to_act(residual)
            rp = residual.ctypes.data_as(C.c_void_p)
        _check(self._lib.rbmoe_forward_host(self.handle, x.ctypes.data_as(C.c_void_p), rows, cols, vp, bp, rp,
                                            out.ctypes.data_as(C.c_void_p)), self.device.handle)
        if self.act_dtype == "bf16":
            out = bf16_bits_to_f32(out).reshape(rows, cols)
        valid_tokens = rows if valid is None else int(valid.sum())
        return out, self.cache(rows, valid_tokens)

    def forward_device(self, x_ptr: int, tokens: int, out_ptr: int, valid_ptr: int = 0, bias_ptr: int = 0,
                       residual_ptr: int = 0) -> None:
        """Enqueue one forward on device pointers (no synchronisation)."""
        _check(self._lib.rbmoe_forward(self.handle, C.c_void_p(x_ptr), tokens, self._d_model,
                                       C.c_void_p(valid_ptr or None), C.c_void_p(bias_ptr or None),
                                       C.c_void_p(residual_ptr or None), C.c_void_p(out_ptr)), self.device.handle)

    def forward_static_device(self, x_ptr: int, tokens: int, out_ptr: int, valid_ptr: int = 0, bias_ptr: int = 0,
                              residual_ptr: int = 0) -> None:
        """``forward_device`` with every intermediate buffer in the library's static device array: the call
        allocates nothing.  Decode-shaped calls only (``Unsupported`` otherwise)."""
        _check(self._lib.rbmoe_forward_static(self.handle, C.c_void_p(x_ptr), tokens, self._d_model,
                                              C.c_void_p(valid_ptr or None), C.c_void_p(bias_ptr or None),
                                              C.c_void_p(residual_ptr or None), C.c_void_p(out_ptr)),
               self.device.handle)

    def forward_timed(self, x_ptr: int, tokens: int, out_ptr: int, valid_ptr: int = 0, bias_ptr: int = 0,
                      residual_ptr: int = 0) -> dict:
        ms = (C.c_float * L.NUM_STAGES)()
        _check(self._lib.rbmoe_forward_timed(self.handle, C.c_void_p(x_ptr), tokens, self._d_model,
                                             C.c_void_p(valid_ptr or None), C.c_void_p(bias_ptr or None),
                                             C.c_void_p(residual_ptr or None), C.c_void_p(out_ptr), ms),
               self.device.handle)
        return {name: float(ms[i]) for i, name in enumerate(L.STAGE_NAMES)}

    def forward_kernel_times(self, x_ptr: int, tokens: int, out_ptr: int, valid_ptr: int = 0, bias_ptr: int = 0,
                             residual_ptr: int = 0) -> dict:
        """One forward whose launches carry their own start/stop events: kernel durations per stage in milliseconds,
        as a kernel trace would report them."""
        ms = (C.c_float * L.NUM_STAGES)()
        _check(self._lib.rbmoe_forward_kernel_times(self.handle, C.c_void_p(x_ptr), tokens, self._d_model,
                                                    C.c_void_p(valid_ptr or None), C.c_void_p(bias_ptr or None),
                                                    C.c_void_p(residual_ptr or None), C.c_void_p(out_ptr), ms),
               self.device.handle)
        return {name: float(ms[i]) for i, name in enumerate(L.STAGE_NAMES)}

    def replay_stage(self, stage: str, launches: int = 20) -> Optional[float]:
        """Average launch time in milliseconds of one stage of the last forward (``_lib.STAGE_NAMES``), replayed
        ``launches`` times between one pair of events; None when the last forward had no launch for the stage."""
        ms = C.c_float()
        rc = self._lib.rbmoe_replay_stage(self.handle, L.STAGE_NAMES.index(stage), launches, C.byref(ms))
        if rc == L.UNSUPPORTED:
            return None
        _check(rc, self.device.handle)
        return float(ms.value)

    def enqueue_stage(self, stage: str, launches: int = 1) -> bool:
        """The launches of one stage of the last forward again, enqueued only (the caller times the sequence)."""
        rc = self._lib.rbmoe_replay_stage(self.handle, L.STAGE_NAMES.index(stage), launches, None)
        if rc == L.UNSUPPORTED:
            return False
        _check(rc, self.device.handle)
        return True

    def losses(self) -> Tuple[float, float]:
        aux, z = C.c_float(), C.c_float()
        _check(self._lib.rbmoe_get_losses(self.handle, C.byref(aux), C.byref(z)), self.device.handle)
        return float(aux.value), float(z.value)

    def cache(self, tokens: int, valid_tokens: Optional[int] = None) -> MoeCache:
        E, k = self.config.num_experts, self.config.experts_per_token
        S = tokens * k
        expert_of = np.full((S,), UNROUTED, np.int32)
        gate_of = np.zeros((S,), np.float32)
        counts = np.zeros((E,), np.int32)
        offsets = np.zeros((E + 1,), np.int32)
        perm_slot = np.full((S,), -1, np.int32)
        perm_token = np.full((S,), -1, np.int32)
        P = np.zeros((tokens, E), np.float32)
        lse = np.zeros((tokens,), np.float32)
        ip, fp = C.POINTER(C.c_int32), C.POINTER(C.c_float)
        r = L.Routing(expert_of.ctypes.data_as(ip), gate_of.ctypes.data_as(fp), counts.ctypes.data_as(ip),
                      offsets.ctypes.data_as(ip), perm_slot.ctypes.data_as(ip), perm_token.ctypes.data_as(ip),
                      P.ctypes.data_as(fp), lse.ctypes.data_as(fp))
        _check(self._lib.rbmoe_get_routing(self.handle, C.byref(r)), self.device.handle)
        aux, z = self.losses()
        R = int(offsets[E])
        if valid_tokens is None:
            valid_tokens = R // k
        assignments = list(zip(expert_of.tolist(), gate_of.tolist()))
        return MoeCache(assignments, expert_of, gate_of, counts, offsets, perm_slot[:R], perm_token[:R], P, lse,
                        valid_tokens, aux, z)

    def expert_rows(self, routed: int) -> Tuple[np.ndarray, np.ndarray]:
        """Hidden rows ``[routed, d_ff]`` and expert output rows ``[routed, d_model]``
        of the last forward in permuted order (f32)."""
        F, d = self.config.d_ff, self._d_model
        h = np.zeros((max(routed, 1), F), np.float32)
        y = np.zeros((max(routed, 1), d), np.float32)
        fp = C.POINTER(C.c_float)
        _check(self._lib.rbmoe_get_expert_rows(self.handle, h.ctypes.data_as(fp), y.ctypes.data_as(fp)),
               self.device.handle)
        return h[:routed], y[:routed]

    # ---- the block's steps either side of the layer (reference src/transformer_block.rs:216-222)
    def set_feed_forward_norm(self, weight: np.ndarray, eps: float = 1e-6) -> None:
        """Weight ``[d_model]`` and eps of the block's ``feed_forward_norm`` (RmsNorm, src/norm.rs:23-37)."""
        w = np.ascontiguousarray(np.asarray(weight, dtype=np.float32).reshape(-1))
        _check(self._lib.rbmoe_set_feed_forward_norm(self.handle, w.ctypes.data_as(C.POINTER(C.c_float)), w.size,
                                                     C.c_float(eps)), self.device.handle)

    def forward_block(self, residual: np.ndarray, layout: Layout = Layout(),
                      router_bias: Optional[np.ndarray] = None) -> Tuple[np.ndarray, MoeCache]:
        """``residual + forward_train(feed_forward_norm(residual))``; the cache describes the normed rows."""
        residual = np.asarray(residual)
        if residual.ndim != 2:
            raise InvalidInput("input must be a [tokens, d_model] matrix")
        rows, cols = residual.shape
        if cols != self._d_model:
            raise InvalidInput(f"input length {cols} does not match expected length {self._d_model}",
                               expected=self._d_model, actual=cols)
        layout.check(rows)
        x = self._to_act(residual)
        out = np.empty_like(x)
        vp = bp = None
        valid = None
        if layout.valid is not None:
            valid = np.ascontiguousarray(np.asarray(layout.valid, dtype=bool).astype(np.uint8))
            vp = valid.ctypes.data_as(C.c_void_p)
        if router_bias is not None:
            router_bias = np.ascontiguousarray(router_bias, dtype=np.float32)
            bp = router_bias.ctypes.data_as(C.c_void_p)
        _check(self._lib.rbmoe_forward_block_host(self.handle, x.ctypes.data_as(C.c_void_p), rows, cols, vp, bp,
                                                  out.ctypes.data_as(C.c_void_p)), self.device.handle)
        if self.act_dtype == "bf16":
            out = bf16_bits_to_f32(out).reshape(rows, cols)
        valid_tokens = rows if valid is None else int(valid.sum())
        return out, self.cache(rows, valid_tokens)

    def forward_block_device(self, x_ptr: int, tokens: int, out_ptr: int, valid_ptr: int = 0,
                             bias_ptr: int = 0) -> None:
        """Enqueue one block step on device pointers (no synchronisation); ``out_ptr`` may equal ``x_ptr``."""
        _check(self._lib.rbmoe_forward_block(self.handle, C.c_void_p(x_ptr), tokens, self._d_model,
                                             C.c_void_p(valid_ptr or None), C.c_void_p(bias_ptr or None),
                                             C.c_void_p(out_ptr)), self.device.handle)

    # ---- backward (reference MoeLayer::backward, src/moe.rs:348-489)
    def enable_training(self) -> None:
        """Makes the forward keep what the backward pass needs and allocates the gradient accumulators.
        Call before the weights are set."""
        _check(self._lib.rbmoe_layer_enable_training(self.handle), self.device.handle)

    def backward(self, grad_output: np.ndarray) -> np.ndarray:
        """Gradient of the last ``forward_train``'s input; weight gradients accumulate (``weight_grad``)."""
        grad_output = np.asarray(grad_output)
        if grad_output.ndim != 2 or grad_output.shape[1] != self._d_model:
            raise InvalidInput(f"grad_output must be [tokens, {self._d_model}]", expected=self._d_model,
                               actual=grad_output.shape[-1] if grad_output.ndim else 0)
        g = self._to_act(grad_output)
        out = np.empty_like(g)
        _check(self._lib.rbmoe_backward_host(self.handle, g.ctypes.data_as(C.c_void_p), g.shape[0], g.shape[1],
                                             out.ctypes.data_as(C.c_void_p)), self.device.handle)
        if self.act_dtype == "bf16":
            out = bf16_bits_to_f32(out).reshape(g.shape)
        return out

    def backward_block(self, grad_output: np.ndarray) -> np.ndarray:
        """Gradient of the last ``forward_block``'s input: through the layer, the norm and the residual
        (reference TransformerBlock::backward, src/transformer_block.rs:257-263)."""
        grad_output = np.asarray(grad_output)
        if grad_output.ndim != 2 or grad_output.shape[1] != self._d_model:
            raise InvalidInput(f"grad_output must be [tokens, {self._d_model}]", expected=self._d_model,
                               actual=grad_output.shape[-1] if grad_output.ndim else 0)
        g = self._to_act(grad_output)
        out = np.empty_like(g)
        _check(self._lib.rbmoe_backward_block_host(self.handle, g.ctypes.data_as(C.c_void_p), g.shape[0], g.shape[1],
                                                   out.ctypes.data_as(C.c_void_p)), self.device.handle)
        if self.act_dtype == "bf16":
            out = bf16_bits_to_f32(out).reshape(g.shape)
        return out

    def backward_block_device(self, grad_output_ptr: int, tokens: int, grad_input_ptr: int) -> None:
        """Enqueue the block step's backward pass on device pointers (no synchronisation); both buffers are
        ``[tokens, d_model]`` and ``tokens`` must be the last forward's."""
        _check(self._lib.rbmoe_backward_block(self.handle, C.c_void_p(grad_output_ptr), tokens, self._d_model,
                                              C.c_void_p(grad_input_ptr)), self.device.handle)

    def backward_device(self, grad_output_ptr: int, tokens: int, grad_input_ptr: int) -> None:
        """Enqueue the backward pass on device pointers (no synchronisation); both buffers are
        ``[tokens, d_model]`` and ``tokens`` must be the last forward's."""
        _check(self._lib.rbmoe_backward(self.handle, C.c_void_p(grad_output_ptr), tokens, self._d_model,
                                        C.c_void_p(grad_input_ptr)), self.device.handle)

    def zero_grads(self) -> None:
        _check(self._lib.rbmoe_zero_grads(self.handle), self.device.handle)

    def weight_grad(self, which: int, expert: int = 0) -> np.ndarray:
        """Accumulated gradient (f32) of one weight matrix: ``which`` is one of ``_lib.W_*``."""
        F, d, Fs = self.config.d_ff, self._d_model, self.shared_d_ff
        shape = {L.W_ROUTER: (self.config.num_experts, d), L.W_GATE: (F, d), L.W_UP: (F, d), L.W_DOWN: (d, F),
                 L.W_SHARED_GATE: (Fs, d), L.W_SHARED_UP: (Fs, d), L.W_SHARED_DOWN: (d, Fs), L.W_NORM: (1, d)}[which]
        g = np.zeros(shape, np.float32)
        _check(self._lib.rbmoe_get_weight_grad(self.handle, which, expert, g.ctypes.data_as(C.POINTER(C.c_float)),
                                               shape[0], shape[1]), self.device.handle)
        return g

    def kernel_name(self) -> str:
        return self._lib.rbmoe_expert_kernel_name(self.handle).decode()

    def close(self) -> None:
        if getattr(self, "handle", None):
            self._lib.rbmoe_layer_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
