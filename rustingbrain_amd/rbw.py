"""Reader (and, for tests, writer) of the reference's binary weight snapshot, `.rbw`.

Format, from the reference's `TransformerLm::save_bin` / `load_bin`
(src/transformer.rs:1806-1932; header struct :503-510; `quantize` :512-519):

    8 bytes   magic  b"RBWTS001"                                   (:488)
    u64 LE    length of the JSON header
    bytes     JSON  {"config": TransformerConfig, "optimizer": ..., "optimizer_step": n,
                     "precision": "F32" | "Q8"}
    u64 LE    number of parameters
    per parameter, in `TransformerLm::params_mut()` order (:1620-1630):
        u64 LE rows, u64 LE cols
        F32:  rows * cols little-endian f32, row-major
        Q8:   per row: f32 scale (= absmax / 127), then cols int8 (`round(w / scale)` clamped to +-127)

Parameter order (src/transformer.rs:1620-1630, src/transformer_block.rs:286-292,
src/attention.rs:911-917, src/moe.rs:516-525, src/ffn.rs:126-131):

    embedding; per block: attention_norm, query, key, value, output, feed_forward_norm,
    then the feed-forward: dense SwiGLU gate, up, down -- or, in a sparse block, router,
    experts[0..E] x (gate, up, down), shared (gate, up, down) when configured;
    final_norm; lm_head unless the embeddings are tied.

Only what the mixture-of-experts layer needs is interpreted: the sparse blocks' parameters
are handed to `MoeLayer`; everything else is parsed (so that positions are right) and
returned untouched.  A Q8 file's expert matrices go to the device as the int8 values and
scales they are stored as (the library's int8 path dequantises in the product); the router,
which the library keeps in f32, is dequantised the way `load_bin` does (`q * scale`).
Snapshots of models with LoRA adapters carry extra parameters per linear layer and are
refused.
"""
from __future__ import annotations

import json
import struct
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np

from .moe import InvalidConfig, InvalidInput, MoeConfig, MoeLayer, NetworkError

MAGIC = b"RBWTS001"


class InvalidSnapshot(NetworkError):
    """Reference: NetworkError::InvalidSnapshot (src/network.rs)."""


@dataclass
class RbwParam:
    rows: int
    cols: int
    values: Optional[np.ndarray] = None   # f32 [rows, cols] (F32 files)
    q: Optional[np.ndarray] = None        # int8 [rows, cols] (Q8 files)
    scales: Optional[np.ndarray] = None   # f32 [rows]         (Q8 files)

    def dequantized(self) -> np.ndarray:
        """f32 values the way `load_bin` restores them: `q as f32 * scale`."""
        if self.values is not None:
            return self.values
        return (self.q.astype(np.float32) * self.scales[:, None]).astype(np.float32)


@dataclass
class RbwFile:
    config: dict
    optimizer: object
    optimizer_step: int
    precision: str
    params: List[RbwParam]


def read(path: str) -> RbwFile:
    with open(path, "rb") as f:
        data = f.read()
    if len(data) < 16 or data[:8] != MAGIC:
        raise InvalidSnapshot("not a RustingBrain weight file")
    pos = 8
    (hlen,) = struct.unpack_from("<Q", data, pos)
    pos += 8
    if pos + hlen + 8 > len(data):
        raise InvalidSnapshot("weight file is truncated inside its header")
    try:
        header = json.loads(data[pos:pos + hlen].decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as e:
        raise InvalidSnapshot(f"weight file header is not JSON: {e}") from None
    pos += hlen
    precision = header.get("precision")
    if precision not in ("F32", "Q8"):
        raise InvalidSnapshot(f"unknown precision {precision!r}")
    (count,) = struct.unpack_from("<Q", data, pos)
    pos += 8
    params: List[RbwParam] = []
    for _ in range(count):
        if pos + 16 > len(data):
            raise InvalidSnapshot("weight file is truncated between parameters")
        rows, cols = struct.unpack_from("<QQ", data, pos)
        pos += 16
        if precision == "F32":
            n = rows * cols * 4
            if pos + n > len(data):
                raise InvalidSnapshot("weight file is truncated inside a parameter")
            v = np.frombuffer(data, dtype="<f4", count=rows * cols, offset=pos).reshape(rows, cols).astype(np.float32)
            params.append(RbwParam(rows, cols, values=v))
            pos += n
        else:
            stride = 4 + cols
            n = rows * stride
            if pos + n > len(data):
                raise InvalidSnapshot("weight file is truncated inside a parameter")
            raw = np.frombuffer(data, dtype=np.uint8, count=n, offset=pos).reshape(rows, stride)
            scales = raw[:, :4].copy().view("<f4").reshape(rows).astype(np.float32)
            q = raw[:, 4:].copy().view(np.int8).reshape(rows, cols)
            params.append(RbwParam(rows, cols, q=q, scales=scales))
            pos += n
    if pos != len(data):
        raise InvalidSnapshot(f"{len(data) - pos} bytes follow the last parameter")
    return RbwFile(header["config"], header.get("optimizer"), int(header.get("optimizer_step", 0)), precision, params)


def quantize_row(row: np.ndarray):
    """`save_bin`'s rule for one row (src/transformer.rs:1839-1847 with `quantize`, :512-519)."""
    absmax = np.float32(np.max(np.abs(row))) if row.size else np.float32(0)
    scale = np.float32(absmax / np.float32(127.0))
    if scale == 0:
        return scale, np.zeros(row.shape, np.int8)
    r = row.astype(np.float32) / scale
    q = np.clip(np.sign(r) * np.floor(np.abs(r) + np.float32(0.5)), -127, 127)  # f32::round: half away from zero
    return scale, q.astype(np.int8)


def write(path: str, config: dict, params: List[np.ndarray], precision: str = "F32", optimizer="Sgd",
          optimizer_step: int = 0) -> None:
    """Writes `params` (f32 matrices in `params_mut()` order) the way `save_bin` does.  Test support: the
    reference is the producer of real files."""
    header = json.dumps({"config": config, "optimizer": optimizer, "optimizer_step": optimizer_step,
                         "precision": precision}).encode("utf-8")
    with open(path, "wb") as f:
        f.write(MAGIC)
        f.write(struct.pack("<Q", len(header)))
        f.write(header)
        f.write(struct.pack("<Q", len(params)))
        for p in params:
            p = np.ascontiguousarray(p, dtype=np.float32)
            rows, cols = p.shape
            f.write(struct.pack("<QQ", rows, cols))
            if precision == "F32":
                f.write(p.astype("<f4").tobytes())
            else:
                for r in range(rows):
                    scale, q = quantize_row(p[r])
                    f.write(struct.pack("<f", float(scale)))
                    f.write(q.tobytes())


@dataclass
class MoeBlockParams:
    """The parameters of one sparse block's feed-forward, in the reference's order (src/moe.rs:516-525)."""
    block: int
    norm: RbwParam          # feed_forward_norm.weight, 1 x d_model (src/norm.rs:30-35)
    router: RbwParam
    experts: List[Dict[str, RbwParam]]
    shared: Optional[Dict[str, RbwParam]]


def _expect(p: RbwParam, rows: int, cols: int, what: str) -> RbwParam:
    if (p.rows, p.cols) != (rows, cols):
        raise InvalidSnapshot(f"weight file has a {p.rows}x{p.cols} parameter where the model has {rows}x{cols} ({what})")
    return p


def moe_blocks(snapshot: RbwFile) -> List[MoeBlockParams]:
    """Walks the parameter list in `params_mut()` order and picks out every sparse block."""
    c = snapshot.config
    if c.get("lora") is not None:
        raise InvalidConfig("snapshots of models with LoRA adapters are not supported")
    d, layers = int(c["d_model"]), int(c["n_layers"])
    heads, kv_heads, head_dim = int(c["n_heads"]), int(c["n_kv_heads"]), int(c["head_dim"])
    d_ff, moe_d_ff = int(c["d_ff"]), int(c["moe_d_ff"])
    E = int(c["num_experts"])
    sparse = set(int(i) for i in c.get("moe_layers", []))
    shared = bool(c.get("shared_expert", False))
    params = snapshot.params
    pos = 0

    def take(rows, cols, what):
        nonlocal pos
        if pos >= len(params):
            raise InvalidSnapshot(f"weight file holds {len(params)} parameters, this configuration builds more")
        p = _expect(params[pos], rows, cols, what)
        pos += 1
        return p

    def take_swiglu(f, what):
        return {"gate": take(f, d, what + ".gate"), "up": take(f, d, what + ".up"), "down": take(d, f, what + ".down")}

    take(int(c["vocab_size"]), d, "embedding")
    out: List[MoeBlockParams] = []
    for b in range(layers):
        pos += 1  # attention_norm (a vector; its orientation does not matter here)
        take(heads * head_dim, d, f"block {b} query")
        take(kv_heads * head_dim, d, f"block {b} key")
        take(kv_heads * head_dim, d, f"block {b} value")
        take(d, heads * head_dim, f"block {b} output")
        ff_norm = params[pos] if pos < len(params) else None
        pos += 1  # feed_forward_norm
        if b in sparse:
            router = take(E, d, f"block {b} router")
            experts = [take_swiglu(moe_d_ff, f"block {b} expert {e}") for e in range(E)]
            sh = take_swiglu(moe_d_ff, f"block {b} shared expert") if shared else None
            out.append(MoeBlockParams(b, ff_norm, router, experts, sh))
        else:
            take_swiglu(d_ff, f"block {b} feed-forward")
    pos += 1  # final_norm
    if not c.get("tie_embeddings", False):
        take(int(c["vocab_size"]), d, "lm_head")
    if pos != len(params):
        raise InvalidSnapshot(f"weight file holds {len(params)} parameters, this configuration builds {pos}")
    return out


def load_moe_layers(path: str, device, max_tokens: int, act_dtype: str = "bf16",
                    weight_dtype: Optional[str] = None) -> List[MoeLayer]:
    """Builds one device `MoeLayer` per sparse block of the snapshot.  `weight_dtype` defaults to "int8" for a
    Q8 file (the stored values and scales are used as they are) and to "bf16" for an F32 file."""
    snap = read(path)
    c = snap.config
    blocks = moe_blocks(snap)
    if weight_dtype is None:
        weight_dtype = "int8" if snap.precision == "Q8" else "bf16"
    cfg = MoeConfig(int(c["num_experts"]), int(c["experts_per_token"]), int(c["moe_d_ff"]),
                    bool(c.get("shared_expert", False)), float(c.get("aux_loss_weight", 0.01)),
                    float(c.get("router_z_loss_weight", 1e-3)))
    layers = []
    for blk in blocks:
        layer = MoeLayer(int(c["d_model"]), cfg, device, act_dtype=act_dtype, weight_dtype=weight_dtype,
                         max_tokens=max_tokens)
        layer.set_router(blk.router.dequantized())
        if blk.norm is not None and blk.norm.rows * blk.norm.cols == int(c["d_model"]):
            # the norm in front of the layer, for MoeLayer.forward_block
            layer.set_feed_forward_norm(blk.norm.dequantized().reshape(-1), float(c.get("rmsnorm_eps", 1e-6)))

        def put(setter_f32, setter_q8, ex):
            if snap.precision == "Q8" and weight_dtype == "int8":
                setter_q8(ex["gate"].q, ex["gate"].scales, ex["up"].q, ex["up"].scales, ex["down"].q, ex["down"].scales)
            else:
                setter_f32(ex["gate"].dequantized(), ex["up"].dequantized(), ex["down"].dequantized())

        for e, ex in enumerate(blk.experts):
            put(lambda g, u, dn, e=e: layer.set_expert(e, g, u, dn),
                lambda gq, gs, uq, us, dq, dsc, e=e: layer.set_expert_q8(e, gq, gs, uq, us, dq, dsc), ex)
        if blk.shared is not None:
            put(layer.set_shared, layer.set_shared_q8, blk.shared)
        layers.append(layer)
    return layers
