"""Shared helpers of the parity tests: build the oracle layer and the GPU layer
from the same tensors."""
from __future__ import annotations

from typing import Optional

import numpy as np

from oracle import rb_oracle as orc
from rustingbrain_amd import synth


def oracle_layer(t: synth.Tensors, aux_w: float = 0.01, z_w: float = 1e-3) -> orc.OracleLayer:
    w = t.workload
    experts = [orc.ExpertWeights(**e) for e in t.experts]
    shared = orc.ExpertWeights(**t.shared) if t.shared is not None else None
    return orc.OracleLayer(w.d_model, w.num_experts, w.experts_per_token, w.d_ff, t.router, experts, shared,
                           w.shared_d_ff if shared is not None else 0, aux_w, z_w)


def small_workload(name="small", d=8, E=4, k=2, F=6, T=7, seed=5, act="f32", wt="f32", shared=False,
                   shared_d_ff=0) -> synth.Workload:
    return synth.Workload(name, d, E, k, F, T, seed, act, wt, shared_expert=shared,
                          shared_d_ff=(shared_d_ff or F) if shared else 0)


def f64_layer_forward(t: synth.Tensors, valid: Optional[np.ndarray] = None,
                      bias: Optional[np.ndarray] = None, routing=None):
    """Textbook float64 evaluation of the layer given a routing decision
    (expert_of, gate_of): out[t] = sum_r gate * swiglu_e(x[t]) + shared(x[t])."""
    w = t.workload
    x = t.x.astype(np.float64)
    T = x.shape[0]
    k = w.experts_per_token
    expert_of, gate_of = routing

    def dense(e, rows):
        if "gate_q" in e:
            g = (rows @ e["gate_q"].astype(np.float64).T) * e["gate_s"].astype(np.float64)
            u = (rows @ e["up_q"].astype(np.float64).T) * e["up_s"].astype(np.float64)
            h = g / (1.0 + np.exp(-g)) * u
            return (h @ e["down_q"].astype(np.float64).T) * e["down_s"].astype(np.float64)
        g = rows @ e["gate"].astype(np.float64).T
        u = rows @ e["up"].astype(np.float64).T
        h = g / (1.0 + np.exp(-g)) * u
        return h @ e["down"].astype(np.float64).T

    out = np.zeros((T, w.d_model))
    for e in range(w.num_experts):
        slots = np.nonzero(expert_of == e)[0]
        if slots.size == 0:
            continue
        toks = slots // k
        y = dense(t.experts[e], x[toks])
        np.add.at(out, toks, y * gate_of[slots].astype(np.float64)[:, None])
    if t.shared is not None:
        out += dense(t.shared, x)
    return out


def gpu_layer(device, t: synth.Tensors, max_tokens: Optional[int] = None, aux_w: float = 0.01,
              z_w: float = 1e-3, training: bool = False):
    import rustingbrain_amd as rb
    w = t.workload
    cfg = rb.MoeConfig(w.num_experts, w.experts_per_token, w.d_ff, w.shared_expert, aux_w, z_w)
    layer = rb.MoeLayer(w.d_model, cfg, device, act_dtype=w.act_dtype, weight_dtype=w.weight_dtype,
                        max_tokens=max_tokens or max(t.x.shape[0], 1),
                        shared_d_ff=w.shared_d_ff if w.shared_expert else 0)
    if training:
        layer.enable_training()
    layer.load_tensors(t)
    return layer


def assert_routing_identical(cache, ref) -> None:
    """Bit-exact comparands: indices, counts, permutation — and, because the
    router arithmetic is a fixed sequence, probabilities, lse and gates too."""
    assert np.array_equal(cache.expert_of, ref.expert_of), "expert_of differs"
    assert np.array_equal(cache.counts, ref.counts), "counts differ"
    assert np.array_equal(cache.offsets, ref.offsets), "offsets differ"
    assert np.array_equal(cache.perm_slot, ref.perm_slot), "perm_slot differs"
    assert np.array_equal(cache.perm_token, ref.perm_token), "perm_token differs"
    assert np.array_equal(cache.probabilities.view(np.uint32), ref.probabilities.view(np.uint32)), \
        "probabilities differ in bits"
    assert np.array_equal(cache.log_sum_exp.view(np.uint32), ref.lse.view(np.uint32)), "lse differs in bits"
    assert np.array_equal(cache.gate_of.view(np.uint32), ref.gate_of.view(np.uint32)), "gates differ in bits"


def tolerance(w: synth.Workload) -> float:
    """rel-L2 bar: 1e-5 for all-f32 layers, 2e-2 when bf16 or int8 is involved."""
    return 1e-5 if (w.act_dtype == "f32" and w.weight_dtype == "f32") else 2e-2
