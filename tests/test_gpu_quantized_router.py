"""What `TransformerLm::quantize()` (reference src/transformer.rs:899-910) does to a MoE layer, on the device: every
Linear - the router included (src/moe.rs:491-500) - quantized in memory by Quantized::from_matrix
(src/quantized.rs:29-51), and the products taken as (sum x * q) * scale (:55-62).  A quantized router changes the
logits, so the routing must equal the oracle's run with the same quantized router in every bit."""
import numpy as np
import pytest

import rustingbrain_amd as rb
from conftest import rel_l2
from helpers import assert_routing_identical, small_workload
from oracle import rb_oracle as orc
from rustingbrain_amd import _lib as L
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu


def quantized_pair(device, t, rule, act, max_tokens=None):
    """The device layer fed f32 weights with quantize-on-upload, and the oracle layer fed the oracle's own quantizer's
    output (mode 1 = in-memory rule, 0 = checkpoint rule)."""
    w = t.workload
    mode = {"in_memory": 1, "checkpoint": 0}[rule]
    cfg = rb.MoeConfig(w.num_experts, w.experts_per_token, w.d_ff, w.shared_expert)
    layer = rb.MoeLayer(w.d_model, cfg, device, act_dtype=act, weight_dtype="int8",
                        max_tokens=max_tokens or t.x.shape[0], shared_d_ff=w.shared_d_ff if w.shared_expert else 0)
    layer.quantize_on_upload(rule, router=True)
    layer.set_router(t.router)
    for e, ew in enumerate(t.experts):
        layer.set_expert(e, ew["gate"], ew["up"], ew["down"])
    if t.shared is not None:
        layer.set_shared(t.shared["gate"], t.shared["up"], t.shared["down"])

    def q(ew):
        out = {}
        for name in ("gate", "up", "down"):
            out[name + "_q"], out[name + "_s"] = orc.q8_quantize(ew[name], mode)
        return orc.ExpertWeights(**out)

    rq, rs = orc.q8_quantize(t.router, mode)
    ref = orc.OracleLayer(w.d_model, w.num_experts, w.experts_per_token, w.d_ff, t.router, [q(ew) for ew in t.experts],
                          q(t.shared) if t.shared is not None else None, w.shared_d_ff if t.shared is not None else 0)
    ref.router_q, ref.router_s = rq, rs
    return layer, ref


@pytest.mark.parametrize("act", ["bf16", "f32"])
@pytest.mark.parametrize("shape", [dict(d=128, E=8, k=2, F=192, T=300, shared=True, shared_d_ff=128),
                                   dict(d=100, E=5, k=2, F=40, T=77),          # widths off the tiles and off the 32 lanes
                                   dict(d=128, E=8, k=2, F=192, T=8)],          # a few tokens
                         ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}".format(**s))
def test_a_layer_quantized_in_memory_routes_like_the_oracle(device, shape, act):
    t = synth.make(small_workload(seed=97, act=act, wt="f32", **shape))
    layer, ref_layer = quantized_pair(device, t, "in_memory", act)
    valid = (np.arange(shape["T"]) % 6 != 2).astype(np.uint8)
    bias = np.linspace(-0.3, 0.3, shape["E"]).astype(np.float32)
    layout = rb.Layout(valid=[bool(v) for v in valid])
    out, cache = layer.forward_train(t.x, layout, router_bias=bias)
    ref = ref_layer.forward(t.x, valid=valid, router_bias=bias, threads=4)
    assert_routing_identical(cache, ref)
    assert rel_l2(out, ref.out) <= 2e-2
    assert abs(cache.aux_loss() - ref.aux_loss) <= 2e-2 * abs(ref.aux_loss) + 1e-7
    assert abs(cache.z_loss() - ref.z_loss) <= 2e-2 * abs(ref.z_loss) + 1e-7
    # the unquantized router of the same weights decides differently somewhere, or at least computes other
    # probabilities: the test would not notice a layer that ignored the switch otherwise
    plain = orc.OracleLayer(ref_layer.d_model, ref_layer.num_experts, ref_layer.experts_per_token, ref_layer.d_ff,
                            t.router, ref_layer.experts, ref_layer.shared, ref_layer.shared_d_ff)
    assert not np.array_equal(plain.forward(t.x, valid=valid, router_bias=bias).probabilities, ref.probabilities)
    layer.close()


def test_router_given_as_int8_rows_and_scales(device):
    t = synth.make(small_workload(d=64, E=6, k=3, F=64, T=50, seed=98, act="bf16", wt="f32"))
    layer, ref_layer = quantized_pair(device, t, "checkpoint", "bf16")
    layer.set_router_q8(ref_layer.router_q, ref_layer.router_s)     # replaces the router quantized on upload: same values
    _, cache = layer.forward_train(t.x)
    ref = ref_layer.forward(t.x, threads=2)
    assert_routing_identical(cache, ref)
    # back to an f32 router: the layer routes on f32 logits again
    layer.set_option(L.OPT_QUANTIZE_ROUTER, 0)
    layer.set_router(t.router)
    _, cache = layer.forward_train(t.x)
    ref_layer.router_q = ref_layer.router_s = None
    assert_routing_identical(cache, ref_layer.forward(t.x, threads=2))
    layer.close()


def test_the_two_quantisation_rules_are_told_apart(device):
    """round(w / scale) and round(w * (1 / scale)) differ where the reciprocal's rounding moves a quotient across a
    half.  A router row is built around such an element; a one-hot token row makes the logit exactly q * scale, so
    the probabilities of that row show which rule the library applied."""
    rng = np.random.default_rng(99)
    E, d = 4, 64
    found = None
    for _ in range(200000):
        absmax = np.float32(rng.uniform(0.5, 2.0))
        scale = np.float32(absmax / np.float32(127.0))
        inverse = np.float32(np.float32(1.0) / scale)
        n = rng.integers(1, 126)
        w = np.float32((n + 0.5) * float(scale))
        for cand in (w, np.nextafter(w, np.float32(0)), np.nextafter(w, np.float32(4))):
            # (positive values: floor(v + 0.5) rounds halves away from zero, as f32::round does)
            qa = np.floor(np.float32(cand / scale) + np.float32(0.5))
            qb = np.floor(np.float32(cand * inverse) + np.float32(0.5))
            if qa != qb and abs(cand) < absmax:
                found = (absmax, np.float32(cand), int(qa), int(qb))
                break
        if found:
            break
    assert found, "no element on which the two rules differ was found"
    absmax, w_special, q_div, q_mul = found
    router = (rng.standard_normal((E, d)) * 0.01).astype(np.float32)
    router[2, 0], router[2, 5] = absmax, w_special                  # row 2: its absmax, and the element in question
    q0, s0 = orc.q8_quantize(router, 0)
    q1, s1 = orc.q8_quantize(router, 1)
    assert (q0[2, 5], q1[2, 5]) == (q_div, q_mul) and q0[2, 5] != q1[2, 5]
    t = synth.make(small_workload(d=d, E=E, k=2, F=64, T=4, seed=99, act="f32", wt="f32"))
    t.router[:] = router
    t.x[:] = 0
    t.x[1, 5] = 1.0                                                   # token 1: logits = q[:, 5] * scale exactly
    for rule, mode in (("checkpoint", 0), ("in_memory", 1)):
        layer, ref_layer = quantized_pair(device, t, rule, "f32")
        _, cache = layer.forward_train(t.x)
        ref = ref_layer.forward(t.x)
        assert_routing_identical(cache, ref)
        other = orc.q8_quantize(router, 1 - mode)
        ref_layer.router_q, ref_layer.router_s = other
        assert not np.array_equal(ref_layer.forward(t.x).probabilities[1], cache.probabilities[1]), rule
        layer.close()


def test_a_quantized_router_is_inference_only(device):
    t = synth.make(small_workload(d=64, E=4, k=2, F=64, T=8, seed=100, act="bf16", wt="bf16"))
    cfg = rb.MoeConfig(4, 2, 64, False)
    layer = rb.MoeLayer(64, cfg, device, act_dtype="bf16", weight_dtype="bf16", max_tokens=8)
    layer.set_option(L.OPT_QUANTIZE_ROUTER, 1)
    with pytest.raises(rb.Unsupported, match="quantized router"):
        layer.enable_training()
    layer.close()
    layer = rb.MoeLayer(64, cfg, device, act_dtype="bf16", weight_dtype="bf16", max_tokens=8)
    layer.enable_training()
    with pytest.raises(rb.Unsupported, match="quantized router"):
        layer.set_option(L.OPT_QUANTIZE_ROUTER, 1)
    q, s = orc.q8_quantize(t.router, 1)
    with pytest.raises(rb.Unsupported, match="quantized router"):
        layer.set_router_q8(q, s)
    layer.close()
