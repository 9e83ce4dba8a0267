"""GPU parity of the block step around the layer (src/transformer_block.rs:216-222): RmsNorm::forward in front
(src/norm.rs:41-61), the residual add behind.  The norm's sum of squares runs in the reference's order on both
sides, so the normed rows - and with them every routing table - must be identical in every bit; outputs within
rel-L2 1e-5 (all-f32 layers) or 2e-2 (bf16 / int8).
"""
import numpy as np
import pytest

import rustingbrain_amd as rb
from conftest import rel_l2
from helpers import assert_routing_identical, gpu_layer, oracle_layer, small_workload, tolerance
from rustingbrain_amd import _lib as L
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu


def norm_weight(d, seed):
    return np.random.default_rng(seed).uniform(0.5, 1.5, d).astype(np.float32)


def check_block(device, t, eps=1e-6, valid=None, bias=None, seed=3, scale=1.0):
    w = t.workload
    nw = norm_weight(w.d_model, seed)
    x = t.x * np.float32(scale)
    if w.act_dtype == "bf16":
        x = synth.round_bf16(x)
    rounder = synth.round_bf16 if w.act_dtype == "bf16" else None
    want, normed, ref = oracle_layer(t).forward_block(x, nw, eps, valid=valid, router_bias=bias, round_normed=rounder)
    layer = gpu_layer(device, t)
    layer.set_feed_forward_norm(nw, eps)
    layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
    out, cache = layer.forward_block(x, layout, router_bias=bias)
    assert_routing_identical(cache, ref)
    tol = tolerance(w)
    assert rel_l2(out, want) <= tol
    # the layer's own share, without the residual that dominates the sum; a bf16 output carries the rounding
    # of the SUM (2^-9 of its size), which weighs more the larger the residual is against the share
    share = float(np.linalg.norm(want - x))
    rounding = 2.0 ** -8 * float(np.linalg.norm(want)) / max(share, 1e-30) if w.act_dtype == "bf16" else 0.0
    assert rel_l2(out - x, want - x) <= 2 * tol + rounding
    layer.close()
    return out, cache, ref


SHAPES = [
    dict(d=8, E=4, k=2, F=6, T=7),
    dict(d=33, E=7, k=3, F=19, T=65),
    dict(d=64, E=8, k=2, F=64, T=200, shared=True),
    dict(d=128, E=16, k=2, F=64, T=513),
    dict(d=768, E=8, k=2, F=128, T=130, shared=True),
]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}".format(**s))
@pytest.mark.parametrize("act,wt", [("f32", "f32"), ("bf16", "bf16"), ("bf16", "int8")])
def test_block_step_matches_the_oracle(device, shape, act, wt):
    t = synth.make(small_workload(seed=41, act=act, wt=wt, **shape))
    check_block(device, t)


def test_block_step_with_padding_rows_bias_and_large_inputs(device):
    t = synth.make(small_workload(d=64, E=6, k=2, F=64, T=90, seed=42, act="bf16", wt="bf16", shared=True))
    valid = (np.arange(90) % 4 != 3).astype(np.uint8)
    bias = np.linspace(-0.3, 0.3, 6).astype(np.float32)
    out, cache, ref = check_block(device, t, eps=1e-5, valid=valid, bias=bias, scale=37.0)
    assert cache.valid_tokens == int(valid.sum())


def test_a_few_tokens_take_the_decode_kernels(device):
    t = synth.make(small_workload(d=128, E=8, k=2, F=128, T=5, seed=43, act="bf16", wt="bf16", shared=True))
    nw = norm_weight(128, 1)
    layer = gpu_layer(device, t, max_tokens=8)
    layer.set_feed_forward_norm(nw, 1e-6)
    want, _, ref = oracle_layer(t).forward_block(t.x, nw, 1e-6, round_normed=synth.round_bf16)
    out, cache = layer.forward_block(t.x)
    assert layer.kernel_name().startswith("mfma_bf16_decode")
    assert_routing_identical(cache, ref)
    assert rel_l2(out, want) <= 2e-2
    layer.close()


@pytest.mark.parametrize("T", [1, 2, 8, 32])
@pytest.mark.parametrize("wt", ["bf16", "int8"])
def test_decode_steps_normalise_inside_the_routing_kernel(device, T, wt):
    # TransformerBlock::forward_cached (src/transformer_block.rs:236-250): norm, layer, residual add on the rows
    # of one decode step.  With one row the reference's Linear takes its eight-lane dot for the router
    # (src/matrix.rs:131-153), the order the oracle uses for every row count.
    t = synth.make(small_workload(d=768, E=8, k=2, F=128, T=T, seed=46 + T, act="bf16", wt=wt, shared=True))
    nw = norm_weight(768, 4)
    x = synth.round_bf16(t.x * np.float32(5.0))
    layer = gpu_layer(device, t, max_tokens=32)
    layer.set_feed_forward_norm(nw, 1e-6)
    want, normed, ref = oracle_layer(t).forward_block(x, nw, 1e-6, round_normed=synth.round_bf16)
    out, cache = layer.forward_block(x)
    assert layer.kernel_name().startswith("mfma_bf16_decode")
    assert_routing_identical(cache, ref)
    assert rel_l2(out, want) <= 2e-2
    # the same call again (the normed rows are rewritten), then a plain forward on the normed rows
    out2, _ = layer.forward_block(x)
    assert np.array_equal(out, out2)
    plain, cache_p = layer.forward_train(normed, residual=x)
    assert_routing_identical(cache_p, ref)
    assert np.array_equal(plain, out)
    layer.close()


def test_in_place_and_device_pointers(device):
    from bench import DeviceBuffer
    t = synth.make(small_workload(d=64, E=4, k=2, F=64, T=300, seed=44, act="bf16", wt="bf16"))
    nw = norm_weight(64, 2)
    layer = gpu_layer(device, t)
    layer.set_feed_forward_norm(nw, 1e-6)
    want, _ = layer.forward_block(t.x)
    bits = synth.f32_to_bf16_bits(t.x)
    buf = DeviceBuffer(device, bits.nbytes).upload(bits)
    layer.forward_block_device(buf.ptr, 300, buf.ptr)     # out == x
    device.synchronize()
    got = synth.bf16_bits_to_f32(buf.download(np.empty_like(bits))).reshape(300, 64)
    assert np.array_equal(got, want)
    buf.free()
    layer.close()


def test_norm_errors(device):
    t = synth.make(small_workload(d=8, E=4, k=2, F=6, T=4, seed=45))
    layer = gpu_layer(device, t)
    with pytest.raises(rb.InvalidConfig):
        layer.forward_block(t.x)                           # norm not set
    with pytest.raises(rb.InvalidInput):
        layer.set_feed_forward_norm(np.ones(7, np.float32))
    layer.set_feed_forward_norm(np.ones(8, np.float32), 1e-6)
    layer.set_feed_forward_norm(np.full(8, 2.0, np.float32), 1e-6)   # replacing it is allowed
    with pytest.raises(rb.InvalidInput):
        layer.forward_block(np.zeros((4, 9), np.float32))
    out, _ = layer.forward_block(np.zeros((4, 8), np.float32))       # zero rows stay finite (eps under the root)
    assert np.isfinite(out).all()
    layer.close()


def test_c3_block_step_at_full_size(device):
    t = synth.make(synth.WORKLOADS["c3_prefill_d768_e16"])
    w = t.workload
    nw = norm_weight(w.d_model, 9)
    # a residual stream with rows of very different size, as after a few blocks
    rng = np.random.default_rng(10)
    x = synth.round_bf16(t.x * rng.uniform(0.25, 8.0, (w.tokens, 1)).astype(np.float32))
    want, normed, ref = oracle_layer(t).forward_block(x, nw, 1e-6, router_bias=t.router_bias, threads=8,
                                                      round_normed=synth.round_bf16)
    layer = gpu_layer(device, t)
    layer.set_feed_forward_norm(nw, 1e-6)
    out, cache = layer.forward_block(x, router_bias=t.router_bias)
    assert_routing_identical(cache, ref)
    assert rel_l2(out, want) <= 2e-2
    share = float(np.linalg.norm(want - x))
    assert rel_l2(out - x, want - x) <= 4e-2 + 2.0 ** -8 * float(np.linalg.norm(want)) / share
    layer.close()


# ------------------------------------------------------------------ backward through the block step
def check_block_backward(device, t, valid=None, bias=None, seed=5, norm_first=True):
    w = t.workload
    bf16 = w.act_dtype == "bf16"
    tol = 2e-2 if bf16 else 1e-5
    nw = norm_weight(w.d_model, seed)
    rng = np.random.default_rng(seed + 1)
    gout = synth.round_bf16(rng.standard_normal(t.x.shape).astype(np.float32))
    rounder = synth.round_bf16 if bf16 else None
    ref_layer = oracle_layer(t)
    want_out, _, ref_f = ref_layer.forward_block(t.x, nw, 1e-6, valid=valid, router_bias=bias, round_normed=rounder,
                                                 threads=8)
    want_g, want_gw, inner = ref_layer.backward_block(t.x, nw, 1e-6, gout, valid=valid, router_bias=bias,
                                                      round_normed=rounder, threads=8)
    cfg = rb.MoeConfig(w.num_experts, w.experts_per_token, w.d_ff, w.shared_expert)
    layer = rb.MoeLayer(w.d_model, cfg, device, act_dtype=w.act_dtype, weight_dtype=w.weight_dtype,
                        max_tokens=t.x.shape[0], shared_d_ff=w.shared_d_ff if w.shared_expert else 0)
    if norm_first:                       # the two set-up calls in either order
        layer.set_feed_forward_norm(nw, 1e-6)
        layer.enable_training()
    else:
        layer.enable_training()
        layer.set_feed_forward_norm(nw, 1e-6)
    layer.load_tensors(t)
    layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
    out, cache = layer.forward_block(t.x, layout, router_bias=bias)
    assert_routing_identical(cache, ref_f)
    assert rel_l2(out, want_out) <= tol
    g = layer.backward_block(gout)
    assert rel_l2(g, want_g) <= tol
    # the branch's share alone (the residual passes grad_output through, which dominates the sum)
    share = float(np.linalg.norm(want_g - gout))
    rounding = 2.0 ** -8 * float(np.linalg.norm(want_g)) / max(share, 1e-30) if bf16 else 0.0
    assert rel_l2(g - gout, want_g - gout) <= 2 * tol + rounding
    assert rel_l2(layer.weight_grad(L.W_NORM).reshape(-1), want_gw) <= tol
    assert rel_l2(layer.weight_grad(L.W_ROUTER), inner.grad_router) <= tol
    assert rel_l2(layer.weight_grad(L.W_DOWN, 0), inner.grad_down[0]) <= tol
    return layer, gout, want_gw


@pytest.mark.parametrize("act", ["bf16", "f32"])
@pytest.mark.parametrize("shape", [dict(d=64, E=4, k=2, F=64, T=70), dict(d=128, E=8, k=2, F=64, T=300, shared=True)],
                         ids=lambda s: "d{d}_E{E}_T{T}".format(**s))
def test_block_backward_matches_the_oracle(device, act, shape):
    t = synth.make(small_workload(seed=51, act=act, wt=act, **shape))
    layer, _, _ = check_block_backward(device, t, norm_first=shape["T"] == 70)
    layer.close()


def test_block_backward_with_padding_accumulation_and_errors(device):
    t = synth.make(small_workload(d=64, E=6, k=2, F=64, T=100, seed=52, act="bf16", wt="bf16", shared=True))
    valid = (np.arange(100) % 6 != 1).astype(np.uint8)
    bias = np.linspace(-0.4, 0.4, 6).astype(np.float32)
    layer, gout, want_gw = check_block_backward(device, t, valid=valid, bias=bias)
    layer.backward_block(gout)                              # the norm's scale gradient accumulates ...
    assert rel_l2(layer.weight_grad(L.W_NORM).reshape(-1), 2.0 * want_gw) <= 2e-2
    layer.zero_grads()                                      # ... until cleared
    assert not layer.weight_grad(L.W_NORM).any()
    layer.forward_train(synth.round_bf16(t.x))              # a plain forward is not a block step
    with pytest.raises(rb.InvalidInput):
        layer.backward_block(gout)
    layer.close()
    plain = gpu_layer(device, t, training=True)             # no norm set
    plain.forward_train(t.x)
    with pytest.raises(rb.InvalidConfig):
        plain.backward_block(gout)
    plain.close()


def test_c3_block_training_step_at_full_size(device):
    t = synth.make(synth.WORKLOADS["c3_prefill_d768_e16"])
    layer, _, _ = check_block_backward(device, t, bias=t.router_bias)
    layer.close()


# ------------------------------------------------------------------ the reference's cached-decode tests, feed-forward half
@pytest.mark.parametrize("act,wt,d,F", [("f32", "f32", 64, 96), ("bf16", "bf16", 128, 192), ("bf16", "int8", 128, 192),
                                        ("f32", "f32", 24, 10)])
def test_a_cached_decode_reproduces_the_full_sequence_forward(device, act, wt, d, F):
    """reference src/transformer.rs:2422-2454: feeding a sequence one token at a time (`forward_cached`), or a
    prefill and then single tokens, must give what the whole sequence gives at once, within 1e-3.  For the
    feed-forward half of the block that is: the block step on one row (the decode-shaped kernels where the layer
    has them) against the same row inside a batch of 70 (the large-batch kernels) - the same experts and
    probabilities in every bit, the same output within 1e-3 for f32 and within the bf16 bar otherwise."""
    T = 70
    t = synth.make(small_workload(d=d, E=8, k=2, F=F, T=T, seed=51, act=act, wt=wt, shared=True))
    nw = norm_weight(d, 51)
    cfg = rb.MoeConfig(8, 2, F, True)
    layer = rb.MoeLayer(d, cfg, device, act_dtype=act, weight_dtype=wt, max_tokens=T)
    layer.set_feed_forward_norm(nw, 1e-5)
    layer.load_tensors(t)
    full, cache_full = layer.forward_block(t.x)
    big_kernels = layer.kernel_name()

    def same_as_full(rows, out, cache):
        k = 2
        assert np.array_equal(cache.expert_of.reshape(-1, k), cache_full.expert_of.reshape(T, k)[rows])
        assert np.array_equal(cache.probabilities.view(np.uint32), cache_full.probabilities[rows].view(np.uint32))
        if act == "f32":
            assert np.max(np.abs(out - full[rows])) < 1e-3
        else:
            assert rel_l2(out, full[rows]) <= 5e-3

    for position in (0, 1, 2, 17, 69):                      # one token at a time
        out, cache = layer.forward_block(t.x[position:position + 1])
        same_as_full(slice(position, position + 1), out, cache)
    if act == "bf16":
        assert layer.kernel_name().startswith("mfma_bf16_decode") and big_kernels.startswith("mfma_bf16_stream")
    out, cache = layer.forward_block(t.x[:40])              # a prefill, then the next token
    same_as_full(slice(0, 40), out, cache)
    out, cache = layer.forward_block(t.x[40:41])
    same_as_full(slice(40, 41), out, cache)
    layer.close()
