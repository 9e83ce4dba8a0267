"""GPU parity of the backward pass (MoeLayer::backward, src/moe.rs:348-489) through the C ABI against the CPU
oracle's backward on the same seeded inputs.  The routing of the forward is bit-identical, so both sides
differentiate the same selection; every gradient must agree within rel-L2 2e-2 for bf16 layers (the oracle
computes in f32 from the same bf16-representable values) and 1e-5 for all-f32 layers.
"""
import numpy as np
import pytest

import rustingbrain_amd as rb
from conftest import rel_l2
from helpers import assert_routing_identical, gpu_layer, oracle_layer, small_workload
from rustingbrain_amd import _lib as L
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu

TOL = 2e-2


def grad_output_for(t, seed):
    rng = np.random.default_rng(seed)
    return synth.round_bf16(rng.standard_normal(t.x.shape).astype(np.float32))


def check_backward(device, t, valid=None, bias=None, aux_w=0.01, z_w=1e-3, seed=1, tol=None, max_tokens=None):
    w = t.workload
    if tol is None:  # f32 rows over bf16 weights multiply on the bf16 matrix cores where the widths allow
        tol = 1e-5 if (w.act_dtype == "f32" and w.weight_dtype == "f32") else TOL
    E = w.num_experts
    gout = grad_output_for(t, seed)
    ref_layer = oracle_layer(t, aux_w=aux_w, z_w=z_w)
    ref_fwd = ref_layer.forward(t.x, valid=valid, router_bias=bias, threads=8)
    ref = ref_layer.backward(t.x, gout, valid=valid, router_bias=bias, threads=8)
    layer = gpu_layer(device, t, max_tokens=max_tokens, aux_w=aux_w, z_w=z_w, training=True)
    layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
    out, cache = layer.forward_train(t.x, layout, router_bias=bias)
    assert_routing_identical(cache, ref_fwd)
    assert rel_l2(out, ref_fwd.out) <= tol
    gin = layer.backward(gout)

    def close(name, got, want):
        if not want.any():
            assert not got.any(), f"{name}: expected exactly zero"
            return
        err = rel_l2(got, want)
        assert err <= tol, f"{name}: rel-L2 {err} > {tol}"

    close("grad_input", gin, ref.grad_input)
    close("grad_router", layer.weight_grad(L.W_ROUTER), ref.grad_router)
    for e in range(E):
        close(f"grad_gate[{e}]", layer.weight_grad(L.W_GATE, e), ref.grad_gate[e])
        close(f"grad_up[{e}]", layer.weight_grad(L.W_UP, e), ref.grad_up[e])
        close(f"grad_down[{e}]", layer.weight_grad(L.W_DOWN, e), ref.grad_down[e])
    if t.shared is not None:
        close("grad_shared_gate", layer.weight_grad(L.W_SHARED_GATE), ref.grad_shared[0])
        close("grad_shared_up", layer.weight_grad(L.W_SHARED_UP), ref.grad_shared[1])
        close("grad_shared_down", layer.weight_grad(L.W_SHARED_DOWN), ref.grad_shared[2])
    return layer, ref, gout


SHAPES = [
    dict(d=64, E=4, k=2, F=64, T=50),
    dict(d=64, E=4, k=1, F=128, T=7),
    dict(d=128, E=8, k=3, F=192, T=300, shared=True, shared_d_ff=128),
    dict(d=192, E=16, k=2, F=64, T=1000, shared=True),
    dict(d=64, E=3, k=3, F=64, T=129),
    dict(d=64, E=24, k=4, F=64, T=333),                                   # 32 lanes per token, two expert batches
    dict(d=256, E=64, k=6, F=128, T=2048, shared=True, shared_d_ff=256),  # C4's proportions, scaled down
    dict(d=64, E=70, k=8, F=64, T=77),                                    # more experts than lanes, ragged batches
    dict(d=320, E=5, k=2, F=192, T=3000),                                 # widths that are not multiples of 256
]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}".format(**s))
def test_backward_matches_the_oracle(device, shape):
    t = synth.make(small_workload(seed=21, act="bf16", wt="bf16", **shape))
    layer, _, _ = check_backward(device, t)
    layer.close()


SHAPES_F32 = [
    dict(d=32, E=4, k=2, F=32, T=50),
    dict(d=64, E=8, k=3, F=96, T=300, shared=True, shared_d_ff=64),
    dict(d=96, E=24, k=2, F=32, T=1000),
    dict(d=512, E=8, k=2, F=1408, T=1024),          # the f32 configuration of the benchmark set (C1)
]


@pytest.mark.parametrize("shape", SHAPES_F32, ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}".format(**s))
def test_backward_of_all_f32_layers(device, shape):
    t = synth.make(small_workload(seed=31, act="f32", wt="f32", **shape))
    valid = (np.arange(shape["T"]) % 7 != 3).astype(np.uint8) if shape["T"] == 300 else None
    layer, ref, gout = check_backward(device, t, valid=valid)
    assert layer.kernel_name() == "mfma_f32"
    # accumulate, clear, overwrite
    once = layer.weight_grad(L.W_DOWN, 1)
    layer.backward(gout)
    assert rel_l2(layer.weight_grad(L.W_DOWN, 1), 2.0 * once) <= 1e-6
    layer.zero_grads()
    layer.backward(gout)
    assert rel_l2(layer.weight_grad(L.W_DOWN, 1), once) <= 1e-6
    layer.close()


def test_backward_with_padding_rows_and_router_bias(device):
    # padding rows get no gradient from the routed experts or the router, only from the shared expert
    # (src/moe.rs:356-361 runs it over every row)
    t = synth.make(small_workload(d=64, E=6, k=2, F=128, T=90, seed=22, act="bf16", wt="bf16", shared=True))
    valid = (np.arange(90) % 5 != 2).astype(np.uint8)
    bias = np.linspace(-0.5, 0.5, 6).astype(np.float32)
    layer, ref, _ = check_backward(device, t, valid=valid, bias=bias)
    layer.close()


def test_an_expert_without_tokens_gets_exactly_zero_gradients(device):
    # reference test src/moe.rs:861-890: gradients reach only the experts a token was routed to
    t = synth.make(small_workload(d=64, E=5, k=2, F=64, T=64, seed=23, act="bf16", wt="bf16"))
    bias = np.zeros(5, np.float32)
    bias[3] = -1e4
    layer, ref, _ = check_backward(device, t, bias=bias)
    assert not ref.grad_gate[3].any()
    for which in (L.W_GATE, L.W_UP, L.W_DOWN):
        assert not layer.weight_grad(which, 3).any()
    layer.close()


def test_router_gradient_of_one_expert_per_token_is_no_further_from_float64_than_the_oracle(device):
    # With k = 1 the gate is p / p, and its gradient reaches the probability as g / total - (g p) / (total total)
    # with total = p (src/moe.rs:427-441): zero in exact arithmetic, the roundings of two quotients of size |g| / p
    # in f32.  That noise is larger than what the two losses contribute, and it depends on the last bits of g (a dot
    # product of d terms), which differ between any two orders of summation: the router gradient of such a layer is
    # compared with its float64 value, where the GPU has to be as close as the oracle is; every other gradient is
    # compared with the oracle as usual.
    T, E = 2049, 2
    t = synth.make(small_workload(d=384, E=E, k=1, F=512, T=T, seed=16026, act="f32", wt="f32"))
    gout = grad_output_for(t, 5)
    ref_layer = oracle_layer(t)
    fwd = ref_layer.forward(t.x, threads=8)
    ref = ref_layer.backward(t.x, gout, threads=8)
    layer = gpu_layer(device, t, training=True)
    out, cache = layer.forward_train(t.x)
    assert_routing_identical(cache, fwd)
    gin = layer.backward(gout)
    assert rel_l2(gin, ref.grad_input) <= 1e-5
    for e in range(E):
        for which, want in ((L.W_GATE, ref.grad_gate), (L.W_UP, ref.grad_up), (L.W_DOWN, ref.grad_down)):
            assert rel_l2(layer.weight_grad(which, e), want[e]) <= 1e-5
    # float64: the gate contributes nothing; balance loss d aux / d p[t, e] = w_aux E load_e / V, z loss
    # d z / d logit[t, e] = 2 w_z lse_t p[t, e] / V (src/moe.rs:421-478), softmax backward, then dlogits^T X
    P = fwd.probabilities.astype(np.float64)
    lse = fwd.lse.astype(np.float64)
    dp = np.broadcast_to(0.01 * E * (fwd.counts.astype(np.float64) / T) / T, (T, E))
    dlogits = P * (dp - (P * dp).sum(1, keepdims=True)) + 1e-3 * 2.0 * lse[:, None] * P / T
    exact = dlogits.T @ t.x.astype(np.float64)
    oracle_off = np.linalg.norm(ref.grad_router.astype(np.float64) - exact)
    gpu_off = np.linalg.norm(layer.weight_grad(L.W_ROUTER).astype(np.float64) - exact)
    print(f"|exact| {np.linalg.norm(exact):.3e}  oracle off by {oracle_off:.3e}  GPU off by {gpu_off:.3e}")
    assert oracle_off > 0.05 * np.linalg.norm(exact), "the case no longer shows the cancellation it is here for"
    assert gpu_off <= 2.0 * oracle_off
    layer.close()


def test_large_auxiliary_loss_weights_reach_the_router(device):
    # reference test src/moe.rs:969-1013: the balance and z losses are differentiated inside backward
    t = synth.make(small_workload(d=64, E=8, k=2, F=64, T=256, seed=24, act="bf16", wt="bf16"))
    layer, ref, _ = check_backward(device, t, aux_w=5.0, z_w=2.0)
    layer.close()
    # with a zero upstream gradient only the two losses drive the router
    ref_layer = oracle_layer(t, aux_w=5.0, z_w=2.0)
    zero = np.zeros_like(t.x)
    want = ref_layer.backward(t.x, zero)
    layer = gpu_layer(device, t, aux_w=5.0, z_w=2.0, training=True)
    layer.forward_train(t.x)
    gin = layer.backward(zero)
    assert want.grad_router.any()
    assert rel_l2(layer.weight_grad(L.W_ROUTER), want.grad_router) <= TOL
    assert rel_l2(gin, want.grad_input) <= TOL
    assert not layer.weight_grad(L.W_DOWN, 0).any()
    layer.close()


def test_weight_gradients_accumulate_until_zeroed(device):
    # Param.grad accumulates across backward calls (src/param.rs:819-821) until zero_grad
    t = synth.make(small_workload(d=64, E=4, k=2, F=64, T=40, seed=25, act="bf16", wt="bf16", shared=True))
    layer, ref, gout = check_backward(device, t)
    once = {w: layer.weight_grad(w, 1 if w in (L.W_GATE, L.W_UP, L.W_DOWN) else 0) for w in range(7)}
    gin1 = layer.backward(gout)
    for w, g in once.items():
        twice = layer.weight_grad(w, 1 if w in (L.W_GATE, L.W_UP, L.W_DOWN) else 0)
        assert rel_l2(twice, 2.0 * g) <= 1e-6, w
    layer.zero_grads()
    for w in range(7):
        assert not layer.weight_grad(w, 1 if w in (L.W_GATE, L.W_UP, L.W_DOWN) else 0).any()
    gin2 = layer.backward(gout)
    assert np.array_equal(gin1, gin2)
    for w, g in once.items():
        again = layer.weight_grad(w, 1 if w in (L.W_GATE, L.W_UP, L.W_DOWN) else 0)
        assert rel_l2(again, g) <= 1e-6, w
    layer.close()


def test_cleared_gradients_are_overwritten_not_added_to(device):
    # zero_grads leaves the expert matrices as they are and marks them clear; the next backward pass must not
    # see the stale values, also for an expert that then gets no rows and for one that is cut into chunks
    t = synth.make(small_workload(d=64, E=5, k=2, F=64, T=600, seed=28, act="bf16", wt="bf16", shared=True))
    layer, ref, gout = check_backward(device, t)               # fills every gradient
    layer.zero_grads()
    for which in (L.W_GATE, L.W_UP, L.W_DOWN):
        assert not layer.weight_grad(which, 2).any()
    bias = np.zeros(5, np.float32)
    bias[3] = -1e4                                             # expert 3 gets nothing ...
    bias[1] = 3.0                                              # ... and expert 1 most rows (cut into chunks)
    ref_layer = oracle_layer(t)
    want = ref_layer.backward(t.x, gout, router_bias=bias)
    layer.forward_train(t.x, router_bias=bias)
    layer.backward(gout)
    for which, w in ((L.W_GATE, want.grad_gate), (L.W_UP, want.grad_up), (L.W_DOWN, want.grad_down)):
        assert not layer.weight_grad(which, 3).any()
        for e in (0, 1, 2, 4):
            assert rel_l2(layer.weight_grad(which, e), w[e]) <= TOL, (which, e)
    assert rel_l2(layer.weight_grad(L.W_SHARED_DOWN), want.grad_shared[2]) <= TOL
    assert rel_l2(layer.weight_grad(L.W_ROUTER), want.grad_router) <= TOL
    layer.close()


@pytest.mark.parametrize("mode", ["default", "uncut", "atomic"])
@pytest.mark.parametrize("act", ["bf16", "f32"])
def test_weight_gradients_of_a_cut_expert(device, monkeypatch, mode, act):
    # One expert far above its share is cut into chunks of rows (a shared expert always is).  By default the
    # chunks meet in a fixed order (the first adds in place, the others store partial matrices that are added in
    # chunk order), so two runs give identical bits - with gradients accumulated over two passes and after
    # zero_grads alike; RBMOE_DETERMINISTIC=1 cuts nothing; RBMOE_ATOMIC_WGRAD=1 adds with f32 atomics (right
    # within the tolerance, in no fixed order).
    if mode == "uncut":
        monkeypatch.setenv("RBMOE_DETERMINISTIC", "1")
    if mode == "atomic":
        monkeypatch.setenv("RBMOE_ATOMIC_WGRAD", "1")
    t = synth.make(small_workload(d=64, E=4, k=2, F=128, T=2600, seed=29, act=act, wt=act, shared=True))
    bias = np.array([2.5, 0.0, 0.0, 0.0], np.float32)          # one expert far above its share
    runs = []
    for _ in range(2):
        layer, ref, gout = check_backward(device, t, bias=bias)
        first = [layer.weight_grad(w, e) for w in (L.W_GATE, L.W_UP, L.W_DOWN) for e in range(4)] + \
                [layer.weight_grad(L.W_ROUTER), layer.weight_grad(L.W_SHARED_DOWN), layer.weight_grad(L.W_SHARED_UP)]
        layer.backward(gout)                                    # a second pass adds to the gradients
        twice = [layer.weight_grad(L.W_DOWN, 0), layer.weight_grad(L.W_SHARED_DOWN)]
        assert rel_l2(twice[0], 2.0 * ref.grad_down[0]) <= (2e-2 if act == "bf16" else 1e-5)
        runs.append(first + twice)
        layer.close()
    if mode != "atomic":
        for a, b in zip(*runs):
            assert np.array_equal(a, b)


def test_plain_f32_weight_gradient_kernel_agrees(device, monkeypatch):
    # RBMOE_WGRAD_GENERIC=1 swaps the matrix-core weight-gradient kernels for the plain f32 one (A/B switch)
    monkeypatch.setenv("RBMOE_WGRAD_GENERIC", "1")
    for act in ("bf16", "f32"):
        t = synth.make(small_workload(d=64, E=4, k=2, F=64, T=150, seed=32, act=act, wt=act, shared=True))
        layer, ref, gout = check_backward(device, t)
        layer.zero_grads()
        layer.backward(gout)             # cleared, then written through the plain kernel's path
        assert rel_l2(layer.weight_grad(L.W_UP, 2), ref.grad_up[2]) <= (1e-5 if act == "f32" else TOL)
        layer.close()


def test_backward_of_degenerate_batches(device):
    # every row padding (nothing routed; only the shared expert sees the rows), then a single row
    t = synth.make(small_workload(d=64, E=4, k=2, F=64, T=40, seed=34, act="bf16", wt="bf16", shared=True))
    layer, ref, gout = check_backward(device, t, valid=np.zeros(40, np.uint8))
    for which in (L.W_GATE, L.W_UP, L.W_DOWN):
        for e in range(4):
            assert not layer.weight_grad(which, e).any()
    assert not layer.weight_grad(L.W_ROUTER).any()
    assert layer.weight_grad(L.W_SHARED_DOWN).any()
    layer.close()
    one = synth.make(small_workload(d=64, E=4, k=2, F=64, T=1, seed=35, act="bf16", wt="bf16"))
    layer, ref, gout = check_backward(device, one)
    assert int((np.abs(ref.grad_down).sum(axis=(1, 2)) > 0).sum()) == 2     # exactly the two selected experts
    layer.close()
    plain = synth.make(small_workload(d=64, E=4, k=2, F=64, T=40, seed=36, act="f32", wt="f32"))
    layer, _, _ = check_backward(device, plain, valid=np.zeros(40, np.uint8))  # no shared expert: all gradients zero
    assert not layer.weight_grad(L.W_DOWN, 0).any()
    layer.close()


def test_backward_follows_the_most_recent_forward(device):
    t = synth.make(small_workload(d=64, E=4, k=2, F=64, T=120, seed=26, act="bf16", wt="bf16"))
    layer = gpu_layer(device, t, training=True)
    ref_layer = oracle_layer(t)
    for rows in (120, 33, 1):
        x = t.x[:rows]
        gout = grad_output_for(t, rows)[:rows]
        layer.zero_grads()
        layer.forward_train(x)
        gin = layer.backward(gout)
        want = ref_layer.backward(x, gout)
        assert rel_l2(gin, want.grad_input) <= TOL
        assert rel_l2(layer.weight_grad(L.W_ROUTER), want.grad_router) <= TOL
        for e in range(4):
            if want.grad_down[e].any():
                assert rel_l2(layer.weight_grad(L.W_DOWN, e), want.grad_down[e]) <= TOL
    layer.close()


def test_training_mode_errors(device):
    cfg = rb.MoeConfig(4, 2, 64)
    t = synth.make(small_workload(d=64, E=4, k=2, F=64, T=8, seed=27, act="bf16", wt="bf16"))
    late = gpu_layer(device, t)
    with pytest.raises(rb.InvalidConfig):
        late.enable_training()         # the transposed copies are made when a weight is set
    with pytest.raises(rb.InvalidConfig):
        late.backward(np.zeros((8, 64), np.float32))
    with pytest.raises(rb.InvalidConfig):
        late.weight_grad(L.W_ROUTER)
    late.close()
    q8 = rb.MoeLayer(64, cfg, device, act_dtype="bf16", weight_dtype="int8", max_tokens=8)
    with pytest.raises(rb.Unsupported):          # quantized experts have no backward pass (src/ffn.rs:87-93)
        q8.enable_training()
    q8.close()
    fresh = rb.MoeLayer(64, cfg, device, act_dtype="bf16", weight_dtype="bf16", max_tokens=8)
    fresh.enable_training()
    fresh.enable_training()            # idempotent
    with pytest.raises(rb.InvalidInput):
        fresh.backward(np.zeros((8, 64), np.float32))   # no forward yet
    fresh.load_tensors(t)
    fresh.forward_train(t.x)
    with pytest.raises(rb.InvalidInput):
        fresh.backward(np.zeros((8, 32), np.float32))
    # buffers that do not have the last forward's rows are refused before a byte of them is touched, on host and
    # on device pointers, with and without the norm in front
    for rows in (7, 9, 0):
        with pytest.raises(rb.InvalidInput, match="rows of the last forward"):
            fresh.backward(np.zeros((rows, 64), np.float32))
    lib = L.load()
    import ctypes as C
    small = np.zeros((1, 64), np.uint16)
    for fn in (lib.rbmoe_backward, lib.rbmoe_backward_host):
        assert fn(fresh.handle, small.ctypes.data_as(C.c_void_p), 9, 64, small.ctypes.data_as(C.c_void_p)) == L.INVALID_INPUT
        assert fn(fresh.handle, small.ctypes.data_as(C.c_void_p), 8, 63, small.ctypes.data_as(C.c_void_p)) == L.INVALID_INPUT
    fresh.set_feed_forward_norm(np.ones(64, np.float32))
    fresh.forward_block(t.x)
    with pytest.raises(rb.InvalidInput, match="rows of the last forward"):
        fresh.backward_block(np.zeros((5, 64), np.float32))
    for fn in (lib.rbmoe_backward_block, lib.rbmoe_backward_block_host):
        assert fn(fresh.handle, small.ctypes.data_as(C.c_void_p), 1, 64, small.ctypes.data_as(C.c_void_p)) == L.INVALID_INPUT
    assert fresh.backward_block(np.zeros((8, 64), np.float32)).shape == (8, 64)
    assert fresh.kernel_name().startswith("mfma_bf16")
    fresh.close()


def test_c3_backward_at_full_size(device):
    # the configuration the headline metric is quoted on; the oracle's f32 backward takes a few seconds here
    t = synth.make(synth.WORKLOADS["c3_prefill_d768_e16"])
    layer, ref, _ = check_backward(device, t)
    layer.close()


@pytest.mark.parametrize("max_tokens,tokens", [(1200, 1024), (2000, 1152)])
def test_backward_of_a_batch_smaller_than_max_tokens_with_two_skewed_experts(device, max_tokens, tokens):
    """The workspace of the ordered weight gradients is sized at creation for max_tokens, the cut limit of a launch
    follows the rows of that launch: at this shape a batch of 1024 tokens cuts out more partial matrices than one
    of 1200 does.  Two experts far above the average share are both cut."""
    t = synth.make(small_workload(d=768, E=16, k=2, F=2048, T=tokens, seed=27, act="bf16", wt="bf16"))
    bias = np.zeros(16, np.float32)
    bias[3], bias[11] = 1.2, 0.9
    layer, ref, gout = check_backward(device, t, bias=bias, max_tokens=max_tokens)
    counts = np.asarray(layer.cache(tokens).counts)
    assert counts[3] > 3 * np.median(counts) and counts[11] > 2 * np.median(counts), counts
    # accumulating over a second pass, and identical bits run to run (the cut experts meet in a fixed order)
    once = layer.weight_grad(L.W_DOWN, 3)
    layer.backward(gout)
    assert rel_l2(layer.weight_grad(L.W_DOWN, 3), 2.0 * once) <= 1e-6
    layer.zero_grads()
    layer.backward(gout)
    assert np.array_equal(layer.weight_grad(L.W_DOWN, 3).view(np.uint32), once.view(np.uint32))
    layer.close()


@pytest.mark.parametrize("shape", [dict(d=128, E=8, k=2, F=192, T=300, shared=True, shared_d_ff=128),
                                   dict(d=768, E=16, k=2, F=1408, T=1024)],
                         ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}".format(**s))
def test_f32_rows_over_bf16_weights_train_on_the_matrix_cores(device, shape):
    """The reference's mixed-precision shape (f32 activations, bf16 expert weights, src/gpu_model.rs:2146-2153): the
    products of both directions run on the bf16 matrix cores over bf16 copies of the rows and of the upstream
    gradient; routing, losses and the router's gradient are those of the f32 rows."""
    t = synth.make(small_workload(seed=33, act="f32", wt="bf16", **shape))
    valid = (np.arange(shape["T"]) % 11 != 5).astype(np.uint8)
    layer, ref, gout = check_backward(device, t, valid=valid, tol=TOL)
    assert layer.kernel_name() == "mfma_bf16_stream"
    once = layer.weight_grad(L.W_GATE, 1)
    layer.backward(gout)
    assert rel_l2(layer.weight_grad(L.W_GATE, 1), 2.0 * once) <= 1e-6
    layer.close()
