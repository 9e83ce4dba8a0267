"""The backward pass on layers of any shape (widths off the matrix-core kernels, mixed dtypes), through the C ABI.

* The reference's own four gradient tests (src/moe.rs:861-1013) at their own shapes (d_model 4 and 6, d_ff 4 and
  5), inputs, epsilon and tolerances, run on the device layer: the finite differences are taken through the
  device's forward pass, the analytic side is `rbmoe_backward`.  The weights are this build's seeded ones (the
  reference draws its own from `StdRng`, which cannot be replayed here).
* `SwiGlu`'s own two gradient tests (src/ffn.rs:274-322) on a layer with one expert, where the gate is exactly 1.
* The same gradients against the CPU oracle at odd shapes, for f32, bf16 and mixed layers, with a shared expert
  of another width, padding rows, an expert without rows, accumulation and the block step's norm.
"""
import numpy as np
import pytest

from conftest import rel_l2
from helpers import gpu_layer, small_workload
from rustingbrain_amd import _lib as L
from rustingbrain_amd import synth
from test_gpu_backward import check_backward
from test_gpu_block import check_block_backward

pytestmark = pytest.mark.gpu


def one_hot_router(E, d, strength):
    w = np.zeros((E, d), np.float32)
    for e in range(E):
        w[e, e % d] = strength
    return w


def device_layer(device, E, k, F, d, T, seed, shared=False, aux_w=0.0, z_w=0.0):
    t = synth.make(small_workload(d=d, E=E, k=k, F=F, T=T, seed=seed, shared=shared))
    layer = gpu_layer(device, t, aux_w=aux_w, z_w=z_w, training=True)
    return t, layer


def test_gradients_reach_only_the_experts_a_token_was_routed_to(device):
    t, layer = device_layer(device, 4, 1, 4, 4, 3, seed=10)
    layer.set_router(one_hot_router(4, 4, 30.0))
    x = np.zeros((3, 4), np.float32)
    x[:, 0] = 1.0  # every token routes to expert 0
    out, cache = layer.forward_train(x)
    assert layer.kernel_name() == "generic"
    assert list(cache.counts) == [3, 0, 0, 0]
    layer.backward(np.ones((3, 4), np.float32))
    assert np.any(layer.weight_grad(L.W_GATE, 0) != 0.0)
    for e in range(1, 4):
        for which in (L.W_GATE, L.W_UP, L.W_DOWN):
            assert np.all(layer.weight_grad(which, e) == 0.0), "an unrouted expert received a gradient"
    layer.close()


def test_backward_matches_finite_differences(device):
    t, layer = device_layer(device, 4, 2, 5, 6, 3, seed=11, shared=True)
    x = np.array([((i * 29) % 17) / 8.0 - 1.0 for i in range(18)], np.float32).reshape(3, 6)
    layer.forward_train(x)
    gin = layer.backward(np.ones((3, 6), np.float32))
    eps = np.float32(1e-3)
    for i in range(x.size):
        hi, lo = x.copy(), x.copy()
        hi.flat[i] += eps
        lo.flat[i] -= eps
        numeric = (layer.forward(hi).sum(dtype=np.float32) - layer.forward(lo).sum(dtype=np.float32)) / (2 * eps)
        assert abs(gin.flat[i] - numeric) < 2e-2, (i, gin.flat[i], numeric)
    layer.close()


def test_router_weight_gradient_matches_finite_differences(device):
    t, layer = device_layer(device, 3, 2, 4, 4, 3, seed=12)
    x = np.array([((i * 13) % 11) / 5.0 - 1.0 for i in range(12)], np.float32).reshape(3, 4)
    layer.forward_train(x)
    layer.backward(np.ones((3, 4), np.float32))
    analytic = layer.weight_grad(L.W_ROUTER)
    eps = np.float32(1e-3)
    for i in range(analytic.size):
        vals = []
        for sgn in (+1, -1):
            probe = t.router.copy()
            probe.flat[i] += sgn * eps
            layer.set_router(probe)
            vals.append(layer.forward(x).sum(dtype=np.float32))
        numeric = (vals[0] - vals[1]) / (2 * eps)
        assert abs(analytic.flat[i] - numeric) < 2e-2, (i, analytic.flat[i], numeric)
    layer.close()


def test_auxiliary_loss_gradient_matches_finite_differences(device):
    t, layer = device_layer(device, 3, 2, 4, 4, 4, seed=13, aux_w=0.01, z_w=1e-3)
    # wide logit gaps: a bump of 1e-3 must not move a token across a top-k boundary, where the counts (and with
    # them the balancing loss) jump
    base = (t.router * 8).astype(np.float32)
    layer.set_router(base)
    x = np.array([((i * 19) % 13) / 6.0 - 1.0 for i in range(16)], np.float32).reshape(4, 4)
    layer.forward_train(x)
    layer.backward(np.zeros((4, 4), np.float32))  # zero upstream: only the two losses reach the router
    analytic = layer.weight_grad(L.W_ROUTER)
    assert np.any(analytic != 0.0)
    eps = np.float32(1e-3)
    for i in range(analytic.size):
        vals = []
        for sgn in (+1, -1):
            probe = base.copy()
            probe.flat[i] += sgn * eps
            layer.set_router(probe)
            _, cache = layer.forward_train(x)
            vals.append(np.float32(cache.aux_loss()) + np.float32(cache.z_loss()))
        numeric = (vals[0] - vals[1]) / (2 * eps)
        assert abs(analytic.flat[i] - numeric) < 1e-3, (i, analytic.flat[i], numeric)
    layer.close()


ODD_SHAPES = [
    # the reference's test shapes, then widths that fit no vector piece and no tile
    dict(d=6, E=4, k=2, F=5, T=3, shared=True, act="f32", wt="f32"),
    dict(d=4, E=3, k=2, F=4, T=4, act="f32", wt="f32"),
    dict(d=33, E=5, k=2, F=50, T=70, shared=True, shared_d_ff=27, act="f32", wt="f32"),
    dict(d=40, E=4, k=2, F=24, T=200, act="f32", wt="f32"),              # 16-byte pieces, no matrix-core tile
    dict(d=7, E=9, k=3, F=11, T=130, act="f32", wt="f32"),
    dict(d=40, E=4, k=2, F=24, T=200, shared=True, act="bf16", wt="bf16"),
    dict(d=33, E=5, k=2, F=50, T=70, shared=True, shared_d_ff=27, act="bf16", wt="bf16"),
    dict(d=72, E=4, k=2, F=56, T=90, shared=True, act="f32", wt="bf16"),   # mixed: f32 rows, bf16 weights, off the tiles
    dict(d=24, E=20, k=4, F=10, T=300, act="f32", wt="bf16"),
]


@pytest.mark.parametrize("shape", ODD_SHAPES,
                         ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}_{act}_{wt}".format(**s))
def test_backward_of_any_shape_matches_the_oracle(device, shape):
    t = synth.make(small_workload(seed=41, **shape))
    T = shape["T"]
    valid = (np.arange(T) % 5 != 2).astype(np.uint8) if T >= 70 else None
    layer, ref, gout = check_backward(device, t, valid=valid)
    assert layer.kernel_name() == "generic"
    tol = 1e-5 if shape["act"] == "f32" else 2e-2
    # accumulate, clear, overwrite
    once = layer.weight_grad(L.W_DOWN, 1)
    router_once = layer.weight_grad(L.W_ROUTER)
    layer.backward(gout)
    assert rel_l2(layer.weight_grad(L.W_DOWN, 1), 2.0 * once) <= 1e-6
    assert rel_l2(layer.weight_grad(L.W_ROUTER), 2.0 * router_once) <= 1e-6
    layer.zero_grads()
    assert not layer.weight_grad(L.W_DOWN, 1).any() and not layer.weight_grad(L.W_ROUTER).any()
    layer.backward(gout)
    assert rel_l2(layer.weight_grad(L.W_DOWN, 1), once) <= 1e-6
    assert rel_l2(layer.weight_grad(L.W_GATE, 0), ref.grad_gate[0]) <= tol
    layer.close()


@pytest.mark.parametrize("act", ["f32", "bf16"])
def test_block_step_of_any_width(device, act):
    """norm -> layer -> residual and back, for a width the 16-byte kernels do not take."""
    t = synth.make(small_workload(d=33, E=4, k=2, F=20, T=50, seed=43, shared=True, act=act, wt=act))
    valid = (np.arange(50) % 6 != 1).astype(np.uint8)
    layer, _, _ = check_block_backward(device, t, valid=valid)
    assert layer.kernel_name() == "generic"
    layer.close()


# ------------------------------------------------------------------ SwiGlu's own gradient tests (src/ffn.rs:274-322)
def single_expert_layer(device, d, F, T, seed):
    """One expert, one expert per token: the gate is exactly 1, so the layer is that expert's SwiGLU."""
    t = synth.make(small_workload(d=d, E=1, k=1, F=F, T=T, seed=seed))
    return t, gpu_layer(device, t, aux_w=0.0, z_w=0.0, training=True)


def test_swiglu_backward_matches_finite_differences(device):
    t, layer = single_expert_layer(device, 4, 6, 2, seed=2)
    x = np.array([0.5, -1.0, 2.0, 0.25, -0.75, 1.5, 0.1, -0.3], np.float32).reshape(2, 4)
    out, cache = layer.forward_train(x)
    assert np.all(cache.gate_of == 1.0)
    gin = layer.backward(np.ones((2, 4), np.float32))
    eps = np.float32(1e-3)
    for i in range(x.size):
        hi, lo = x.copy(), x.copy()
        hi.flat[i] += eps
        lo.flat[i] -= eps
        numeric = (layer.forward(hi).sum(dtype=np.float32) - layer.forward(lo).sum(dtype=np.float32)) / (2 * eps)
        assert abs(gin.flat[i] - numeric) < 1e-2, (i, gin.flat[i], numeric)
    layer.close()


def test_swiglu_gate_weight_gradient_matches_finite_differences(device):
    t, layer = single_expert_layer(device, 3, 4, 2, seed=3)
    x = np.array([0.4, -0.8, 1.2, 0.9, 0.3, -1.1], np.float32).reshape(2, 3)
    layer.forward_train(x)
    layer.backward(np.ones((2, 3), np.float32))
    analytic = layer.weight_grad(L.W_GATE, 0)
    assert np.any(analytic != 0.0)
    w = t.experts[0]
    eps = np.float32(1e-3)
    for i in range(analytic.size):
        sums = []
        for sgn in (+1, -1):
            gate = w["gate"].copy()
            gate.flat[i] += sgn * eps
            layer.set_expert(0, gate, w["up"], w["down"])
            sums.append(layer.forward(x).sum(dtype=np.float32))
        numeric = (sums[0] - sums[1]) / (2 * eps)
        assert abs(analytic.flat[i] - numeric) < 1e-2, (i, analytic.flat[i], numeric)
    layer.close()
