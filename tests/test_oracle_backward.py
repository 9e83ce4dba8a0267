"""Pins of the oracle's backward pass (MoeLayer::backward, src/moe.rs:348-489).

* the reference's own four tests (src/moe.rs:861-1013), with their inputs and tolerances: gradients reach only the
  experts a token was routed to; grad_input, the router gradient and the auxiliary-loss gradient against central
  finite differences of the oracle's f32 forward (epsilon 1e-3; 2e-2, 2e-2, 1e-3);
* an independent float64 evaluation of the layer (softmax, renormalised top-k gates with the selection held fixed,
  SwiGLU experts, shared expert, both losses) differentiated by finite differences in float64, for every kind of
  parameter, a weighted output sum as the objective (so that no term cancels), padding rows included.
No GPU."""
import numpy as np
import pytest

from helpers import oracle_layer, small_workload
from oracle import rb_oracle as orc
from rustingbrain_amd import synth


def one_hot_router(E, d, strength):
    w = np.zeros((E, d), np.float32)
    for e in range(E):
        w[e, e % d] = strength
    return w


def make(E, k, F, d, T, seed, shared=False, aux_w=0.0, z_w=0.0):
    t = synth.make(small_workload(d=d, E=E, k=k, F=F, T=T, seed=seed, shared=shared))
    return t, oracle_layer(t, aux_w=aux_w, z_w=z_w)


def test_gradients_reach_only_the_experts_a_token_was_routed_to():
    t, layer = make(4, 1, 4, 4, 3, seed=10)
    layer.router = one_hot_router(4, 4, 30.0)
    x = np.zeros((3, 4), np.float32)
    x[:, 0] = 1.0  # every token routes to expert 0
    g = layer.backward(x, np.ones((3, 4), np.float32))
    assert np.any(g.grad_gate[0] != 0.0)
    for e in range(1, 4):
        assert np.all(g.grad_gate[e] == 0.0) and np.all(g.grad_up[e] == 0.0) and np.all(g.grad_down[e] == 0.0)


def test_backward_matches_finite_differences():
    t, layer = make(4, 2, 5, 6, 3, seed=11, shared=True)
    x = np.array([((i * 29) % 17) / 8.0 - 1.0 for i in range(18)], np.float32).reshape(3, 6)
    g = layer.backward(x, np.ones((3, 6), np.float32))
    eps = np.float32(1e-3)
    for i in range(x.size):
        hi, lo = x.copy(), x.copy()
        hi.flat[i] += eps
        lo.flat[i] -= eps
        numeric = (layer.forward(hi).out.sum(dtype=np.float32) - layer.forward(lo).out.sum(dtype=np.float32)) / (2 * eps)
        assert abs(g.grad_input.flat[i] - numeric) < 2e-2, (i, g.grad_input.flat[i], numeric)


def test_router_weight_gradient_matches_finite_differences():
    t, layer = make(3, 2, 4, 4, 3, seed=12)
    x = np.array([((i * 13) % 11) / 5.0 - 1.0 for i in range(12)], np.float32).reshape(3, 4)
    g = layer.backward(x, np.ones((3, 4), np.float32))
    eps = np.float32(1e-3)
    base = layer.router.copy()
    for i in range(base.size):
        vals = []
        for s in (+1, -1):
            layer.router = base.copy()
            layer.router.flat[i] += s * eps
            vals.append(layer.forward(x).out.sum(dtype=np.float32))
        numeric = (vals[0] - vals[1]) / (2 * eps)
        assert abs(g.grad_router.flat[i] - numeric) < 2e-2, (i, g.grad_router.flat[i], numeric)
    layer.router = base


def test_auxiliary_loss_gradient_matches_finite_differences():
    t, layer = make(3, 2, 4, 4, 4, seed=13, aux_w=0.01, z_w=1e-3)
    # wide logit gaps: a bump of 1e-3 must not move a token across a top-k boundary, where the counts (and
    # with them the balancing loss) jump
    layer.router = (layer.router * 8).astype(np.float32)
    x = np.array([((i * 19) % 13) / 6.0 - 1.0 for i in range(16)], np.float32).reshape(4, 4)
    g = layer.backward(x, np.zeros((4, 4), np.float32))  # zero upstream: only the two losses reach the router
    eps = np.float32(1e-3)
    base = layer.router.copy()
    for i in range(base.size):
        vals = []
        for s in (+1, -1):
            layer.router = base.copy()
            layer.router.flat[i] += s * eps
            r = layer.forward(x)
            vals.append(np.float32(r.aux_loss) + np.float32(r.z_loss))
        numeric = (vals[0] - vals[1]) / (2 * eps)
        assert abs(g.grad_router.flat[i] - numeric) < 1e-3, (i, g.grad_router.flat[i], numeric)
    layer.router = base


# ------------------------------------------------------------------ float64 cross-check
def f64_objective(x, router, experts, shared, sel, valid, counts, k, aux_w, z_w, R):
    """sum(out * R) + aux + z in float64, the top-k selection `sel` [T, k] and the load counts held fixed."""
    T, d = x.shape
    E = router.shape[0]
    logits = x @ router.T
    mx = logits.max(axis=1, keepdims=True)
    ex = np.exp(logits - mx)
    ssum = ex.sum(axis=1, keepdims=True)
    P = ex / ssum
    lse = (mx + np.log(ssum))[:, 0]

    def swiglu(w, rows):
        g = rows @ w[0].T
        u = rows @ w[1].T
        return (g / (1.0 + np.exp(-g)) * u) @ w[2].T

    out = np.zeros((T, d))
    for t in range(T):
        if not valid[t]:
            continue
        p = P[t, sel[t]]
        gates = p / p.sum()
        for r in range(k):
            out[t] += gates[r] * swiglu(experts[sel[t, r]], x[t:t + 1])[0]
    if shared is not None:
        out += swiglu(shared, x)
    V = int(valid.sum())
    aux = z = 0.0
    if V > 0:
        load = counts / (V * k)
        mass = P[valid.astype(bool)].sum(axis=0) / V
        aux = (load * mass).sum() * E * aux_w
        z = z_w * (lse[valid.astype(bool)] ** 2).sum() / V
    return (out * R).sum() + aux + z


@pytest.mark.parametrize("shared", [False, True])
def test_every_gradient_against_float64_finite_differences(shared):
    E, k, F, d, T = 5, 2, 7, 6, 9
    t, layer = make(E, k, F, d, T, seed=21, shared=shared, aux_w=0.05, z_w=0.02)
    layer.router = (layer.router * 20).astype(np.float32)  # spread the logits: no near-ties, meaningful softmax
    x = t.x.astype(np.float32)
    valid = np.ones(T, np.uint8)
    valid[[2, 7]] = 0
    Rm = synth.normal((T, d), 1.0, 5, 77).astype(np.float32)
    fwd = layer.forward(x, valid=valid)
    g = layer.backward(x, Rm, valid=valid)
    sel = fwd.expert_of.reshape(T, k)
    counts = fwd.counts.astype(np.float64)
    experts = [[w.gate.astype(np.float64), w.up.astype(np.float64), w.down.astype(np.float64)] for w in layer.experts]
    sh = None if layer.shared is None else [layer.shared.gate.astype(np.float64), layer.shared.up.astype(np.float64),
                                            layer.shared.down.astype(np.float64)]
    x64, r64 = x.astype(np.float64), layer.router.astype(np.float64)

    def objective():
        return f64_objective(x64, r64, experts, sh, sel, valid, counts, k, 0.05, 0.02, Rm.astype(np.float64))

    def fd(arr, analytic, name, stride=1):
        eps = 1e-6
        worst = 0.0
        for i in range(0, arr.size, stride):
            keep = arr.flat[i]
            arr.flat[i] = keep + eps
            hi = objective()
            arr.flat[i] = keep - eps
            lo = objective()
            arr.flat[i] = keep
            numeric = (hi - lo) / (2 * eps)
            worst = max(worst, abs(analytic.flat[i] - numeric))
        scale = max(np.max(np.abs(analytic)), 1e-3)
        assert worst <= 2e-4 * scale + 2e-5, (name, worst, scale)

    fd(x64, g.grad_input, "input")
    assert np.all(g.grad_input[[2, 7]] == 0.0) or shared  # padding rows get a gradient only through the shared expert
    fd(r64, g.grad_router, "router")
    used = int(np.argmax(fwd.counts))
    fd(experts[used][0], g.grad_gate[used], "gate", stride=3)
    fd(experts[used][1], g.grad_up[used], "up", stride=3)
    fd(experts[used][2], g.grad_down[used], "down", stride=3)
    if shared:
        fd(sh[0], g.grad_shared[0], "shared gate", stride=3)
        fd(sh[2], g.grad_shared[2], "shared down", stride=3)
    # slots of padding rows carry no gate gradient, and the weight gradients of an unused expert stay zero
    assert np.all(g.grad_gates.reshape(T, k)[[2, 7]] == 0.0)
    for e in range(E):
        if fwd.counts[e] == 0:
            assert np.all(g.grad_gate[e] == 0.0)
