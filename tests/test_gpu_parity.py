"""GPU parity: the HIP layer through the C ABI against the CPU oracle on the same
seeded inputs.  Routing tables (and, since the router arithmetic is a fixed
sequence, probabilities / lse / gates) must be identical in every bit; layer
outputs and auxiliary losses must agree within rel-L2 1e-5 for all-f32 layers
and 2e-2 when bf16 or int8 is involved.
"""
import numpy as np
import pytest

import rustingbrain_amd as rb
from conftest import rel_l2
from helpers import (assert_routing_identical, f64_layer_forward, gpu_layer, oracle_layer, small_workload,
                     tolerance)
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu


def check_parity(device, t, valid=None, bias=None, residual=None, threads=8, check_rows=True):
    w = t.workload
    ref = oracle_layer(t).forward(t.x, valid=valid, router_bias=bias, threads=threads)
    layer = gpu_layer(device, t)
    layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
    out, cache = layer.forward_train(t.x, layout, router_bias=bias, residual=residual)
    assert_routing_identical(cache, ref)
    tol = tolerance(w)
    want = ref.out if residual is None else ref.out + residual
    assert out.shape == want.shape
    err = rel_l2(out, want)
    assert err <= tol, f"output rel-L2 {err} > {tol}"
    assert abs(cache.aux_loss() - ref.aux_loss) <= tol * max(abs(ref.aux_loss), 1e-6)
    assert abs(cache.z_loss() - ref.z_loss) <= tol * max(abs(ref.z_loss), 1e-6)
    if check_rows and ref.perm_slot.size:
        h, y = layer.expert_rows(int(ref.offsets[-1]))
        assert rel_l2(h, ref.hidden) <= tol
        assert rel_l2(y, ref.expert_out) <= tol
    layer.close()
    return out, cache, ref


# ------------------------------------------------------------------ small shapes, every dtype
SMALL = [
    dict(d=8, E=4, k=2, F=6, T=7),
    dict(d=8, E=4, k=1, F=6, T=6),
    dict(d=8, E=6, k=3, F=4, T=9),
    dict(d=6, E=4, k=2, F=5, T=3, shared=True),
    dict(d=4, E=3, k=2, F=4, T=4),
    dict(d=16, E=5, k=5, F=12, T=33),
    dict(d=24, E=16, k=2, F=40, T=100, shared=True, shared_d_ff=56),
    dict(d=64, E=8, k=2, F=32, T=512),
    dict(d=40, E=64, k=6, F=24, T=129, shared=True),
    dict(d=8, E=1, k=1, F=8, T=5),
    dict(d=128, E=200, k=8, F=16, T=70),
    dict(d=33, E=7, k=3, F=19, T=65),
]


@pytest.mark.parametrize("shape", SMALL, ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}".format(**s))
@pytest.mark.parametrize("act,wt", [("f32", "f32"), ("bf16", "bf16"), ("bf16", "int8"), ("f32", "int8")])
def test_small_shapes_match_the_oracle(device, shape, act, wt):
    t = synth.make(small_workload(seed=11, act=act, wt=wt, **shape))
    check_parity(device, t)


def test_padding_rows_are_routed_nowhere_and_left_out_of_the_losses(device):
    # reference device test src/gpu_transformer.rs:1762-1786 (aux on a padded batch)
    t = synth.make(small_workload(d=16, E=4, k=2, F=12, T=40, seed=3, shared=True))
    valid = (np.arange(40) % 4 != 1).astype(np.uint8)
    out, cache, ref = check_parity(device, t, valid=valid)
    assert np.all(cache.expert_of.reshape(40, 2)[valid == 0] == rb.UNROUTED)
    assert not cache.gate_of.reshape(40, 2)[valid == 0].any()
    assert cache.valid_tokens == int(valid.sum())


def test_all_rows_padding(device):
    t = synth.make(small_workload(d=8, E=4, k=2, F=6, T=5, seed=4))
    out, cache, ref = check_parity(device, t, valid=np.zeros(5, np.uint8), check_rows=False)
    assert not out.any() and cache.aux_loss() == 0.0 and cache.z_loss() == 0.0
    assert not cache.counts.any()


def test_zero_tokens(device):
    t = synth.make(small_workload(d=8, E=4, k=2, F=6, T=3, seed=4))
    layer = gpu_layer(device, t)
    out, cache = layer.forward_train(np.zeros((0, 8), np.float32))
    assert out.shape == (0, 8) and cache.aux_loss() == 0.0 and cache.z_loss() == 0.0
    assert cache.counts.tolist() == [0, 0, 0, 0] and cache.offsets.tolist() == [0] * 5
    layer.close()


def test_single_token_uses_the_reference_gemv_order(device):
    # one row: the reference computes the logits with its eight-lane `dot` (src/matrix.rs:131-153)
    t = synth.make(small_workload(d=72, E=8, k=2, F=16, T=1, seed=8))
    check_parity(device, t)


def test_router_bias_and_residual(device):
    t = synth.make(small_workload(d=16, E=8, k=2, F=12, T=64, seed=6, act="bf16", wt="bf16"))
    bias = np.zeros(8, np.float32)
    bias[3] = 2.0
    residual = synth.round_bf16(synth.normal((64, 16), 1.0, 6, 99))
    out, cache, ref = check_parity(device, t, bias=bias, residual=residual)
    assert cache.counts[3] > 40


def test_extreme_logits_keep_probabilities_identical(device):
    # huge logit gaps push exp() into the subnormal range and to zero
    w = small_workload(d=4, E=4, k=2, F=4, T=6, seed=2)
    t = synth.make(w)
    t.router = np.zeros((4, 4), np.float32)
    for e, s in enumerate((1.0, 30.0, 95.0, 200.0)):
        t.router[e, e] = s
    t.x = np.array([[1, 0, 0, 0], [0, 1, 0, 0], [0, 0, 1, 0], [0, 0, 0, 1], [1, 1, 1, 1], [0, 0, 0, 0]], np.float32)
    check_parity(device, t)


def test_exact_ties_go_to_the_lower_expert(device):
    t = synth.make(small_workload(d=8, E=6, k=3, F=4, T=4, seed=2))
    t.router = np.zeros((6, 8), np.float32)  # all logits equal -> experts 0, 1, 2
    out, cache, ref = check_parity(device, t)
    assert cache.expert_of.reshape(4, 3).tolist() == [[0, 1, 2]] * 4
    t.router[4] = t.router[2] = 0.5 * np.ones(8, np.float32)  # two equal winners
    t.x = np.abs(t.x)
    out, cache, ref = check_parity(device, t)
    assert cache.expert_of.reshape(4, 3)[:, :2].tolist() == [[2, 4]] * 4


def test_nan_row_routes_in_index_order(device):
    t = synth.make(small_workload(d=8, E=5, k=2, F=4, T=3, seed=2))
    t.x[1, 0] = np.nan
    ref = oracle_layer(t).forward(t.x)
    layer = gpu_layer(device, t)
    out, cache = layer.forward_train(t.x)
    assert np.array_equal(cache.expert_of, ref.expert_of)
    assert cache.expert_of.reshape(3, 2)[1].tolist() == [0, 1]
    assert np.array_equal(np.isnan(cache.probabilities), np.isnan(ref.probabilities))
    layer.close()


@pytest.mark.parametrize("T,act", [(40, "f32"), (40, "bf16"), (3, "bf16")])   # (3, bf16): the single-workgroup routing
def test_rows_whose_logits_overflow_route_like_the_cpu_path(device, T, act):
    """A row of huge values gives infinite logits: `v - max` is inf - inf = NaN for the winners and -inf for the
    rest, the sum of exponentials is NaN, `sum > 0` is false and the row is left un-normalised
    (src/activations.rs:56-70); no NaN is ever 'greater', so the row routes to experts 0..k-1
    (src/moe.rs:566-581).  A row of zeros beside it is the plain uniform case."""
    d = 16 if act == "f32" else 64
    t = synth.make(small_workload(d=d, E=6, k=2, F=8 if act == "f32" else 64, T=T, seed=4, act=act, wt=act))
    t.x[1, :] = synth.round_bf16(np.float32(3.0e38))
    t.x[2, :] = 0.0
    t.router[0, :] = 2.0                                  # +inf
    t.router[1, :] = -2.0                                 # -inf
    t.router[2, :] = np.where(np.arange(d) % 2, 2.0, -2.0)  # inf - inf = NaN
    t.router[3, :] = 2.0                                  # +inf again
    ref = oracle_layer(t).forward(t.x)
    layer = gpu_layer(device, t)
    out, cache = layer.forward_train(t.x)
    assert np.array_equal(cache.expert_of, ref.expert_of)
    assert np.array_equal(cache.probabilities.view(np.uint32) & 0x7fffffff == 0x7f800000,
                          ref.probabilities.view(np.uint32) & 0x7fffffff == 0x7f800000)
    assert np.array_equal(np.isnan(cache.probabilities), np.isnan(ref.probabilities))
    finite = ~np.isnan(ref.probabilities)
    assert np.array_equal(cache.probabilities[finite], ref.probabilities[finite])
    assert cache.expert_of.reshape(T, 2)[2].tolist() == [0, 1]          # all-equal probabilities: lowest indices
    assert np.array_equal(cache.counts, ref.counts) and np.array_equal(cache.perm_slot, ref.perm_slot)
    assert layer.kernel_name() == {"f32": "generic", "bf16": "mfma_bf16_decode" if T <= 32 else "mfma_bf16_stream"}[act]
    layer.close()


# ------------------------------------------------------------------ the reference's own MoE tests, on the GPU
def one_hot_router(E, d, strength):
    w = np.zeros((E, d), np.float32)
    for e in range(E):
        w[e, e % d] = strength
    return w


def one_hot_rows(rows, width):
    x = np.zeros((len(rows), width), np.float32)
    for r, c in enumerate(rows):
        x[r, c] = 1.0
    return x


def make_layer(device, E, k, F, d, seed, z_w=1e-3, aux_w=0.01, shared=False, T=16):
    t = synth.make(small_workload(d=d, E=E, k=k, F=F, T=T, seed=seed, shared=shared))
    return gpu_layer(device, t, max_tokens=max(T, 16), aux_w=aux_w, z_w=z_w), t


def test_output_keeps_the_model_dimension(device):
    # reference src/moe.rs:696-702
    layer, t = make_layer(device, 4, 2, 6, 8, 1, T=5)
    assert layer.forward(t.x).shape == (5, 8)


@pytest.mark.parametrize("k", [1, 2, 3, 4])
def test_gate_weights_sum_to_one_per_token(device, k):
    # reference src/moe.rs:726-754
    layer, t = make_layer(device, 4, k, 6, 8, 3, T=7)
    _, cache = layer.forward_train(t.x)
    sums = cache.gate_of.reshape(7, k).sum(axis=1)
    assert np.all(np.abs(sums - 1.0) < 1e-5)
    if k == 1:
        assert len(cache.assignments) == 7 and np.all(np.abs(cache.gate_of - 1.0) < 1e-6)


def test_every_token_reaches_exactly_top_k_experts(device):
    # reference src/moe.rs:757-765
    layer, t = make_layer(device, 6, 3, 4, 8, 5, T=9)
    _, cache = layer.forward_train(t.x)
    assert sum(len(v) for v in cache.expert_tokens) == 9 * 3


def test_balanced_and_collapsed_routing_losses(device):
    # reference src/moe.rs:768-802
    layer, _ = make_layer(device, 4, 1, 4, 4, 6, z_w=0.0)
    layer.set_router(one_hot_router(4, 4, 30.0))
    _, cache = layer.forward_train(one_hot_rows([0, 1, 2, 3], 4))
    assert abs(cache.aux_loss() - 0.01) < 1e-3
    assert all(abs(f - 0.25) < 1e-6 for f in cache.load_fractions())
    _, cache = layer.forward_train(one_hot_rows([0, 0, 0, 0], 4))
    assert abs(cache.aux_loss() - 0.04) < 1e-3 and cache.aux_loss() > 0.01
    assert cache.load_fractions() == [1.0, 0.0, 0.0, 0.0]


def test_z_loss_grows_with_the_logits_and_a_disabled_z_loss_is_zero(device):
    # reference src/moe.rs:805-836
    x = one_hot_rows([0, 1, 2, 3], 4)
    layer, _ = make_layer(device, 4, 1, 4, 4, 7)
    layer.set_router(one_hot_router(4, 4, 1.0))
    quiet = layer.forward_train(x)[1].z_loss()
    layer.set_router(one_hot_router(4, 4, 20.0))
    loud = layer.forward_train(x)[1].z_loss()
    assert loud > quiet > 0.0
    layer, t = make_layer(device, 4, 2, 6, 8, 8, z_w=0.0, T=4)
    _, cache = layer.forward_train(t.x)
    assert cache.z_loss() == 0.0 and cache.auxiliary_loss() == cache.aux_loss()


def test_the_shared_expert_contributes_to_every_token(device):
    # reference src/moe.rs:839-859
    plain, t = make_layer(device, 4, 1, 6, 8, 9, T=4)
    shared, ts = make_layer(device, 4, 1, 6, 8, 9, shared=True, T=4)
    a, b = plain.forward(t.x), shared.forward(ts.x)
    assert np.all(np.any(np.abs(a - b) > 1e-6, axis=1))


def test_identical_tokens_collapse_onto_two_experts(device):
    # reference tutorials/15_mixture_of_experts.md:296-312
    layer, _ = make_layer(device, 8, 2, 32, 64, 7, T=512)
    x = np.repeat(synth.uniform((1, 64), 1.0, 7, 5), 512, axis=0)
    _, cache = layer.forward_train(x)
    assert sorted(cache.load_fractions()) == [0.0] * 6 + [0.5, 0.5]


def test_wrong_width_is_invalid_input_and_too_many_tokens_are_refused(device):
    # reference src/moe.rs:248-253
    layer, t = make_layer(device, 4, 2, 6, 8, 1, T=5)
    with pytest.raises(rb.InvalidInput) as info:
        layer.forward(np.zeros((3, 5), np.float32))
    assert (info.value.expected, info.value.actual) == (8, 5)
    with pytest.raises(rb.InvalidInput):
        layer.forward(np.zeros((layer.max_tokens + 1, 8), np.float32))
    with pytest.raises(rb.InvalidInput):
        layer.set_expert(0, np.zeros((3, 3), np.float32), np.zeros((6, 8), np.float32), np.zeros((8, 6), np.float32))


def test_memory_budget_refuses_before_allocating():
    # reference src/param.rs:172-189, src/gpu_transformer.rs:2050-2066
    dev = rb.Device.open(0, budget_mib=1)
    with pytest.raises(rb.MemoryBudget, match="exceeds budget 1 MiB"):
        rb.MoeLayer(768, rb.MoeConfig.new(8, 2, 1408), dev, max_tokens=1024)
    dev.close()


def test_forward_is_reproducible_bit_for_bit(device):
    t = synth.make(small_workload(d=64, E=8, k=2, F=48, T=300, seed=12, act="bf16", wt="bf16", shared=True))
    layer = gpu_layer(device, t)
    a, ca = layer.forward_train(t.x)
    b, cb = layer.forward_train(t.x)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert ca.aux_loss() == cb.aux_loss() and ca.z_loss() == cb.z_loss()


def test_builder_surface_builds_the_sparse_layers(device):
    layers = (rb.TransformerBuilder().d_model(16).n_layers(4).experts(4, 2).moe_layers([1, 3]).moe_d_ff(12)
              .shared_expert(True).build_moe_layers(device, max_tokens=8))
    assert sorted(layers) == [1, 3]
    assert layers[1].num_parameters() == 4 * 16 + 5 * 3 * 16 * 12
    assert layers[1].active_parameters() == 4 * 16 + 3 * 3 * 16 * 12


def test_many_router_blocks_take_the_separate_layout_scan(device):
    # 66 router blocks x 64 experts is past the size up to which the layout scan rides in the dispatch launch
    t = synth.make(small_workload(d=16, E=64, k=3, F=8, T=2100, seed=17))
    valid = (np.arange(2100) % 13 != 5).astype(np.uint8)
    out, cache, ref = check_parity(device, t, valid=valid)
    assert int(cache.offsets[-1]) == int(valid.sum()) * 3


@pytest.mark.parametrize("T", [8, 200, 512, 600])
@pytest.mark.parametrize("act", ["f32", "bf16"])
def test_the_largest_expert_count_keeps_both_losses(device, T, act):
    # 256 experts is the routing kernels' limit and the workgroup size of the fused dispatch launch, where no
    # thread is numbered E: the z-loss (the sum of lse^2 folded by one thread) must still come out.  With bf16
    # rows T = 8 takes the single-workgroup routing; 200 and 512 take the fused dispatch launch, 600 the
    # separate layout scan.
    t = synth.make(small_workload(d=64, E=256, k=3, F=64, T=T, seed=23, act=act, wt=act))
    ref = oracle_layer(t, z_w=0.7).forward(t.x, threads=8)
    layer = gpu_layer(device, t, z_w=0.7)
    out, cache = layer.forward_train(t.x)
    assert_routing_identical(cache, ref)
    assert ref.z_loss > 1e-3
    assert abs(cache.z_loss() - ref.z_loss) <= 1e-5 * abs(ref.z_loss)
    assert abs(cache.aux_loss() - ref.aux_loss) <= 1e-5 * max(abs(ref.aux_loss), 1e-6)
    assert rel_l2(out, ref.out) <= tolerance(t.workload)
    if act == "bf16":
        assert layer.kernel_name() == ("mfma_bf16_decode" if T <= 32 else "mfma_bf16_stream")
    layer.close()
