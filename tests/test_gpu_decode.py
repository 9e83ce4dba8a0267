"""The decode-shaped path (at most 32 tokens, packed bf16 / int8 weights): one routing workgroup and two
weight-streaming launches, against the oracle and against the large-batch path of the same library."""
import os

import numpy as np
import pytest

import rustingbrain_amd as rb
from conftest import rel_l2
from helpers import assert_routing_identical, gpu_layer, oracle_layer, small_workload
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture
def env():
    keys = ("RBMOE_NO_DECODE_PATH", "RBMOE_NO_DECODE_FRONT", "RBMOE_NO_DECODE_COMBINE_FOLD", "RBMOE_NO_DECODE_DOWN_BY_EXPERT")
    saved = {k: os.environ.get(k) for k in keys}
    yield os.environ
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v


def run(device, t, valid=None, bias=None, residual=None):
    ref = oracle_layer(t).forward(t.x, valid=valid, router_bias=bias, threads=4)
    layer = gpu_layer(device, t)
    layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
    out, cache = layer.forward_train(t.x, layout, router_bias=bias, residual=residual)
    name = layer.kernel_name()
    assert_routing_identical(cache, ref)
    R = int(ref.offsets[-1])
    if R:
        h, y = layer.expert_rows(R)
        assert rel_l2(h, ref.hidden) <= 2e-2, "hidden rows"
        assert rel_l2(y, ref.expert_out) <= 2e-2, "expert output rows"
    want = ref.out if residual is None else ref.out + residual
    assert rel_l2(out, want) <= 2e-2
    assert abs(cache.aux_loss() - ref.aux_loss) <= 1e-6 + 1e-5 * abs(ref.aux_loss)
    assert abs(cache.z_loss() - ref.z_loss) <= 1e-6 + 1e-5 * abs(ref.z_loss)
    layer.close()
    return name, out, cache


# widths are multiples of 64: the packed-weight kernels need that in both directions
SHAPES = [dict(d=64, E=4, k=1, F=64, T=1), dict(d=128, E=8, k=2, F=128, T=8), dict(d=192, E=6, k=3, F=192, T=7),
          dict(d=256, E=64, k=6, F=64, T=32), dict(d=128, E=5, k=2, F=320, T=19),
          dict(d=64, E=24, k=5, F=64, T=20),     # a wave per token, 40 lanes idle
          dict(d=64, E=16, k=16, F=64, T=9),     # every expert selected, 16 lanes per token
          dict(d=64, E=100, k=4, F=64, T=16)]    # more experts than lanes: one thread per token


@pytest.mark.parametrize("wt", ["bf16", "int8"])
@pytest.mark.parametrize("shared", [False, True])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}".format(**s))
def test_decode_path_matches_the_oracle(device, env, shape, shared, wt):
    env.pop("RBMOE_NO_DECODE_PATH", None)
    t = synth.make(small_workload(seed=23, act="bf16", wt=wt, shared=shared, shared_d_ff=shape["F"] + 64, **shape))
    name, _, _ = run(device, t)
    assert name.startswith("mfma_bf16_decode"), name


def test_decode_path_with_padding_bias_and_residual(device, env):
    env.pop("RBMOE_NO_DECODE_PATH", None)
    shape = dict(d=128, E=8, k=2, F=128, T=13)
    t = synth.make(small_workload(seed=29, act="bf16", wt="bf16", shared=True, **shape))
    valid = (np.arange(13) % 4 != 1).astype(np.uint8)
    bias = np.zeros(8, np.float32)
    bias[5] = 3.0  # nearly every token takes expert 5 first
    residual = synth.round_bf16(synth.normal((13, 128), 1.0, 7, 5))
    name, out, cache = run(device, t, valid=valid, bias=bias, residual=residual)
    assert name.startswith("mfma_bf16_decode")
    assert cache.counts[5] >= 8
    assert (cache.expert_of.reshape(13, 2)[valid == 0] == -1).all()


def test_decode_path_all_tokens_on_one_expert_fill_one_tile(device, env):
    env.pop("RBMOE_NO_DECODE_PATH", None)
    t = synth.make(small_workload(seed=31, act="bf16", wt="bf16", d=64, E=4, k=1, F=64, T=32))
    bias = np.array([0, 50, 0, 0], np.float32)
    name, out, cache = run(device, t, bias=bias)
    assert name.startswith("mfma_bf16_decode")
    assert cache.counts.tolist() == [0, 32, 0, 0]


def test_decode_path_ties_and_nan_rows(device, env):
    env.pop("RBMOE_NO_DECODE_PATH", None)
    t = synth.make(small_workload(seed=2, act="bf16", wt="bf16", d=64, E=6, k=3, F=64, T=4))
    t.router = np.zeros((6, 64), np.float32)  # all logits equal -> experts 0, 1, 2
    name, out, cache = run(device, t)
    assert name.startswith("mfma_bf16_decode")
    assert cache.expert_of.reshape(4, 3).tolist() == [[0, 1, 2]] * 4
    t = synth.make(small_workload(seed=2, act="bf16", wt="bf16", d=64, E=5, k=2, F=64, T=3))
    t.x[1, 0] = np.nan
    ref = oracle_layer(t).forward(t.x)
    layer = gpu_layer(device, t)
    out, cache = layer.forward_train(t.x)
    assert layer.kernel_name().startswith("mfma_bf16_decode")
    assert np.array_equal(cache.expert_of, ref.expert_of)
    assert cache.expert_of.reshape(3, 2)[1].tolist() == [0, 1]
    assert np.array_equal(np.isnan(cache.probabilities), np.isnan(ref.probabilities))
    layer.close()


def test_decode_and_large_batch_paths_agree(device, env):
    shape = dict(d=128, E=8, k=2, F=192, T=24)
    t = synth.make(small_workload(seed=37, act="bf16", wt="bf16", shared=True, **shape))
    env.pop("RBMOE_NO_DECODE_PATH", None)
    small = gpu_layer(device, t)
    out_s, cache_s = small.forward_train(t.x)
    assert small.kernel_name() == "mfma_bf16_decode_front"   # 48 slots on 8 experts: routing beside the gate/up products
    env["RBMOE_NO_DECODE_PATH"] = "1"
    large = gpu_layer(device, t)
    out_l, cache_l = large.forward_train(t.x)
    assert large.kernel_name() == "mfma_bf16_stream"
    for f in ("expert_of", "counts", "offsets", "perm_slot", "perm_token"):
        assert np.array_equal(getattr(cache_s, f), getattr(cache_l, f)), f
    assert np.array_equal(cache_s.probabilities.view(np.uint32), cache_l.probabilities.view(np.uint32))
    assert np.array_equal(cache_s.gate_of.view(np.uint32), cache_l.gate_of.view(np.uint32))
    assert rel_l2(out_s, out_l) <= 5e-3
    small.close()
    large.close()


@pytest.mark.parametrize("wt", ["bf16", "int8"])
def test_routing_beside_the_products_changes_nothing_but_the_launch_count(device, env, wt):
    # When most experts are about to be touched (tokens * k >= 2 E) the routing workgroup runs in the same launch as
    # the gate/up products, which are then taken for every expert over every row; the routing tables are the same
    # bits, the routed hidden rows and outputs the same within the reduction order of the products (8 waves
    # split the reduction there, 4 in the product launch of its own).
    shape = dict(d=256, E=8, k=2, F=192, T=11)
    t = synth.make(small_workload(seed=41, act="bf16", wt=wt, shared=True, shared_d_ff=128, **shape))
    valid = (np.arange(11) % 5 != 3).astype(np.uint8)
    bias = synth.normal((8,), 0.5, 41, 98)
    env.pop("RBMOE_NO_DECODE_PATH", None)
    env.pop("RBMOE_NO_DECODE_FRONT", None)
    name_f, out_f, cache_f = run(device, t, valid=valid, bias=bias)
    assert name_f.startswith("mfma_bf16_decode_front")
    env["RBMOE_NO_DECODE_FRONT"] = "1"
    name_p, out_p, cache_p = run(device, t, valid=valid, bias=bias)
    assert name_p.startswith("mfma_bf16_decode") and "front" not in name_p
    for f in ("expert_of", "counts", "offsets", "perm_slot", "perm_token"):
        assert np.array_equal(getattr(cache_f, f), getattr(cache_p, f)), f
    assert np.array_equal(cache_f.probabilities.view(np.uint32), cache_p.probabilities.view(np.uint32))
    assert np.array_equal(cache_f.gate_of.view(np.uint32), cache_p.gate_of.view(np.uint32))
    assert cache_f.aux_loss() == cache_p.aux_loss() and cache_f.z_loss() == cache_p.z_loss()
    assert rel_l2(out_f, out_p) <= 5e-3
    # few slots on many experts: the launches stay apart (an unrouted expert's weights would be fetched for nothing)
    t = synth.make(small_workload(seed=41, act="bf16", wt=wt, d=64, E=16, k=2, F=64, T=4))
    env.pop("RBMOE_NO_DECODE_FRONT", None)
    name, _, _ = run(device, t)
    assert name.startswith("mfma_bf16_decode") and "front" not in name


@pytest.mark.parametrize("case", [
    dict(act="bf16", wt="bf16", shared=True, T=13, k=2, pad="some", residual=True),
    dict(act="bf16", wt="int8", shared=False, T=32, k=3, pad="none", residual=False),
    dict(act="bf16", wt="bf16", shared=False, T=6, k=2, pad="all", residual=True),    # no workgroup writes a row
    dict(act="bf16", wt="bf16", shared=True, T=6, k=2, pad="all", residual=False),    # only the shared expert does
    dict(act="f32", wt="bf16", shared=True, T=9, k=4, pad="some", residual=True),     # f32 rows over bf16 weights
], ids=lambda c: "{act}_{wt}_T{T}_k{k}_pad-{pad}".format(**c))
def test_the_combine_inside_the_down_launch_gives_the_bits_of_the_combine_launch(device, env, case):
    """The last workgroup of a column block to finish sums the block: same order and roundings as the combine
    kernel, so the outputs agree in every bit - twice in a row (the arrival counters must be back at zero), with
    padding rows, with nothing routed at all, with a residual, with f32 rows."""
    T, k = case["T"], case["k"]
    t = synth.make(small_workload(d=128, E=8, k=k, F=192, T=T, seed=83, act=case["act"], wt=case["wt"],
                                  shared=case["shared"], shared_d_ff=128))
    valid = {"none": None, "some": (np.arange(T) % 3 != 1).astype(np.uint8), "all": np.zeros(T, np.uint8)}[case["pad"]]
    residual = synth.round_bf16(synth.normal((T, 128), 1.0, 83, 7)) if case["residual"] else None
    layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
    outs = {}
    for fold in (True, False):
        if fold:
            env.pop("RBMOE_NO_DECODE_COMBINE_FOLD", None)
        else:
            env["RBMOE_NO_DECODE_COMBINE_FOLD"] = "1"
        layer = gpu_layer(device, t)
        a, _ = layer.forward_train(t.x, layout, residual=residual)
        b, _ = layer.forward_train(t.x, layout, residual=residual)
        assert layer.kernel_name().startswith("mfma_bf16_decode")
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        outs[fold] = a
        layer.close()
    assert np.array_equal(outs[True].view(np.uint32), outs[False].view(np.uint32))
    ref = oracle_layer(t).forward(t.x, valid=valid, threads=4)
    want = ref.out if residual is None else ref.out + residual
    assert rel_l2(outs[True], want) <= 2e-2 if np.any(want) else not np.any(outs[True])


BY_EXPERT_CASES = [
    dict(act="bf16", wt="bf16", shared=True, d=256, E=8, k=2, F=192, T=11, pad="some", bias=True, residual=True),
    dict(act="bf16", wt="int8", shared=False, d=128, E=8, k=3, F=192, T=21, pad="none", bias=False, residual=False),
    dict(act="bf16", wt="bf16", shared=False, d=768, E=8, k=2, F=1408, T=8, pad="none", bias=False, residual=False),  # the decode workload of the benchmark
    dict(act="bf16", wt="bf16", shared=False, d=128, E=8, k=4, F=64, T=32, pad="none", bias=False, residual=True),   # 128 slots, full tiles
    dict(act="bf16", wt="bf16", shared=False, d=128, E=4, k=2, F=192, T=6, pad="all", bias=False, residual=True),   # no workgroup writes a row
    dict(act="bf16", wt="bf16", shared=True, d=128, E=4, k=2, F=192, T=6, pad="all", bias=False, residual=False),   # only the shared expert does
    dict(act="bf16", wt="bf16", shared=True, d=64, E=2, k=1, F=64, T=5, pad="some", bias=True, residual=False,
         shared_d_ff=192),                                                                                         # a shared expert wider than the routed ones
    dict(act="bf16", wt="bf16", shared=False, d=64, E=16, k=4, F=64, T=8, pad="none", bias=True, residual=False,
         lopsided=True),                                                                                           # most experts without a row
]


@pytest.mark.parametrize("case", BY_EXPERT_CASES,
                         ids=lambda c: "{wt}_d{d}_E{E}_k{k}_F{F}_T{T}_pad-{pad}".format(**c))
def test_down_launch_by_expert_gives_the_bits_of_the_tile_table_launch(device, env, case):
    """Behind the launch that routes beside the gate/up products, the down launch has one row of workgroups per
    expert (weights requested at once, the expert's rows read off its token bits behind them, the combine's
    positions and gates fetched early): routing tables, losses and outputs are those of the launch that walks the
    tile table, in every bit - three calls in a row, the last one with fewer tokens."""
    T, k, E, d = case["T"], case["k"], case["E"], case["d"]
    t = synth.make(small_workload(d=d, E=E, k=k, F=case["F"], T=T, seed=59, act=case["act"], wt=case["wt"],
                                  shared=case["shared"], shared_d_ff=case.get("shared_d_ff", 128)))
    valid = {"none": None, "some": (np.arange(T) % 4 != 2).astype(np.uint8), "all": np.zeros(T, np.uint8)}[case["pad"]]
    bias = synth.normal((E,), 0.5, 59, 98) if case["bias"] else None
    if case.get("lopsided"):
        bias = np.where(np.arange(E) < 5, 30.0, -30.0).astype(np.float32)
    residual = synth.round_bf16(synth.normal((T, d), 1.0, 59, 7)) if case["residual"] else None
    layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
    T2 = max(1, T // 2)
    while T2 * k < 2 * E and T2 < T:   # the shorter call takes the same kernels
        T2 += 1
    layout2 = rb.Layout(valid=None if valid is None else [bool(v) for v in valid[:T2]])
    got = {}
    for by_expert in (True, False):
        if by_expert:
            env.pop("RBMOE_NO_DECODE_DOWN_BY_EXPERT", None)
        else:
            env["RBMOE_NO_DECODE_DOWN_BY_EXPERT"] = "1"
        layer = gpu_layer(device, t)
        a, ca = layer.forward_train(t.x, layout, router_bias=bias, residual=residual)
        assert layer.kernel_name().startswith("mfma_bf16_decode_front")
        b, _ = layer.forward_train(t.x, layout, router_bias=bias, residual=residual)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        c, cc = layer.forward_train(t.x[:T2], layout2, router_bias=bias, residual=None if residual is None else residual[:T2])
        got[by_expert] = (a, ca, c, cc)
        layer.close()
    for i in (0, 2):
        assert np.array_equal(got[True][i].view(np.uint32), got[False][i].view(np.uint32)), "outputs"
    for i in (1, 3):
        cw, cp = got[True][i], got[False][i]
        for f in ("expert_of", "counts", "offsets", "perm_slot", "perm_token"):
            assert np.array_equal(getattr(cw, f), getattr(cp, f)), f
        assert np.array_equal(cw.gate_of.view(np.uint32), cp.gate_of.view(np.uint32))
        assert cw.aux_loss() == cp.aux_loss() and cw.z_loss() == cp.z_loss()
    ref = oracle_layer(t).forward(t.x, valid=valid, router_bias=bias, threads=4)
    assert_routing_identical(got[True][1], ref)
    if case.get("lopsided"):
        assert int((ref.counts > 0).sum()) <= 5
    want = ref.out if residual is None else ref.out + residual
    assert rel_l2(got[True][0], want) <= 2e-2 if np.any(want) else not np.any(got[True][0])
