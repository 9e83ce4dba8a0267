"""The bf16 matrix-core path of the grouped expert products against the oracle,
ragged groups, partial tiles in both directions, padding rows, empty experts, a shared expert of another
width, int8 weights, and the explicit-gather variant."""
import os

import numpy as np
import pytest

import rustingbrain_amd as rb
from conftest import rel_l2
from helpers import assert_routing_identical, gpu_layer, oracle_layer, small_workload
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu



@pytest.fixture
def kernel_env():
    keys = ("RBMOE_GROUP_M", "RBMOE_EXPLICIT_GATHER", "RBMOE_FORCE_GENERIC")
    saved = {k: os.environ.get(k) for k in keys}
    yield os.environ
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v


def run(device, t, valid=None, bias=None):
    ref = oracle_layer(t).forward(t.x, valid=valid, router_bias=bias, threads=8)
    layer = gpu_layer(device, t)
    assert layer.kernel_name().startswith("mfma") or layer.kernel_name() == "none"
    layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
    out, cache = layer.forward_train(t.x, layout, router_bias=bias)
    assert layer.kernel_name().startswith("mfma")
    assert_routing_identical(cache, ref)
    h, y = layer.expert_rows(int(ref.offsets[-1]))
    assert rel_l2(h, ref.hidden) <= 2e-2, "hidden rows"
    assert rel_l2(y, ref.expert_out) <= 2e-2, "expert output rows"
    err = rel_l2(out, ref.out)
    assert err <= 2e-2, err
    name = layer.kernel_name()
    layer.close()
    return name


@pytest.mark.parametrize("wt", ["bf16", "int8"])
@pytest.mark.parametrize("shape", [dict(d=128, E=6, k=2, F=192, T=700), dict(d=64, E=3, k=1, F=64, T=130),
                                   dict(d=256, E=16, k=4, F=128, T=333), dict(d=192, E=5, k=2, F=320, T=1000)],
                         ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}".format(**s))
def test_matrix_core_kernels(device, kernel_env, shape, wt):
    E = shape["E"]
    t = synth.make(small_workload(seed=19, act="bf16", wt=wt, shared=True, shared_d_ff=shape["F"] + 64, **shape))
    bias = np.zeros(E, np.float32)
    bias[1] = 1.5
    bias[E - 1] = -50
    T = shape["T"]
    valid = (np.arange(T) % 9 != 4).astype(np.uint8)
    layer_name = run(device, t, valid=valid, bias=bias)


@pytest.mark.parametrize("group_m", [1, 3, 8])
def test_scheduling_group_size_does_not_change_results(device, kernel_env, group_m):
    kernel_env["RBMOE_GROUP_M"] = str(group_m)
    t = synth.make(small_workload(d=64, E=8, k=2, F=128, T=1500, seed=23, act="bf16", wt="bf16"))
    run(device, t)


def test_explicit_gather_gives_the_same_bits_as_gathering_in_the_product(device, kernel_env):
    t = synth.make(small_workload(d=128, E=8, k=3, F=256, T=900, seed=29, act="bf16", wt="bf16"))
    layer = gpu_layer(device, t)
    a, _ = layer.forward_train(t.x)
    layer.close()
    kernel_env["RBMOE_EXPLICIT_GATHER"] = "1"
    layer = gpu_layer(device, t)
    b, _ = layer.forward_train(t.x)
    layer.close()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_matrix_core_and_generic_paths_agree(device, kernel_env):
    t = synth.make(small_workload(d=64, E=4, k=2, F=64, T=257, seed=31, act="bf16", wt="bf16", shared=True))
    layer = gpu_layer(device, t)
    a, _ = layer.forward_train(t.x)
    assert layer.kernel_name() == "mfma_bf16_stream"
    layer.close()
    kernel_env["RBMOE_FORCE_GENERIC"] = "1"
    layer = gpu_layer(device, t)
    b, _ = layer.forward_train(t.x)
    assert layer.kernel_name() == "generic"
    layer.close()
    assert rel_l2(a, b) < 1e-2


@pytest.mark.parametrize("T", [1, 8, 33, 127, 128, 129])
def test_small_token_counts(device, T):
    t = synth.make(small_workload(d=64, E=8, k=2, F=64, T=T, seed=37, act="bf16", wt="bf16", shared=True))
    run(device, t)


@pytest.mark.parametrize("wt", ["bf16", "int8"])
@pytest.mark.parametrize("T", [8, 700])
def test_f32_rows_with_bf16_or_int8_weights_run_on_the_matrix_cores(device, wt, T):
    # What a caller with f32 matrices and a bf16 or quantized checkpoint has (Matrix is f32, src/matrix.rs:13-18;
    # after TransformerLm::quantize() the Linear layers take the Quantized branch on f32 inputs,
    # src/param.rs:778-780, src/quantized.rs:55-99).  The router reads the f32 rows (identical routing), the expert
    # products read their bf16 copy: the same 2e-2 bar as bf16 rows.  T = 8: the decode-shaped kernels.
    t = synth.make(small_workload(d=768, E=8, k=2, F=1408, T=T, seed=29, act="f32", wt=wt, shared=True,
                                  shared_d_ff=704))
    name = run(device, t)
    assert name == ("mfma_bf16_decode" if T <= 32 else "mfma_bf16_stream") + ("_int8w" if wt == "int8" else "")
    valid = (np.arange(T) % 5 != 2).astype(np.uint8)
    bias = synth.normal((8,), 0.5, 29, 98)
    run(device, t, valid=valid, bias=bias)


def test_f32_rows_block_step_on_the_matrix_cores(device):
    # norm in front, residual behind, f32 on the boundary, int8 experts on the matrix cores, both kernel sets
    from helpers import small_workload as sw
    from oracle import rb_oracle as orc
    for T in (5, 300):
        t = synth.make(sw(d=128, E=8, k=2, F=192, T=T, seed=31, act="f32", wt="int8", shared=True, shared_d_ff=64))
        layer = gpu_layer(device, t)
        w = (1.0 + 0.1 * synth.normal((128,), 1.0, 31, 97)).astype(np.float32)
        layer.set_feed_forward_norm(w, 1e-6)
        out, cache = layer.forward_block(t.x)
        assert layer.kernel_name().startswith("mfma_bf16")
        normed = orc.rmsnorm(t.x, w, 1e-6)
        ref = oracle_layer(t).forward(normed, threads=4)
        assert_routing_identical(cache, ref)
        assert rel_l2(out, ref.out + t.x) <= 2e-2
        layer.close()


def test_shared_expert_beside_the_routing_gives_the_bits_of_one_stream(device):
    """From 1024 tokens on the shared expert's two products run on the context's second stream, beside the routing
    kernels.  Same kernels, same operands: the output must not differ in a single bit from the one-stream order,
    and both stay within the bar of the oracle."""
    from rustingbrain_amd import _lib as L
    t = synth.make(small_workload(d=128, E=8, k=2, F=192, T=1500, seed=43, act="bf16", wt="bf16", shared=True,
                                  shared_d_ff=256))
    ref = oracle_layer(t).forward(t.x, threads=8)
    outs = []
    for side in (1, 0):
        layer = gpu_layer(device, t)
        layer.set_option(L.OPT_SIDE_STREAM, side)
        for _ in range(3):   # repeated: a missing join would show as a stale row sooner or later
            out, cache = layer.forward_train(t.x)
        assert_routing_identical(cache, ref)
        assert rel_l2(out, ref.out) <= 2e-2
        outs.append(out)
        layer.close()
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
