"""The f32 matrix-core path of the grouped expert products (all-f32 layers) against the oracle at the
1e-5 bar: ragged groups, partial feature tiles, shared expert of another width, padding rows; and
agreement with the generic kernels."""
import os

import numpy as np
import pytest

import rustingbrain_amd as rb
from conftest import rel_l2
from helpers import assert_routing_identical, gpu_layer, oracle_layer, small_workload
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu

# widths are multiples of 32 (the reduction slice); 96 and 224 leave a partial tile of 64 features
SHAPES = [dict(d=32, E=4, k=2, F=64, T=70), dict(d=64, E=3, k=1, F=64, T=130), dict(d=128, E=16, k=4, F=96, T=333),
          dict(d=96, E=5, k=2, F=224, T=257), dict(d=512, E=8, k=2, F=1408, T=96)]


@pytest.mark.parametrize("shared", [False, True])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "d{d}_E{E}_k{k}_F{F}_T{T}".format(**s))
def test_f32_matrix_core_path(device, shape, shared):
    t = synth.make(small_workload(seed=41, act="f32", wt="f32", shared=shared, shared_d_ff=shape["F"] + 32, **shape))
    T, E = shape["T"], shape["E"]
    valid = (np.arange(T) % 11 != 3).astype(np.uint8)
    bias = np.zeros(E, np.float32)
    bias[E - 1] = -50  # an expert nobody picks
    ref = oracle_layer(t).forward(t.x, valid=valid, router_bias=bias, threads=8)
    layer = gpu_layer(device, t)
    out, cache = layer.forward_train(t.x, rb.Layout(valid=[bool(v) for v in valid]), router_bias=bias)
    assert layer.kernel_name() == "mfma_f32"
    assert_routing_identical(cache, ref)
    h, y = layer.expert_rows(int(ref.offsets[-1]))
    assert rel_l2(h, ref.hidden) <= 1e-5, "hidden rows"
    assert rel_l2(y, ref.expert_out) <= 1e-5, "expert output rows"
    assert rel_l2(out, ref.out) <= 1e-5
    layer.close()


def test_f32_matrix_core_and_generic_kernels_agree(device):
    saved = os.environ.get("RBMOE_FORCE_GENERIC")
    try:
        t = synth.make(small_workload(seed=43, act="f32", wt="f32", d=64, E=6, k=2, F=96, T=200, shared=True))
        os.environ.pop("RBMOE_FORCE_GENERIC", None)
        a = gpu_layer(device, t)
        out_a, cache_a = a.forward_train(t.x)
        assert a.kernel_name() == "mfma_f32"
        os.environ["RBMOE_FORCE_GENERIC"] = "1"
        b = gpu_layer(device, t)
        out_b, cache_b = b.forward_train(t.x)
        assert b.kernel_name() == "generic"
        assert np.array_equal(cache_a.perm_slot, cache_b.perm_slot)
        assert rel_l2(out_a, out_b) <= 2e-6
        a.close()
        b.close()
    finally:
        if saved is None:
            os.environ.pop("RBMOE_FORCE_GENERIC", None)
        else:
            os.environ["RBMOE_FORCE_GENERIC"] = saved
