"""rbmoe_forward_static: the decode-shaped forward with every intermediate buffer in the library's static device
array, for callers that cannot allocate.  Through the C ABI it must give the same bits as rbmoe_forward (the same
kernels run, only the buffers lie elsewhere), stay within the layer's tolerance of the CPU oracle, keep doing so
on a second call with a smaller input (the array keeps the first call's contents), and refuse what it cannot
take with a clear error."""
import ctypes as C

import numpy as np
import pytest

import rustingbrain_amd as rb
from bench import DeviceBuffer
from conftest import rel_l2
from helpers import assert_routing_identical, gpu_layer, oracle_layer, small_workload
from rustingbrain_amd import _lib as L
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu


def run_both(device, layer, t, rows, valid=None, bias=None, residual=None):
    """One call of each entry point on the same device buffers; returns (out, cache) of both."""
    x = synth.f32_to_bf16_bits(t.x[:rows])
    xb = DeviceBuffer(device, x.nbytes).upload(x)
    ob = DeviceBuffer(device, x.nbytes)
    vb = DeviceBuffer(device, rows).upload(valid.astype(np.uint8)) if valid is not None else None
    bb = DeviceBuffer(device, 4 * len(bias)).upload(bias.astype(np.float32)) if bias is not None else None
    rb_ = DeviceBuffer(device, x.nbytes).upload(synth.f32_to_bf16_bits(residual)) if residual is not None else None
    got = []
    for fn in (layer.forward_device, layer.forward_static_device):
        ob.upload(np.zeros_like(x))
        fn(xb.ptr, rows, ob.ptr, valid_ptr=vb.ptr if vb else 0, bias_ptr=bb.ptr if bb else 0,
           residual_ptr=rb_.ptr if rb_ else 0)
        device.synchronize()
        out = ob.download(np.empty_like(x)).copy()
        cache = layer.cache(rows, int(valid.sum()) if valid is not None else None)
        routed = int(cache.offsets[-1])
        h, y = layer.expert_rows(routed)
        got.append((out, cache, h.copy(), y.copy()))
    for b in (xb, ob, vb, bb, rb_):
        if b:
            b.free()
    return got


def same(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


@pytest.mark.parametrize("wt", ["bf16", "int8"])
def test_static_forward_matches_the_allocating_one_twice_in_a_row(device, wt):
    t = synth.make(small_workload(d=128, E=8, k=2, F=192, T=24, seed=71, act="bf16", wt=wt, shared=True,
                                  shared_d_ff=64))
    layer = gpu_layer(device, t)
    ref_layer = oracle_layer(t)
    bias = synth.normal((8,), 0.5, 71, 98)
    residual = synth.round_bf16(synth.normal((24, 128), 1.0, 71, 99))
    # the first call fills the static array; the second, smaller one must not see anything of it
    for rows, valid in ((24, None), (5, np.array([1, 0, 1, 1, 1], np.uint8))):
        (out_a, cache_a, h_a, y_a), (out_s, cache_s, h_s, y_s) = run_both(device, layer, t, rows, valid=valid,
                                                                          bias=bias, residual=residual[:rows])
        assert layer.kernel_name().startswith("mfma_bf16_decode")
        assert same(out_s, out_a), f"{rows} rows: outputs differ between the two entry points"
        for name in ("expert_of", "gate_of", "counts", "offsets", "perm_slot", "perm_token", "probabilities",
                     "log_sum_exp"):
            assert same(getattr(cache_s, name), getattr(cache_a, name)), f"{rows} rows: {name}"
        assert cache_s.aux_loss() == cache_a.aux_loss() and cache_s.z_loss() == cache_a.z_loss()
        assert same(h_s, h_a) and same(y_s, y_a)
        ref = ref_layer.forward(t.x[:rows], valid=valid, router_bias=bias, threads=4)
        assert_routing_identical(cache_s, ref)
        want = ref.out + residual[:rows]
        assert rel_l2(synth.bf16_bits_to_f32(out_s).reshape(rows, 128), want) <= 2e-2
        assert abs(cache_s.aux_loss() - ref.aux_loss) <= 2e-2 * max(abs(ref.aux_loss), 1e-6)
        assert abs(cache_s.z_loss() - ref.z_loss) <= 2e-2 * max(abs(ref.z_loss), 1e-6)
    layer.close()


def test_static_forward_over_f32_rows_keeps_their_bf16_copy_in_the_static_array_too(device):
    """f32 rows over bf16 weights: the bf16 copy of the rows that the products read is one more buffer of the
    call and lies in the static array like the others; same bits as the allocating entry point, twice in a row."""
    t = synth.make(small_workload(d=128, E=8, k=2, F=192, T=24, seed=73, act="f32", wt="bf16", shared=True,
                                  shared_d_ff=64))
    layer = gpu_layer(device, t)
    ref_layer = oracle_layer(t)
    for rows in (24, 7):
        x = np.ascontiguousarray(t.x[:rows], dtype=np.float32)
        xb, ob = DeviceBuffer(device, x.nbytes).upload(x), DeviceBuffer(device, x.nbytes)
        got = []
        for fn in (layer.forward_device, layer.forward_static_device):
            ob.upload(np.zeros_like(x))
            fn(xb.ptr, rows, ob.ptr)
            device.synchronize()
            got.append((ob.download(np.empty_like(x)).copy(), layer.cache(rows)))
        assert layer.kernel_name().startswith("mfma_bf16_decode")
        (out_a, cache_a), (out_s, cache_s) = got
        assert same(out_s, out_a), f"{rows} rows: outputs differ between the two entry points"
        for name in ("expert_of", "gate_of", "counts", "offsets", "perm_slot", "perm_token", "probabilities"):
            assert same(getattr(cache_s, name), getattr(cache_a, name)), f"{rows} rows: {name}"
        ref = ref_layer.forward(t.x[:rows], threads=4)
        assert_routing_identical(cache_s, ref)
        assert rel_l2(out_s.reshape(rows, 128), ref.out) <= 2e-2
        xb.free()
        ob.free()
    layer.close()


def test_static_forward_refuses_what_it_cannot_take(device):
    t = synth.make(small_workload(d=64, E=4, k=2, F=64, T=40, seed=72, act="bf16", wt="bf16"))
    layer = gpu_layer(device, t)
    x = synth.f32_to_bf16_bits(t.x)
    xb, ob = DeviceBuffer(device, x.nbytes).upload(x), DeviceBuffer(device, x.nbytes)
    with pytest.raises(rb.Unsupported, match="decode-shaped"):
        layer.forward_static_device(xb.ptr, 40, ob.ptr)            # more than 32 tokens
    with pytest.raises(rb.Unsupported, match="decode-shaped"):
        layer.forward_static_device(xb.ptr, 0, ob.ptr)
    layer.forward_static_device(xb.ptr, 32, ob.ptr)                # the limit itself is fine
    device.synchronize()
    layer.close()
    f32 = gpu_layer(device, synth.make(small_workload(d=64, E=4, k=2, F=64, T=8, seed=72)))
    with pytest.raises(rb.Unsupported, match="decode-shaped"):
        f32.forward_static_device(xb.ptr, 8, ob.ptr)               # not a matrix-core bf16 layer
    f32.close()
    # hidden rows of 32 tokens x 8 experts each x 16448 features: more than the static array holds
    cfg = rb.MoeConfig(8, 8, 16448)
    wide = rb.MoeLayer(64, cfg, device, act_dtype="bf16", weight_dtype="bf16", max_tokens=32)
    with pytest.raises(rb.Unsupported, match="bytes of scratch"):
        wide.forward_static_device(xb.ptr, 32, ob.ptr)
    wide.forward_static_device(xb.ptr, 8, ob.ptr)                  # a quarter of the rows fits
    device.synchronize()
    wide.close()
    xb.free()
    ob.free()
