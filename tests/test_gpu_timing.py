"""The measuring entry points change nothing but the clock: a forward whose launches carry their own events
(rbmoe_forward_kernel_times), a forward with events between the stages (rbmoe_forward_timed) and the replay of one
stage (rbmoe_replay_stage) leave the same output bits and the same routing tables as a plain forward."""
import numpy as np
import pytest

from bench import DeviceBuffer
from helpers import gpu_layer, small_workload
from rustingbrain_amd import _lib as L
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [dict(d=128, E=8, k=2, F=192, T=700, shared=True),     # large-batch kernels
                                   dict(d=128, E=8, k=2, F=192, T=16, shared=True),      # decode-shaped, routing beside
                                   dict(d=64, E=40, k=2, F=64, T=8)],                    # decode-shaped, four launches
                         ids=["batch", "decode_front", "decode"])
def test_measuring_entry_points_leave_the_results_alone(device, shape):
    t = synth.make(small_workload(seed=91, act="bf16", wt="bf16", **shape))
    T = shape["T"]
    layer = gpu_layer(device, t)
    x = synth.f32_to_bf16_bits(t.x)
    xb, ob = DeviceBuffer(device, x.nbytes).upload(x), DeviceBuffer(device, x.nbytes)

    def snapshot():
        device.synchronize()
        out = ob.download(np.empty_like(x)).copy()
        c = layer.cache(T)
        return out, c.expert_of.copy(), c.perm_token.copy(), c.gate_of.copy(), layer.losses()

    def same(a, b):
        return all(np.array_equal(np.asarray(u).view(np.uint8), np.asarray(v).view(np.uint8)) for u, v in zip(a, b))

    layer.forward_device(xb.ptr, T, ob.ptr)
    plain = snapshot()
    ob.upload(np.zeros_like(x))
    kt = layer.forward_kernel_times(xb.ptr, T, ob.ptr)
    assert same(snapshot(), plain)
    decode = "decode" in layer.kernel_name()   # decode-shaped: the combine rides in the down launch
    assert kt["gate_up"] > 0 and kt["down"] > 0 and (kt["combine"] > 0) != decode and kt["empty"] == 0
    assert abs(kt["total"] - sum(v for k, v in kt.items() if k != "total")) <= 1e-6
    assert kt["total"] < 5.0          # milliseconds: these are kernel durations, not garbage
    if shape["shared"] if "shared" in shape else False:
        assert kt["shared"] > 0 or "decode" in layer.kernel_name()   # decode-shaped: the shared expert rides in the product launches
    ob.upload(np.zeros_like(x))
    st = layer.forward_timed(xb.ptr, T, ob.ptr)
    assert same(snapshot(), plain) and st["total"] > 0
    # one stage again, by itself
    for stage in ("gate_up", "down", "combine"):
        ob.upload(np.zeros_like(x))
        layer.forward_device(xb.ptr, T, ob.ptr)
        ms = layer.replay_stage(stage, 5)
        if stage == "combine" and decode:
            assert ms is None
            continue
        assert ms is not None and 0 < ms < 5.0
        assert layer.enqueue_stage(stage, 2)
        assert same(snapshot(), plain), stage
    front = layer.kernel_name().startswith("mfma_bf16_decode_front")
    assert (layer.replay_stage("router", 2) is None) == front   # the routing has no launch of its own there
    assert (layer.replay_stage("dispatch", 2) is None) == ("decode" in layer.kernel_name())
    assert layer.replay_stage("empty", 2) is None
    layer.close()
    xb.free()
    ob.free()
