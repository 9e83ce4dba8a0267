"""The entry points that take device pointers enqueue kernels and device-to-device copies only (no allocation, no
host synchronisation, no memset nodes), so a caller can capture them into a HIP graph.  Each test captures one call
sequence on a stream of its own, replays the graph several times with eager work and synchronisations in between,
and wants every replay identical to the eager result."""
import ctypes as C

import numpy as np
import pytest

import rustingbrain_amd as rb
from bench import DeviceBuffer
from helpers import gpu_layer, small_workload
from rustingbrain_amd import _lib as L
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    return C.CDLL("libamdhip64.so")


def ck(rc, what):
    assert rc == 0, f"{what} failed with hipError {rc}"


class Capture:
    """Captures what `enqueue()` puts on a fresh stream that the context is switched to."""

    def __init__(self, hip, device, enqueue):
        self.hip, self.device = hip, device
        self.stream = C.c_void_p()
        ck(hip.hipStreamCreateWithFlags(C.byref(self.stream), 1), "hipStreamCreateWithFlags")  # non-blocking
        device.synchronize()
        device.set_stream(self.stream.value)
        ck(hip.hipStreamBeginCapture(self.stream, 0), "hipStreamBeginCapture")                # global mode
        enqueue()
        self.graph = C.c_void_p()
        ck(hip.hipStreamEndCapture(self.stream, C.byref(self.graph)), "hipStreamEndCapture")
        self.exe = C.c_void_p()
        ck(hip.hipGraphInstantiate(C.byref(self.exe), self.graph, None, None, 0), "hipGraphInstantiate")

    def replay(self):
        ck(self.hip.hipGraphLaunch(self.exe, self.stream), "hipGraphLaunch")
        ck(self.hip.hipStreamSynchronize(self.stream), "hipStreamSynchronize")

    def close(self):
        self.device.set_stream(None)
        ck(self.hip.hipGraphExecDestroy(self.exe), "hipGraphExecDestroy")
        ck(self.hip.hipGraphDestroy(self.graph), "hipGraphDestroy")
        ck(self.hip.hipStreamDestroy(self.stream), "hipStreamDestroy")


def bits(t, a):
    return synth.f32_to_bf16_bits(a) if t.workload.act_dtype == "bf16" else np.ascontiguousarray(a, np.float32)


@pytest.mark.parametrize("shape,block", [
    (dict(d=768, E=8, k=2, F=128, T=8, shared=True), False),     # decode-shaped kernels
    (dict(d=768, E=8, k=2, F=128, T=8, shared=True), True),      # ... with the norm inside the routing kernel
    (dict(d=128, E=8, k=2, F=64, T=600, shared=True), False),    # large-batch kernels
    (dict(d=128, E=8, k=2, F=64, T=600), True),                  # ... behind the norm kernel, residual added
    (dict(d=128, E=8, k=2, F=64, T=1100, shared=True), False),   # the shared expert forked onto the side stream and
    (dict(d=128, E=8, k=2, F=64, T=1100, shared=True), True),    # joined again inside the capture
])
def test_forward_replays_identically(device, hip, shape, block):
    t = synth.make(small_workload(seed=61, act="bf16", wt="bf16", **shape))
    T = shape["T"]
    layer = gpu_layer(device, t, max_tokens=T)
    layer.set_feed_forward_norm(np.linspace(0.5, 1.5, shape["d"]).astype(np.float32), 1e-6)
    xh = bits(t, t.x)
    x = DeviceBuffer(device, xh.nbytes).upload(xh)
    out_e, out_g = DeviceBuffer(device, xh.nbytes), DeviceBuffer(device, xh.nbytes)
    run = (lambda o: layer.forward_block_device(x.ptr, T, o.ptr)) if block else \
          (lambda o: layer.forward_device(x.ptr, T, o.ptr))
    run(out_e)
    device.synchronize()
    eager = out_e.download(np.empty_like(xh)).copy()
    cap = Capture(hip, device, lambda: run(out_g))
    other = bits(t, t.x[::-1].copy())
    x2 = DeviceBuffer(device, xh.nbytes).upload(other)
    for _ in range(3):
        cap.replay()
        assert np.array_equal(out_g.download(np.empty_like(xh)), eager)
        # eager work on other rows in between: the layer's buffers hold something else before the next replay
        layer.forward_device(x2.ptr, T, out_e.ptr)
        device.synchronize()
    cap.close()
    for b in (x, x2, out_e, out_g):
        b.free()
    layer.close()


def test_training_step_replays_identically(device, hip, monkeypatch):
    # zero_grads, forward, backward (with its side stream forked and joined inside the capture); deterministic
    # mode so that the weight gradients can be compared bit for bit
    monkeypatch.setenv("RBMOE_DETERMINISTIC", "1")
    t = synth.make(small_workload(d=128, E=8, k=2, F=64, T=500, seed=62, act="bf16", wt="bf16", shared=True))
    T = 500
    layer = gpu_layer(device, t, training=True)
    xh = bits(t, t.x)
    gh = bits(t, np.random.default_rng(1).standard_normal(t.x.shape).astype(np.float32))
    x, g = DeviceBuffer(device, xh.nbytes).upload(xh), DeviceBuffer(device, xh.nbytes).upload(gh)
    out, gin = DeviceBuffer(device, xh.nbytes), DeviceBuffer(device, xh.nbytes)

    def step():
        layer.zero_grads()
        layer.forward_device(x.ptr, T, out.ptr)
        layer.backward_device(g.ptr, T, gin.ptr)

    step()
    device.synchronize()
    want_gin = gin.download(np.empty_like(xh)).copy()
    want = [layer.weight_grad(w, 3) for w in (L.W_GATE, L.W_DOWN)] + [layer.weight_grad(L.W_ROUTER),
                                                                      layer.weight_grad(L.W_SHARED_UP)]
    cap = Capture(hip, device, step)
    for _ in range(3):
        layer.backward_device(g.ptr, T, gin.ptr)        # eager work in between: gradients now hold twice the values
        device.synchronize()
        cap.replay()
        assert np.array_equal(gin.download(np.empty_like(xh)), want_gin)
        got = [layer.weight_grad(w, 3) for w in (L.W_GATE, L.W_DOWN)] + [layer.weight_grad(L.W_ROUTER),
                                                                         layer.weight_grad(L.W_SHARED_UP)]
        for a, b in zip(got, want):
            assert np.array_equal(a, b)
    cap.close()
    for b in (x, g, out, gin):
        b.free()
    layer.close()
