#!/usr/bin/env python3
"""Benchmark of the mixture-of-experts layer forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-backward]

A step is one forward pass of the layer (router, dispatch, grouped SwiGLU expert
products, combine, auxiliary losses) over one batch of seeded synthetic tokens
already resident in HBM.  Prints ONE JSON line: tokens/s for the whole layer, the
roofline of the dominant kernel (the grouped gate/up product) measured with HIP
events on the library's stream, per-stage figures, and the CPU restatement of
the reference's rayon path timed on this machine's host cores.  With --backward
a second layer in training mode is also timed (unless --no-backward): forward
with the backward pass's state kept, the backward pass, and both (a "backward"
object in the same line).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import rustingbrain_amd as rb  # noqa: E402
from rustingbrain_amd import _lib as L  # noqa: E402
from rustingbrain_amd import synth  # noqa: E402

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3     # MI355X fp32 matrix
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# HBM-side bytes per launch of the dominant kernel come from rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE), which
# cannot be taken inside this program: profiles/hbm_traffic.json records them, each with the summary file it was read
# from and a digest of the kernel sources at the time.  A record whose digest is not that of the sources beside this
# file describes other kernels and is reported as null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
KERNEL_SOURCES = ("grouped_stream.hip", "decode_kernels.hip", "grouped_f32.hip")


def kernel_digest() -> str:
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "rustingbrain_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload: str, kernel: str):
    """(bytes per launch or None, where the figure comes from)."""
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None, "no profiles/hbm_traffic.json"
    rec = table.get(workload)
    if not rec or rec.get("kernel") != kernel:
        return None, "no counter run recorded for this workload and kernel"
    if rec.get("kernel_digest") != kernel_digest():
        return None, f"{rec.get('source')} was measured on other kernel sources (digest {rec.get('kernel_digest')})"
    return float(rec["bytes_per_launch"]), rec.get("source")


class DeviceBuffer:
    def __init__(self, dev: rb.Device, nbytes: int):
        self.dev, self.nbytes = dev, nbytes
        p = C.c_void_p()
        rc = dev._lib.rbmoe_device_alloc(dev.handle, nbytes, C.byref(p))
        if rc != L.OK:
            raise RuntimeError(dev._lib.rbmoe_last_error(dev.handle).decode())
        self.ptr = p.value

    def upload(self, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        rc = self.dev._lib.rbmoe_copy_to_device(self.dev.handle, C.c_void_p(self.ptr), a.ctypes.data_as(C.c_void_p),
                                                a.nbytes)
        assert rc == L.OK
        return self

    def download(self, a: np.ndarray) -> np.ndarray:
        rc = self.dev._lib.rbmoe_copy_to_host(self.dev.handle, a.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr),
                                              a.nbytes)
        assert rc == L.OK
        return a

    def free(self):
        if self.ptr:
            self.dev._lib.rbmoe_device_free(self.dev.handle, C.c_void_p(self.ptr))
            self.ptr = None


def algorithmic(w: synth.Workload, T: int, routed: int, touched_experts: int) -> dict:
    """Algorithmic flops / bytes per launch of each stage (padding and recomputation never count)."""
    d, F, E, k = w.d_model, w.d_ff, w.num_experts, w.experts_per_token
    Fs = w.shared_d_ff if w.shared_expert else 0
    sa = 2 if w.act_dtype == "bf16" else 4
    sw = {"f32": 4, "bf16": 2, "int8": 1}[w.weight_dtype]
    S = routed
    return {
        "router_bytes": T * d * sa + E * d * 4 + T * k * 8,
        # permutation only (the gather of the rows is part of the gate/up operand load): expert_of and
        # rank_in_block read, per-block histograms read, perm_slot / perm_token / inv_pos written
        "dispatch_bytes": 2 * T * k * 4 + ((T + 31) // 32) * E * 4 + 3 * S * 4,
        "combine_bytes": S * d * sa + 2 * S * 4 + T * d * sa,
        "gate_up_flops": 4 * d * F * S,
        "down_flops": 2 * d * F * S,
        "shared_flops": 6 * d * Fs * T,
        "gemm_flops": 6 * d * F * S + 6 * d * Fs * T,
        "layer_bytes_decode": touched_experts * 3 * d * F * sw + 3 * d * Fs * sw + E * d * 4 + 2 * T * d * sa + S * 8,
        # decode-shaped products: every touched expert's weights once, token rows in, hidden / output rows out
        "decode_gate_up_bytes": touched_experts * 2 * d * F * sw + 2 * d * Fs * sw + (S + T) * d * sa
                                + (S * F + T * Fs) * sa,
        "decode_down_bytes": touched_experts * d * F * sw + d * Fs * sw + (S * F + T * Fs) * sa + (S + T) * d * sa,
    }


def cpu_baseline(t: synth.Tensors, budget_s: float = 20.0) -> dict:
    """The CPU restatement of the reference's rayon path (oracle/, C++), timed
    on the host cores of this machine.  Only this function touches oracle/."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from helpers import oracle_layer
    threads = max(1, min(16, os.cpu_count() or 1))   # the GPU box gives one job 16 cores' worth
    layer = oracle_layer(t)
    T = t.x.shape[0]
    layer.forward(t.x, router_bias=t.router_bias, threads=threads)  # warm-up
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 20 and (time.perf_counter() < t_end or len(times) < 2):
        t0 = time.perf_counter()
        layer.forward(t.x, router_bias=t.router_bias, threads=threads)
        times.append(time.perf_counter() - t0)
    best = float(np.median(times))
    return {"value": T / best, "unit": "tokens/s", "cores": threads, "os_cpu_count": os.cpu_count(), "kind": "port",
            "sample": f"whole workload ({T} tokens), median of {len(times)} forwards after 1 warm-up; "
                      "C++ restatement of the reference's rayon path, not the Rust binary",
            "ms_per_forward": best * 1e3}


def cpu_baseline_backward(t: synth.Tensors, grad_output: np.ndarray) -> dict:
    """The CPU restatement's forward + backward (oracle/, C++, one task per expert on the host cores), one call.
    With cpu_baseline, the only code of this file that touches oracle/."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from helpers import oracle_layer
    threads = max(1, min(16, os.cpu_count() or 1))
    layer = oracle_layer(t)
    t0 = time.perf_counter()
    layer.backward(t.x, grad_output, router_bias=t.router_bias, threads=threads)
    ms = (time.perf_counter() - t0) * 1e3
    return {"value": t.x.shape[0] / (ms * 1e-3), "unit": "tokens/s", "cores": threads, "os_cpu_count": os.cpu_count(),
            "kind": "port",
            "sample": "whole workload, one forward + backward call of the C++ restatement (experts as parallel "
                      "tasks, like the reference's par_iter over experts)", "ms": ms}


def backward_leg(dev, w, t, x, out, bp, args, alg, with_cpu: bool) -> dict:
    """Times MoeLayer::backward (reference src/moe.rs:348-489) on a second layer in training mode: K forwards
    that keep the backward pass's state, K backward passes of the last forward (accumulating, as Param.grad does,
    and after zero_grads), and K training steps (zero_grads, forward, backward)."""
    if (w.act_dtype, w.weight_dtype) not in (("bf16", "bf16"), ("f32", "f32")):
        return {"skipped": "the backward pass exists for bf16 layers and for all-f32 layers"}
    bf16 = w.act_dtype == "bf16"
    T = w.tokens
    cfg = rb.MoeConfig(w.num_experts, w.experts_per_token, w.d_ff, w.shared_expert)
    layer = rb.MoeLayer(w.d_model, cfg, dev, act_dtype=w.act_dtype, weight_dtype=w.weight_dtype, max_tokens=T,
                        shared_d_ff=w.shared_d_ff if w.shared_expert else 0)
    layer.enable_training()
    layer.load_tensors(t)
    rng = np.random.default_rng(w.seed + 1000)
    gh = synth.round_bf16(rng.standard_normal(t.x.shape).astype(np.float32))
    g = DeviceBuffer(dev, x.nbytes).upload(synth.f32_to_bf16_bits(gh) if bf16 else gh)
    gin = DeviceBuffer(dev, x.nbytes)

    def fwd():
        layer.forward_device(x.ptr, T, out.ptr, bias_ptr=bp)

    def bwd():
        layer.backward_device(g.ptr, T, gin.ptr)

    def timed(fn, n):
        dev.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        dev.synchronize()
        return (time.perf_counter() - t0) * 1e3 / n

    for _ in range(max(3, args.warmup // 4)):
        fwd()
        bwd()
    n = max(5, args.steps // 4)
    ms_f = timed(fwd, n)
    ms_b_acc = timed(bwd, n)                                     # every pass adds to the gradients
    ms_b = timed(lambda: (layer.zero_grads(), bwd()), n)         # as in a training loop: cleared, then written
    ms_fb = timed(lambda: (layer.zero_grads(), fwd(), bwd()), n)
    # products of the backward pass: twice the forward's (grad_input and weight gradients)
    flops = 2 * alg["gemm_flops"]
    res = {"ms_forward_training": ms_f, "ms_backward": ms_b, "ms_backward_accumulating": ms_b_acc,
           "ms_forward_backward": ms_fb,
           "tokens_per_s_forward_backward": T / (ms_fb * 1e-3), "steps": n,
           "backward_product_flops": flops, "backward_tflops": flops / (ms_b * 1e-3) / 1e12,
           "backward_frac_of_peak": flops / (ms_b * 1e-3) / 1e12 / (PEAK_BF16_TFLOPS if bf16 else PEAK_F32_TFLOPS),
           "note": "ms_backward and ms_forward_backward include zero_grads, as a training step does (the expert "
                   "gradients, f32, are then written once); ms_backward_accumulating adds to them (read and write)"}
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline_backward(t, gh)
    layer.close()
    g.free()
    gin.free()
    return res


class Tools:
    """The benchmark's helpers (librbmoe_bench.so): one stream that the layer's kernels, the cache flush and the
    event timer share, set on the device context."""

    def __init__(self, dev):
        self.lib = L.load_bench()
        self.dev = dev
        self.stream, self.timer, self._flush = C.c_void_p(), C.c_void_p(), None
        self._ck(self.lib.rbbench_stream_create(C.byref(self.stream)), "rbbench_stream_create")
        self._ck(self.lib.rbbench_timer_create(C.byref(self.timer)), "rbbench_timer_create")
        dev.set_stream(self.stream.value)

    @staticmethod
    def _ck(rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed with code {rc}")

    def use_stream(self):
        self.dev.set_stream(self.stream.value)

    def start(self):
        self._ck(self.lib.rbbench_timer_start(self.timer, self.stream), "rbbench_timer_start")

    def stop(self) -> float:
        ms = C.c_float()
        self._ck(self.lib.rbbench_timer_stop(self.timer, self.stream, C.byref(ms)), "rbbench_timer_stop")
        return float(ms.value)

    def flush(self):
        """Evict L2 and the 256 MiB Infinity Cache with a read-only sweep of 512 MiB (no dirty lines are left to
        drain while the next kernel runs)."""
        if self._flush is None:
            self._flush = C.c_void_p()
            self._ck(self.lib.rbbench_flush_create(512 << 20, C.byref(self._flush)), "rbbench_flush_create")
        self._ck(self.lib.rbbench_flush(self._flush, self.stream), "rbbench_flush")

    def flush_handle(self):
        if self._flush is None:
            self.flush()
            self.dev.synchronize()
        return self._flush

    def close(self):
        self.dev.synchronize()
        self.dev.set_stream(None)
        if self._flush is not None:
            self.lib.rbbench_flush_destroy(self._flush)
        self.lib.rbbench_timer_destroy(self.timer)
        self.lib.rbbench_stream_destroy(self.stream)


class ForwardGraph:
    """One forward captured into a HIP graph on a stream of its own (the entry points that take device pointers only
    enqueue kernels, so they can be captured); a replay is one step without the host's launch calls."""

    def __init__(self, dev, tools, enqueue):
        self.hip = C.CDLL("libamdhip64.so")
        self.dev, self.tools = dev, tools
        self.stream, self.graph, self.exe = C.c_void_p(), C.c_void_p(), C.c_void_p()
        self._ck(self.hip.hipStreamCreateWithFlags(C.byref(self.stream), 1), "hipStreamCreateWithFlags")
        dev.synchronize()
        dev.set_stream(self.stream.value)
        self._ck(self.hip.hipStreamBeginCapture(self.stream, 0), "hipStreamBeginCapture")
        enqueue()
        self._ck(self.hip.hipStreamEndCapture(self.stream, C.byref(self.graph)), "hipStreamEndCapture")
        self._ck(self.hip.hipGraphInstantiate(C.byref(self.exe), self.graph, None, None, 0), "hipGraphInstantiate")
        n = C.c_size_t()
        self.nodes = None
        if self.hip.hipGraphGetNodes(self.graph, None, C.byref(n)) == 0:
            self.nodes = int(n.value)

    @staticmethod
    def _ck(rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed with hipError {rc}")

    def replay(self):
        self._ck(self.hip.hipGraphLaunch(self.exe, self.stream), "hipGraphLaunch")

    def synchronize(self):
        self._ck(self.hip.hipStreamSynchronize(self.stream), "hipStreamSynchronize")

    def close(self):
        self.synchronize()
        self.tools.use_stream()
        self.hip.hipGraphExecDestroy(self.exe)
        self.hip.hipGraphDestroy(self.graph)
        self.hip.hipStreamDestroy(self.stream)


REPLAY_STAGES = ("router", "dispatch", "gate_up", "down", "combine")


def weight_bytes(w: synth.Workload) -> int:
    sw = {"f32": 4, "bf16": 2, "int8": 1}[w.weight_dtype]
    Fs = w.shared_d_ff if w.shared_expert else 0
    return w.num_experts * 3 * w.d_model * w.d_ff * sw + 3 * w.d_model * Fs * sw + w.num_experts * w.d_model * 4


def measure(dev, tools, name: str, steps: int, warmup: int, repeats: int, act_override: str = None,
            plain: bool = False) -> dict:
    """One workload.
    * `repeats` loops of `steps` forwards of one layer back to back (median loop -> ms_per_step): weights that fit
      the 256 MiB Infinity Cache stay there;
    * the launch time of each stage by itself: the stage's launches of the last forward replayed 20 times between
      ONE pair of events (rbmoe_replay_stage), median of three such runs -> the roofline of the dominant kernel;
    * the same two measurements over several layers with their own copies of the weights (more than the Infinity
      Cache holds in all), forwards and stage launches issued in rotation: every launch finds its weights in HBM;
    * forwards with L2 and Infinity Cache flushed by a read-only sweep before each one, each forward timed by an
      event pair of its own (raw interval);
    * per-stage event intervals inside one forward (rbmoe_forward_timed), kept for comparison.
    With `plain` only the first measurement and the kernels' own durations inside those forwards are taken (the
    program then issues nothing but plain forwards: what a kernel trace or a counter run of it sees is the layer
    as a model runs it)."""
    w = synth.WORKLOADS[name]
    t = synth.make(w)
    if act_override:
        w = synth.Workload(**{**w.__dict__, "act_dtype": act_override})
    T = w.tokens
    cfg = rb.MoeConfig(w.num_experts, w.experts_per_token, w.d_ff, w.shared_expert)

    def new_layer():
        layer = rb.MoeLayer(w.d_model, cfg, dev, act_dtype=w.act_dtype, weight_dtype=w.weight_dtype, max_tokens=T,
                            shared_d_ff=w.shared_d_ff if w.shared_expert else 0)
        layer.load_tensors(t)
        return layer

    layer = new_layer()
    bf16 = w.act_dtype == "bf16"
    xh = synth.f32_to_bf16_bits(t.x) if bf16 else t.x
    x = DeviceBuffer(dev, xh.nbytes).upload(xh)
    out = DeviceBuffer(dev, xh.nbytes)
    bias = DeviceBuffer(dev, 4 * w.num_experts).upload(t.router_bias) if t.router_bias is not None else None
    bp = bias.ptr if bias else 0

    def fwd(lay=None):
        (lay or layer).forward_device(x.ptr, T, out.ptr, bias_ptr=bp)

    def wall_loops(fn, n_steps, n_repeats, sync):
        loops = []
        for _ in range(n_repeats):
            t0 = time.perf_counter()
            for i in range(n_steps):
                fn(i)
            sync()
            loops.append((time.perf_counter() - t0) * 1e3 / n_steps)
        return loops

    for _ in range(warmup):
        fwd()
    dev.synchronize()
    loops = wall_loops(lambda i: fwd(), steps, repeats, dev.synchronize)
    ms_per_step = float(np.median(loops))

    decode = "decode" in layer.kernel_name()   # the library takes the decode-shaped kernels up to 32 tokens
    graph = None
    if decode and not plain:
        # A decode step is three short launches: issued one by one from this interpreter, the host's launch calls
        # are part of the step.  The same forward replayed from a HIP graph, timed the same way:
        g = ForwardGraph(dev, tools, fwd)
        for _ in range(warmup):
            g.replay()
        g.synchronize()
        gl = wall_loops(lambda i: g.replay(), steps, repeats, g.synchronize)
        graph = {"ms_per_step": float(np.median(gl)), "nodes": g.nodes}
        g.close()

    # ---- each stage by itself, one event pair over 20 launches
    fwd()
    dev.synchronize()
    launch_ms = {}
    for st in REPLAY_STAGES:
        v = [None] if plain else [layer.replay_stage(st, 20) for _ in range(3)]
        launch_ms[st] = None if v[0] is None else float(np.median(v))

    # ---- kernel durations inside a forward: every launch carries its own start / stop events, which receive the
    # dispatch's own begin and end time stamps (what a kernel trace reports for the same launch)
    nprof = max(10, min(50, steps))

    def kernel_times(flush: bool):
        acc = {}
        for _ in range(nprof):
            if flush:
                tools.flush()
            for nm, v in layer.forward_kernel_times(x.ptr, T, out.ptr, bias_ptr=bp).items():
                acc.setdefault(nm, []).append(v)
        return {nm: float(np.mean(v)) for nm, v in acc.items()}, {nm: float(np.min(v)) for nm, v in acc.items()}

    kernel_ms, kernel_ms_min = kernel_times(False)
    # ---- event intervals between the stages of one forward (each carries the cost of an event pair: `empty`)
    acc = {}
    for _ in range(0 if plain else nprof):
        for nm, v in layer.forward_timed(x.ptr, T, out.ptr, bias_ptr=bp).items():
            acc.setdefault(nm, []).append(v)
    raw_ms = {nm: float(np.mean(v)) for nm, v in acc.items()} if acc else {"empty": 0.0}
    over = raw_ms["empty"]

    # ---- caches flushed (a read-only sweep of 512 MiB) before every forward
    cold_kernel_ms = kernel_ms if plain else kernel_times(True)[0]
    flushed = [0.0]
    for _ in range(0 if plain else max(10, min(30, steps))):
        tools.flush()
        tools.start()
        fwd()
        flushed.append(tools.stop())
    if len(flushed) > 1:
        flushed = flushed[1:]
    cold_flush = {"kernel_ms": cold_kernel_ms, "ms_per_step_raw_interval": float(np.median(flushed)),
                  "event_interval_overhead_ms": over,
                  "note": "a read-only sweep of 512 MiB before every forward.  kernel_ms: the dispatches' own time "
                          "stamps, per stage; ms_per_step_raw_interval: one event pair around the whole forward, "
                          "nothing subtracted"}

    # ---- several layers with their own copies of the weights, in rotation
    wb = weight_bytes(w)
    nlayers = 1 if plain else int(max(4, min(16, -(-(512 << 20) // wb))))
    layers = [layer] + [new_layer() for _ in range(nlayers - 1)]
    for lay in layers:
        fwd(lay)
    dev.synchronize()
    rr_steps = max(nlayers * 2, (max(20, steps // 2) // nlayers) * nlayers)
    rr_loops = [ms_per_step] if plain else wall_loops(lambda i: fwd(layers[i % nlayers]), rr_steps,
                                                      max(3, min(repeats, 5)), dev.synchronize)
    rr_ms = float(np.median(rr_loops))
    rr_launch = {}
    rounds = max(1, 20 // nlayers)
    for st in REPLAY_STAGES:
        if launch_ms[st] is None:
            rr_launch[st] = None
            continue
        v = []
        for _ in range(3):
            for lay in layers:      # untimed: the rotation is in steady state when the interval starts
                lay.enqueue_stage(st)
            tools.start()
            for _ in range(rounds):
                for lay in layers:
                    lay.enqueue_stage(st)
            v.append(tools.stop() / (rounds * nlayers))
        rr_launch[st] = float(np.median(v))
    for lay in layers[1:]:
        lay.close()
    round_robin = {"layers": nlayers, "weight_bytes_per_layer": wb, "weight_bytes_total": wb * nlayers,
                   "ms_per_step": rr_ms, "tokens_per_s": T / (rr_ms * 1e-3), "stage_launch_ms": rr_launch,
                   "note": "layers with their own copies of the weights (same values, distinct addresses, more than "
                           "the 256 MiB Infinity Cache in all), forwards issued in rotation; stage_launch_ms: the "
                           "stage's launches of all layers in rotation between one pair of events"}

    cache = layer.cache(T)
    routed = int(cache.offsets[-1])
    touched = int((cache.counts > 0).sum())
    alg = algorithmic(w, T, routed, touched)
    peak_tf = PEAK_F32_TFLOPS if (w.weight_dtype == "f32") else PEAK_BF16_TFLOPS

    def tflops(flops, ms):
        return flops / (ms * 1e-3) / 1e12 if ms and ms > 0 else 0.0

    def gbs(nbytes, ms):
        return nbytes / (ms * 1e-3) / 1e9 if ms and ms > 0 else 0.0

    kname = layer.kernel_name()
    traffic, traffic_source = measured_traffic(w.name, kname)
    timing = ("start / stop events carried by the launch itself (the dispatch's own begin and end time stamps, as in a "
              "kernel trace), mean over %d forwards" % nprof)
    if decode:
        # the dominant kernel of the decode-shaped path streams the gate/up weights of the touched experts (and of
        # the shared expert) once: it is bound by HBM, and is measured where its weights come from HBM
        ms_gu = cold_kernel_ms["gate_up"]
        gu_gbs = gbs(alg["decode_gate_up_bytes"], ms_gu)
        roofline = {"bound": "hbm", "kernel": "decode gate/up product + SwiGLU, routed and shared (" + kname +
                                              "), caches flushed before every forward",
                    "achieved": gu_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gu_gbs / PEAK_HBM_GBS,
                    "traffic": traffic, "traffic_source": traffic_source,
                    "bytes_per_launch": alg["decode_gate_up_bytes"], "avg_launch_ms": ms_gu, "timing": timing,
                    "touched_experts": touched,
                    "frac_layers_in_rotation": gbs(alg["decode_gate_up_bytes"], rr_launch["gate_up"]) / PEAK_HBM_GBS,
                    "cache_resident_gbs": gbs(alg["decode_gate_up_bytes"], kernel_ms["gate_up"])}
    else:
        gu = tflops(alg["gate_up_flops"], kernel_ms["gate_up"])
        roofline = {"bound": "mfma", "kernel": "grouped gate/up product + SwiGLU (" + kname + ")",
                    "achieved": gu, "peak": peak_tf, "unit": "TFLOP/s", "frac": gu / peak_tf,
                    "traffic": traffic, "traffic_source": traffic_source,
                    "flops_per_launch": alg["gate_up_flops"], "avg_launch_ms": kernel_ms["gate_up"],
                    "min_launch_ms": kernel_ms_min["gate_up"], "timing": timing,
                    "frac_back_to_back": tflops(alg["gate_up_flops"], launch_ms["gate_up"]) / peak_tf,
                    "frac_weights_from_hbm": tflops(alg["gate_up_flops"], cold_kernel_ms["gate_up"]) / peak_tf}
    prod_ms = kernel_ms["gate_up"] + kernel_ms["down"]
    stages = {
        "kernel_ms": kernel_ms, "kernel_ms_min": kernel_ms_min, "kernel_ms_timing": timing,
        "launch_ms_back_to_back": launch_ms,
        "launch_ms_back_to_back_timing": "20 launches of the stage between one pair of HIP events, median of 3 runs "
                                         "(sustained: the clocks settle lower than inside a forward)",
        "ms_mean_raw_intervals": raw_ms, "event_interval_overhead_ms": over,
        "gate_up_tflops": tflops(alg["gate_up_flops"], kernel_ms["gate_up"]),
        "down_tflops": tflops(alg["down_flops"], kernel_ms["down"]),
        "down_frac_of_peak": tflops(alg["down_flops"], kernel_ms["down"]) / peak_tf,
        # the routed experts' two products
        "grouped_gemms_tflops": tflops(alg["gate_up_flops"] + alg["down_flops"], prod_ms),
        "grouped_gemms_frac_of_peak": tflops(alg["gate_up_flops"] + alg["down_flops"], prod_ms) / peak_tf,
        "router_gbs": gbs(alg["router_bytes"], kernel_ms["router"]),
        "dispatch_gbs": gbs(alg["dispatch_bytes"], kernel_ms["dispatch"]),
        "dispatch_note": "latency-bound: a few hundred KB of indices per launch, no rows are moved",
        "combine_gbs": gbs(alg["combine_bytes"], kernel_ms["combine"]),
        "combine_frac_of_hbm": gbs(alg["combine_bytes"], kernel_ms["combine"]) / PEAK_HBM_GBS,
        "launch_gaps_ms": ms_per_step - kernel_ms["total"],
    }
    if decode:
        cold_kernels = cold_kernel_ms["total"]
        stages.update({
            "whole_layer_bytes": alg["layer_bytes_decode"],
            "cold_kernel_ms": cold_kernel_ms,
            "cold_decode_down_frac_of_hbm": gbs(alg["decode_down_bytes"], cold_kernel_ms["down"]) / PEAK_HBM_GBS,
            "cold_whole_layer_ms": cold_kernels,
            "cold_whole_layer_frac_of_hbm": gbs(alg["layer_bytes_decode"], cold_kernels) / PEAK_HBM_GBS,
            "rotation_whole_layer_frac_of_hbm_per_step": gbs(alg["layer_bytes_decode"], rr_ms) / PEAK_HBM_GBS,
            "cache_resident_whole_layer_gbs": gbs(alg["layer_bytes_decode"], ms_per_step),
            "note": "value / ms_per_step are back-to-back forwards of one layer (weights stay in the 256 MiB "
                    "Infinity Cache); cold_* figures flush L2 and Infinity Cache before every forward and sum the "
                    "kernels' own durations; rotation_*: layers with their own weights in rotation, whole step "
                    "(launch gaps included)"})
    config = {"workload": w.name, "d_model": w.d_model, "num_experts": w.num_experts,
              "experts_per_token": w.experts_per_token, "d_ff": w.d_ff, "tokens": T,
              "shared_expert": w.shared_expert, "weight_dtype": w.weight_dtype, "act_dtype": w.act_dtype,
              "seed": w.seed, "expert0_share": float(cache.load_fractions()[0]), "routed_slots": routed}
    if plain:
        roofline["note"] = stages["note_plain"] = ("--plain: only back-to-back forwards and the kernels' own durations "
                                                   "inside them were measured; every cold / rotation / replay figure "
                                                   "repeats those")
    return {"w": w, "t": t, "layer": layer, "x": x, "out": out, "bias": bias, "bp": bp, "alg": alg,
            "ms_per_step": ms_per_step, "loops_ms": loops, "roofline": roofline, "stages": stages, "config": config,
            "bf16": bf16, "decode": decode, "graph": graph, "cold_flush": cold_flush, "round_robin": round_robin}


def two_in_flight(w, t, steps: int, warmup: int, repeats: int) -> dict:
    """Throughput with two independent batches in flight: two contexts (a stream each), a layer with the same weights
    on each, forwards issued alternately.  The routing kernels of one forward (vector units, latency) then run beside
    the expert products of the other (matrix cores).  Not the headline figure: inside one model consecutive layers
    depend on each other; this is what independent micro-batches get."""
    T = w.tokens
    devs = [rb.Device.open(0) for _ in range(2)]
    layers, bufs = [], []
    xh = synth.f32_to_bf16_bits(t.x) if w.act_dtype == "bf16" else t.x
    for dev in devs:
        cfg = rb.MoeConfig(w.num_experts, w.experts_per_token, w.d_ff, w.shared_expert)
        layer = rb.MoeLayer(w.d_model, cfg, dev, act_dtype=w.act_dtype, weight_dtype=w.weight_dtype, max_tokens=T,
                            shared_d_ff=w.shared_d_ff if w.shared_expert else 0)
        layer.load_tensors(t)
        x, out = DeviceBuffer(dev, xh.nbytes).upload(xh), DeviceBuffer(dev, xh.nbytes)
        bias = DeviceBuffer(dev, 4 * w.num_experts).upload(t.router_bias) if t.router_bias is not None else None
        layers.append(layer)
        bufs.append((x, out, bias))

    def run(n):
        for i in range(n):
            x, out, bias = bufs[i % 2]
            layers[i % 2].forward_device(x.ptr, T, out.ptr, bias_ptr=bias.ptr if bias else 0)
        for dev in devs:
            dev.synchronize()

    run(2 * warmup)
    loops = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        run(steps)
        loops.append((time.perf_counter() - t0) * 1e3 / steps)
    ms = float(np.median(loops))
    for layer in layers:
        layer.close()
    for x, out, bias in bufs:
        for b in (x, out, bias):
            if b:
                b.free()
    for dev in devs:
        dev.close()
    return {"ms_per_forward": ms, "tokens_per_s": T / (ms * 1e-3), "steps": steps, "repeats": repeats,
            "note": "two contexts and two layers with the same weights, forwards issued alternately; not the headline value"}


def release(m: dict) -> None:
    m["layer"].close()
    for b in (m["x"], m["out"], m["bias"]):
        if b:
            b.free()


def summary(m: dict) -> dict:
    """The short form of one workload for the `workloads` object of the report."""
    r, st, rr = m["roofline"], m["stages"], m["round_robin"]
    s = {"tokens_per_s": m["config"]["tokens"] / (m["ms_per_step"] * 1e-3), "ms_per_step": m["ms_per_step"],
         "kernel": r["kernel"], "bound": r["bound"], "frac": r["frac"], "achieved": r["achieved"], "unit": r["unit"],
         "peak": r["peak"], "avg_launch_ms": r["avg_launch_ms"], "traffic": r["traffic"],
         "kernel_ms": {k: round(v, 5) for k, v in st["kernel_ms"].items()},
         "launch_gaps_ms": st["launch_gaps_ms"],
         "down_frac_of_peak": st["down_frac_of_peak"],
         "grouped_gemms_frac_of_peak": st["grouped_gemms_frac_of_peak"],
         "cold": m["cold_flush"],
         "layers_round_robin": {"layers": rr["layers"], "ms_per_step": rr["ms_per_step"],
                                "tokens_per_s": rr["tokens_per_s"],
                                "stage_launch_ms": {k: (None if v is None else round(v, 5))
                                                    for k, v in rr["stage_launch_ms"].items()}},
         "config": m["config"]}
    if m["decode"]:
        s["cold"] = dict(m["cold_flush"], gate_up_frac_of_hbm=r["frac"], gate_up_ms=r["avg_launch_ms"],
                         down_frac_of_hbm=st["cold_decode_down_frac_of_hbm"], whole_layer_ms=st["cold_whole_layer_ms"],
                         whole_layer_frac_of_hbm=st["cold_whole_layer_frac_of_hbm"],
                         rotation_whole_layer_frac_of_hbm_per_step=st["rotation_whole_layer_frac_of_hbm_per_step"])
        s["warm"] = {"gate_up_gbs": r["cache_resident_gbs"], "whole_layer_ms": m["ms_per_step"],
                     "whole_layer_gbs": st["cache_resident_whole_layer_gbs"],
                     "whole_layer_ms_graph_replay": m["graph"]["ms_per_step"] if m["graph"] else None,
                     "graph_nodes": m["graph"]["nodes"] if m["graph"] else None}
    return s


def library_gemm_child(slots: int, d_ff: int, d_model: int) -> int:
    """The measuring half of library_gemm: a process of its own (torch brings its own copy of the HIP runtime, which
    finds no device in a process where this program's library has already opened one).  Prints one JSON object."""
    import torch
    out = {"library": f"torch {torch.__version__} matmul (bf16 x bf16 -> bf16)", "runs": "20 launches between one pair "
           "of events, median of 5 runs, in a process of its own"}
    for name, (M, N, K) in (("gate_up", (slots, 2 * d_ff, d_model)), ("down", (slots, d_model, d_ff))):
        a = torch.randn(M, K, device="cuda:0", dtype=torch.bfloat16)
        b = torch.randn(N, K, device="cuda:0", dtype=torch.bfloat16)
        for _ in range(5):
            a @ b.t()
        torch.cuda.synchronize()
        runs = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                a @ b.t()
            e1.record()
            torch.cuda.synchronize()
            runs.append(e0.elapsed_time(e1) / 20)
        ms = statistics.median(runs)
        tf = 2.0 * M * N * K / (ms * 1e-3) / 1e12
        out[name] = {"M": M, "N": N, "K": K, "avg_launch_ms": ms, "tflops": tf, "frac_of_peak": tf / PEAK_BF16_TFLOPS}
    print(json.dumps(out))
    return 0


def library_gemm(w) -> dict:
    """The vendor library's bf16 product on the dense shapes of the two grouped products of workload `w` (all routed
    rows as one group), measured by a child process (library_gemm_child)."""
    import subprocess
    cmd = [sys.executable, os.path.abspath(__file__), "--library-gemm-child", str(w.tokens * w.experts_per_token),
           str(w.d_ff), str(w.d_model)]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    if res.returncode != 0:
        return {"error": (res.stderr or "").strip().splitlines()[-1:] or ["child failed"]}
    return json.loads(res.stdout.strip().splitlines()[-1])


def main() -> int:
    if sys.argv[1:2] == ["--library-gemm-child"]:
        return library_gemm_child(int(sys.argv[2]), int(sys.argv[3]), int(sys.argv[4]))
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=0,
                    help="loops of --steps forwards; ms_per_step is their median (default: 5, more for short loops, so "
                         "that about 300 forwards are timed in all - a loop of 20 forwards lasts 3 ms, less than "
                         "the device takes to settle at its clocks)")
    ap.add_argument("--workload", default="c3_prefill_d768_e16", choices=list(synth.WORKLOADS),
                    help="the workload of the top-level figures (the metric is quoted on the default)")
    ap.add_argument("--only", action="store_true", help="skip the `workloads` object (the other four workloads)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--plain", action="store_true",
                    help="issue nothing but plain forwards of the chosen workload (timed loops, then forwards whose "
                         "launches carry their own events): the command to run under a kernel trace or a counter pass")
    ap.add_argument("--no-backward", action="store_true",
                    help="skip the training-step figures (the `backward` object: forward in training mode, backward "
                         "pass, both; bf16 layers and all-f32 layers)")
    ap.add_argument("--backward", action="store_true", help="(the training-step figures are on by default)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (the plain copy that FETCH_SIZE / "
                         "WRITE_SIZE readings are scaled by when this command runs under rocprofv3 --pmc)")
    ap.add_argument("--calibrate-mfma", action="store_true",
                    help="also run the multiply-only kernel: the rate the matrix cores sustain (`calibration.mfma`)")
    ap.add_argument("--calibrate-read", action="store_true",
                    help="also run a plain 39 MiB read with cold and warm caches (`calibration.read`): what a launch "
                         "the size of the decode gate/up product can get out of HBM")
    ap.add_argument("--calibrate-library-gemm", action="store_true",
                    help="also time the vendor library's bf16 matrix product (torch.matmul, i.e. hipBLASLt) on the dense "
                         "shapes of the workload's two grouped products (`calibration.library_gemm`): what a plain "
                         "product of these shapes - no gather, no ragged groups, no SwiGLU - gets out of the matrix cores")
    args = ap.parse_args()
    if args.repeats <= 0:
        args.repeats = max(5, min(25, 300 // max(args.steps, 1)))
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    dev = rb.Device.open(0)
    tools = Tools(dev)
    if args.plain:
        args.only = args.no_cpu = args.no_backward = True
    m = measure(dev, tools, args.workload, args.steps, args.warmup, args.repeats, plain=args.plain)
    w, T = m["w"], m["w"].tokens
    result = {
        "metric": "MoE-layer fwd tokens/sec at d768 E16 k2; grouped-GEMM % of bf16 MFMA peak",
        "value": T / (m["ms_per_step"] * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "repeats": args.repeats, "ms_per_step": m["ms_per_step"],
        "ms_per_step_loops": m["loops_ms"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if w.weight_dtype != "f32" else "f32", "data": "synthetic",
        "config": m["config"], "roofline": m["roofline"], "stages": m["stages"], "cold": m["cold_flush"],
        "layers_round_robin": m["round_robin"],
    }
    if m["graph"] is not None:
        result["graph_replay"] = m["graph"]
    if args.calibrate_copy:
        n = 256 << 20
        a, b = DeviceBuffer(dev, n), DeviceBuffer(dev, n)
        assert dev._lib.rbmoe_copy_device(dev.handle, C.c_void_p(b.ptr), C.c_void_p(a.ptr), n) == L.OK
        a.free()
        b.free()
    calibration = {}
    if args.calibrate_mfma:
        tf, ms = C.c_double(), C.c_double()
        assert tools.lib.rbbench_mfma_only(tools.stream, 10, C.byref(tf), C.byref(ms)) == 0
        calibration["mfma"] = {"tflops": tf.value, "avg_launch_ms": ms.value, "frac_of_published_peak":
                               tf.value / PEAK_BF16_TFLOPS, "kernel": "mfma_only_kernel: 32x32x16 bf16 multiplies only, "
                               "two waves per SIMD, 10 launches between one pair of events"}
    if args.calibrate_read:
        n = 39 * (1 << 20)
        rd = {}
        for label, flush in (("cold", tools.flush_handle()), ("warm", None)):
            g, ms = C.c_double(), C.c_double()
            assert tools.lib.rbbench_read(tools.stream, n, 20, flush, C.byref(g), C.byref(ms)) == 0
            rd[label] = {"gbs": g.value, "avg_launch_ms": ms.value, "frac_of_hbm_peak": g.value / PEAK_HBM_GBS}
        rd["bytes"] = n
        rd["note"] = ("warm: 20 launches of read_only_kernel between one pair of events; cold: a read-only sweep of "
                      "512 MiB before every launch, each launch in an event pair of its own, raw interval")
        calibration["read"] = rd
    if args.calibrate_library_gemm:
        calibration["library_gemm"] = library_gemm(w)
    if calibration:
        result["calibration"] = calibration
    if not args.no_backward:
        result["backward"] = backward_leg(dev, w, m["t"], m["x"], m["out"], m["bp"], args, m["alg"],
                                          with_cpu=args.backward and not args.no_cpu)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(m["t"])
    release(m)
    if not m["decode"] and not args.plain:
        tools.close()
        result["two_batches_in_flight"] = two_in_flight(w, m["t"], args.steps, args.warmup, max(3, min(args.repeats, 5)))
        tools = Tools(dev)
    if not args.only:
        # the other workloads, shorter loops: parity-test cases as far as the metric goes, reported for their
        # kernels' rooflines (C2: the decode-shaped target, with weights from HBM and cache-resident)
        others = {}
        for name in synth.WORKLOADS:
            if name == args.workload:
                continue
            o = measure(dev, tools, name, max(20, args.steps // 4), max(5, args.warmup // 2), max(3, min(args.repeats, 5)))
            others[name] = summary(o)
            release(o)
        # the int8 workload with f32 rows on the boundary: what a caller with f32 matrices and a quantized
        # checkpoint runs (the router reads the f32 rows, the products their bf16 copy)
        o = measure(dev, tools, "c5_int8_d768_e8", max(20, args.steps // 4), max(5, args.warmup // 2), 3, act_override="f32")
        others["c5_int8_d768_e8_f32_rows"] = summary(o)
        release(o)
        result["workloads"] = others
    tools.close()
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
