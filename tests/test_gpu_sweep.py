"""Seeded sweeps of the forward and the backward pass against the CPU oracle, through the C ABI: shapes on and off
every kernel set's tiles, 1 to 100 experts, every dtype mix, padding masks (none, alternating, random, all rows
padding), a router bias, a shared expert of another width, and rows that stress the routing rules - NaN values,
values whose logits overflow to +-inf and NaN, zero rows, identical rows, identical router rows (ties), a NaN in
the router.  Routing tables, probabilities, log-sum-exp and gates must be identical in every bit (NaN in the same
places); outputs, losses and gradients within the layer's tolerance."""
import numpy as np
import pytest

import rustingbrain_amd as rb
from helpers import gpu_layer, oracle_layer, small_workload
from rustingbrain_amd import _lib as L
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu


def same_bits_or_same_nans(a, b):
    return np.array_equal(np.isnan(a), np.isnan(b)) and np.array_equal(a[~np.isnan(a)], b[~np.isnan(b)])


def rel_finite(a, b):
    if not np.array_equal(np.isfinite(a), np.isfinite(b)):
        return float("inf")
    m = np.isfinite(b)
    den = np.linalg.norm(b[m].astype(np.float64))
    return float(np.linalg.norm((a[m] - b[m]).astype(np.float64)) / max(den, 1e-30))


def draw_layer(rng, seed, modes, token_counts_generic):
    mode = str(rng.choice(modes))
    if mode in ("stream", "stream_i8", "decode", "decode_i8"):
        d, F, act = int(rng.choice([64, 128, 192, 320])), int(rng.choice([64, 128, 192])), "bf16"
        wt = "int8" if mode.endswith("i8") else "bf16"
        T = int(rng.integers(1, 33)) if mode.startswith("decode") else int(rng.choice([33, 64, 65, 127, 200, 513]))
    elif mode == "f32mc":
        d, F, act, wt = int(rng.choice([32, 64, 96])), int(rng.choice([32, 64, 160])), "f32", "f32"
        T = int(rng.choice([1, 7, 64, 65, 300]))
    elif mode == "mixed":
        d, F, act, wt = int(rng.choice([8, 24, 64])), int(rng.choice([6, 32, 64])), "f32", "bf16"
        T = int(rng.choice([1, 5, 33, 70]))
    else:
        d, F = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        act = wt = "f32" if mode == "generic_f32" else "bf16"
        T = int(rng.choice(token_counts_generic))
    E = int(rng.choice([1, 2, 3, 5, 8, 16, 17, 33, 64, 65, 100]))
    k = int(rng.integers(1, min(E, 8) + 1))
    shared = bool(rng.integers(0, 2))
    sdf = 0
    if shared:
        if mode in ("generic_f32", "generic_bf16", "mixed"):
            sdf = int(rng.integers(1, 40))
        else:
            sdf = int(rng.choice([64, 128])) if act == "bf16" else int(rng.choice([32, 64]))
    t = synth.make(small_workload(d=d, E=E, k=k, F=F, T=T, seed=int(seed), act=act, wt=wt, shared=shared,
                                  shared_d_ff=sdf))
    vm = str(rng.choice(["none", "alt", "all_padding", "random"], p=[0.5, 0.2, 0.1, 0.2]))
    valid = {"none": None, "alt": (np.arange(T) % 2 == 0).astype(np.uint8), "all_padding": np.zeros(T, np.uint8),
             "random": rng.integers(0, 2, T).astype(np.uint8)}[vm]
    bias = synth.normal((E,), 0.5, int(seed), 99) if rng.integers(0, 3) == 0 else None
    what = f"seed {seed}: {mode} d{d} F{F} E{E} k{k} T{T} shared {sdf if shared else 'no'} valid {vm} bias {bias is not None}"
    return t, valid, bias, what


FORWARD_MODES = ["generic_f32", "generic_bf16", "stream", "stream_i8", "f32mc", "decode", "decode_i8"]


@pytest.mark.parametrize("first", range(0, 240, 40))
def test_forward_sweep(device, first):
    for seed in range(first, first + 40):
        rng = np.random.default_rng(seed)
        t, valid, bias, what = draw_layer(rng, seed, FORWARD_MODES, [1, 2, 5, 31, 32, 33, 70])
        w = t.workload
        T, d, E = w.tokens, w.d_model, w.num_experts
        special = str(rng.choice(["none", "nan", "huge", "zeros", "same_rows", "same_router_rows", "overflow",
                                  "nan_in_router"], p=[0.23, 0.11, 0.11, 0.11, 0.11, 0.11, 0.11, 0.11]))
        x = t.x
        huge = synth.round_bf16(np.float32(3e38))
        if special == "nan":
            x[rng.integers(0, T), rng.integers(0, d)] = np.nan
        elif special == "huge":
            x[rng.integers(0, T), :] = huge if rng.integers(0, 2) else -huge
        elif special == "zeros":
            x[::2, :] = 0
        elif special == "same_rows" and T > 1:
            x[1:, :] = x[0:1, :]
        elif special == "same_router_rows" and E > 1:
            t.router[E - 1] = t.router[0]
        elif special == "overflow":
            x[rng.integers(0, T), :] = huge
            for e in range(E):
                pattern = rng.integers(0, 4)
                if pattern == 0:
                    t.router[e, :] = 2.0
                elif pattern == 1:
                    t.router[e, :] = -2.0
                elif pattern == 2:
                    t.router[e, :] = np.where(np.arange(d) % 2, 2.0, -2.0)
        elif special == "nan_in_router" and E > 1:
            t.router[rng.integers(0, E), rng.integers(0, d)] = np.nan
        what += f" rows {special}"
        ref = oracle_layer(t).forward(x, valid=valid, router_bias=bias, threads=4)
        layer = gpu_layer(device, t)
        layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
        out, cache = layer.forward_train(x, layout, router_bias=bias)
        n = int(ref.offsets[-1])
        for name in ("expert_of", "counts", "offsets"):
            assert np.array_equal(getattr(cache, name), getattr(ref, name)), f"{what}: {name}"
        assert np.array_equal(cache.perm_slot[:n], ref.perm_slot[:n]), f"{what}: perm_slot"
        assert np.array_equal(cache.perm_token[:n], ref.perm_token[:n]), f"{what}: perm_token"
        assert same_bits_or_same_nans(cache.probabilities, ref.probabilities), f"{what}: probabilities"
        assert same_bits_or_same_nans(cache.gate_of, ref.gate_of), f"{what}: gates"
        assert same_bits_or_same_nans(cache.log_sum_exp, ref.lse), f"{what}: log-sum-exp"
        tol = 1e-5 if (w.act_dtype == "f32" and w.weight_dtype == "f32") else 2e-2
        assert rel_finite(out, ref.out) <= tol, f"{what}: output"
        for name, got, want in (("aux", cache.aux_loss(), ref.aux_loss), ("z", cache.z_loss(), ref.z_loss)):
            if np.isfinite(want):
                assert abs(got - want) <= tol * max(abs(want), 1e-6), f"{what}: {name} {got} vs {want}"
            else:   # NaN, or the same infinity
                assert (np.isnan(got) and np.isnan(want)) or got == want, f"{what}: {name} {got} vs {want}"
        layer.close()


BACKWARD_MODES = ["generic_f32", "generic_bf16", "mixed", "stream", "f32mc"]


@pytest.mark.parametrize("first", range(0, 160, 40))
def test_backward_sweep(device, first):
    for seed in range(first, first + 40):
        rng = np.random.default_rng(1000 + seed)
        t, valid, bias, what = draw_layer(rng, 1000 + seed, BACKWARD_MODES, [1, 2, 5, 31, 32, 33, 70])
        w = t.workload
        aux_w, z_w = float(rng.choice([0.0, 0.01, 1.0])), float(rng.choice([0.0, 1e-3, 0.5]))
        gout = synth.round_bf16(rng.standard_normal(t.x.shape).astype(np.float32))
        if rng.integers(0, 5) == 0:
            gout[:] = 0     # only the two losses drive the router
        what += f" loss weights {aux_w}/{z_w}"
        ref = oracle_layer(t, aux_w=aux_w, z_w=z_w).backward(t.x, gout, valid=valid, router_bias=bias, threads=4)
        layer = gpu_layer(device, t, aux_w=aux_w, z_w=z_w, training=True)
        layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
        layer.forward_train(t.x, layout, router_bias=bias)
        gin = layer.backward(gout)
        all_f32 = w.act_dtype == "f32" and w.weight_dtype == "f32"
        # (f32 rows over bf16 weights multiply on the bf16 matrix cores where the widths allow: the bf16 bar)
        tol = 1e-5 if all_f32 else 2e-2
        # With one expert per token the gate is p / p: its gradient is an exact zero on paper and the difference
        # of two nearly equal quotients in f32 (src/moe.rs:438-441), so what reaches the router through it is
        # rounding noise of the size of the cancelled terms - in the reference as in both implementations here.
        # Differences are therefore measured against that size as well as against the result.
        floor = (1e-7 if all_f32 else 1e-3) * float(np.linalg.norm(gout)) * float(np.linalg.norm(t.x))

        def close(name, got, want):
            err = float(np.linalg.norm((got - want).astype(np.float64)))
            assert err <= tol * float(np.linalg.norm(want.astype(np.float64))) + floor, f"{what}: {name} off by {err}"

        close("grad_input", gin, ref.grad_input)
        close("router", layer.weight_grad(L.W_ROUTER), ref.grad_router)
        for e in range(min(w.num_experts, 6)):
            close(f"gate {e}", layer.weight_grad(L.W_GATE, e), ref.grad_gate[e])
            close(f"up {e}", layer.weight_grad(L.W_UP, e), ref.grad_up[e])
            close(f"down {e}", layer.weight_grad(L.W_DOWN, e), ref.grad_down[e])
        if t.shared is not None:
            close("shared gate", layer.weight_grad(L.W_SHARED_GATE), ref.grad_shared[0])
            close("shared down", layer.weight_grad(L.W_SHARED_DOWN), ref.grad_shared[2])
        layer.close()


@pytest.mark.parametrize("first", range(0, 120, 40))
def test_block_step_sweep(device, first):
    """x + layer(rmsnorm(x)): the norm in front (its own kernel, or inside the routing kernel of a few tokens) must
    hand the router the very rows the CPU path normalises, whatever the rows hold."""
    for seed in range(first, first + 40):
        rng = np.random.default_rng(5000 + seed)
        t, valid, bias, what = draw_layer(rng, 5000 + seed, FORWARD_MODES, [1, 2, 5, 31, 32, 33, 70])
        w = t.workload
        T, d = w.tokens, w.d_model
        bf16 = w.act_dtype == "bf16"
        rounder = synth.round_bf16 if bf16 else None
        norm_weight = (np.float32(1) + synth.normal((d,), 0.2, seed, 77)).astype(np.float32)
        eps = float(rng.choice([1e-6, 1e-5, 1e-2]))
        x = (t.x * np.float32(rng.choice([1.0, 1e-3, 50.0]))).astype(np.float32)
        if bf16:
            x = synth.round_bf16(x)
        special = str(rng.choice(["none", "nan", "huge", "zeros", "tiny"]))
        if special == "nan":
            x[rng.integers(0, T), rng.integers(0, d)] = np.nan
        elif special == "huge":      # the sum of squares overflows: inverse rms 0, normed row 0
            x[rng.integers(0, T), :] = synth.round_bf16(np.float32(3e38))
        elif special == "zeros":     # eps alone under the root
            x[::2, :] = 0
        elif special == "tiny":      # squares underflow
            x[rng.integers(0, T), :] = synth.round_bf16(np.float32(1e-30))
        what += f" rows {special} eps {eps}"
        want, _, ref = oracle_layer(t).forward_block(x, norm_weight, eps, valid=valid, router_bias=bias, threads=4,
                                                     round_normed=rounder)
        cfg = rb.MoeConfig(w.num_experts, w.experts_per_token, w.d_ff, w.shared_expert)
        layer = rb.MoeLayer(d, cfg, device, act_dtype=w.act_dtype, weight_dtype=w.weight_dtype, max_tokens=T,
                            shared_d_ff=w.shared_d_ff if w.shared_expert else 0)
        layer.set_feed_forward_norm(norm_weight, eps)
        layer.load_tensors(t)
        layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
        out, cache = layer.forward_block(x, layout, router_bias=bias)
        for name in ("expert_of", "counts", "offsets"):
            assert np.array_equal(getattr(cache, name), getattr(ref, name)), f"{what}: {name}"
        assert same_bits_or_same_nans(cache.probabilities, ref.probabilities), f"{what}: probabilities"
        assert same_bits_or_same_nans(cache.gate_of, ref.gate_of), f"{what}: gates"
        tol = 1e-5 if (w.act_dtype == "f32" and w.weight_dtype == "f32") else 2e-2
        assert rel_finite(out, want) <= tol, f"{what}: output"
        layer.close()


@pytest.mark.parametrize("first", range(0, 60, 20))
def test_call_sequences_on_one_layer(device, first):
    """One layer sized for 300 rows, seven calls of other sizes in a row (no rows, a few rows on the decode-shaped
    path, hundreds on the large-batch path, the full size), with and without padding masks and bias, a backward
    pass after some of them with the gradients cleared or accumulating: no call may see what an earlier one left
    behind."""
    for seed in range(first, first + 20):
        rng = np.random.default_rng(9000 + seed)
        mode = str(rng.choice(["stream", "stream_i8", "f32mc", "generic_f32", "generic_bf16"]))
        training = bool(rng.integers(0, 2)) and mode != "stream_i8"
        if mode.startswith("stream"):
            d, F, act = int(rng.choice([64, 128])), int(rng.choice([64, 128])), "bf16"
            wt = "int8" if mode.endswith("i8") else "bf16"
        elif mode == "f32mc":
            d, F, act, wt = int(rng.choice([32, 64])), int(rng.choice([32, 96])), "f32", "f32"
        else:
            d, F = int(rng.integers(1, 40)), int(rng.integers(1, 40))
            act = wt = "f32" if mode == "generic_f32" else "bf16"
        E = int(rng.choice([1, 3, 8, 17, 64]))
        k = int(rng.integers(1, min(E, 6) + 1))
        shared = bool(rng.integers(0, 2))
        sdf = (int(rng.integers(1, 40)) if mode.startswith("generic") else (64 if act == "bf16" else 32)) if shared else 0
        rows = 300
        t = synth.make(small_workload(d=d, E=E, k=k, F=F, T=rows, seed=9000 + seed, act=act, wt=wt, shared=shared,
                                      shared_d_ff=sdf))
        about = f"seed {seed}: {mode} training {training} d{d} F{F} E{E} k{k} shared {sdf}"
        oracle = oracle_layer(t)
        layer = gpu_layer(device, t, max_tokens=rows, training=training)
        tol = 1e-5 if (act == "f32" and wt == "f32") else 2e-2
        for call in range(7):
            T = int(rng.choice([0, 1, 3, 8, 32, 33, 100, 257, 300]))
            x = t.x[rng.permutation(rows)[:T]].copy()
            valid = None if rng.integers(0, 2) else rng.integers(0, 2, T).astype(np.uint8)
            bias = synth.normal((E,), 0.5, seed, call) if rng.integers(0, 3) == 0 else None
            what = f"{about} call {call} T{T} mask {valid is not None} bias {bias is not None}"
            layout = rb.Layout(valid=None if valid is None else [bool(v) for v in valid])
            out, cache = layer.forward_train(x, layout, router_bias=bias)
            if T == 0:
                assert out.shape == (0, d), what
                continue
            ref = oracle.forward(x, valid=valid, router_bias=bias, threads=4)
            for name in ("expert_of", "counts", "offsets"):
                assert np.array_equal(getattr(cache, name), getattr(ref, name)), f"{what}: {name}"
            assert same_bits_or_same_nans(cache.probabilities, ref.probabilities), f"{what}: probabilities"
            assert rel_finite(out, ref.out) <= tol, f"{what}: output"
            assert abs(cache.aux_loss() - ref.aux_loss) <= tol * max(abs(ref.aux_loss), 1e-6), f"{what}: aux"
            if not (training and rng.integers(0, 2)):
                continue
            gout = synth.round_bf16(rng.standard_normal(x.shape).astype(np.float32))
            watched = ((L.W_ROUTER, 0), (L.W_DOWN, 0), (L.W_GATE, E - 1))
            if rng.integers(0, 2):
                layer.zero_grads()
                before = [0.0, 0.0, 0.0]
            else:
                before = [layer.weight_grad(which, e) for which, e in watched]
            gin = layer.backward(gout)
            want = oracle.backward(x, gout, valid=valid, router_bias=bias, threads=4)
            floor = (1e-7 if act == "f32" else 1e-3) * float(np.linalg.norm(gout)) * float(np.linalg.norm(x))

            def close(name, got, wanted):
                err = float(np.linalg.norm((got - wanted).astype(np.float64)))
                assert err <= tol * float(np.linalg.norm(wanted.astype(np.float64))) + floor, f"{what}: {name} off by {err}"

            close("grad_input", gin, want.grad_input)
            for (which, e), old, wanted in zip(watched, before, (want.grad_router, want.grad_down[0], want.grad_gate[E - 1])):
                close(f"weight {which}/{e}", layer.weight_grad(which, e) - old, wanted)
        layer.close()
