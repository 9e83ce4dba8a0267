"""Pins of the oracle's RmsNorm::forward (src/norm.rs:41-61, :128-131) and of the block step built on it
(src/transformer_block.rs:216-222).

* the reference's three forward tests (src/norm.rs:138-170), with their inputs and tolerances;
* a float64 closed form on random rows (a dropped eps, a mean taken over the wrong length, a missing weight or
  a subtracted mean each fails it);
* the summation order: the sum of squares is taken in index order in f32 (a row built so that pairwise or
  reversed summation gives different bits);
* the block step: output = moe(normed) + residual, checked against the oracle's own layer on the normed rows
  (composition only; the layer itself is pinned elsewhere).
No GPU."""
import numpy as np

from helpers import oracle_layer, small_workload
from oracle import rb_oracle as orc
from rustingbrain_amd import synth


def test_forward_normalizes_to_unit_rms():
    out = orc.rmsnorm(np.array([[1.0, 2.0, 3.0, 4.0]], np.float32), np.ones(4, np.float32), 1e-6)
    assert abs(float((out * out).sum(dtype=np.float32)) / 4.0 - 1.0) < 1e-4


def test_forward_does_not_subtract_the_mean():
    out = orc.rmsnorm(np.full((1, 3), 5.0, np.float32), np.ones(3, np.float32), 1e-6)
    assert np.all(np.abs(out - 1.0) < 1e-4)


def test_weight_scales_each_channel():
    out = orc.rmsnorm(np.ones((1, 2), np.float32), np.array([2.0, 0.5], np.float32), 1e-6)
    assert abs(out[0, 0] - 2.0) < 1e-4 and abs(out[0, 1] - 0.5) < 1e-4


def test_matches_the_closed_form_in_float64():
    rng = np.random.default_rng(5)
    for T, d, eps in ((7, 33, 1e-6), (3, 768, 1e-5), (1, 1, 1e-6), (4, 64, 0.5)):
        x = (rng.standard_normal((T, d)) * 3.0).astype(np.float32)
        w = rng.uniform(0.5, 1.5, d).astype(np.float32)
        got = orc.rmsnorm(x, w, eps)
        x64 = x.astype(np.float64)
        want = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + np.float64(np.float32(eps))) * w.astype(np.float64)
        assert np.max(np.abs(got - want)) <= 2e-6 * np.max(np.abs(want))


def test_large_eps_is_not_dropped():
    x = np.array([[3.0, 4.0]], np.float32)       # mean square 12.5
    out = orc.rmsnorm(x, np.ones(2, np.float32), 12.5)
    assert np.allclose(out, x / 5.0, rtol=1e-6)  # sqrt(12.5 + 12.5) = 5


def test_sum_of_squares_runs_in_index_order():
    # 1 followed by many tiny squares: added one by one after the 1 they vanish; any tree or reversed order keeps them
    d = 4097
    x = np.full((1, d), 2.0 ** -13, np.float32)
    x[0, 0] = 1.0
    got = orc.rmsnorm(x, np.ones(d, np.float32), 0.0)
    seq = np.float32(1.0)
    for _ in range(d - 1):
        seq = np.float32(seq + np.float32(2.0 ** -26))
    assert seq == np.float32(1.0)
    inv = np.float32(1.0) / np.sqrt(np.float32(seq / np.float32(d)))
    assert got[0, 0] == np.float32(np.float32(1.0) * inv)
    pairwise = np.float32(1.0 + (d - 1) * 2.0 ** -26)
    assert pairwise != seq


def test_zero_row_stays_zero():
    out = orc.rmsnorm(np.zeros((2, 8), np.float32), np.ones(8, np.float32), 1e-6)
    assert not out.any()


def test_block_step_is_norm_then_layer_then_residual():
    t = synth.make(small_workload(d=16, E=4, k=2, F=12, T=9, seed=31, shared=True))
    layer = oracle_layer(t)
    rng = np.random.default_rng(6)
    w = rng.uniform(0.5, 1.5, 16).astype(np.float32)
    out, normed, res = layer.forward_block(t.x, w, 1e-6)
    assert np.array_equal(normed, orc.rmsnorm(t.x, w, 1e-6))
    again = layer.forward(normed)
    assert np.array_equal(res.expert_of, again.expert_of)
    assert np.array_equal(out, again.out + t.x)
    # padding rows: the residual passes through (plus the shared expert of the normed row, src/moe.rs:313-319)
    valid = np.array([1, 0, 1, 1, 0, 1, 1, 1, 1], np.uint8)
    outp, _, resp = layer.forward_block(t.x, w, 1e-6, valid=valid)
    assert np.all(resp.expert_of.reshape(9, 2)[valid == 0] == -1)
    assert np.array_equal(outp, resp.out + t.x)
