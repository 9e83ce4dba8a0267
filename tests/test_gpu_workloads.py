"""The five benchmark workloads at full size on the GPU against the oracle:
bit-exact routing, outputs and losses within the stated rel-L2, plus properties
that do not need the oracle (permutation is a bijection, counts add up, a token
never meets the same expert twice)."""
import os

import numpy as np
import pytest

import rustingbrain_amd as rb
from conftest import rel_l2
from helpers import assert_routing_identical, gpu_layer, oracle_layer, tolerance
from rustingbrain_amd import synth

pytestmark = pytest.mark.gpu

THREADS = min(16, os.cpu_count() or 8)


def routing_properties(cache, T, E, k):
    R = int(cache.offsets[E])
    assert R == T * k == int(cache.counts.sum())
    assert np.array_equal(np.sort(cache.perm_slot), np.arange(T * k))
    assert np.array_equal(cache.offsets, np.concatenate([[0], np.cumsum(cache.counts)]))
    assert np.array_equal(cache.perm_token, cache.perm_slot // k)
    experts = cache.expert_of.reshape(T, k)
    assert np.all(np.sort(experts, axis=1)[:, 1:] != np.sort(experts, axis=1)[:, :-1]) if k > 1 else True
    for e in range(E):
        seg = cache.perm_slot[cache.offsets[e]:cache.offsets[e + 1]]
        assert np.all(np.diff(seg) > 0)
        assert np.all(cache.expert_of[seg] == e)
    g = cache.gate_of.reshape(T, k)
    assert np.all(np.abs(g.sum(axis=1) - 1.0) < 1e-5)
    assert np.all(np.diff(cache.probabilities[np.arange(T)[:, None], experts], axis=1) <= 0)


@pytest.mark.parametrize("name", list(synth.WORKLOADS))
def test_workload_matches_the_oracle(device, name):
    t = synth.make(name)
    w = t.workload
    ref = oracle_layer(t).forward(t.x, router_bias=t.router_bias, threads=THREADS)
    layer = gpu_layer(device, t)
    out, cache = layer.forward_train(t.x, router_bias=t.router_bias)
    assert_routing_identical(cache, ref)
    routing_properties(cache, w.tokens, w.num_experts, w.experts_per_token)
    tol = tolerance(w)
    err = rel_l2(out, ref.out)
    print(f"{name}: kernel={layer.kernel_name()} out rel-L2 {err:.3e} aux {cache.aux_loss():.6f}/{ref.aux_loss:.6f} "
          f"z {cache.z_loss():.6f}/{ref.z_loss:.6f} near-ties(4ulp) "
          f"{__import__('oracle.rb_oracle', fromlist=['x']).near_ties(ref.probabilities, w.experts_per_token, 4)}")
    assert err <= tol
    assert abs(cache.aux_loss() - ref.aux_loss) <= tol * abs(ref.aux_loss)
    assert abs(cache.z_loss() - ref.z_loss) <= tol * abs(ref.z_loss)
    if w.skew_share:
        assert abs(cache.load_fractions()[0] - w.skew_share) < 0.011
    layer.close()
