"""The routing decisions of the five benchmark workloads do not hinge on the last bits of the logits.

The oracle computes a logit in the reference's eight-lane f32 order (src/matrix.rs:26-40); the reference itself
takes matrixmultiply's order for more than one row, and libm's exp (both outside its repository).  If the choice of
experts depended on such last-place differences, bit-exact parity between the device path and the oracle would say
little about parity with the Rust binary.  So: the same routing from a float64 evaluation (numpy product, float64
softmax, stable descending sort = top-k with ties to the lower index, src/moe.rs:566-581) must pick the same
experts for every token that the census of near ties (k-th and (k+1)-th probability within 4 ulp) does not list
- and the census is empty for all five workloads.  No GPU."""
import numpy as np
import pytest

from oracle import rb_oracle as orc
from rustingbrain_amd import synth


@pytest.mark.parametrize("name", list(synth.WORKLOADS))
def test_float64_routing_picks_the_same_experts(name):
    t = synth.make(name)
    w = t.workload
    k, E = w.experts_per_token, w.num_experts
    logits = orc.router_logits(t.x, t.router, t.router_bias)
    P, _ = orc.softmax_rows(logits)
    expert_of, _ = orc.route(P, k)
    l64 = t.x.astype(np.float64) @ t.router.astype(np.float64).T
    if t.router_bias is not None:
        l64 += t.router_bias.astype(np.float64)
    # the oracle's own float64 logits (a plain sum in index order) agree with numpy's
    assert np.max(np.abs(orc.router_logits_f64(t.x, t.router, t.router_bias) - l64)) < 1e-9
    assert np.max(np.abs(logits - l64)) < 1e-4
    p64 = np.exp(l64 - l64.max(axis=1, keepdims=True))
    p64 /= p64.sum(axis=1, keepdims=True)
    want = np.argsort(-p64, axis=1, kind="stable")[:, :k].astype(np.int32)
    got = expert_of.reshape(-1, k)
    differing = np.nonzero((want != got).any(axis=1))[0]
    ties = orc.near_ties(P, k, 4)
    print(f"{name}: {differing.size} of {got.shape[0]} tokens route differently in float64; near ties (4 ulp): {ties}")
    assert ties == 0
    assert differing.size == 0
