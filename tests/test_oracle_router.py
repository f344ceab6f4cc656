"""The oracle's router top-k against the numpy formulas of the reference's own router test
(tests/test_moe_glu.py:453-551): softmax / sqrt-softplus scores, stable argsort for the picks, renormalised
mixing weights, shared-expert sigmoid.  CPU only."""
import numpy as np
import pytest

import oracle_lib as O


def _softmax(l):
    p = np.exp(l - l.max(-1, keepdims=True))
    return p / p.sum(-1, keepdims=True)


@pytest.mark.parametrize("e,r,norm", [(256, 8, True), (256, 8, False), (128, 4, True), (16, 2, True)])
def test_softmax_with_shared_gate(e, r, norm):
    rng = np.random.default_rng(5)
    logits = rng.standard_normal((5, e + 1)).astype(np.float32)
    idx, sc = O.router_topk(logits, "float32", r, norm, True)
    p = _softmax(logits[:, :e].astype(np.float64))
    top = np.argsort(-p, axis=-1, kind="stable")[:, :r]
    assert np.array_equal(idx, top)  # picks come out in rank order
    for t in range(5):
        pk = p[t, idx[t]]
        assert np.allclose(sc[t, :r], pk / (pk.sum() if norm else 1.0), rtol=1e-5, atol=1e-6)
        assert abs(sc[t, r] - 1.0 / (1.0 + np.exp(-logits[t, e]))) < 1e-6


@pytest.mark.parametrize("e,r", [(128, 8), (16, 4)])
def test_per_expert_scale_without_shared_gate(e, r):
    rng = np.random.default_rng(6)
    logits = rng.standard_normal((5, e)).astype(np.float32)
    pes = rng.uniform(0.5, 1.5, e).astype(np.float32)
    idx, sc = O.router_topk(logits, "float32", r, True, False, pes=pes)
    assert sc.shape == (5, r)
    p = _softmax(logits.astype(np.float64))
    assert np.array_equal(idx, np.argsort(-p, axis=-1, kind="stable")[:, :r])
    for t in range(5):
        pk = p[t, idx[t]]
        assert np.allclose(sc[t], pk / pk.sum() * pes[idx[t]], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("e,r,spread", [(256, 6, 1.0), (256, 6, 30.0), (64, 4, 1.0)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sqrtsoftplus_bias_scale_and_ties(e, r, spread, dtype):
    rng = np.random.default_rng(7)
    logits = (rng.standard_normal((7, e)) * spread).astype(np.float32)
    logits[5, 10:20] = logits[5, 10]  # exact ties at the boundary: smallest index wins
    bias = rng.standard_normal(e).astype(np.float32)
    stored = O.f32_to_bits(logits, dtype)
    lf = O.bits_to_f32(stored, dtype).astype(np.float64)
    idx, sc = O.router_topk(stored, dtype, r, True, False, bias=bias, scoring=1, scale=1.5)
    p = np.sqrt(np.logaddexp(lf, 0.0))
    top = np.argsort(-(p + bias), axis=-1, kind="stable")[:, :r]
    for t in range(7):
        if set(idx[t]) != set(top[t]):  # f32 softplus ulp noise at the boundary
            assert np.allclose(np.sort((p + bias)[t, idx[t]]), np.sort((p + bias)[t, top[t]]), rtol=0, atol=3e-6)
        pk = p[t, idx[t]]
        assert np.allclose(sc[t], pk / (pk.sum() + 1e-20) * 1.5, rtol=1e-5, atol=1e-6)
    tie_rank = (p + bias)[5]
    picked = [i for i in idx[5] if 10 <= i < 20]
    assert picked == sorted(picked)
    neg = (-np.abs(logits) - 50.0).astype(np.float32)
    _, sc = O.router_topk(neg, "float32", r, True, False, bias=bias, scoring=1, scale=1.5)
    assert np.all(np.isfinite(sc))
