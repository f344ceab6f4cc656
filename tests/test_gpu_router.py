"""GPU parity of kq.moe_router_topk against the CPU oracle: identical picks, scores within 1e-5 (the
reference's own tolerance; the f32 sums run in a different order)."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import bits_to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _check(kq, logits_f32, dtype, r, norm, shared, pes=None, bias=None, scoring="softmax", scale=1.0):
    stored = O.f32_to_bits(logits_f32, dtype)
    want_i, want_s = O.router_topk(stored, dtype, r, norm, shared, pes, bias, 1 if scoring == "sqrtsoftplus" else 0, scale)
    dev = lambda a: None if a is None else torch.from_numpy(a).cuda()
    got_i, got_s = kq.moe_router_topk(bits_to_dev(stored, dtype), r, norm, shared_gate=shared, per_expert_scale=dev(pes),
                                      bias=dev(bias), scoring=scoring, scale=scale)
    assert got_i.dtype == torch.int32 and tuple(got_i.shape) == want_i.shape
    assert got_s.dtype == torch.float32 and tuple(got_s.shape) == want_s.shape
    gi, gs = got_i.cpu().numpy().view(np.uint32), got_s.cpu().numpy()
    same = np.all(gi == want_i, axis=1)
    # rows whose picks differ may only differ through f32 summation-order noise in the scores that rank them
    assert same.mean() > 0.98, same.mean()
    assert np.allclose(gs[same], want_s[same], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
@pytest.mark.parametrize("e,r,norm", [(256, 8, True), (256, 8, False), (128, 4, True), (16, 2, True), (1024, 16, True),
                                      (5, 5, True)])
def test_softmax_shared_gate(kq, dtype, e, r, norm):
    logits = np.random.default_rng(e + r).standard_normal((37, e + 1)).astype(np.float32) * 2.0
    _check(kq, logits, dtype, r, norm, True)


@pytest.mark.parametrize("e,r", [(128, 8), (16, 4)])
def test_per_expert_scale(kq, e, r):
    rng = np.random.default_rng(8)
    logits = rng.standard_normal((9, e)).astype(np.float32)
    _check(kq, logits, "float32", r, True, False, pes=rng.uniform(0.5, 1.5, e).astype(np.float32))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("e,r,spread", [(256, 6, 1.0), (256, 6, 30.0), (64, 4, 1.0)])
def test_sqrtsoftplus_bias_ties(kq, dtype, e, r, spread):
    rng = np.random.default_rng(9)
    logits = (rng.standard_normal((7, e)) * spread).astype(np.float32)
    logits[5, 10:20] = logits[5, 10]
    bias = rng.standard_normal(e).astype(np.float32)
    _check(kq, logits, dtype, r, True, False, bias=bias, scoring="sqrtsoftplus", scale=1.5)
    _check(kq, (-np.abs(logits) - 50.0).astype(np.float32), "float32", r, True, False, bias=bias, scoring="sqrtsoftplus",
           scale=1.5)


def test_feeds_the_fused_moe_ops(kq):
    """indices / scores come out in the form the fused MoE ops take."""
    from gpu_util import make_x, wire_to_dev
    E, N, K, T, R = 8, 64, 512, 6, 2
    wire = O.synth_wire("q4_k", E * N * K // 256, 3).reshape(E, N, K // 256 * 144)
    logits = torch.randn((T, E), device="cuda:0")
    idx, sc = kq.moe_router_topk(logits, R, True, shared_gate=False)
    _, xt = make_x((T, K), "bfloat16", seed=4, scale=0.1)
    h = kq.moe_glu_gather_kq(xt, wire_to_dev(wire), wire_to_dev(wire[::-1].copy()), "q4_k", idx)
    assert tuple(h.shape) == (T, R, N) and torch.isfinite(h.float()).all()
    assert torch.allclose(sc.sum(-1), torch.ones(T, device="cuda:0"), atol=1e-5)


def test_validation(kq):
    l = torch.zeros((2, 9), device="cuda:0")
    with pytest.raises(ValueError):
        kq.moe_router_topk(l, 9, True)  # top_k > E (E = 8 with the shared gate)
    with pytest.raises(ValueError):
        kq.moe_router_topk(l, 2, False, scoring="sqrtsoftplus")
    with pytest.raises(ValueError):
        kq.moe_router_topk(l, 2, True, scoring="sigmoid")
    with pytest.raises(ValueError):
        kq.moe_router_topk(l[0], 2, True)
    with pytest.raises(ValueError):
        kq.moe_router_topk(l, 2, True, bias=torch.zeros(7, device="cuda:0"))
