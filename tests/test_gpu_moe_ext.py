"""GPU parity of the shared-expert GLU op and the slot-mixing down projections against the CPU oracle
(rel-L2 <= 1e-3 on the rounded outputs), over the kernel routes they can take: up to 16 pairs (gathered
kernels) and more (expert-grouped kernels), K-quant / other codecs, mixed shared-expert codecs."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import dev_to_bits, make_x, rel_l2, wire_to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _stack(codec, E, N, K, seed):
    wpb, bpb = O.geometry(codec)
    return O.synth_wire(codec, E * N * (K // wpb), seed).reshape(E, N, K // wpb * bpb)


def _idx_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a).astype(np.int64)).cuda()


@pytest.mark.parametrize("codec,shexp", [("q4_k", ""), ("q4_k", "q6_k"), ("q2_k", "q8_0"), ("iq4_xs", "q8_0"),
                                          ("mxfp4", ""), ("q8_0", "q6_k")])
@pytest.mark.parametrize("T,R", [(1, 4), (5, 3), (40, 2)])
@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_moe_glu_gather_shexp(kq, codec, shexp, T, R, act):
    E, N = 6, 72
    K = 512 if codec != "mxfp4" else 288
    sc = shexp or codec
    gate, up = _stack(codec, E, N, K, 21), _stack(codec, E, N, K, 22)
    sg, su = _stack(sc, 1, N, K, 23)[0], _stack(sc, 1, N, K, 24)[0]
    idx = np.random.default_rng(25).integers(0, E, (T, R))
    for dtype in ("bfloat16", "float16"):
        xb, xt = make_x((T, K), dtype, seed=26, scale=0.05)
        got = kq.moe_glu_gather_shexp_kq(xt, wire_to_dev(gate), wire_to_dev(up), wire_to_dev(sg), wire_to_dev(su), codec,
                                         _idx_dev(idx), act=act, shexp_kquant_type=shexp)
        assert tuple(got.shape) == (T, R + 1, N)
        want = O.moe_glu_gather_shexp(xb, gate, up, sg, su, codec, sc, idx, act, dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, shexp, T, R, act, dtype)
        # the routed slots are exactly what moe_glu_gather_kq gives
        plain = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act=act)
        assert torch.equal(got[:, :R], plain)


@pytest.mark.parametrize("codec,shexp", [("q6_k", ""), ("q4_k", "q8_0"), ("q3_k", "q6_k"), ("iq3_s", "q8_0"), ("mxfp4", "")])
@pytest.mark.parametrize("T,S", [(1, 5), (3, 4), (30, 3)])
def test_gather_qmv_mix(kq, codec, shexp, T, S):
    E, N = 5, 80
    K = 512 if codec != "mxfp4" else 288
    sc_codec = shexp or codec
    w, sw = _stack(codec, E, N, K, 31), _stack(sc_codec, 1, N, K, 32)[0]
    rng = np.random.default_rng(33)
    idx = rng.integers(0, E, (T, S - 1))
    scores = rng.uniform(0.05, 1.0, (T, S)).astype(np.float32)
    for dtype in ("bfloat16", "float16"):
        xb, xt = make_x((T, S, K), dtype, seed=34, scale=0.05)
        got = kq.gather_qmv_mix_kq(xt, wire_to_dev(w), wire_to_dev(sw), codec, _idx_dev(idx), torch.from_numpy(scores).cuda(),
                                   shexp_kquant_type=shexp)
        assert tuple(got.shape) == (T, N)
        want = O.gather_qmv_mix(xb, w, sw, codec, sc_codec, idx, scores, dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, shexp, T, S, dtype)


@pytest.mark.parametrize("codec", ["q4_k", "q6_k", "q2_k", "iq2_xxs", "q8_0", "mxfp4"])
@pytest.mark.parametrize("T,S", [(1, 8), (4, 4), (25, 2), (40, 2), (70, 2)])
def test_gather_qmv_mix_ns(kq, codec, T, S):
    E, N = 7, 64
    K = 768 if codec != "mxfp4" else 320
    w = _stack(codec, E, N, K, 41)
    rng = np.random.default_rng(42)
    idx = rng.integers(0, E, (T, S))
    scores = rng.uniform(0.05, 1.0, (T, S)).astype(np.float32)
    xb, xt = make_x((T, S, K), "bfloat16", seed=43, scale=0.05)
    got = kq.gather_qmv_mix_ns_kq(xt, wire_to_dev(w), codec, _idx_dev(idx), torch.from_numpy(scores).cuda())
    want = O.gather_qmv_mix(xb, w, None, codec, None, idx, scores, "bfloat16")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (codec, T, S)
    # one slot with score 1 is the plain gathered matvec, rounded once either way
    one = kq.gather_qmv_mix_ns_kq(xt[:, :1].contiguous(), wire_to_dev(w), codec, _idx_dev(idx[:, :1]),
                                  torch.ones((T, 1), device="cuda:0"))
    plain = kq.gather_qmv_kq(xt[:, :1].contiguous(), wire_to_dev(w), codec, _idx_dev(idx[:, :1]))[:, 0]
    if T > 64:
        # above 64 entries both ops run the same gathered kernels (the mix reads their f32 sums): bit-equal
        assert torch.equal(one, plain), (codec, T)
    else:
        # up to 64 entries the mix runs a kernel of its own: the f32 sums add in another order, so an element may
        # round to the neighbouring bf16 (2^-8 relative), or by the same absolute amount where the sum cancels
        a, b = one.float(), plain.float()
        bound = 2.0 ** -7 * torch.maximum(a.abs(), b.abs()) + 2.0 ** -8 * a.abs().mean()
        assert bool(((a - b).abs() <= bound).all()), (codec, T, float((a - b).abs().max()))


@pytest.mark.parametrize("T", [1, 3, 20])
@pytest.mark.parametrize("shared", [False, True])
def test_gather_qmv_mix_skips_expert_ids_outside_the_stack(kq, shared, T):
    """A slot whose expert id is >= E adds nothing, i.e. the result is the one with that slot's score set to zero
    (one token: the one-kernel form; 20: gathered matmuls into f32 slot rows, then the mix)."""
    codec, E, N, K, S = "q4_k", 4, 96, 512, 4
    w, sw = _stack(codec, E, N, K, 51), _stack(codec, 1, N, K, 52)[0]
    rng = np.random.default_rng(53)
    routed = S - 1 if shared else S
    idx = rng.integers(0, E, (T, routed))
    scores = rng.uniform(0.05, 1.0, (T, S)).astype(np.float32)
    bad, zeroed = idx.copy(), scores.copy()
    bad[0, 1], bad[T - 1, 0] = E, 0xFFFFFFF
    zeroed[0, 1] = zeroed[T - 1, 0] = 0.0
    _, xt = make_x((T, S, K), "bfloat16", seed=54, scale=0.05)

    def run(i, sc):
        if shared:
            return kq.gather_qmv_mix_kq(xt, wire_to_dev(w), wire_to_dev(sw), codec, _idx_dev(i), torch.from_numpy(sc).cuda())
        return kq.gather_qmv_mix_ns_kq(xt, wire_to_dev(w), codec, _idx_dev(i), torch.from_numpy(sc).cuda())

    assert torch.equal(run(bad, scores), run(idx, zeroed))


def test_validation(kq):
    x = torch.zeros((2, 3, 512), dtype=torch.bfloat16, device="cuda:0")
    w = torch.zeros((4, 8, 288), dtype=torch.uint8, device="cuda:0")
    sw = torch.zeros((8, 288), dtype=torch.uint8, device="cuda:0")
    idx2, idx3 = torch.zeros((2, 2), dtype=torch.int64, device="cuda:0"), torch.zeros((2, 3), dtype=torch.int64, device="cuda:0")
    sc = torch.ones((2, 3), device="cuda:0")
    with pytest.raises(ValueError):
        kq.gather_qmv_mix_kq(x, w, sw, "q4_k", idx3, sc)  # indices must be [T, S - 1]
    with pytest.raises(ValueError):
        kq.gather_qmv_mix_ns_kq(x, w, "q4_k", idx2, sc)  # indices must be [T, S]
    with pytest.raises(ValueError):
        kq.gather_qmv_mix_kq(x, w, sw, "q4_k", idx2, sc, shexp_kquant_type="q5_k")  # shared codec: same, q6_k or q8_0
    with pytest.raises(ValueError):
        kq.moe_glu_gather_shexp_kq(x[:, 0], w, w, sw, sw, "q4_k", idx2, act="silu_limit")
    with pytest.raises(ValueError):
        kq.moe_glu_gather_shexp_kq(x[:, 0], w, w, sw[:4], sw, "q4_k", idx2)
