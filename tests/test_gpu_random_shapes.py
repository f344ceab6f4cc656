"""Seeded random shapes through every op against the CPU oracle: a net under the shape-specific tests, for the
seams between kernels (row tiles that do not divide N, K of odd block counts, one pair, 16 / 17 pairs, an
idle expert, a single expert, M on both sides of every routing threshold)."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import bits_to_dev, dev_to_bits, make_x, rel_l2, wire_to_dev

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


def _rand_k(rng, codec):
    wpb, _ = O.geometry(codec)
    return int(wpb * rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 24, 32] if wpb == 256 else [8, 9, 16, 24, 40, 64, 72, 90]))


@pytest.mark.parametrize("seed", range(40))
def test_random_dense(kq, seed):
    rng = np.random.default_rng(1000 + seed)
    codec = O.ALL_CODECS[seed % len(O.ALL_CODECS)]
    M = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 9, 16, 31, 32, 33, 70]))
    N = int(rng.choice([1, 7, 8, 31, 32, 33, 100, 127, 128, 129, 500, 1000]))
    K = _rand_k(rng, codec)
    dtype = "bfloat16" if seed % 2 else "float16"
    wire = _stack(codec, 1, N, K, seed)[0]
    xb, xt = make_x((M, K), dtype, seed=seed, scale=float(rng.choice([0.01, 1.0, 30.0])))
    got = kq.quantized_matmul(xt, wire_to_dev(wire), None, codec)
    assert rel_l2(dev_to_bits(got), O.qmm(xb, wire, codec, True, dtype), dtype) <= TOL, (codec, M, N, K, dtype)


@pytest.mark.parametrize("seed", range(40))
def test_random_moe(kq, seed):
    rng = np.random.default_rng(2000 + seed)
    codec = O.ALL_CODECS[(seed * 5) % len(O.ALL_CODECS)]
    E = int(rng.choice([1, 2, 5, 9]))
    N = int(rng.choice([8, 24, 64, 72, 136, 200]))
    K = _rand_k(rng, codec)
    T, R = int(rng.choice([1, 2, 4, 5, 8, 9, 17, 40])), int(rng.choice([1, 2, 4]))
    dtype = "bfloat16" if seed % 2 else "float16"
    gate, up = _stack(codec, E, N, K, seed), _stack(codec, E, N, K, seed + 500)
    idx = rng.integers(0, max(E - 1, 1), (T, R))  # the last expert stays idle when E > 1
    xb, xt = make_x((T, K), dtype, seed=seed, scale=0.05)
    act = ["silu", "gelu"][seed % 2]
    h = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act=act)
    want = O.moe_glu_gather(xb, gate, up, codec, idx, act, 0.0, None, None, 0.0, dtype)
    assert rel_l2(dev_to_bits(h), want, dtype) <= TOL, ("glu", codec, E, N, K, T, R, dtype)
    xb3, xt3 = make_x((T, R, K), dtype, seed=seed + 1, scale=0.05)
    y = kq.gather_qmv_kq(xt3, wire_to_dev(gate), codec, _idx_dev(idx))
    assert rel_l2(dev_to_bits(y), O.gather_qmv(xb3, gate, codec, idx, None, dtype), dtype) <= TOL, ("qmv", codec, E, N, K, T, R)
    lhs = rng.integers(0, T, T * R)
    g = kq.gather_qmm(xt3[:, :1], wire_to_dev(gate), None, codec, lhs_indices=_idx_dev(lhs), rhs_indices=_idx_dev(idx.reshape(-1)))
    wantg = O.gather_qmm(xb3[:, :1], gate, codec, lhs, idx.reshape(-1), True, dtype)
    assert rel_l2(dev_to_bits(g), wantg, dtype) <= TOL, ("gather_qmm", codec, E, N, K, T, R)
