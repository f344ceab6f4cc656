"""The oracle's shared-expert GLU and slot-mixing down projection against numpy compositions (float64
dequantize + matmul), the way the reference's own test states them (tests/test_moe_glu.py:234-310).  CPU only."""
import numpy as np
import pytest

import oracle_lib as O


def _stack(codec, E, N, K, seed):
    wpb, bpb = O.geometry(codec)
    return O.synth_wire(codec, E * N * (K // wpb), seed).reshape(E, N, K // wpb * bpb)


def _deq(wire, codec, K):
    return O.dequantize(wire.reshape(-1, wire.shape[-1]), codec).reshape(*wire.shape[:-1], K).astype(np.float64)


def _silu(g):
    return g / (1.0 + np.exp(-g))


@pytest.mark.parametrize("codec,shexp", [("q4_k", "q4_k"), ("q4_k", "q6_k"), ("iq4_xs", "q8_0")])
def test_shexp_glu(codec, shexp):
    E, N, K, T, R = 5, 24, 512, 4, 3
    gate, up = _stack(codec, E, N, K, 1), _stack(codec, E, N, K, 2)
    sg, su = _stack(shexp, 1, N, K, 3)[0], _stack(shexp, 1, N, K, 4)[0]
    idx = np.random.default_rng(5).integers(0, E, (T, R))
    xb = O.f32_to_bits((np.random.default_rng(6).standard_normal((T, K)) * 0.1).astype(np.float32), "bfloat16")
    got = O.bits_to_f32(O.moe_glu_gather_shexp(xb, gate, up, sg, su, codec, shexp, idx), "bfloat16")
    x = O.bits_to_f32(xb, "bfloat16").astype(np.float64)
    G, U, SG, SU = _deq(gate, codec, K), _deq(up, codec, K), _deq(sg, shexp, K), _deq(su, shexp, K)
    want = np.empty((T, R + 1, N))
    for t in range(T):
        for r in range(R):
            want[t, r] = _silu(x[t] @ G[idx[t, r]].T) * (x[t] @ U[idx[t, r]].T)
        want[t, R] = _silu(x[t] @ SG.T) * (x[t] @ SU.T)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 4e-3  # bf16 rounding of the outputs


@pytest.mark.parametrize("codec,shexp", [("q6_k", "q6_k"), ("q4_k", "q8_0"), ("mxfp4", None)])
def test_mix(codec, shexp):
    E, N, T, S = 6, 40, 3, 4
    K = 512 if codec != "mxfp4" else 288
    w = _stack(codec, E, N, K, 11)
    sw = None if shexp is None else _stack(shexp, 1, N, K, 12)[0]
    rng = np.random.default_rng(13)
    idx = rng.integers(0, E, (T, S - 1 if sw is not None else S))
    sc = rng.uniform(0.05, 1.0, (T, S)).astype(np.float32)
    xb = O.f32_to_bits((rng.standard_normal((T, S, K)) * 0.1).astype(np.float32), "bfloat16")
    got = O.bits_to_f32(O.gather_qmv_mix(xb, w, sw, codec, shexp, idx, sc), "bfloat16")
    x = O.bits_to_f32(xb, "bfloat16").astype(np.float64)
    W = _deq(w, codec, K)
    want = np.zeros((T, N))
    for t in range(T):
        for s in range(S):
            m = W[idx[t, s]] if (sw is None or s < S - 1) else _deq(sw, shexp, K)
            want[t] += sc[t, s] * (x[t, s] @ m.T)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 4e-3
