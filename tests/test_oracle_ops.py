"""Pins the oracle's matmul / gather / fused-MoE functions against plain numpy float64 maths on the
oracle's (separately pinned) decoded weights: `x @ deq(W).T`, the per-entry gather definition of the
reference's tests/test_gather.py:171-176 and the GLU formulas of tests/test_moe_glu.py:139-160."""
import numpy as np
import pytest

import oracle_lib as O


def _wire(codec, N, K, seed):
    wpb, bpb = O.geometry(codec)
    return O.synth_wire(codec, N * (K // wpb), seed).reshape(N, K // wpb * bpb)


def _rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b) / np.linalg.norm(b))


@pytest.mark.parametrize("codec", ["q4_k", "q6_k", "iq2_xxs", "mxfp4", "q5_1"])
@pytest.mark.parametrize("M", [1, 16, 17, 40])  # both sides of the fused / dequant-then-GEMM switch
def test_qmm_matches_numpy(codec, M):
    N, K = 48, 512 if codec != "mxfp4" else 288
    wire = _wire(codec, N, K, seed=3)
    x = np.random.default_rng(M).standard_normal((M, K)).astype(np.float32)
    w = O.dequantize(wire, codec).astype(np.float64)
    got = O.qmm(x, wire, codec, True, "float32")
    assert _rel(got, x.astype(np.float64) @ w.T) < 5e-6
    # half types: one rounding of the f32 result, activations upcast exactly
    for dt in ("float16", "bfloat16"):
        xb = O.f32_to_bits(x, dt)
        xf = O.bits_to_f32(xb, dt)
        got = O.qmm(xb, wire, codec, True, dt)
        assert np.array_equal(got, O.f32_to_bits(O.qmm(xf, wire, codec, True, "float32"), dt))


def test_qmm_no_transpose_matches_numpy():
    K, N, M = 24, 512, 3
    wire = _wire("q4_k", K, N, seed=4)  # decodes to [K, N]
    x = np.random.default_rng(0).standard_normal((M, K)).astype(np.float32)
    w = O.dequantize(wire, "q4_k").astype(np.float64)
    assert _rel(O.qmm(x, wire, "q4_k", False, "float32"), x.astype(np.float64) @ w) < 5e-6


def test_gather_matches_per_entry_definition_and_dedupes():
    codec, E, N, K, M = "q5_k", 4, 32, 256, 2
    wire = np.stack([_wire(codec, N, K, seed=10 + e) for e in range(E)])
    x = np.random.default_rng(1).standard_normal((6, M, K)).astype(np.float32)
    lhs = np.array([5, 5, 0, 3, 5, 1, 2, 2, 4])
    rhs = np.array([1, 1, 3, 0, 1, 2, 2, 2, 0])
    got = O.gather_qmm(x, wire, codec, lhs, rhs, True, "float32")
    for i in range(len(lhs)):
        w = O.dequantize(wire[rhs[i]], codec).astype(np.float64)
        assert _rel(got[i], x[lhs[i]].astype(np.float64) @ w.T) < 5e-6
    assert np.array_equal(got[0], got[1]) and np.array_equal(got[0], got[4]) and np.array_equal(got[6], got[7])
    # a large group (rows * M > 16) goes down the dequant-then-GEMM path; same definition
    lhs2 = np.arange(40) % 6
    rhs2 = np.zeros(40, dtype=np.int64)
    got2 = O.gather_qmm(x, wire, codec, lhs2, rhs2, True, "float32")
    w0 = O.dequantize(wire[0], codec).astype(np.float64)
    for i in range(40):
        assert _rel(got2[i], x[lhs2[i]].astype(np.float64) @ w0.T) < 5e-6


def _act_np(g, act):
    if act == "gelu":
        return 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
    return g / (1.0 + np.exp(-g))


def _glu_np(g, u, act, limit=0.0, alpha=1.0):
    if act == "swiglu_clamp":
        g = np.minimum(g, limit)
        u = np.clip(u, -limit, limit)
        return (g / (1.0 + np.exp(-alpha * g))) * (u + 1.0)
    if act == "silu_limit":
        g = np.minimum(g, limit)
        u = np.clip(u, -limit, limit)
        act = "silu"
    return _act_np(g, act) * u


@pytest.mark.parametrize("act,limit,alpha,biased", [("silu", 0, 0, False), ("gelu", 0, 0, False),
                                                    ("silu_limit", 0.7, 0, False), ("swiglu_clamp", 7.0, 1.702, True)])
def test_moe_glu_matches_numpy(act, limit, alpha, biased):
    codec = "mxfp4" if biased else "q4_k"
    E, N, K, T, R = 3, 24, 512 if not biased else 288, 4, 2
    gate = np.stack([_wire(codec, N, K, seed=20 + e) for e in range(E)])
    up = np.stack([_wire(codec, N, K, seed=30 + e) for e in range(E)])
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((T, K)) * 0.3).astype(np.float32)
    idx = rng.integers(0, E, (T, R))
    gb = (rng.standard_normal((E, N)) * 0.01).astype(np.float32) if biased else None
    ub = (rng.standard_normal((E, N)) * 0.01).astype(np.float32) if biased else None
    xb = O.f32_to_bits(x, "bfloat16")
    xf = O.bits_to_f32(xb, "bfloat16").astype(np.float64)
    got = O.bits_to_f32(O.moe_glu_gather(xb, gate, up, codec, idx, act, limit, gb, ub, alpha, "bfloat16"), "bfloat16")
    want = np.zeros((T, R, N))
    for t in range(T):
        for r in range(R):
            e = idx[t, r]
            g = xf[t] @ O.dequantize(gate[e], codec).astype(np.float64).T
            u = xf[t] @ O.dequantize(up[e], codec).astype(np.float64).T
            if biased:
                g, u = g + gb[e], u + ub[e]
            want[t, r] = _glu_np(g, u, act, limit, alpha if alpha else 1.0)
    # bf16 output rounding alone is ~1.7e-3 relative; the f32 pipeline underneath is what is pinned
    assert _rel(got, want) < 3e-3
    want_b = O.bits_to_f32(O.f32_to_bits(want.astype(np.float32), "bfloat16"), "bfloat16")
    big = np.abs(want) > 1e-3  # f32 tanh/exp saturate where float64 keeps a ~1e-14 residue
    assert np.mean(got[big] != want_b[big]) < 0.02  # only rounding-boundary flips may differ
    # gather_qmv
    h = (rng.standard_normal((T, R, K)) * 0.3).astype(np.float32)
    hb = O.f32_to_bits(h, "float16")
    hf = O.bits_to_f32(hb, "float16").astype(np.float64)
    got = O.bits_to_f32(O.gather_qmv(hb, gate, codec, idx, gb, "float16"), "float16")
    want = np.stack([np.stack([hf[t, r] @ O.dequantize(gate[idx[t, r]], codec).astype(np.float64).T
                               + (gb[idx[t, r]] if biased else 0) for r in range(R)]) for t in range(T)])
    assert _rel(got, want) < 1e-3


def test_glu_epilogue_scalar_values():
    f = O.lib.kq_oracle_glu_epilogue
    for g, u in [(-3.0, 2.0), (0.0, 1.0), (0.5, -0.25), (9.0, 10.0)]:
        assert abs(f(0, g, u, 0.0, 0.0) - g / (1 + np.exp(-g)) * u) < 1e-6 * max(1, abs(g * u))
        assert abs(f(1, g, u, 0.0, 0.0) - _act_np(np.float64(g), "gelu") * u) < 2e-6 * max(1, abs(g * u))
        assert abs(f(2, g, u, 1.5, 0.0) - _glu_np(np.float64(g), np.float64(u), "silu_limit", 1.5)) < 1e-6 * 10
        assert abs(f(3, g, u, 7.0, 1.702) - _glu_np(np.float64(g), np.float64(u), "swiglu_clamp", 7.0, 1.702)) < 1e-5
