"""GPU parity of the batched MoE ops on mxfp4 stacks, which run on the block-scaled matrix instruction (wire blocks
undecoded, activations as e4m3 terms with a power-of-two scale per 32): against the CPU oracle on the same inputs,
rel-L2 <= 1e-3 on the rounded outputs.  Covers both activation dtypes (two / three terms), K with a tail of
blocks, ragged N, both segment forms (up to 16 pairs per workgroup, two m-tiles per workgroup), expert ids out of
range, biases with swiglu_clamp, activations of wide dynamic range inside a 32-block, zero blocks, and scale bytes
at the ends of the e8m0 range the reference decodes as finite numbers."""
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


def _stack(E, N, K, seed):
    return O.synth_wire("mxfp4", E * N * K // 32, seed=seed).reshape(E, N, K // 32 * 17)


def _idx_dev(idx):
    return torch.from_numpy(np.ascontiguousarray(idx, dtype=np.int64)).cuda()


@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
@pytest.mark.parametrize("E,N,K,T,R", [(4, 136, 288, 9, 1),      # 9 pairs: the smallest batch this kernel takes (K tail)
                                       (8, 200, 2880 // 5, 12, 4),  # 48 pairs, K = 576 = 4 steps + 2 blocks
                                       (2, 64, 1024, 20, 2),     # 40 pairs on 2 experts: two m-tiles per workgroup
                                       (3, 72, 160, 70, 1)])     # segments of 32 and a ragged rest
def test_fp4_gather_qmv(kq, dtype, E, N, K, T, R):
    wire = _stack(E, N, K, seed=3)
    rng = np.random.default_rng(4)
    idx = rng.integers(0, E, (T, R))
    bias = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
    xb, xt = make_x((T, R, K), dtype, seed=5, scale=0.3)
    for b in (None, bias):
        got = kq.gather_qmv_kq(xt, wire_to_dev(wire), "mxfp4", _idx_dev(idx), bias=None if b is None else torch.from_numpy(b).cuda())
        want = O.gather_qmv(xb, wire, "mxfp4", idx, b, dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (dtype, E, N, K, T, R, b is not None)


@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
@pytest.mark.parametrize("act", ["silu", "gelu", "swiglu_clamp"])
def test_fp4_moe_glu(kq, dtype, act):
    E, N, K, T, R = 5, 104, 352, 24, 3
    gate, up = _stack(E, N, K, seed=6), _stack(E, N, K, seed=7)
    rng = np.random.default_rng(8)
    idx = rng.integers(0, E, (T, R))
    xb, xt = make_x((T, K), dtype, seed=9, scale=0.2)
    kw, okw = {}, {}
    if act == "swiglu_clamp":
        gb = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
        ub = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
        kw = dict(limit=7.0, alpha=1.702, gate_bias=torch.from_numpy(gb).cuda(), up_bias=torch.from_numpy(ub).cuda())
        okw = dict(limit=7.0, alpha=1.702, gate_bias=gb, up_bias=ub)
    got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), "mxfp4", _idx_dev(idx), act=act, **kw)
    want = O.moe_glu_gather(xb, gate, up, "mxfp4", idx, act, dtype=dtype, **okw)
    assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (dtype, act)


def test_fp4_out_of_range_experts_are_skipped(kq):
    """Pairs whose expert id is outside the stack leave their output rows untouched; the others are right."""
    E, N, K, T, R = 3, 64, 256, 30, 1
    wire = _stack(E, N, K, seed=10)
    rng = np.random.default_rng(11)
    idx = rng.integers(0, E, (T, R))
    bad = [2, 11, 29]
    idx_dev = idx.copy()
    idx_dev[bad, 0] = [E, E + 7, 2 ** 31 - 1]
    xb, xt = make_x((T, R, K), "bfloat16", seed=12, scale=0.3)
    got = dev_to_bits(kq.gather_qmv_kq(xt, wire_to_dev(wire), "mxfp4", _idx_dev(idx_dev)))
    want = O.gather_qmv(xb, wire, "mxfp4", idx, None, "bfloat16")
    keep = [t for t in range(T) if t not in bad]
    assert rel_l2(got[keep], want[keep], "bfloat16") <= TOL


def test_fp4_activation_range_inside_a_block_and_extreme_scales(kq):
    """Activations that span many binades inside one 32-block (the e4m3 terms share one power of two per block),
    all-zero activation blocks, and wire scale bytes from 1 to 254: every output row within tolerance on its own."""
    E, N, K, T = 2, 48, 512, 20
    wire = _stack(E, N, K, seed=13).reshape(E, N, K // 32, 17).copy()
    rng = np.random.default_rng(14)
    wire[0, :, 3, 0] = 1          # 2^-127 blocks
    wire[0, :, 5, 0] = 150
    wire[1, :, 2, 0] = 90
    wire[1, 7, :, 0] = 140
    wire = wire.reshape(E, N, K // 32 * 17)
    x = rng.standard_normal((T, 1, K)).astype(np.float32)
    x *= np.exp2(rng.integers(-12, 3, (T, 1, K))).astype(np.float32)      # wide range inside every block
    x[3, 0, 64:96] = 0.0                                                     # a zero block
    x[4, 0, :] *= 2.0 ** 40                                                  # a huge row
    x[5, 0, :] *= 2.0 ** -60                                                 # a tiny row
    xb = O.f32_to_bits(x, "bfloat16")
    idx = rng.integers(0, E, (T, 1))
    got = dev_to_bits(kq.gather_qmv_kq(bits_to_dev(xb, "bfloat16"), wire_to_dev(wire), "mxfp4", _idx_dev(idx)))
    want = O.gather_qmv(xb, wire, "mxfp4", idx, None, "bfloat16")
    g = O.bits_to_f32(got, "bfloat16").astype(np.float64).reshape(T, N)
    w_ = O.bits_to_f32(want, "bfloat16").astype(np.float64).reshape(T, N)
    assert np.isfinite(g).all()
    rel_rows = np.linalg.norm(g - w_, axis=1) / np.maximum(np.linalg.norm(w_, axis=1), 1e-300)
    assert rel_rows.max() <= TOL, rel_rows


def test_fp4_matches_per_entry_route_at_the_threshold(kq):
    """8 pairs run here, 7 on the per-entry kernels: both agree with the oracle on the same stack (K has a tail)."""
    E, N, K = 6, 80, 2880 // 10
    wire = _stack(E, N, K, seed=15)
    for T in (7, 8):
        idx = np.random.default_rng(16 + T).integers(0, E, (T, 1))
        xb, xt = make_x((T, 1, K), "bfloat16", seed=17, scale=0.3)
        got = kq.gather_qmv_kq(xt, wire_to_dev(wire), "mxfp4", _idx_dev(idx))
        assert rel_l2(dev_to_bits(got), O.gather_qmv(xb, wire, "mxfp4", idx, None, "bfloat16"), "bfloat16") <= TOL, T
