"""GPU parity: gather_qmm, moe_glu_gather_kq, gather_qmv_kq (HIP) vs the CPU oracle."""
import os

import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import bits_to_dev, dev_to_bits, make_x, rel_l2, wire_to_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _stack(codec, E, N, K, seed):
    wpb, bpb = O.geometry(codec)
    return O.synth_wire(codec, E * N * (K // wpb), seed).reshape(E, N, K // wpb * bpb)


def _idx_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a).astype(np.int64)).cuda()


@pytest.mark.parametrize("codec", ["q4_k", "q6_k", "q2_k", "iq3_s", "mxfp4", "q8_0"])
@pytest.mark.parametrize("M", [1, 5])
def test_gather_qmm(kq, codec, M):
    E, N, K, B = 4, 128, 512 if codec != "mxfp4" else 288, 8
    wire = _stack(codec, E, N, K, seed=41)
    xb, xt = make_x((B, M, K), "float16", seed=42)
    rng = np.random.default_rng(43)
    rhs = rng.integers(0, E, B)
    # arange lhs (rhs only given)
    got = kq.gather_qmm(xt, wire_to_dev(wire), None, codec, rhs_indices=_idx_dev(rhs))
    want = O.gather_qmm(xb, wire, codec, np.arange(B), rhs, True, "float16")
    assert tuple(got.shape) == (B, M, N)
    assert rel_l2(dev_to_bits(got), want, "float16") <= TOL
    # reversed lhs with repeats, 2-D index arrays
    lhs = np.array([7, 6, 5, 4, 3, 3, 1, 0]).reshape(2, 4)
    got = kq.gather_qmm(xt, wire_to_dev(wire), None, codec, lhs_indices=_idx_dev(lhs),
                        rhs_indices=_idx_dev(rhs.reshape(2, 4)))
    want = O.gather_qmm(xb, wire, codec, lhs.reshape(-1), rhs, True, "float16")
    assert tuple(got.shape) == (2, 4, M, N)
    assert rel_l2(dev_to_bits(got).reshape(B, M, N), want, "float16") <= TOL


@pytest.mark.parametrize("codec", ["q4_k", "q5_k", "q6_k", "q3_k", "iq4_xs", "iq2_xxs", "q8_0", "mxfp4", "nvfp4"])
@pytest.mark.parametrize("M", [1, 3])
def test_gather_qmm_batched(kq, codec, M):
    """More than 16 output rows: entries are gathered and grouped by expert on the device (the
    sort-by-expert arm of KQuantGatherQMM::eval_cpu, src/kquant_gather.cpp:584-593).  General lhs with
    repeats, an expert nobody picks, 2-D index arrays, both half dtypes."""
    E, N, K, B, XB = 6, 136, 768 if codec not in ("mxfp4", "nvfp4") else 320, 44, 9
    wire = _stack(codec, E, N, K, seed=61)
    rng = np.random.default_rng(62)
    lhs = rng.integers(0, XB, B)
    rhs = rng.integers(0, E - 1, B)  # expert E-1 stays idle
    for dtype in ("bfloat16", "float16"):
        xb, xt = make_x((XB, M, K), dtype, seed=63, scale=0.5)
        got = kq.gather_qmm(xt, wire_to_dev(wire), None, codec, lhs_indices=_idx_dev(lhs.reshape(4, 11)),
                            rhs_indices=_idx_dev(rhs.reshape(4, 11)))
        want = O.gather_qmm(xb, wire, codec, lhs, rhs, True, dtype)
        assert tuple(got.shape) == (4, 11, M, N)
        assert rel_l2(dev_to_bits(got).reshape(B, M, N), want, dtype) <= TOL, (codec, M, dtype)


@pytest.mark.parametrize("codec", ["q4_k", "q2_k", "iq4_xs", "mxfp4", "nvfp4", "q8_0"])
@pytest.mark.parametrize("B,M", [(10, 3), (3, 12)])
def test_gather_qmm_few_entries_of_several_rows(kq, codec, B, M):
    """17 ... 48 output rows made of entries with several activation rows each: the one-row-per-entry kernels do not
    apply, whatever the pair count says."""
    E, N, K = 5, 136, 512 if codec not in ("mxfp4", "nvfp4") else 320
    wire = _stack(codec, E, N, K, seed=161)
    rng = np.random.default_rng(162)
    lhs, rhs = rng.integers(0, B, B), rng.integers(0, E, B)
    xb, xt = make_x((B, M, K), "bfloat16", seed=163, scale=0.5)
    got = kq.gather_qmm(xt, wire_to_dev(wire), None, codec, lhs_indices=_idx_dev(lhs), rhs_indices=_idx_dev(rhs))
    want = O.gather_qmm(xb, wire, codec, lhs, rhs, True, "bfloat16")
    assert tuple(got.shape) == (B, M, N)
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (codec, B, M)


@pytest.mark.parametrize("codec", ["q4_k", "q6_k", "q2_k", "q8_0"])
def test_single_entry_picks_its_expert(kq, codec):
    """A gathered call of ONE entry must still honour its expert index (it must not take the dense-call
    kernels, which read the stack's first matrix)."""
    E, N, K = 4, 64, 1024
    wire = _stack(codec, E, N, K, seed=71)
    xb, xt = make_x((1, 1, K), "bfloat16", seed=72)
    for e in (0, 3):
        got = kq.gather_qmm(xt, wire_to_dev(wire), None, codec, rhs_indices=_idx_dev(np.array([e])))
        want = O.gather_qmm(xb, wire, codec, np.array([0]), np.array([e]), True, "bfloat16")
        assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (codec, e)
        got = kq.gather_qmv_kq(xt, wire_to_dev(wire), codec, _idx_dev(np.array([[e]])))
        assert rel_l2(dev_to_bits(got), O.gather_qmv(xb, wire, codec, np.array([[e]]), None, "bfloat16"), "bfloat16") <= TOL


@pytest.mark.parametrize("codec", ["q4_k", "q8_0", "iq4_nl", "q6_k"])
def test_gather_qmm_no_transpose(kq, codec):
    """transpose=False: every expert decodes to [K, N] (the MLA / LoRA-vjp orientation)."""
    E, K, N, B, M = 3, 48, 512, 6, 4
    wire = _stack(codec, E, K, N, seed=46)  # [E, K, N / wpb * bpb]
    xb, xt = make_x((B, M, K), "float16", seed=47)
    rng = np.random.default_rng(48)
    lhs, rhs = rng.integers(0, B, B), rng.integers(0, E, B)
    got = kq.gather_qmm(xt, wire_to_dev(wire), None, codec, lhs_indices=_idx_dev(lhs), rhs_indices=_idx_dev(rhs),
                        transpose=False)
    want = O.gather_qmm(xb, wire, codec, lhs, rhs, False, "float16")
    assert tuple(got.shape) == (B, M, N)
    assert rel_l2(dev_to_bits(got), want, "float16") <= TOL


@pytest.mark.parametrize("codec", ["q4_k", "q8_0", "iq3_s"])
def test_gather_qmm_no_transpose_many_rows_per_entry(kq, codec):
    """transpose=False with 100 activation rows per entry (the kernel that shares a step's decode over 128 rows),
    repeated lhs rows and an expert id outside the stack (that entry's rows stay untouched)."""
    E, K, N, B, M = 3, 48, 512, 5, 100
    wire = _stack(codec, E, K, N, seed=146)
    xb, xt = make_x((B, M, K), "bfloat16", seed=147)
    lhs, rhs = np.array([4, 0, 0, 2, 1]), np.array([2, 0, 7, 1, 1])
    out = kq.gather_qmm(xt, wire_to_dev(wire), None, codec, lhs_indices=_idx_dev(lhs), rhs_indices=_idx_dev(rhs),
                        transpose=False)
    keep = [0, 1, 3, 4]
    want = O.gather_qmm(xb, wire, codec, lhs[keep], rhs[keep], False, "bfloat16")
    assert tuple(out.shape) == (B, M, N)
    assert rel_l2(dev_to_bits(out[keep]), want, "bfloat16") <= TOL


def test_gather_qmm_reference_moe_fixture_and_strided_experts(kq):
    wire = np.load(os.path.join(GOLD, "q4_k_moe.npz"))["wire"]  # [4, 128, 288]
    E, N, K, B = 4, 128, 512, 64
    xb, xt = make_x((B, 1, K), "bfloat16", seed=44)
    rhs = np.sort(np.random.default_rng(45).integers(0, E, B))
    got = kq.gather_qmm(xt, wire_to_dev(wire), None, "q4_k", rhs_indices=_idx_dev(rhs), sorted_indices=True)
    want = O.gather_qmm(xb, wire, "q4_k", np.arange(B), rhs, True, "bfloat16")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL
    # gate half of a fused gate_up stack: expert stride is twice the matrix size
    fused = np.concatenate([wire, wire[::-1]], axis=1)  # [4, 256, 288]
    got = kq.gather_qmm(xt, wire_to_dev(fused)[:, :128, :], None, "q4_k", rhs_indices=_idx_dev(rhs))
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL
    # duplicate (x, expert) entries give bit-identical rows
    lhs = np.zeros(B, dtype=np.int64)
    got = dev_to_bits(kq.gather_qmm(xt, wire_to_dev(wire), None, "q4_k", lhs_indices=_idx_dev(lhs),
                                    rhs_indices=_idx_dev(np.zeros(B, dtype=np.int64))))
    assert all(np.array_equal(got[0], got[i]) for i in range(B))


def _glu_truth(codec, xb, gate, up, idx, act, limit=0.0, alpha=0.0, gb=None, ub=None, dtype="bfloat16"):
    return O.moe_glu_gather(xb, gate, up, codec, idx, act, limit, gb, ub, alpha, dtype)


@pytest.mark.parametrize("codec", O.ALL_CODECS)
def test_moe_glu_all_codecs(kq, codec):
    E, N, K, T, R = 4, 64, 512 if codec not in ("mxfp4",) else 288, 3, 2
    gate = _stack(codec, E, N, K, seed=51)
    up = gate[::-1].copy()
    idx = np.random.default_rng(52).integers(0, E, (T, R))
    for dtype in ("float16", "bfloat16"):
        xb, xt = make_x((T, K), dtype, seed=53, scale=0.1)
        got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx))
        want = _glu_truth(codec, xb, gate, up, idx, "silu", dtype=dtype)
        assert tuple(got.shape) == (T, R, N)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype)
        hb, ht = make_x((T, R, K), dtype, seed=54, scale=0.1)
        got = kq.gather_qmv_kq(ht, wire_to_dev(gate), codec, _idx_dev(idx))
        want = O.gather_qmv(hb, gate, codec, idx, None, dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype)


@pytest.mark.parametrize("act,limit", [("gelu", 0.0), ("silu_limit", 0.5), ("silu", 0.0)])
def test_moe_glu_activations(kq, act, limit):
    codec, E, N, K, T, R = "q6_k", 4, 64, 512, 5, 3
    gate = _stack(codec, E, N, K, seed=55)
    up = _stack(codec, E, N, K, seed=56)
    idx = np.random.default_rng(57).integers(0, E, (T, R))
    xb, xt = make_x((T, K), "bfloat16", seed=58, scale=0.3)
    got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act=act, limit=limit)
    want = _glu_truth(codec, xb, gate, up, idx, act, limit)
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL


@pytest.mark.parametrize("codec", ["q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("E,N,K,T,R", [(6, 136, 768, 1, 4), (8, 2048, 512, 4, 2), (3, 72, 4352, 5, 3), (128, 64, 256, 1, 8)])
def test_moe_tuned_gathered_shapes(kq, codec, E, N, K, T, R):
    """The MFMA gathered kernels: gate/up tiles that do not divide N, 1 / 3 / 17 superblocks, many experts."""
    gate = _stack(codec, E, N, K, seed=71)
    up = _stack(codec, E, N, K, seed=72)
    rng = np.random.default_rng(73)
    idx = np.stack([rng.permutation(E)[:R] for _ in range(T)]) if R <= E else rng.integers(0, E, (T, R))
    for dtype, act, limit in (("bfloat16", "silu", 0.0), ("float16", "gelu", 0.0), ("bfloat16", "silu_limit", 0.4)):
        xb, xt = make_x((T, K), dtype, seed=74, scale=0.02)
        got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act=act, limit=limit)
        want = _glu_truth(codec, xb, gate, up, idx, act, limit, dtype=dtype)
        assert tuple(got.shape) == (T, R, N)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype, act)
    hb, ht = make_x((T, R, K), "bfloat16", seed=75, scale=0.02)
    got = kq.gather_qmv_kq(ht, wire_to_dev(gate), codec, _idx_dev(idx))
    want = O.gather_qmv(hb, gate, codec, idx, None, "bfloat16")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, codec


@pytest.mark.parametrize("codec,T", [("q2_k", 50), ("q2_k", 80), ("q3_k", 50), ("q3_k", 80), ("iq4_xs", 15),
                                     ("iq4_xs", 20), ("iq3_s", 15), ("iq3_s", 20), ("iq2_xxs", 15), ("iq2_xxs", 20),
                                     ("q8_0", 15), ("q8_0", 20), ("mxfp4", 15), ("mxfp4", 20), ("q4_0", 15),
                                     ("q4_0", 20), ("iq4_nl", 15), ("iq4_nl", 20), ("nvfp4", 50), ("nvfp4", 80)])
def test_moe_low_bit_routes_either_side_of_the_entry_threshold(kq, codec, T):
    """q2_k / q3_k / nvfp4 stacks run entry by entry on the streamed kernel up to 256 (token, expert) pairs, on the
    any-codec kernel above; iq4_xs / iq3_s / iq2_xxs / q8_0 / mxfp4 / q4_0 / iq4_nl switch to the code-level grouped
    kernel above 64 pairs.  The
    token counts (x 4 experts each) sit on either side.  (128 experts: the pair limits shrink with shorter stacks.)"""
    E, N, K, R = 128, 136, 768, 4
    gate = _stack(codec, E, N, K, seed=91)
    up = _stack(codec, E, N, K, seed=92)
    rng = np.random.default_rng(93)
    idx = np.stack([rng.permutation(E)[:R] for _ in range(T)])
    xb, xt = make_x((T, K), "bfloat16", seed=94, scale=0.05)
    got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act="silu")
    want = _glu_truth(codec, xb, gate, up, idx, "silu", 0.0, dtype="bfloat16")
    assert tuple(got.shape) == (T, R, N)
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (codec, T)
    hb, ht = make_x((T, R, K), "float16", seed=95, scale=0.05)
    got = kq.gather_qmv_kq(ht, wire_to_dev(gate), codec, _idx_dev(idx))
    want = O.gather_qmv(hb, gate, codec, idx, None, "float16")
    assert rel_l2(dev_to_bits(got), want, "float16") <= TOL, (codec, T)


@pytest.mark.parametrize("codec", ["mxfp4", "q4_0", "q8_0", "iq4_nl"])
@pytest.mark.parametrize("E,N,K,T,R", [(6, 136, 288, 1, 4), (5, 72, 2880, 3, 2), (130, 40, 480, 4, 4)])
def test_moe_decode_k_ends_inside_a_unit(kq, codec, E, N, K, T, R):
    """MoE decode (a few pairs, entry by entry on the streamed kernel) on stacks whose K is not a multiple of 256:
    fused gate / up and the down form, both activation dtypes; mxfp4 also with biases and swiglu_clamp."""
    gate, up = _stack(codec, E, N, K, seed=151), _stack(codec, E, N, K, seed=152)
    rng = np.random.default_rng(153)
    idx = np.stack([rng.permutation(E)[:R] for _ in range(T)])
    for dtype in ("bfloat16", "float16"):
        xb, xt = make_x((T, K), dtype, seed=154, scale=0.05)
        got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act="silu")
        assert rel_l2(dev_to_bits(got), _glu_truth(codec, xb, gate, up, idx, "silu", dtype=dtype), dtype) <= TOL, (codec, dtype)
        hb, ht = make_x((T, R, K), dtype, seed=155, scale=0.05)
        got = kq.gather_qmv_kq(ht, wire_to_dev(up), codec, _idx_dev(idx))
        assert rel_l2(dev_to_bits(got), O.gather_qmv(hb, up, codec, idx, None, dtype), dtype) <= TOL, (codec, dtype)
    if codec == "mxfp4":
        gb = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
        ub = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
        xb, xt = make_x((T, K), "bfloat16", seed=156, scale=0.05)
        got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act="swiglu_clamp",
                                   limit=7.0, alpha=1.702, gate_bias=torch.from_numpy(gb).cuda(),
                                   up_bias=torch.from_numpy(ub).cuda())
        want = _glu_truth(codec, xb, gate, up, idx, "swiglu_clamp", 7.0, 1.702, gb, ub)
        assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL
        hb, ht = make_x((T, R, K), "bfloat16", seed=157, scale=0.05)
        got = kq.gather_qmv_kq(ht, wire_to_dev(up), codec, _idx_dev(idx), bias=torch.from_numpy(gb).cuda())
        assert rel_l2(dev_to_bits(got), O.gather_qmv(hb, up, codec, idx, gb, "bfloat16"), "bfloat16") <= TOL


@pytest.mark.parametrize("T", [4, 16])
def test_moe_routes_on_32_experts_of_2880_square(kq, T):
    """A stack unlike the one the entry-by-entry limits were measured on (32 experts of 2880 x 2880 in mxfp4, top-4,
    biases with swiglu_clamp): 16 pairs run entry by entry, 64 on the expert-grouped kernels; the fused gate / up
    projection and the biased down projection agree with the oracle on both."""
    codec, E, N, K, R = "mxfp4", 32, 2880, 2880, 4
    gate, up = _stack(codec, E, N, K, seed=131), _stack(codec, E, N, K, seed=132)
    rng = np.random.default_rng(133)
    idx = np.stack([rng.permutation(E)[:R] for _ in range(T)])
    gb = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
    ub = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
    xb, xt = make_x((T, K), "bfloat16", seed=134, scale=0.05)
    got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act="swiglu_clamp", limit=7.0,
                               alpha=1.702, gate_bias=torch.from_numpy(gb).cuda(), up_bias=torch.from_numpy(ub).cuda())
    want = _glu_truth(codec, xb, gate, up, idx, "swiglu_clamp", 7.0, 1.702, gb, ub)
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, T
    hb, ht = make_x((T, R, K), "bfloat16", seed=135, scale=0.05)
    got = kq.gather_qmv_kq(ht, wire_to_dev(up), codec, _idx_dev(idx), bias=torch.from_numpy(gb).cuda())
    assert rel_l2(dev_to_bits(got), O.gather_qmv(hb, up, codec, idx, gb, "bfloat16"), "bfloat16") <= TOL, T


@pytest.mark.parametrize("E,T,R", [(8, 2, 4), (8, 20, 4), (4, 40, 2)])
@pytest.mark.parametrize("N,K", [(200, 736), (64, 2880)])
def test_moe_mxfp4_block_scaled_forms(kq, E, T, R, N, K):
    """The three forms of the block-scaled kernels on stacks whose K ends inside a step and inside a 256-weight unit
    (736 = 23 blocks; 2880) and whose last column group is ragged (200 columns): 8 pairs (two-wave workgroups on 32
    columns), 80 pairs on 8 experts (four waves, one m-tile per pass), 80 pairs on 4 experts (two m-tiles on the same
    weight registers); fused op with biases and swiglu_clamp and plain op with a bias, both activation dtypes."""
    codec = "mxfp4"
    gate, up = _stack(codec, E, N, K, seed=161), _stack(codec, E, N, K, seed=162)
    rng = np.random.default_rng(163)
    idx = np.stack([rng.permutation(E)[:R] for _ in range(T)])
    gb = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
    ub = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
    for dtype in ("bfloat16", "float16"):
        xb, xt = make_x((T, K), dtype, seed=164, scale=0.05)
        got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act="swiglu_clamp",
                                   limit=7.0, alpha=1.702, gate_bias=torch.from_numpy(gb).cuda(),
                                   up_bias=torch.from_numpy(ub).cuda())
        want = _glu_truth(codec, xb, gate, up, idx, "swiglu_clamp", 7.0, 1.702, gb, ub, dtype=dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (E, T, R, N, K, dtype)
        hb, ht = make_x((T, R, K), dtype, seed=165, scale=0.05)
        got = kq.gather_qmv_kq(ht, wire_to_dev(up), codec, _idx_dev(idx), bias=torch.from_numpy(gb).cuda())
        assert rel_l2(dev_to_bits(got), O.gather_qmv(hb, up, codec, idx, gb, dtype), dtype) <= TOL, (E, T, R, N, K, dtype)


@pytest.mark.parametrize("T", [16, 40])
@pytest.mark.parametrize("off", [1, 2, 3])
def test_moe_mxfp4_stacks_at_any_byte_offset_use_nothing_past_their_end(kq, off, T):
    """The block-scaled kernel fetches aligned dwords around every 17-byte block.  Stacks that start at an odd byte
    offset end inside a dword: the result must not depend on the bytes that follow the stack (two fillings), and
    equals the result on the same stacks at an aligned address bit for bit (16 tokens: one m-tile per segment, 40:
    two)."""
    codec, E, N, K, R = "mxfp4", 4, 64, 288, 2
    gate, up = _stack(codec, E, N, K, seed=141), _stack(codec, E, N, K, seed=142)
    rng = np.random.default_rng(143)
    idx = np.stack([rng.permutation(E)[:R] for _ in range(T)])
    xb, xt = make_x((T, K), "bfloat16", seed=144, scale=0.05)
    hb, ht = make_x((T, R, K), "bfloat16", seed=145, scale=0.05)
    want = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx))
    want_d = kq.gather_qmv_kq(ht, wire_to_dev(up), codec, _idx_dev(idx))
    assert rel_l2(dev_to_bits(want), _glu_truth(codec, xb, gate, up, idx, "silu"), "bfloat16") <= TOL

    def placed(stack, fill):
        buf = torch.full((off + stack.size + 64,), fill, dtype=torch.uint8, device="cuda")
        buf[off:off + stack.size] = wire_to_dev(stack).reshape(-1)
        return buf[off:off + stack.size].view(stack.shape)

    for fill in (0x00, 0xFF):
        got = kq.moe_glu_gather_kq(xt, placed(gate, fill), placed(up, fill), codec, _idx_dev(idx))
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (off, T, fill)
        got = kq.gather_qmv_kq(ht, placed(up, fill), codec, _idx_dev(idx))
        assert torch.equal(got.view(torch.int16), want_d.view(torch.int16)), (off, T, fill)


@pytest.mark.parametrize("N,K,T", [(1536, 2048, 5), (2048, 2560, 5), (1536, 2048, 10)])
def test_moe_q4k_routes_by_pairs_per_expert_and_bytes_read_again(kq, N, K, T):
    """64 experts in q4_k, top-4.  20 pairs of 1536 x 2048 matrices run entry by entry; the same 20 pairs of
    2048 x 2560 matrices would read more bytes again than the grouped route's prologue costs, and 40 pairs are more
    pairs per expert than were measured to pay: both go to the expert-grouped kernels.  All agree with the oracle;
    an activation matrix that starts 2 bytes off a 16-byte boundary (which the streamed and the grouped kernels both
    decline) still does."""
    codec, E, R = "q4_k", 64, 4
    gate, up = _stack(codec, E, N, K, seed=141), _stack(codec, E, N, K, seed=142)
    rng = np.random.default_rng(143)
    idx = np.stack([rng.permutation(E)[:R] for _ in range(T)])
    xb, xt = make_x((T, K), "bfloat16", seed=144, scale=0.03)
    want = _glu_truth(codec, xb, gate, up, idx, "silu")
    got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act="silu")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (N, K, T)
    off = torch.empty(T * K + 8, dtype=xt.dtype, device=xt.device)
    shifted = off[1:1 + T * K].view(T, K)
    shifted.copy_(xt)
    assert shifted.data_ptr() % 16 == 2
    got = kq.moe_glu_gather_kq(shifted, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act="silu")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL, (N, K, T, "shifted")


@pytest.mark.parametrize("codec", ["q4_k", "q5_k", "q6_k"])
@pytest.mark.parametrize("E,N,K,T,R", [(6, 136, 768, 20, 3), (8, 200, 512, 100, 2), (128, 64, 256, 8, 8),
                                       (5, 72, 4352, 9, 2)])
def test_moe_grouped_batched_shapes(kq, codec, E, N, K, T, R):
    """More than 16 pairs: the expert-sorted MFMA path (segments of <= 32 pairs; experts with none, one
    partial or several segments; column slabs that do not divide N)."""
    gate = _stack(codec, E, N, K, seed=81)
    up = _stack(codec, E, N, K, seed=82)
    rng = np.random.default_rng(83)
    idx = rng.integers(0, E, (T, R))
    if E == 8:
        idx[:, 0] = 3  # one hot expert: 100+ pairs = four segments; expert 5 gets none
        idx[idx == 5] = 6
    for dtype, act, limit in (("bfloat16", "silu", 0.0), ("float16", "gelu", 0.0), ("bfloat16", "silu_limit", 0.4)):
        xb, xt = make_x((T, K), dtype, seed=84, scale=0.02)
        got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act=act, limit=limit)
        want = _glu_truth(codec, xb, gate, up, idx, act, limit, dtype=dtype)
        assert tuple(got.shape) == (T, R, N)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype, act)
    for dtype in ("bfloat16", "float16"):
        hb, ht = make_x((T, R, K), dtype, seed=85, scale=0.02)
        got = kq.gather_qmv_kq(ht, wire_to_dev(gate), codec, _idx_dev(idx))
        want = O.gather_qmv(hb, gate, codec, idx, None, dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype)


@pytest.mark.parametrize("codec", O.ALL_CODECS)
def test_moe_batched_every_codec(kq, codec):
    """More than 16 pairs for every codec: the batched paths (tuned K-quant or any-codec matrix-core)."""
    wpb, _ = O.geometry(codec)
    E, N, K, T, R = 5, 72, (288 if wpb == 32 else 512), 12, 3
    gate = _stack(codec, E, N, K, seed=91)
    up = _stack(codec, E, N, K, seed=92)
    idx = np.random.default_rng(93).integers(0, E, (T, R))
    for dtype in ("bfloat16", "float16"):
        xb, xt = make_x((T, K), dtype, seed=94, scale=0.02)
        got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx))
        want = _glu_truth(codec, xb, gate, up, idx, "silu", dtype=dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype)
        hb, ht = make_x((T, R, K), dtype, seed=95, scale=0.02)
        got = kq.gather_qmv_kq(ht, wire_to_dev(gate), codec, _idx_dev(idx))
        want = O.gather_qmv(hb, gate, codec, idx, None, dtype)
        assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype)


@pytest.mark.parametrize("codec", ["mxfp4", "nvfp4"])
def test_moe_batched_swiglu_clamp_bias(kq, codec):
    """Biased fp4 experts with swiglu_clamp on the batched path (64 tokens, top-4), K not a multiple of 256."""
    E, N, K, T, R = 8, 136, 576, 64, 4
    gate = _stack(codec, E, N, K, seed=96)
    up = _stack(codec, E, N, K, seed=97)
    rng = np.random.default_rng(98)
    gb = (rng.standard_normal((E, N)) * 0.01).astype(np.float32)
    ub = (rng.standard_normal((E, N)) * 0.01).astype(np.float32)
    idx = np.stack([rng.permutation(E)[:R] for _ in range(T)])
    xb, xt = make_x((T, K), "bfloat16", seed=99, scale=0.2)
    got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act="swiglu_clamp",
                               limit=7.0, gate_bias=torch.from_numpy(gb).cuda(), up_bias=torch.from_numpy(ub).cuda(),
                               alpha=1.702)
    want = _glu_truth(codec, xb, gate, up, idx, "swiglu_clamp", 7.0, 1.702, gb, ub)
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL
    hb, ht = make_x((T, R, K), "bfloat16", seed=100, scale=0.2)
    got = kq.gather_qmv_kq(ht, wire_to_dev(gate), codec, _idx_dev(idx), bias=torch.from_numpy(gb).cuda())
    want = O.gather_qmv(hb, gate, codec, idx, gb, "bfloat16")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL


def test_moe_grouped_matches_per_pair_path_bitwise(kq):
    """A pair's row does not depend on which other pairs share the call: rows of a 64-pair call equal the
    rows of the same pairs computed in 4-pair calls (different kernels, same exact products)."""
    codec, E, N, K, T, R = "q4_k", 8, 128, 1024, 32, 2
    gate = _stack(codec, E, N, K, seed=86)
    up = _stack(codec, E, N, K, seed=87)
    idx = np.random.default_rng(88).integers(0, E, (T, R))
    xb, xt = make_x((T, K), "bfloat16", seed=89, scale=0.02)
    g, u = wire_to_dev(gate), wire_to_dev(up)
    big = O.bits_to_f32(dev_to_bits(kq.moe_glu_gather_kq(xt, g, u, codec, _idx_dev(idx))), "bfloat16")
    small = np.concatenate([O.bits_to_f32(dev_to_bits(kq.moe_glu_gather_kq(xt[t:t + 2], g, u, codec,
                                                                         _idx_dev(idx[t:t + 2]))), "bfloat16")
                            for t in range(0, T, 2)])
    # both are exact products accumulated in f32 in different orders: agreement to a few bf16 ulps
    assert np.linalg.norm(big - small) / np.linalg.norm(small) <= 2e-3
    assert np.mean(big != small) < 0.2


@pytest.mark.parametrize("codec", ["mxfp4", "nvfp4"])
def test_moe_swiglu_clamp_bias(kq, codec):
    E, N, K, T, R = 4, 64, 576, 4, 2
    gate = _stack(codec, E, N, K, seed=61)
    up = _stack(codec, E, N, K, seed=62)
    rng = np.random.default_rng(63)
    gb = (rng.standard_normal((E, N)) * 0.01).astype(np.float32)
    ub = (rng.standard_normal((E, N)) * 0.01).astype(np.float32)
    idx = rng.integers(0, E, (T, R))
    xb, xt = make_x((T, K), "bfloat16", seed=64, scale=0.2)
    got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act="swiglu_clamp",
                               limit=7.0, gate_bias=torch.from_numpy(gb).cuda(), up_bias=torch.from_numpy(ub).cuda(),
                               alpha=1.702)
    want = _glu_truth(codec, xb, gate, up, idx, "swiglu_clamp", 7.0, 1.702, gb, ub)
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL
    hb, ht = make_x((T, R, K), "bfloat16", seed=65, scale=0.2)
    got = kq.gather_qmv_kq(ht, wire_to_dev(gate), codec, _idx_dev(idx), bias=torch.from_numpy(gb).cuda())
    want = O.gather_qmv(hb, gate, codec, idx, gb, "bfloat16")
    assert rel_l2(dev_to_bits(got), want, "bfloat16") <= TOL


@pytest.mark.parametrize("codec", ["mxfp4", "nvfp4"])
@pytest.mark.parametrize("T,R", [(1, 4), (3, 4), (10, 4), (15, 4), (20, 4)])
@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
def test_moe_swiglu_clamp_bias_on_the_streamed_kernel(kq, codec, T, R, dtype):
    """Biased fp4 experts with swiglu_clamp and K a multiple of 256: up to 64 (mxfp4) or 256 (nvfp4) pairs run entry
    by entry on the streamed kernel, whose epilogue adds the f32 biases; 80 pairs of mxfp4 take the grouped kernel.
    Ragged N (two tiles + 8 rows), a limit small enough to clamp, the down op with its bias."""
    E, N, K = 128, 72, 768
    gate = _stack(codec, E, N, K, seed=261)
    up = _stack(codec, E, N, K, seed=262)
    rng = np.random.default_rng(263)
    gb = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
    ub = (rng.standard_normal((E, N)) * 0.05).astype(np.float32)
    idx = np.stack([rng.permutation(E)[:R] for _ in range(T)])
    xb, xt = make_x((T, K), dtype, seed=264, scale=0.2)
    g, u, ix = wire_to_dev(gate), wire_to_dev(up), _idx_dev(idx)
    gbt, ubt = torch.from_numpy(gb).cuda(), torch.from_numpy(ub).cuda()
    got = kq.moe_glu_gather_kq(xt, g, u, codec, ix, act="swiglu_clamp", limit=7.0, gate_bias=gbt, up_bias=ubt, alpha=1.702)
    want = _glu_truth(codec, xb, gate, up, idx, "swiglu_clamp", 7.0, 1.702, gb, ub, dtype=dtype)
    assert rel_l2(dev_to_bits(got), want, dtype) <= TOL
    got = kq.moe_glu_gather_kq(xt, g, u, codec, ix, act="swiglu_clamp", limit=0.75, gate_bias=ubt, up_bias=gbt, alpha=1.2)
    want = _glu_truth(codec, xb, gate, up, idx, "swiglu_clamp", 0.75, 1.2, ub, gb, dtype=dtype)
    assert rel_l2(dev_to_bits(got), want, dtype) <= TOL
    hb, ht = make_x((T, R, K), dtype, seed=265, scale=0.2)
    got = kq.gather_qmv_kq(ht, g, codec, ix, bias=gbt)
    want = O.gather_qmv(hb, gate, codec, idx, gb, dtype)
    assert rel_l2(dev_to_bits(got), want, dtype) <= TOL


def test_moe_validation_errors(kq):
    d = torch.device("cuda:0")
    E, N, K = 2, 16, 256
    w = torch.zeros((E, N, 144), dtype=torch.uint8, device=d)
    x = torch.zeros((3, K), dtype=torch.float16, device=d)
    idx = torch.zeros((3, 2), dtype=torch.int64, device=d)
    with pytest.raises(ValueError):
        kq.moe_glu_gather_kq(x.float(), w, w, "q4_k", idx)
    with pytest.raises(ValueError):
        kq.moe_glu_gather_kq(x, w, w, "q4_k", idx, act="relu")
    with pytest.raises(ValueError):
        kq.moe_glu_gather_kq(x, w, w, "q4_k", idx, act="silu_limit")
    with pytest.raises(ValueError):
        kq.moe_glu_gather_kq(x, w, w, "q4_k", idx, gate_bias=torch.zeros((E, N), device=d))
    with pytest.raises(ValueError):
        kq.moe_glu_gather_kq(x, w, w[:, :8], "q4_k", idx)
    with pytest.raises(ValueError):
        kq.moe_glu_gather_kq(x, w[:, :, :100], w[:, :, :100], "q4_k", idx)
    with pytest.raises(ValueError):
        kq.gather_qmv_kq(x, w, "q4_k", idx)
    with pytest.raises(ValueError):
        kq.gather_qmv_kq(x.reshape(3, 1, K).expand(3, 2, K), w, "q4_k", idx, bias=torch.zeros((E, N), device=d))


@pytest.mark.parametrize("codec", ["q4_1", "q5_0", "iq4_nl", "iq2_s", "iq1_m", "mxfp4", "nvfp4"])
def test_moe_decode_entries_ragged_shapes(kq, codec):
    """One-row entries of the legacy / IQ / fp4 codecs (MoE decode): N that is no multiple of the 16- / 32-column
    tiles, K that is no multiple of 256 where the codec allows, repeated experts, both half dtypes; then
    gather_qmm with lhs indices that pick rows out of order."""
    wpb = O.geometry(codec)[0]
    E, N, T, R = 5, 72, 2, 3
    K = 320 if wpb == 32 else 384 if wpb == 64 else 512
    gate = _stack(codec, E, N, K, seed=71)
    up = _stack(codec, E, N, K, seed=72)
    idx = np.array([[4, 0, 4], [1, 1, 3]])
    for dtype in ("float16", "bfloat16"):
        xb, xt = make_x((T, K), dtype, seed=73, scale=0.1)
        for act in ("silu", "gelu"):
            got = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act=act)
            want = _glu_truth(codec, xb, gate, up, idx, act, dtype=dtype)
            assert rel_l2(dev_to_bits(got), want, dtype) <= TOL, (codec, dtype, act)
        hb, ht = make_x((T, R, K), dtype, seed=74, scale=0.1)
        got = kq.gather_qmv_kq(ht, wire_to_dev(gate), codec, _idx_dev(idx))
        assert rel_l2(dev_to_bits(got), O.gather_qmv(hb, gate, codec, idx, None, dtype), dtype) <= TOL, (codec, dtype)
    xb, xt = make_x((6, 1, K), "float16", seed=75, scale=0.1)
    lhs, rhs = np.array([5, 0, 3, 3, 1]), np.array([2, 2, 0, 4, 1])
    got = kq.gather_qmm(xt, wire_to_dev(gate), None, codec, lhs_indices=_idx_dev(lhs), rhs_indices=_idx_dev(rhs))
    want = O.gather_qmm(xb, gate, codec, lhs, rhs, True, "float16")
    assert rel_l2(dev_to_bits(got), want, "float16") <= TOL, codec


@pytest.mark.parametrize("codec", ["q8_0", "q4_k"])
def test_rhs_gather_more_than_32767_rows(kq, codec):
    """A single sorted gather of 33000 one-row entries (more than a 16-bit row count, no multiple of any tile),
    long uneven per-expert runs: every row against the oracle (reference tests/test_gather.py:197-250)."""
    E, N, K, B = 8, 64, 256, 33000
    wire = _stack(codec, E, N, K, seed=81)
    rng = np.random.default_rng(82)
    rhs = np.sort(rng.integers(0, E, B))
    xb, xt = make_x((B, 1, K), "float16", seed=83, scale=0.1)
    got = kq.gather_qmm(xt, wire_to_dev(wire), None, codec, rhs_indices=_idx_dev(rhs), sorted_indices=True)
    assert tuple(got.shape) == (B, 1, N)
    want = O.gather_qmm(xb, wire, codec, np.arange(B), rhs, True, "float16")
    gb = dev_to_bits(got)
    assert rel_l2(gb, want, "float16") <= TOL
    assert rel_l2(gb[:64], want[:64], "float16") <= TOL and rel_l2(gb[-64:], want[-64:], "float16") <= TOL


@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
@pytest.mark.parametrize("codec", ["q4_k", "q5_k", "q6_k", "q2_k", "q3_k", "iq4_xs", "iq3_s", "iq2_xxs", "q8_0", "iq4_nl",
                                   "q4_0", "mxfp4", "nvfp4"])
@pytest.mark.parametrize("N,K,T,R,act", [
    (72, 768, 1, 8, "silu"),       # ragged rows (72 = 2 tiles + 8), three superblocks: four-wave form, one unit a wave
    (96, 3072, 2, 4, "gelu"),      # twelve superblocks: eight-wave fused form, two tokens share the activations
    (40, 4096, 1, 3, "silu"),      # sixteen superblocks, the longest K of the fused form
    (64, 6144, 2, 2, "silu"),      # past it for the fused form (older kernel), inside the plain form's 32
    (64, 1024, 10, 4, "silu"),     # 40 entries: still one workgroup per (entry, tile) for q4_k / q5_k / q6_k
])
def test_moe_decode_entries_on_the_streamed_kernel(kq, codec, N, K, T, R, act, dtype):
    """Up to 16 (token, expert) entries of a stack in one of the streamed kernel's codecs (48 for q4_k / q5_k / q6_k)
    run its gathered mode: fused gate / up (two units per superblock) and the plain down projection."""
    E = 5 if T * R <= 16 else 130  # beyond 16 entries the per-entry route needs a tall stack
    gate, up, down = _stack(codec, E, N, K, 201), _stack(codec, E, N, K, 202), _stack(codec, E, N, K, 203)
    rng = np.random.default_rng(204)
    idx = rng.integers(0, E, (T, R))
    xb, xt = make_x((T, K), dtype, seed=205, scale=0.1)
    h = kq.moe_glu_gather_kq(xt, wire_to_dev(gate), wire_to_dev(up), codec, _idx_dev(idx), act=act)
    assert tuple(h.shape) == (T, R, N)
    assert rel_l2(dev_to_bits(h), _glu_truth(codec, xb, gate, up, idx, act, dtype=dtype), dtype) <= TOL
    xb2, xt2 = make_x((T, R, K), dtype, seed=206, scale=0.1)
    y = kq.gather_qmv_kq(xt2, wire_to_dev(down), codec, _idx_dev(idx))
    assert tuple(y.shape) == (T, R, N)
    assert rel_l2(dev_to_bits(y), O.gather_qmv(xb2, down, codec, idx, None, dtype), dtype) <= TOL
    # the entries agree with a dense matmul against the expert's matrix (the dense streamed kernel)
    e0 = int(idx[0, 0])
    dense = kq.quantized_matmul(xt2[0, :1].contiguous(), wire_to_dev(down[e0]), None, codec)
    assert rel_l2(dev_to_bits(y[0, 0:1]), dev_to_bits(dense), dtype) <= TOL
