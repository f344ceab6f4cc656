"""GPU parity at the exact shapes of the benchmark configurations, through the library's own (automatic) kernel
choice: these are the shapes at which the split-K plans, the persistent streamed kernel, the 128 x 256 prefill
tiles and the grouped MoE kernels are selected.  The oracle runs on a fixed sample of weight rows (output
columns) or tokens so that the CPU side stays within seconds; the sample always holds the first and last rows."""
import numpy as np
import pytest
import torch

import oracle_lib as O
from gpu_util import bits_to_dev, dev_to_bits, make_x, rel_l2, synth_wire_dev

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


def _sample_rows(N, count, seed):
    rng = np.random.default_rng(seed)
    rows = np.unique(np.concatenate([np.arange(min(N, 40)), np.arange(max(0, N - 40), N),
                                     rng.integers(0, N, count)]))
    return rows


def _check_matmul(kq, codec, M, N, K, dtype, seed, sample=None):
    w = synth_wire_dev(codec, N, K, seed)
    xb, xt = make_x((M, K), dtype, seed=seed + 1)
    got = dev_to_bits(kq.quantized_matmul(xt, w, None, codec))
    assert got.shape == (M, N)
    rows = np.arange(N) if sample is None else _sample_rows(N, sample, seed + 2)
    wire = w[torch.from_numpy(rows).to(w.device)].cpu().numpy()
    want = O.qmm(xb, wire, codec, True, dtype)
    err = rel_l2(got[:, rows], want, dtype)
    assert err <= TOL, (codec, M, N, K, dtype, err)
    return err


def test_config1_q4k_4096_square_f16(kq):
    """4096 x 4096 q4_k, one f16 row: dequantize to f16 bit-exact on the whole matrix, matmul on all columns."""
    N = K = 4096
    w = synth_wire_dev("q4_k", N, K, 70)
    wire = w.cpu().numpy()
    got = dev_to_bits(kq.dequantize(w, None, "q4_k"))
    assert np.array_equal(got, O.dequantize(wire, "q4_k", "float16"))
    xb, xt = make_x((1, K), "float16", seed=71)
    y = dev_to_bits(kq.quantized_matmul(xt, w, None, "q4_k"))
    assert rel_l2(y, O.qmm(xb, wire, "q4_k", True, "float16"), "float16") <= TOL


@pytest.mark.parametrize("M", [1, 8])
@pytest.mark.parametrize("name,codec,N,K,sample", [
    ("q_proj", "q4_k", 4096, 4096, None), ("gate_up", "q4_k", 14336, 4096, None),
    ("down", "q6_k", 4096, 14336, None), ("lm_head", "q6_k", 128256, 4096, 600)])
def test_config2_decode_projections(kq, name, codec, N, K, sample, M):
    _check_matmul(kq, codec, M, N, K, "bfloat16", 72, sample)


@pytest.mark.parametrize("M", [512, 2048])
@pytest.mark.parametrize("codec", ["q4_k", "q5_k"])
def test_config3_prefill_8192_to_28672(kq, codec, M):
    _check_matmul(kq, codec, M, 28672, 8192, "bfloat16", 74, 48)


@pytest.mark.parametrize("codec", ["iq2_xxs", "iq3_s", "iq1_s"])
def test_prefill_iq_tile_choice(kq, codec):
    """Codebook codecs at the prefill benchmark shape through the automatic tile choice of their tall-tile kernel."""
    _check_matmul(kq, codec, 2048, 28672, 8192, "bfloat16", 96, 48)


@pytest.mark.parametrize("codec", ["mxfp4", "nvfp4"])
@pytest.mark.parametrize("M,N,K,dtype", [(2048, 28672, 8192, "bfloat16"), (512, 28672, 2880, "float16")])
def test_prefill_fp4_tile_choice(kq, codec, M, N, K, dtype):
    """mxfp4 / nvfp4 prefill through the automatic tile choice of the single-term kernel (nvfp4 blocks hold 64
    weights: K = 2880 is 45 of them)."""
    _check_matmul(kq, codec, M, N, K, dtype, 94, 48)


@pytest.mark.parametrize("codec", ["q8_0", "q4_0", "iq4_nl", "q4_1", "q5_0", "q5_1"])
@pytest.mark.parametrize("M,N,K", [(2048, 28672, 8192), (512, 28672, 2880), (1024, 8192, 8192)])
def test_prefill_block32_tile_choice(kq, codec, M, N, K):
    """q8_0 / q4_0 / iq4_nl / q5_0 / q4_1 / q5_1 prefill through the automatic tile choice of the two-term kernel: whole rounds of 256-row tiles
    plus a round of 128-row tiles, 256-row tiles alone (K = 2880: 45 steps), 128-row tiles alone."""
    _check_matmul(kq, codec, M, N, K, "bfloat16", 92, 48)


@pytest.mark.parametrize("M,N,K", [(2048, 28672, 8192), (512, 28672, 8192), (1024, 8192, 8192), (1024, 4096, 14336)])
def test_prefill_q6k_tile_choice(kq, M, N, K):
    """q6_k prefill through the automatic tile choice: whole rounds of 256-row tiles plus a round of 128-row tiles,
    256-row tiles alone, 128-row tiles alone, and the 64-row kernel for a matrix of few tiles."""
    _check_matmul(kq, "q6_k", M, N, K, "bfloat16", 90, 48)


@pytest.mark.parametrize("dtype", ["bfloat16", "float16"])
@pytest.mark.parametrize("codec", ["q2_k", "q3_k", "iq4_xs"])
@pytest.mark.parametrize("M,N,K", [(2048, 28672, 8192), (300, 16400, 512), (256, 32768, 256)])
def test_prefill_q2k_q3k_128x256_tiles(kq, codec, M, N, K, dtype):
    """q2_k / q3_k / iq4_xs prefill on the 128 x 256 tile kernel (M >= 256, 256 or more tiles): the benchmark shape, a ragged
    shape (M and N off the tile sizes, two superblocks) and a single-superblock K."""
    _check_matmul(kq, codec, M, N, K, dtype, 78, 48)


@pytest.mark.parametrize("codec", ["iq2_xxs", "iq3_s", "iq4_xs", "q2_k", "q3_k"])
def test_config5_lowbit_8192_square(kq, codec):
    _check_matmul(kq, codec, 1, 8192, 8192, "bfloat16", 76, None)


def _topk_routing(T, E, k, seed):
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    return np.argsort(-logits, axis=1)[:, :k].astype(np.int64)


@pytest.mark.parametrize("T", [1, 256])
def test_config4_moe_128_experts_top8(kq, T):
    """128 experts, top-8, hidden 2048, intermediate 768: fused gate/up GLU in q4_k, then the down projection in
    q6_k on the GLU output; the oracle recomputes a sample of tokens (each token's result is independent)."""
    E, H, I, R = 128, 2048, 768, 8
    gate = synth_wire_dev("q4_k", E * I, H, 80).reshape(E, I, -1)
    up = synth_wire_dev("q4_k", E * I, H, 81).reshape(E, I, -1)
    down = synth_wire_dev("q6_k", E * H, I, 82).reshape(E, H, -1)
    idx = _topk_routing(T, E, R, 83)
    xb, xt = make_x((T, H), "bfloat16", seed=84, scale=0.5)
    idx_dev = torch.from_numpy(idx).cuda()
    h = kq.moe_glu_gather_kq(xt, gate, up, "q4_k", idx_dev)
    y = kq.gather_qmv_kq(h, down, "q6_k", idx_dev)
    assert tuple(h.shape) == (T, R, I) and tuple(y.shape) == (T, R, H)
    toks = np.arange(T) if T <= 16 else np.unique(np.concatenate([[0, T - 1], np.random.default_rng(85).integers(0, T, 14)]))
    hb, yb = dev_to_bits(h), dev_to_bits(y)
    want_h = O.moe_glu_gather(xb[toks], gate.cpu().numpy(), up.cpu().numpy(), "q4_k", idx[toks], "silu", dtype="bfloat16")
    assert rel_l2(hb[toks], want_h, "bfloat16") <= TOL
    want_y = O.gather_qmv(hb[toks], down.cpu().numpy(), "q6_k", idx[toks], dtype="bfloat16")
    assert rel_l2(yb[toks], want_y, "bfloat16") <= TOL


def test_config5_moe_mxfp4_32_experts_top4_biased(kq):
    """32 experts of 2880 -> 2880 in mxfp4, top-4, 64 tokens, f32 biases, swiglu_clamp (alpha 1.702, limit 7)."""
    E, H, R, T = 32, 2880, 4, 64
    gate = synth_wire_dev("mxfp4", E * H, H, 90).reshape(E, H, -1)
    up = synth_wire_dev("mxfp4", E * H, H, 91).reshape(E, H, -1)
    down = synth_wire_dev("mxfp4", E * H, H, 92).reshape(E, H, -1)
    rng = np.random.default_rng(93)
    gb, ub, db = (rng.standard_normal((E, H)).astype(np.float32) * 0.01 for _ in range(3))
    idx = _topk_routing(T, E, R, 94)
    xb, xt = make_x((T, H), "bfloat16", seed=95, scale=0.5)
    idx_dev = torch.from_numpy(idx).cuda()
    h = kq.moe_glu_gather_kq(xt, gate, up, "mxfp4", idx_dev, act="swiglu_clamp", limit=7.0,
                             gate_bias=torch.from_numpy(gb).cuda(), up_bias=torch.from_numpy(ub).cuda(), alpha=1.702)
    y = kq.gather_qmv_kq(h, down, "mxfp4", idx_dev, bias=torch.from_numpy(db).cuda())
    toks = np.unique(np.concatenate([[0, T - 1], rng.integers(0, T, 6)]))
    hb, yb = dev_to_bits(h), dev_to_bits(y)
    want_h = O.moe_glu_gather(xb[toks], gate.cpu().numpy(), up.cpu().numpy(), "mxfp4", idx[toks], "swiglu_clamp", 7.0, gb,
                              ub, 1.702, dtype="bfloat16")
    assert rel_l2(hb[toks], want_h, "bfloat16") <= TOL
    want_y = O.gather_qmv(hb[toks], down.cpu().numpy(), "mxfp4", idx[toks], bias=db, dtype="bfloat16")
    assert rel_l2(yb[toks], want_y, "bfloat16") <= TOL
