"""GPU parity: kq.dequantize (HIP) vs the CPU oracle -- bit-exact for every codec and dtype."""
import os

import numpy as np
import pytest
import torch

import oracle_lib as O
import wire_pack
from gpu_util import dev_to_bits, wire_to_dev, TORCH_DT

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    assert os.path.exists(_kq.lib_path())
    return _kq


@pytest.mark.parametrize("codec", O.ALL_CODECS)
@pytest.mark.parametrize("dtype", ["float32", "float16", "bfloat16"])
def test_dequantize_bit_exact_synth(kq, codec, dtype):
    # 1037 blocks: not a multiple of the per-workgroup block run -> exercises the ragged tail
    wire = O.synth_wire(codec, 1037, seed=11)
    got = kq.dequantize(wire_to_dev(wire), None, codec, dtype=TORCH_DT[dtype])
    want = O.dequantize(wire, codec, dtype)
    assert got.shape == want.shape
    gb = dev_to_bits(got)
    if dtype == "float32":
        assert np.array_equal(gb.view(np.uint32), want.view(np.uint32)), codec
    else:
        assert np.array_equal(gb, want), codec


@pytest.mark.parametrize("codec", O.ALL_CODECS)
def test_dequantize_known_answer_blocks(kq, codec):
    wire, want = wire_pack.make(codec, 96, seed=500 + O.codec_id(codec))
    got = dev_to_bits(kq.dequantize(wire_to_dev(wire), None, codec, dtype=torch.float32))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), codec


@pytest.mark.parametrize("codec", ["q2_k", "q3_k", "q4_k", "q5_k", "q6_k"])
def test_dequantize_reference_fixtures(kq, codec):
    wire = np.load(os.path.join(GOLD, f"{codec}.npz"))["wire"]
    got = dev_to_bits(kq.dequantize(wire_to_dev(wire), None, codec, dtype=torch.float32))
    assert np.array_equal(got.view(np.uint32), O.dequantize(wire, codec).view(np.uint32))
    moe = np.load(os.path.join(GOLD, f"{codec}_moe.npz"))["wire"]
    got = kq.dequantize(wire_to_dev(moe), None, codec)  # default dtype float16, 3-D input
    assert got.dtype == torch.float16 and tuple(got.shape) == (4, 128, 512)
    assert np.array_equal(dev_to_bits(got), O.dequantize(moe, codec, "float16"))


def test_dequantize_edge_cases(kq):
    d = torch.device("cuda:0")
    out = kq.dequantize(torch.empty((0, 144), dtype=torch.uint8, device=d), None, "q4_k")
    assert tuple(out.shape) == (0, 256)
    one = O.synth_wire("q6_k", 1, seed=5)
    got = dev_to_bits(kq.dequantize(wire_to_dev(one[0]), None, "q6_k", dtype=torch.float32))
    assert np.array_equal(got, O.dequantize(one, "q6_k")[0])
    # non-contiguous view and a byte-misaligned start
    wire = O.synth_wire("iq2_xxs", 64, seed=6)
    big = torch.zeros(64 * 66 + 3, dtype=torch.uint8, device=d)
    big[3:] = wire_to_dev(wire).reshape(-1)
    got = dev_to_bits(kq.dequantize(big[3:].reshape(64, 66), None, "iq2_xxs", dtype=torch.float32))
    assert np.array_equal(got.view(np.uint32), O.dequantize(wire, "iq2_xxs").view(np.uint32))
    with pytest.raises(ValueError):
        kq.dequantize(torch.zeros(145, dtype=torch.uint8, device=d), None, "q4_k")
    with pytest.raises(ValueError):
        kq.dequantize(torch.zeros(144, dtype=torch.uint8, device=d), None, "q9_z")
    with pytest.raises(ValueError):
        kq.dequantize(torch.zeros(144, dtype=torch.float16, device=d), None, "q4_k")
    with pytest.raises(RuntimeError):
        kq.dequantize(torch.zeros(144, dtype=torch.uint8), None, "q4_k")


def test_dequantize_config1_size(kq):
    # the reference CPU-runnable configuration, 4096 x 4096 q4_k -> f16; full size through block independence:
    # the 4096 rows are 512 distinct rows tiled, compared with the oracle on those rows.
    base = O.synth_wire("q4_k", 512 * 16, seed=21).reshape(512, 16 * 144)
    wire = np.tile(base, (8, 1))
    got = dev_to_bits(kq.dequantize(wire_to_dev(wire), None, "q4_k"))
    want = O.dequantize(base, "q4_k", "float16")
    assert got.shape == (4096, 4096)
    for r in range(8):
        assert np.array_equal(got[512 * r:512 * (r + 1)], want)


@pytest.mark.parametrize("codec", ["q4_k", "q6_k", "iq2_xxs", "iq4_xs"])
def test_dequantize_large_tensor_chunking(kq, codec):
    """Tensors of 64 Mi weights and more take the 16384-weight workgroup chunk; 262176 superblocks leave a
    ragged last workgroup (32 of 64 blocks).  Compared in slices to keep the host copies small."""
    nblk = 262176
    wire = O.synth_wire(codec, nblk, seed=77)
    got = dev_to_bits(kq.dequantize(wire_to_dev(wire), None, codec, dtype=torch.float16)).reshape(-1)
    step = 32768
    for b0 in range(0, nblk, step):
        want = O.dequantize(wire.reshape(nblk, -1)[b0:b0 + step], codec, "float16").reshape(-1)
        assert np.array_equal(got[b0 * 256:b0 * 256 + want.size], want), (codec, b0)
