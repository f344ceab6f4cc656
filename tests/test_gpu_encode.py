"""GPU parity: the device encoder behind kq.quantize reproduces the reference's own fixture bytes inside the
reference's x86-vs-Metal band, writes the host encoder's bytes, and what it writes decodes within the codec's bound."""
import os

import numpy as np
import pytest
import torch

import oracle_lib as O

pytestmark = pytest.mark.gpu
DEV_CODECS = ["q8_0", "q4_0", "q4_1", "q5_0", "q5_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k"]
# round-trip rel-L2 bounds on N(0, 1) rows: loose sanity limits per bit width
BOUND = {"q8_0": 0.02, "q4_0": 0.2, "q4_1": 0.2, "q5_0": 0.1, "q5_1": 0.1, "q2_k": 0.5, "q3_k": 0.3, "q4_k": 0.15,
         "q5_k": 0.08, "q6_k": 0.05}


@pytest.fixture(scope="module")
def kq():
    import kq as _kq
    return _kq


@pytest.mark.parametrize("codec", DEV_CODECS)
def test_device_encoder_writes_host_bytes(kq, codec):
    rng = np.random.default_rng(100 + O.codec_id(codec))
    rows, K = 37, 1024
    w = rng.standard_normal((rows, K)).astype(np.float32)
    w[3] = 0.0                                 # an all-zero row
    w[5, :256] = 0.0                           # a zero superblock inside a live row
    w[7] *= 1e-6                               # tiny magnitudes
    w[9, ::7] *= 40.0                          # outliers
    im = (np.abs(rng.standard_normal(K)) + 0.1).astype(np.float32)
    wt = torch.from_numpy(w)
    for imat in (None, im):
        it = None if imat is None else torch.from_numpy(imat)
        host, _ = kq.quantize(wt, codec, it)
        dev, scales = kq.quantize(wt.cuda(), codec, None if it is None else it.cuda())
        assert dev.is_cuda and dev.dtype == torch.uint8 and tuple(dev.shape) == tuple(host.shape)
        assert tuple(scales.shape) == (1,)
        assert np.array_equal(dev.cpu().numpy(), host.numpy()), (codec, imat is not None)
    back = O.dequantize(dev.cpu().numpy(), codec).reshape(rows, K)
    live = [r for r in range(rows) if r not in (3, 9)]  # the outlier row is covered by the byte comparison only
    assert np.linalg.norm(back[live] - w[live]) / np.linalg.norm(w[live]) < BOUND[codec]
    assert not back[3].any()


GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
KCODECS = ["q2_k", "q3_k", "q4_k", "q5_k", "q6_k"]


@pytest.mark.parametrize("codec", KCODECS)
def test_device_encoder_reproduces_reference_fixture_bytes(kq, codec):
    """The device encoder against the reference's own vectors, directly: the committed wire fixtures were minted
    by the reference's encoder from default_rng(1234) (tests/gen_fixtures.py:62-63) on Metal, and the reference's
    x86 encoder lands within a few ULP-tie bytes of them (tests/test_encode.py:203-250).  kq.quantize on cuda:0
    must land in the same band, and what it writes must decode to what the fixture decodes to."""
    gold = np.load(os.path.join(GOLD, f"{codec}.npz"))["wire"]
    w = (np.random.default_rng(1234).standard_normal((256, 512)) * 0.1).astype(np.float32)
    dev, _ = kq.quantize(torch.from_numpy(w).cuda(), codec)
    mine = dev.cpu().numpy()
    assert mine.shape == gold.shape
    frac = np.mean(mine != gold)
    assert frac < 2e-3, (codec, frac)
    a, b = O.dequantize(mine, codec), O.dequantize(gold, codec)
    assert np.linalg.norm(a - b) / np.linalg.norm(b) < 2e-2
    # the fixture's bytes, decoded on the device, are the oracle's decode bit for bit
    got = kq.dequantize(torch.from_numpy(gold).cuda(), None, codec, dtype=torch.float32).cpu().numpy()
    assert np.array_equal(got.view(np.uint32).ravel(), b.view(np.uint32).ravel())


def test_device_encoder_reproduces_reference_moe_fixture_bytes(kq):
    """Same for the expert-stack fixtures (default_rng(4321), four experts of 128 x 512, tests/gen_fixtures.py:80-89)."""
    rng = np.random.default_rng(4321)
    ws = [(rng.standard_normal((128, 512)) * 0.1).astype(np.float32) for _ in range(4 * len(KCODECS))]
    for ci, codec in enumerate(KCODECS):
        gold = np.load(os.path.join(GOLD, f"{codec}_moe.npz"))["wire"]
        stack = np.stack(ws[4 * ci:4 * ci + 4])
        dev, _ = kq.quantize(torch.from_numpy(stack).cuda(), codec)   # leading (expert) dimension kept
        mine = dev.cpu().numpy()
        assert mine.shape == gold.shape
        for e in range(4):
            assert np.mean(mine[e] != gold[e]) < 3e-3, (codec, e)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_device_encoder_half_inputs_and_stacks(kq, dtype):
    """16-bit inputs are widened exactly as the host path widens them; leading dimensions are kept."""
    rng = np.random.default_rng(7)
    w = torch.from_numpy(rng.standard_normal((3, 5, 512)).astype(np.float32) * 0.05).to(dtype)
    for codec in ("q4_k", "q6_k", "q8_0"):
        host, _ = kq.quantize(w, codec)
        dev, _ = kq.quantize(w.cuda(), codec)
        assert tuple(dev.shape) == tuple(host.shape) and dev.shape[:2] == (3, 5)
        assert torch.equal(dev.cpu(), host)


def test_host_encoder_still_reachable_and_iq_stays_on_host(kq):
    rng = np.random.default_rng(8)
    w = torch.from_numpy(rng.standard_normal((4, 512)).astype(np.float32)).cuda()
    a, _ = kq.quantize(w, "q4_k", stream="cpu")          # forced host encoder, result back on the GPU
    b, _ = kq.quantize(w, "q4_k")
    assert a.is_cuda and torch.equal(a, b)
    lib = kq._load()
    assert lib.kq_quantize_dev_supported(lib.kq_codec_id(b"q4_k")) == 1
    assert lib.kq_quantize_dev_supported(lib.kq_codec_id(b"iq4_xs")) == 0
    c, _ = kq.quantize(w, "iq4_xs")                      # host encoder behind the same call
    assert c.is_cuda and tuple(c.shape) == (4, 272)
    assert lib.kq_quantize_dev(w.data_ptr(), 0, None, c.data_ptr(), 4, 512, lib.kq_codec_id(b"iq4_xs"), None) == -2


def test_device_encoder_large_matrix_speed_sanity(kq):
    """A Llama gate/up sized matrix: bytes equal the host's on a sample of rows; prints both times."""
    import time
    rng = np.random.default_rng(9)
    w = torch.from_numpy((rng.standard_normal((2048, 4096)) * 0.02).astype(np.float32))
    wd = w.cuda()
    kq.quantize(wd[:8], "q4_k")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    dev, _ = kq.quantize(wd, "q4_k")
    torch.cuda.synchronize()
    t_dev = time.perf_counter() - t0
    t0 = time.perf_counter()
    host, _ = kq.quantize(w, "q4_k")
    t_host = time.perf_counter() - t0
    print(f"q4_k 2048 x 4096: device {t_dev * 1e3:.1f} ms, host {t_host * 1e3:.1f} ms")
    assert torch.equal(dev.cpu(), host)
