"""kq.quantize (host encoders): pinned against the reference's own encoder output -- the committed
wire fixtures were minted by the reference from default_rng(1234)/(4321) (tests/gen_fixtures.py:62-89)
-- and against the reference's round-trip bounds (tests/test_encode.py:34-45).  CPU only."""
import os
import sys

import numpy as np
import pytest
import torch

import oracle_lib as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "mlx-kquant_amd"))
import kq  # noqa: E402

GOLD = os.path.join(ROOT, "tests", "golden")
KCODECS = ["q2_k", "q3_k", "q4_k", "q5_k", "q6_k"]
RT_BOUND = {"q8_0": 0.02, "q4_0": 0.15, "q4_1": 0.15, "q5_0": 0.10, "q5_1": 0.10, "q6_k": 0.05, "q5_k": 0.08,
            "q4_k": 0.12, "q3_k": 0.25, "q2_k": 0.40}


def _enc(w, codec, imatrix=None):
    wq, scales = kq.quantize(torch.from_numpy(w), codec, None if imatrix is None else torch.from_numpy(imatrix))
    assert scales.dtype == torch.uint8 and tuple(scales.shape) == (1,)
    return wq.numpy()


@pytest.mark.parametrize("codec", KCODECS)
def test_reproduces_reference_fixture_bytes(codec):
    """The fixtures were encoded on Metal; the reference's x86 encoder reproduces them up to a few
    ULP-tie bytes (FMA / reduction order).  A faithful restatement must land in the same band; any
    algorithmic deviation changes a large fraction of the bytes."""
    gold = np.load(os.path.join(GOLD, f"{codec}.npz"))["wire"]
    w = (np.random.default_rng(1234).standard_normal((256, 512)) * 0.1).astype(np.float32)
    mine = _enc(w, codec)
    assert mine.shape == gold.shape
    frac = np.mean(mine != gold)
    assert frac < 2e-3, (codec, frac)
    # and the decoded tensors agree to well under the quantisation step
    a, b = O.dequantize(mine, codec), O.dequantize(gold, codec)
    assert np.linalg.norm(a - b) / np.linalg.norm(b) < 2e-2  # a flipped scale nibble moves 16 coarse weights


def test_reproduces_reference_moe_fixture_bytes():
    rng = np.random.default_rng(4321)
    for codec in KCODECS:
        gold = np.load(os.path.join(GOLD, f"{codec}_moe.npz"))["wire"]
        for e in range(4):
            w = (rng.standard_normal((128, 512)) * 0.1).astype(np.float32)
            assert np.mean(_enc(w, codec) != gold[e]) < 3e-3, (codec, e)


@pytest.mark.parametrize("codec", list(RT_BOUND))
def test_round_trip_bounds(codec):
    w = (np.random.default_rng(7).standard_normal((64, 1024)) * 0.02).astype(np.float32)
    wire = _enc(w, codec)
    wpb, bpb = O.geometry(codec)
    assert wire.dtype == np.uint8 and wire.shape == (64, 1024 // wpb * bpb)
    rel = np.linalg.norm(O.dequantize(wire, codec) - w) / np.linalg.norm(w)
    assert rel < RT_BOUND[codec], (codec, rel)
    assert np.array_equal(wire, _enc(w, codec))  # deterministic (also across the block-parallel split)


def test_imatrix_changes_kquant_bytes_only():
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((8, 512)) * 0.05).astype(np.float32)
    im = rng.uniform(0.1, 10.0, 512).astype(np.float32)
    for codec in KCODECS:
        assert not np.array_equal(_enc(w, codec), _enc(w, codec, im)), codec
        rel = np.linalg.norm(O.dequantize(_enc(w, codec, im), codec) - w) / np.linalg.norm(w)
        assert rel < 1.5 * RT_BOUND[codec]
    for codec in ("q8_0", "q4_0", "q4_1", "q5_0", "q5_1"):
        assert np.array_equal(_enc(w, codec), _enc(w, codec, im)), codec


def test_edge_cases_and_errors():
    z = np.zeros((2, 256), np.float32)
    for codec in RT_BOUND:
        assert np.all(O.dequantize(_enc(z, codec), codec) == 0), codec
    w3 = (np.random.default_rng(1).standard_normal((2, 3, 256)) * 0.1).astype(np.float32)
    assert _enc(w3, "q4_k").shape == (2, 3, 144)
    assert _enc(np.zeros((0, 256), np.float32), "q6_k").shape == (0, 210)
    with pytest.raises(ValueError):
        _enc(np.zeros((2, 100), np.float32), "q4_k")
    with pytest.raises(ValueError):
        kq.quantize(torch.zeros((2, 256)), "nope")
    with pytest.raises(ValueError):
        kq.quantize(torch.zeros((2, 256)), "mxfp4")  # decode-only codec
    with pytest.raises(ValueError):
        kq.quantize(torch.zeros((2, 256)), "iq2_xxs")  # imatrix-required codec
    with pytest.raises(ValueError):
        kq.quantize(torch.zeros((2, 256)), "q4_k", torch.ones(128))


def test_legacy_closed_forms():
    x = (np.random.default_rng(3).standard_normal((16, 32)) * 0.3).astype(np.float32)
    wire = _enc(x, "q8_0")
    d = wire[:, :2].copy().view(np.float16).astype(np.float32)[:, 0]
    assert np.allclose(d, np.abs(x).max(1) / 127, rtol=1e-3)
    assert np.all(np.abs(O.dequantize(wire, "q8_0") - x) <= d[:, None] * 0.5 + 1e-6 + np.abs(x) * 1e-3)
    wire = _enc(x, "q4_1")
    m = wire[:, 2:4].copy().view(np.float16).astype(np.float32)[:, 0]
    assert np.allclose(m, x.min(1), rtol=1e-3, atol=1e-4)
