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
            "q4_k": 0.12, "q3_k": 0.25, "q2_k": 0.40, "iq4_nl": 0.12, "iq4_xs": 0.12}  # iq4: tests/test_iq_encode.py:34-35
KV_IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float32)


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
    for codec in KCODECS + ["iq4_nl", "iq4_xs"]:  # every IQ codec is importance-weighted, flat-32 iq4_nl included
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


def test_iq4_known_answer_blocks():
    """Blocks that ARE codebook points must come back as exactly those levels and scales: a perfect fit
    maximises the weighted correlation the scale search ranks by, so neither the first guess nor any of
    the 15 trial scales can displace it.  Pins the codebook search, the fp16 scale slot, the 6-bit
    scale split of iq4_xs (scales_l nibbles, scales_h pairs) and the nibble packing."""
    rng = np.random.default_rng(11)
    # iq4_nl: 40 blocks, scale d exactly representable in fp16, one weight at the -127 end
    lv = rng.integers(0, 16, (40, 32))
    lv[:, 5] = 0
    d = (rng.integers(1, 64, 40) / 4096.0).astype(np.float32) * rng.choice([-1.0, 1.0], 40).astype(np.float32)
    x = d[:, None] * KV_IQ4NL[lv]
    wire = _enc(x.reshape(40, 32), "iq4_nl")
    assert np.array_equal(wire[:, :2].copy().view(np.float16)[:, 0].astype(np.float32), d)
    assert np.array_equal(wire[:, 2:] & 15, lv[:, :16]) and np.array_equal(wire[:, 2:] >> 4, lv[:, 16:])
    # iq4_xs: super-scale D, block scales D * l with l in [-32, 31] and one block at -32
    nsb = 12
    lv = rng.integers(0, 16, (nsb, 8, 32))
    lv[:, :, 9] = 0
    lb = rng.integers(-32, 32, (nsb, 8))
    lb[lb == 0] = 3
    lb[:, 2] = -32
    D = (rng.integers(1, 32, nsb) / 65536.0).astype(np.float32)
    x = (D[:, None, None] * lb[:, :, None]) * KV_IQ4NL[lv]
    wire = _enc(x.reshape(nsb, 256).astype(np.float32), "iq4_xs")
    assert np.array_equal(wire[:, :2].copy().view(np.float16)[:, 0].astype(np.float32), D)
    u = lb + 32
    sl = wire[:, 4:8]
    got_lo = np.stack([sl[:, i // 2] >> (4 * (i & 1)) & 15 for i in range(8)], axis=1)
    sh = wire[:, 2].astype(np.uint32) | (wire[:, 3].astype(np.uint32) << 8)
    got_hi = np.stack([(sh >> (2 * i)) & 3 for i in range(8)], axis=1)
    assert np.array_equal(got_lo | (got_hi << 4), u)
    qs = wire[:, 8:].reshape(nsb, 8, 16)
    assert np.array_equal(qs & 15, lv[:, :, :16]) and np.array_equal(qs >> 4, lv[:, :, 16:])
    # and the decoder agrees with the pre-image exactly
    assert np.array_equal(O.dequantize(wire, "iq4_xs"), x.reshape(nsb, 256).astype(np.float32))


# ------------------------------------------------------------------ codebook codecs (iq2_xxs, iq3_xxs, iq3_s)
CB_BOUND = {"iq2_xxs": 0.45, "iq2_xs": 0.45, "iq2_s": 0.45, "iq3_xxs": 0.30, "iq3_s": 0.30,
            "iq1_s": 0.65, "iq1_m": 0.65}  # reference tests/test_iq_encode.py:36-43
# The reference's bounds carry about 1.3x headroom over what its encoder measures on this recipe (0.36 for iq2_xxs,
# 0.076 for the 4-bit pair; tests/test_iq_encode.py:28-32).  The encoders here are a different search over the same
# lattices, so their bytes differ from the reference's; what is pinned instead is that they are at least as close
# to the input as the reference's measured figures, with the values measured here (+3 %) as regression ceilings.
CB_MEASURED = {"iq2_xxs": 0.3553, "iq2_xs": 0.3131, "iq2_s": 0.2576, "iq3_xxs": 0.1915, "iq3_s": 0.1419,
               "iq1_s": 0.5075, "iq1_m": 0.4806, "iq4_nl": 0.0761, "iq4_xs": 0.0767}
REF_MEASURED = {"iq2_xxs": 0.36, "iq4_nl": 0.076 * 1.01, "iq4_xs": 0.076 * 1.01}


@pytest.mark.parametrize("codec", list(CB_MEASURED))
def test_iq_round_trip_quality_ceilings(codec):
    rng = np.random.default_rng(11)
    w = (rng.standard_normal((256, 512)) * 0.1).astype(np.float32)
    im = (np.abs(rng.standard_normal(512)) + 0.1).astype(np.float32)
    rel = np.linalg.norm(O.dequantize(_enc(w, codec, im), codec) - w) / np.linalg.norm(w)
    assert rel <= CB_MEASURED[codec] * 1.03, (codec, rel)
    if codec in REF_MEASURED:
        assert rel <= REF_MEASURED[codec], (codec, rel)


@pytest.mark.parametrize("codec", list(CB_BOUND))
def test_codebook_round_trip_bounds(codec):
    """Same data recipe and bounds as the reference's IQ round-trip gate (gaussian * 0.1, |gaussian| + 0.1
    importance, 256 x 512; tests/test_iq_encode.py:44-60, 77-96): measured there 0.36 for iq2_xxs."""
    rng = np.random.default_rng(11)
    w = (rng.standard_normal((256, 512)) * 0.1).astype(np.float32)
    im = (np.abs(rng.standard_normal(512)) + 0.1).astype(np.float32)
    wire = _enc(w, codec, im)
    wpb, bpb = O.geometry(codec)
    assert wire.shape == (256, 512 // wpb * bpb)
    rel = np.linalg.norm(O.dequantize(wire, codec) - w) / np.linalg.norm(w)
    assert rel < CB_BOUND[codec], (codec, rel)
    assert rel > 0.02  # a 2-3 bit codec cannot be this good: guards against a vacuous decode
    assert np.array_equal(wire, _enc(w, codec, im))
    if codec in ("iq2_xxs", "iq2_xs", "iq1_s"):
        with pytest.raises(ValueError):
            kq.quantize(torch.from_numpy(w), codec)  # imatrix-required, as ggml_quantize_requires_imatrix
    else:
        rel = np.linalg.norm(O.dequantize(_enc(w, codec), codec) - w) / np.linalg.norm(w)
        assert rel < CB_BOUND[codec], (codec, rel)


def _synth_lattice_wire(codec, nsb, seed):
    """Random but structurally exact wire: every sub-block scale nibble is set, block 0 carries the
    largest one (15), super-scale d is a power of two."""
    rng = np.random.default_rng(seed)
    wpb, bpb = O.geometry(codec)
    wire = O.synth_wire(codec, nsb, seed).reshape(nsb, bpb).copy()
    wire[:, 0:2] = np.frombuffer(np.float16(2.0 ** -6).tobytes(), dtype=np.uint8)
    if codec == "iq2_xxs":
        for ib in range(8):  # scale nibble = top 4 bits of the second word of a sub-block
            wire[:, 2 + 8 * ib + 7] = (wire[:, 2 + 8 * ib + 7] & 0x0F) | ((15 if ib == 0 else rng.integers(3, 15)) << 4)
    return wire


def test_iq2_xxs_known_answer_blocks():
    """Weights that ARE codebook points (decode of a valid wire) must come back as the same codebook entries
    and signs: the rounded lattice point of every group is an entry and the sign parity is even by
    construction.  Checks the codebook index built from the decode tables, the level <-> value map and the
    entry / 7-bit sign packing.  Magnitudes are not exact: the search fits scale * (1, 3, 5) while the decode
    values are (8, 25, 43), as in ggml."""
    wire = _synth_lattice_wire("iq2_xxs", 24, 5)
    x = O.dequantize(wire, "iq2_xxs").reshape(24, 256)
    mine = _enc(x, "iq2_xxs", np.ones(256, np.float32))
    a, b = wire[:, 2:].reshape(24, 8, 8), mine[:, 2:].reshape(24, 8, 8)
    assert np.mean(a[:, :, :4] == b[:, :, :4]) > 0.97  # codebook entries
    sa = a[:, :, 4:].copy().view(np.uint32) & 0x0FFFFFFF
    sb = b[:, :, 4:].copy().view(np.uint32) & 0x0FFFFFFF
    assert np.mean(sa == sb) > 0.99  # 4 x 7 sign bits
    back = O.dequantize(mine, "iq2_xxs").reshape(24, 256)
    assert np.linalg.norm(back - x) / np.linalg.norm(x) < 0.10


@pytest.mark.parametrize("codec", ["iq2_xs", "iq2_s"])
def test_iq2_16_known_answer_blocks(codec):
    """As above for the 16-weight sub-block codecs: decoded codebook points re-encode to the same entries
    (9- / 10-bit indices split over qs and the u16 / qh fields) and the same sign bits."""
    nsb = 24
    wire = O.synth_wire(codec, nsb, 8).reshape(nsb, -1).copy()
    wire[:, 0:2] = np.frombuffer(np.float16(2.0 ** -6).tobytes(), dtype=np.uint8)
    soff = 66 if codec == "iq2_xs" else 74
    wire[:, soff:soff + 8] |= 0x33  # no sub-block scale below 3: keeps every sub-block well above the noise floor
    wire[:, soff] |= 0x0F
    x = O.dequantize(wire, codec).reshape(nsb, 256)
    mine = _enc(x, codec, np.ones(256, np.float32))
    if codec == "iq2_xs":
        a, b = wire[:, 2:66].copy().view(np.uint16), mine[:, 2:66].copy().view(np.uint16)
        assert np.mean((a & 511) == (b & 511)) > 0.95 and np.mean((a >> 9) == (b >> 9)) > 0.99
    else:
        assert np.mean(wire[:, 2:34] == mine[:, 2:34]) > 0.95    # entry low bytes
        assert np.mean(wire[:, 66:74] == mine[:, 66:74]) > 0.90  # entry bits 8-9, four groups per byte
        assert np.mean(wire[:, 34:66] == mine[:, 34:66]) > 0.99  # sign bytes
    back = O.dequantize(mine, codec).reshape(nsb, 256)
    assert np.linalg.norm(back - x) / np.linalg.norm(x) < 0.12


@pytest.mark.parametrize("codec", ["iq3_xxs", "iq3_s"])
def test_iq3_lattice_points_keep_their_shape(codec):
    """Decode of a valid wire re-encodes to the same lattice points up to the per-sub-block scale (ggml
    inflates d by 1.0125 / 1.033 on purpose, so magnitudes move by that factor at most)."""
    wire = O.synth_wire(codec, 16, 6).reshape(16, -1).copy()
    wire[:, 0:2] = np.frombuffer(np.float16(2.0 ** -5).tobytes(), dtype=np.uint8)
    x = O.dequantize(wire, codec).reshape(16, 256)
    back = O.dequantize(_enc(x, codec, np.ones(256, np.float32)), codec).reshape(16, 256)
    assert np.mean(np.sign(back) == np.sign(x)) > 0.999
    rel = np.linalg.norm(back - x) / np.linalg.norm(x)
    assert rel < 0.08, (codec, rel)


def test_codebook_zero_and_imatrix():
    for codec in CB_BOUND:
        z = np.zeros((2, 256), np.float32)
        wire = _enc(z, codec, np.ones(256, np.float32))
        assert not wire.any()
        assert not O.dequantize(wire, codec).any()
    rng = np.random.default_rng(12)
    w = (rng.standard_normal((8, 512)) * 0.05).astype(np.float32)
    flat = np.ones(512, np.float32)
    steep = rng.uniform(0.05, 20.0, 512).astype(np.float32)
    for codec in CB_BOUND:
        a, b = _enc(w, codec, flat), _enc(w, codec, steep)
        assert not np.array_equal(a, b), codec
        # the importance-weighted error is what the search minimises: it must not get worse under its own weights
        ea = np.sum(steep * (O.dequantize(a, codec) - w) ** 2)
        eb = np.sum(steep * (O.dequantize(b, codec) - w) ** 2)
        assert eb < ea * 1.02, (codec, ea, eb)


def test_iq1_s_known_answer_blocks():
    """Ternary codebook points (decode of a valid wire) re-encode to the same entries and shift signs: checks the
    int8 level map of the 2048-entry codebook, the 11-bit entry split over qs / qh and the shift bit."""
    nsb = 24
    wire = O.synth_wire("iq1_s", nsb, 9).reshape(nsb, 50).copy()
    wire[:, 0:2] = np.frombuffer(np.float16(2.0 ** -5).tobytes(), dtype=np.uint8)
    qh = wire[:, 34:50].copy().view(np.uint16)
    qh[:] = (qh & 0x8FFF) | (np.random.default_rng(10).integers(2, 8, qh.shape).astype(np.uint16) << 12)
    qh[:, 0] |= 0x7000
    wire[:, 34:50] = qh.view(np.uint8)
    x = O.dequantize(wire, "iq1_s").reshape(nsb, 256)
    mine = _enc(x, "iq1_s", np.ones(256, np.float32))
    mq = mine[:, 34:50].copy().view(np.uint16)
    assert np.mean(wire[:, 2:34] == mine[:, 2:34]) > 0.97          # entry low bytes
    assert np.mean((qh & 0x0FFF) == (mq & 0x0FFF)) > 0.95          # 4 x 3 entry high bits
    assert np.mean((qh & 0x8000) == (mq & 0x8000)) > 0.97          # shift signs
    back = O.dequantize(mine, "iq1_s").reshape(nsb, 256)
    assert np.linalg.norm(back - x) / np.linalg.norm(x) < 0.15


def test_iq1_m_known_answer_blocks():
    """As above for the 16-weight sub-blocks of iq1_m: entries, the two shift-sign bits per sub-block (qh bits 3 and
    7) and the 3-bit scales come back, and the f16 block scale scattered over the four top nibbles decodes to
    within the encoder's 1.1125 fudge of the original."""
    nsb = 24
    rng = np.random.default_rng(12)
    wire = O.synth_wire("iq1_m", nsb, 13).reshape(nsb, 56).copy()
    sc = wire[:, 48:56].copy().view(np.uint16)
    lv = rng.integers(2, 8, (nsb, 16))
    lv[:, 0] = 7
    du = int(np.frombuffer(np.float16(2.0 ** -5).tobytes(), dtype=np.uint16)[0])
    for k in range(4):
        word = np.zeros(nsb, np.uint16)
        for j in range(4):
            word |= (lv[:, 4 * k + j] << (3 * j)).astype(np.uint16)
        sc[:, k] = word | np.uint16(((du >> (4 * k)) & 15) << 12)
    wire[:, 48:56] = sc.view(np.uint8)
    x = O.dequantize(wire, "iq1_m").reshape(nsb, 256)
    mine = _enc(x, "iq1_m", np.ones(256, np.float32))
    assert np.mean(wire[:, 0:32] == mine[:, 0:32]) > 0.98                      # entry low bytes
    assert np.mean((wire[:, 32:48] & 0x77) == (mine[:, 32:48] & 0x77)) > 0.98  # entry high bits
    assert np.mean((wire[:, 32:48] & 0x88) == (mine[:, 32:48] & 0x88)) > 0.98  # shift signs
    assert np.mean((mine[:, 48:56].copy().view(np.uint16) & 0xFFF) == (sc & 0xFFF)) > 0.98  # 3-bit scales
    back = O.dequantize(mine, "iq1_m").reshape(nsb, 256)
    assert np.linalg.norm(back - x) / np.linalg.norm(x) < 0.15
    # without an importance matrix the x^2 weighting still lands on the same structure
    back = O.dequantize(_enc(x, "iq1_m"), "iq1_m").reshape(nsb, 256)
    assert np.linalg.norm(back - x) / np.linalg.norm(x) < 0.15
