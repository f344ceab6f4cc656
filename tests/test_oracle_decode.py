"""Pins the CPU oracle's block decoders and half-precision casts (no GPU needed).

Checks, in order of strength:
  * known-answer blocks from independent packers (tests/wire_pack.py): exact f32 equality;
  * the reference's own wire fixtures (tests/golden/*.npz, minted by its encoder from
    default_rng(1234)/(4321), tests/gen_fixtures.py:62-89): the decode must land within
    the reference's round-trip bounds (tests/test_encode.py:34-45) of the regenerated
    pre-image -- an index, order or scale mistake gives an error of order 1;
  * casts against numpy's IEEE float16 and an integer-arithmetic bf16 round-to-nearest-even;
  * structural invariants (block independence, prefix property, half = rne(f32)).
"""
import hashlib
import os

import numpy as np
import pytest

import oracle_lib as O
import wire_pack

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
KCODECS = ["q2_k", "q3_k", "q4_k", "q5_k", "q6_k"]
RT_BOUND = {"q6_k": 0.05, "q5_k": 0.08, "q4_k": 0.12, "q3_k": 0.25, "q2_k": 0.40}
RT_FLOOR = {"q6_k": 0.005, "q5_k": 0.01, "q4_k": 0.02, "q3_k": 0.05, "q2_k": 0.1}


def test_registry_geometry():
    # src/kquant_codec.cpp:12-37
    want = {"q2_k": (256, 84), "q3_k": (256, 110), "q4_k": (256, 144), "q5_k": (256, 176), "q6_k": (256, 210),
            "q4_0": (32, 18), "q4_1": (32, 20), "q5_0": (32, 22), "q5_1": (32, 24), "q8_0": (32, 34),
            "iq4_nl": (32, 18), "iq4_xs": (256, 136), "iq3_s": (256, 110), "iq3_xxs": (256, 98),
            "iq2_xxs": (256, 66), "iq2_xs": (256, 74), "iq2_s": (256, 82), "iq1_s": (256, 50), "iq1_m": (256, 56),
            "mxfp4": (32, 17), "nvfp4": (64, 36)}
    assert O.ALL_CODECS == list(want)
    for k, v in want.items():
        assert O.geometry(k) == v


def test_grid_blob_digest_and_structure():
    blob = open(os.path.join(O.ROOT, "mlx-kquant_amd", "data", "kq_iq_grids.bin"), "rb").read()
    assert len(blob) == 33792
    assert hashlib.sha256(blob).hexdigest() == "0e3d3ad9db09472d55cdd43268068d9f86c0875f02567e2c499ffbb70f1e1d4b"
    g = wire_pack.GRIDS
    for name in ("iq2_xxs", "iq2_xs", "iq2_s"):
        assert set(np.unique(g[name])) <= {0x08, 0x19, 0x2B}
        assert len({bytes(r) for r in g[name]}) == len(g[name])
    assert set(np.unique(g["iq1"])) <= {-1, 0, 1}
    assert set(np.unique(g["iq3_xxs"])) == {4, 12, 20, 28, 36, 44, 52, 62}
    assert set(np.unique(g["iq3_s"])) == {1, 3, 5, 7, 9, 11, 13, 15}
    for name in ("iq3_xxs", "iq3_s"):
        assert len({bytes(r) for r in g[name]}) == len(g[name])


@pytest.mark.skipif(not os.path.exists("/root/reference/src/kquant_iq_tables.h"), reason="reference not mounted")
def test_grid_blob_matches_reference_header_text():
    import re
    import struct
    src = open("/root/reference/src/kquant_iq_tables.h").read()
    blob = b""
    for name, fmt in (("iq2xxs_grid", "Q"), ("iq2xs_grid", "Q"), ("iq2s_grid", "Q"), ("iq1s_grid", "Q"),
                      ("iq3xxs_grid", "I"), ("iq3s_grid", "I")):
        m = re.search(r"inline constexpr \w+ " + name + r"\[(\d+)\] = \{(.*?)\};", src, re.S)
        vals = [int(t, 0) for t in re.findall(r"0x[0-9a-fA-F]+|\d+", m.group(2))]
        assert len(vals) == int(m.group(1))
        blob += struct.pack("<%d%s" % (len(vals), fmt), *vals)
    assert blob == open(os.path.join(O.ROOT, "mlx-kquant_amd", "data", "kq_iq_grids.bin"), "rb").read()


def test_f16_to_f32_all_patterns():
    h = np.arange(65536, dtype=np.uint16)
    got = np.array([O.lib.kq_oracle_f16_to_f32(int(v)) for v in h], dtype=np.float32)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def _bf16_rne_int(x):
    """round-to-nearest-even to 8 significant bits using exact integer comparison."""
    u = x.view(np.uint32).astype(np.uint64)
    lo = u & ~np.uint64(0xFFFF)
    rem = u & np.uint64(0xFFFF)
    up = (rem > 0x8000) | ((rem == 0x8000) & (((lo >> 16) & 1) == 1))
    return ((lo >> 16) + up.astype(np.uint64)).astype(np.uint16)


def test_f32_to_half_roundings():
    rng = np.random.default_rng(3)
    bits = rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32)
    # dense coverage of the f16 normal/subnormal/overflow boundaries and exact ties
    h = rng.integers(0, 0x7C00, 50000).astype(np.uint16).view(np.float16).astype(np.float32)
    ties = (h.view(np.uint32) + 0x1000).view(np.float32)  # exactly halfway to the next f16
    x = np.concatenate([bits.view(np.float32), h, ties, -ties, (h.view(np.uint32) + 0xFFF).view(np.float32),
                        np.array([65504., 65519.99, 65520., 1e-8, 2.0 ** -25, 2.0 ** -24, 0.0, -0.0], np.float32)])
    x = x[np.isfinite(x)]
    want16 = x.astype(np.float16).view(np.uint16)
    got16 = np.array([O.lib.kq_oracle_f32_to_f16(float(v)) for v in x[:60000]], dtype=np.uint16)
    assert np.array_equal(got16, want16[:60000])
    tail = x[-150008:]
    got16 = O.f32_to_bits(tail, "float16")
    assert np.array_equal(got16, tail.astype(np.float16).view(np.uint16))
    gotb = np.array([O.lib.kq_oracle_f32_to_bf16(float(v)) for v in x[:60000]], dtype=np.uint16)
    assert np.array_equal(gotb, _bf16_rne_int(x[:60000]))
    assert np.array_equal(O.f32_to_bits(x, "bfloat16"), _bf16_rne_int(x))


@pytest.mark.parametrize("codec", O.ALL_CODECS)
def test_known_answer_blocks(codec):
    wire, want = wire_pack.make(codec, 64, seed=100 + O.codec_id(codec))
    assert wire.shape[1] == O.geometry(codec)[1] and want.shape[1] == O.geometry(codec)[0]
    got = O.dequantize(wire, codec, "float32")
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), codec


def test_q4k_unit_block():
    # d = 1, dmin = 0, every scale 1 -> output equals the nibbles in sub-block order
    b = np.zeros(144, np.uint8)
    b[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    b[4:8] = 1
    b[12:16] = 1  # scales 4..7 low nibbles
    q = np.arange(256) % 16
    for g in range(4):
        b[16 + 32 * g:48 + 32 * g] = q[64 * g:64 * g + 32] | (q[64 * g + 32:64 * g + 64] << 4)
    assert np.array_equal(O.dequantize(b[None], "q4_k")[0], q.astype(np.float32))


def test_mxfp4_scale127_is_e2m1_table():
    b = np.zeros(17, np.uint8)
    b[0] = 128  # 2^(128-127)/2 = 1 -> doubled-table values
    b[1:17] = np.arange(16) | (np.arange(16)[::-1] << 4)
    out = O.dequantize(b[None], "mxfp4")[0]
    e2m1x2 = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.float32)
    assert np.array_equal(out[:16], e2m1x2) and np.array_equal(out[16:], e2m1x2[::-1])
    b[0] = 127  # true OCP scale 1.0: table holds 2x E2M1 and the decoder folds the 0.5
    assert np.array_equal(O.dequantize(b[None], "mxfp4")[0][:16], e2m1x2 * 0.5)


@pytest.mark.parametrize("codec", KCODECS)
def test_reference_fixture_roundtrip_dense(codec):
    z = np.load(os.path.join(GOLD, f"{codec}.npz"))
    wire = z["wire"]
    w = (np.random.default_rng(1234).standard_normal((256, 512)) * 0.1).astype(np.float32)
    deq = O.dequantize(wire, codec)
    rel = np.linalg.norm(deq - w) / np.linalg.norm(w)
    assert RT_FLOOR[codec] < rel < RT_BOUND[codec], (codec, rel)


def test_reference_fixture_roundtrip_moe():
    rng = np.random.default_rng(4321)
    for codec in KCODECS:  # the generator draws experts codec by codec from one stream
        wire = np.load(os.path.join(GOLD, f"{codec}_moe.npz"))["wire"]
        for e in range(4):
            w = (rng.standard_normal((128, 512)) * 0.1).astype(np.float32)
            deq = O.dequantize(wire[e], codec)
            rel = np.linalg.norm(deq - w) / np.linalg.norm(w)
            assert RT_FLOOR[codec] < rel < RT_BOUND[codec], (codec, e, rel)


def test_reference_fixture_manifest():
    for line in open(os.path.join(GOLD, "REFERENCE_SHA256SUMS")):
        digest, path = line.split()
        data = open(os.path.join(GOLD, os.path.basename(path)), "rb").read()
        assert hashlib.sha256(data).hexdigest() == digest


@pytest.mark.parametrize("codec", O.ALL_CODECS)
def test_invariants(codec):
    wire = O.synth_wire(codec, 48, seed=7)
    f = O.dequantize(wire, codec)
    assert np.all(np.isfinite(f))
    # half outputs are a single RNE rounding of the f32 value
    assert np.array_equal(O.dequantize(wire, codec, "float16"), O.f32_to_bits(f, "float16"))
    assert np.array_equal(O.dequantize(wire, codec, "bfloat16"), O.f32_to_bits(f, "bfloat16"))
    # block independence + prefix property
    perm = np.random.default_rng(1).permutation(48)
    assert np.array_equal(O.dequantize(wire[perm], codec), f[perm])
    assert np.array_equal(O.dequantize(wire[:5], codec), f[:5])
    # N-d shapes: leading dims pass through
    assert np.array_equal(O.dequantize(wire.reshape(4, 12 * wire.shape[1]), codec).reshape(48, -1), f)
