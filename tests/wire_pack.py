"""Independent *packers* for every wire codec, written in the encode direction from the
GGUF block layouts (field -> byte position), plus the closed-form value each logical
weight must decode to.  Used to build known-answer blocks: random logical fields are
packed here, decoded by the code under test, and compared with `expected`.

A decoder that swaps nibble order, sub-block order, scale packing, sign bits or a
bias constant fails these; nothing here shares code with the decoders.
All float maths is numpy float32 (separately rounded multiplies/adds), so equality is
exact.
"""
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_BLOB = np.fromfile(os.path.join(ROOT, "mlx-kquant_amd", "data", "kq_iq_grids.bin"), dtype=np.uint8)
GRIDS = {
    "iq2_xxs": _BLOB[0:2048].reshape(256, 8),
    "iq2_xs": _BLOB[2048:6144].reshape(512, 8),
    "iq2_s": _BLOB[6144:14336].reshape(1024, 8),
    "iq1": _BLOB[14336:30720].view(np.int8).reshape(2048, 8),
    "iq3_xxs": _BLOB[30720:31744].reshape(256, 4),
    "iq3_s": _BLOB[31744:33792].reshape(512, 4),
}
KV_IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)
E2M1_X2 = np.array([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], np.float32)

f32 = np.float32


def _h(rng, n, lo=0.004, hi=0.02):
    return rng.uniform(lo, hi, n).astype(np.float16)


def _hb(h):
    return h.view(np.uint8).reshape(-1, 2)


def _sign_pattern7(s7):
    """7-bit sign index -> 8 sign bits (bit 7 = parity so the number of minus signs is even)."""
    s7 = s7.astype(np.uint32)
    par = np.zeros_like(s7)
    for b in range(7):
        par ^= (s7 >> b) & 1
    return s7 | (par << 7)


def _bits8(a):
    """[..] uint -> [.., 8] of 0/1, bit j at position j."""
    return ((a[..., None].astype(np.uint32) >> np.arange(8)) & 1).astype(np.int32)


def make(codec, nb, seed):
    """Return (wire uint8 [nb, bytes_per_block], expected float32 [nb, weights_per_block])."""
    rng = np.random.default_rng(seed)
    R = lambda hi, shape: rng.integers(0, hi, size=shape, dtype=np.int64)  # noqa: E731

    if codec in ("q4_k", "q5_k"):
        bits = 4 if codec == "q4_k" else 5
        d, dm = _h(rng, nb), _h(rng, nb)
        s, m = R(64, (nb, 8)), R(64, (nb, 8))
        q = R(1 << bits, (nb, 8, 32))
        sb = np.zeros((nb, 12), np.uint8)
        for j in range(4):
            sb[:, j] = (s[:, j] & 63) | ((s[:, j + 4] >> 4) << 6)
            sb[:, j + 4] = (m[:, j] & 63) | ((m[:, j + 4] >> 4) << 6)
            sb[:, j + 8] = (s[:, j + 4] & 15) | ((m[:, j + 4] & 15) << 4)
        qs = np.zeros((nb, 4, 32), np.uint8)
        for g in range(4):
            qs[:, g] = (q[:, 2 * g] & 15) | ((q[:, 2 * g + 1] & 15) << 4)
        parts = [_hb(d), _hb(dm), sb]
        if bits == 5:
            qh = np.zeros((nb, 32), np.uint8)
            for j in range(8):
                qh |= (((q[:, j] >> 4) & 1) << j).astype(np.uint8)
            parts.append(qh)
        parts.append(qs.reshape(nb, 128))
        sc = d.astype(f32)[:, None] * s.astype(f32)
        mn = dm.astype(f32)[:, None] * m.astype(f32)
        exp = sc[:, :, None] * q.astype(f32) - mn[:, :, None]
        return np.concatenate(parts, 1), exp.reshape(nb, 256).astype(f32)

    if codec == "q6_k":
        d = _h(rng, nb)
        sc = R(256, (nb, 16)).astype(np.int64) - 128
        q = R(64, (nb, 256))  # stored value; decoded as q - 32
        ql = np.zeros((nb, 128), np.uint8)
        qh = np.zeros((nb, 64), np.uint8)
        for h in range(2):
            for l in range(32):
                a = q[:, 128 * h + l]
                b = q[:, 128 * h + l + 32]
                c = q[:, 128 * h + l + 64]
                e = q[:, 128 * h + l + 96]
                ql[:, 64 * h + l] = (a & 15) | ((c & 15) << 4)
                ql[:, 64 * h + l + 32] = (b & 15) | ((e & 15) << 4)
                qh[:, 32 * h + l] = (a >> 4) | ((b >> 4) << 2) | ((c >> 4) << 4) | ((e >> 4) << 6)
        wire = np.concatenate([ql, qh, sc.astype(np.int8).view(np.uint8), _hb(d)], 1)
        scw = np.repeat(sc, 16, axis=1).astype(f32)  # scale index = weight // 16
        exp = (d.astype(f32)[:, None] * scw) * (q.astype(f32) - f32(32))
        return wire, exp.astype(f32)

    if codec in ("q3_k", "q2_k"):
        d = _h(rng, nb)
        q = R(4, (nb, 256))
        qs = np.zeros((nb, 64), np.uint8)
        # weight index w = 128*half + 32*shift_idx + l  lives in qs[32*half + l] at bits 2*shift_idx
        for half in range(2):
            for si in range(4):
                for l in range(32):
                    qs[:, 32 * half + l] |= (q[:, 128 * half + 32 * si + l] << (2 * si)).astype(np.uint8)
        if codec == "q2_k":
            dm = _h(rng, nb)
            s, m = R(16, (nb, 16)), R(16, (nb, 16))
            scb = (s | (m << 4)).astype(np.uint8)
            wire = np.concatenate([scb, qs, _hb(d), _hb(dm)], 1)
            dl = d.astype(f32)[:, None] * s.astype(f32)
            ml = dm.astype(f32)[:, None] * m.astype(f32)
            exp = np.repeat(dl, 16, 1) * q.astype(f32) - np.repeat(ml, 16, 1)
            return wire, exp.astype(f32)
        hb = R(2, (nb, 256))  # high bit set -> no -4
        hm = np.zeros((nb, 32), np.uint8)
        for half in range(2):
            for si in range(4):
                for l in range(32):
                    hm[:, l] |= (hb[:, 128 * half + 32 * si + l] << (4 * half + si)).astype(np.uint8)
        s = R(64, (nb, 16))
        sb = np.zeros((nb, 12), np.uint8)
        for k in range(4):
            sb[:, k] = (s[:, k] & 15) | ((s[:, k + 8] & 15) << 4)
            sb[:, k + 4] = (s[:, k + 4] & 15) | ((s[:, k + 12] & 15) << 4)
            sb[:, k + 8] = (s[:, k] >> 4) | ((s[:, k + 4] >> 4) << 2) | ((s[:, k + 8] >> 4) << 4) | (
                (s[:, k + 12] >> 4) << 6)
        wire = np.concatenate([hm, qs, sb, _hb(d)], 1)
        dl = d.astype(f32)[:, None] * (s.astype(f32) - f32(32))
        exp = np.repeat(dl, 16, 1) * (q.astype(f32) - f32(4) * (1 - hb).astype(f32))
        return wire, exp.astype(f32)

    if codec in ("q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "iq4_nl", "mxfp4"):
        d = _h(rng, nb)
        if codec == "q8_0":
            q = R(256, (nb, 32)) - 128
            return (np.concatenate([_hb(d), q.astype(np.int8).view(np.uint8)], 1),
                    (d.astype(f32)[:, None] * q.astype(f32)).astype(f32))
        bits = 5 if codec in ("q5_0", "q5_1") else 4
        q = R(1 << bits, (nb, 32))
        qs = ((q[:, :16] & 15) | ((q[:, 16:] & 15) << 4)).astype(np.uint8)
        parts = [_hb(d)]
        mval = None
        if codec in ("q4_1", "q5_1"):
            mh = _h(rng, nb)
            parts.append(_hb(mh))
            mval = mh.astype(f32)[:, None]
        if bits == 5:
            qh = np.zeros(nb, np.uint32)
            for i in range(32):
                qh |= ((q[:, i] >> 4) & 1).astype(np.uint32) << i
            parts.append(qh.view(np.uint8).reshape(nb, 4))
        df = d.astype(f32)[:, None]
        if codec == "mxfp4":
            e = R(9, nb) + 121
            e[0] = 0
            if nb > 1:
                e[1] = 1
            if nb > 2:
                e[2] = 254
            parts = [e.astype(np.uint8)[:, None]]
            df = np.ldexp(np.float64(0.5), e - 127).astype(f32)[:, None]
            exp = df * E2M1_X2[q]
        elif codec == "iq4_nl":
            exp = df * KV_IQ4NL[q]
        elif codec == "q4_0":
            exp = df * (q.astype(f32) - f32(8))
        elif codec == "q5_0":
            exp = df * (q.astype(f32) - f32(16))
        else:
            exp = df * q.astype(f32) + mval
        parts.append(qs)
        return np.concatenate(parts, 1), exp.astype(f32)

    if codec == "nvfp4":
        sc = R(0x78, (nb, 4)) + 1  # 1..0x78, never 0x7f
        sc[0, 0] = 0
        sc[0, 1] = 0x7F
        q = R(16, (nb, 4, 16))
        qs = ((q[:, :, :8] & 15) | ((q[:, :, 8:] & 15) << 4)).astype(np.uint8)
        ex, man = (sc >> 3) & 15, sc & 7
        val = np.where(ex == 0, man * 2.0 ** -9, (1 + man / 8.0) * 2.0 ** (ex - 7.0)) * 0.5
        val = np.where((sc == 0) | (sc == 0x7F), 0.0, val).astype(f32)
        exp = val[:, :, None] * E2M1_X2[q]
        return np.concatenate([sc.astype(np.uint8), qs.reshape(nb, 32)], 1), exp.reshape(nb, 64).astype(f32)

    if codec == "iq4_xs":
        d = _h(rng, nb)
        ls = R(64, (nb, 8))
        q = R(16, (nb, 8, 32))
        sh = np.zeros(nb, np.uint16)
        sl = np.zeros((nb, 4), np.uint8)
        for ib in range(8):
            sh |= ((ls[:, ib] >> 4) << (2 * ib)).astype(np.uint16)
            sl[:, ib // 2] |= ((ls[:, ib] & 15) << (4 * (ib % 2))).astype(np.uint8)
        qs = ((q[:, :, :16] & 15) | ((q[:, :, 16:] & 15) << 4)).astype(np.uint8)
        wire = np.concatenate([_hb(d), sh.view(np.uint8).reshape(nb, 2), sl, qs.reshape(nb, 128)], 1)
        dl = d.astype(f32)[:, None] * (ls.astype(f32) - f32(32))
        return wire, (dl[:, :, None] * KV_IQ4NL[q]).reshape(nb, 256).astype(f32)

    d = _h(rng, nb, 0.004, 0.01)
    df = d.astype(f32)
    if codec in ("iq2_xxs", "iq3_xxs"):
        ng, gw = (32, 8) if codec == "iq2_xxs" else (64, 4)  # grid lookups per block, bytes each
        gi = R(256, (nb, ng))
        s7 = R(128, (nb, 8, 4))
        sc = R(16, (nb, 8))
        aux = (s7[:, :, 0] | (s7[:, :, 1] << 7) | (s7[:, :, 2] << 14) | (s7[:, :, 3] << 21) | (sc << 28)).astype(
            np.uint32)
        auxb = aux.view(np.uint8).reshape(nb, 8, 4)
        g = GRIDS[codec][gi].reshape(nb, 256).astype(f32)
        sign = 1 - 2 * _bits8(_sign_pattern7(s7)).reshape(nb, 256)
        if codec == "iq2_xxs":
            body = np.concatenate([gi.reshape(nb, 8, 4).astype(np.uint8), auxb], 2).reshape(nb, 64)
            db = df[:, None] * (f32(0.5) + sc.astype(f32)) * f32(0.25)
        else:
            body = np.concatenate([gi.astype(np.uint8), auxb.reshape(nb, 32)], 1)
            db = df[:, None] * (f32(0.5) + sc.astype(f32)) * f32(0.5)
        exp = np.repeat(db, 32, 1) * g * sign.astype(f32)
        return np.concatenate([_hb(d), body], 1), exp.astype(f32)

    if codec == "iq2_xs":
        gi, s7 = R(512, (nb, 32)), R(128, (nb, 32))
        sc = R(16, (nb, 16))  # one 4-bit scale per 16 weights
        qs = (gi | (s7 << 9)).astype(np.uint16)
        scb = (sc[:, 0::2] | (sc[:, 1::2] << 4)).astype(np.uint8)
        g = GRIDS["iq2_xs"][gi].reshape(nb, 256).astype(f32)
        sign = 1 - 2 * _bits8(_sign_pattern7(s7)).reshape(nb, 256)
        db = df[:, None] * (f32(0.5) + sc.astype(f32)) * f32(0.25)
        exp = np.repeat(db, 16, 1) * g * sign.astype(f32)
        return np.concatenate([_hb(d), qs.view(np.uint8).reshape(nb, 64), scb], 1), exp.astype(f32)

    if codec == "iq2_s":
        gi, s8 = R(1024, (nb, 32)), R(256, (nb, 32))
        sc = R(16, (nb, 16))
        qh = np.zeros((nb, 8), np.uint8)
        for ib in range(8):
            for l in range(4):
                qh[:, ib] |= ((gi[:, 4 * ib + l] >> 8) << (2 * l)).astype(np.uint8)
        scb = (sc[:, 0::2] | (sc[:, 1::2] << 4)).astype(np.uint8)
        g = GRIDS["iq2_s"][gi].reshape(nb, 256).astype(f32)
        sign = 1 - 2 * _bits8(s8).reshape(nb, 256)
        db = df[:, None] * (f32(0.5) + sc.astype(f32)) * f32(0.25)
        exp = np.repeat(db, 16, 1) * g * sign.astype(f32)
        wire = np.concatenate([_hb(d), (gi & 255).astype(np.uint8), s8.astype(np.uint8), qh, scb], 1)
        return wire, exp.astype(f32)

    if codec == "iq3_s":
        gi, s8 = R(512, (nb, 64)), R(256, (nb, 32))
        sc = R(16, (nb, 8))
        qh = np.zeros((nb, 8), np.uint8)
        for ib in range(8):
            for k in range(8):
                qh[:, ib] |= ((gi[:, 8 * ib + k] >> 8) << k).astype(np.uint8)
        scb = (sc[:, 0::2] | (sc[:, 1::2] << 4)).astype(np.uint8)
        g = GRIDS["iq3_s"][gi].reshape(nb, 256).astype(f32)
        sign = 1 - 2 * _bits8(s8).reshape(nb, 256)
        db = df[:, None] * (f32(1) + f32(2) * sc.astype(f32))
        exp = np.repeat(db, 32, 1) * g * sign.astype(f32)
        wire = np.concatenate([_hb(d), (gi & 255).astype(np.uint8), qh, s8.astype(np.uint8), scb], 1)
        return wire, exp.astype(f32)

    if codec == "iq1_s":
        gi = R(2048, (nb, 32))
        sc, neg = R(8, (nb, 8)), R(2, (nb, 8))
        qh = np.zeros((nb, 8), np.uint16)
        for l in range(4):
            qh |= ((gi[:, l::4] >> 8) << (3 * l)).astype(np.uint16)
        qh |= (sc << 12).astype(np.uint16) | (neg << 15).astype(np.uint16)
        g = GRIDS["iq1"][gi].reshape(nb, 256).astype(f32)
        dl = df[:, None] * (f32(2) * sc.astype(f32) + f32(1))
        delta = np.where(neg == 1, f32(-0.125), f32(0.125)).astype(f32)
        exp = np.repeat(dl, 32, 1) * (g + np.repeat(delta, 32, 1))
        wire = np.concatenate([_hb(d), (gi & 255).astype(np.uint8), qh.view(np.uint8).reshape(nb, 16)], 1)
        return wire, exp.astype(f32)

    if codec == "iq1_m":
        gi = R(2048, (nb, 32))
        neg = R(2, (nb, 32))  # one delta sign per 8 weights
        sc = R(8, (nb, 16))  # one 3-bit scale per 16 weights
        qh = np.zeros((nb, 16), np.uint8)
        for k in range(32):
            nib = ((gi[:, k] >> 8) | (neg[:, k] << 3)).astype(np.uint8)
            qh[:, k // 2] |= nib << (4 * (k % 2))
        dbits = d.view(np.uint16).astype(np.uint32)
        scw = np.zeros((nb, 4), np.uint16)
        for w in range(4):
            v = np.zeros(nb, np.uint32)
            for t in range(4):
                v |= (sc[:, 4 * w + t].astype(np.uint32)) << (3 * t)
            v |= ((dbits >> (4 * w)) & 15) << 12
            scw[:, w] = v.astype(np.uint16)
        g = GRIDS["iq1"][gi].reshape(nb, 256).astype(f32)
        dl = df[:, None] * (f32(2) * sc.astype(f32) + f32(1))
        delta = np.where(neg == 1, f32(-0.125), f32(0.125)).astype(f32)
        exp = np.repeat(dl, 16, 1) * (g + np.repeat(delta, 8, 1))
        wire = np.concatenate([(gi & 255).astype(np.uint8), qh, scw.view(np.uint8).reshape(nb, 8)], 1)
        return wire, exp.astype(f32)

    raise ValueError(codec)
