"""ctypes front end of the CPU oracle (oracle/kq_oracle.c). Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(ROOT, "oracle", "_build", "libkq_oracle.so")

DT = {"float32": 0, "float16": 1, "bfloat16": 2}
ACT = {"silu": 0, "gelu": 1, "silu_limit": 2, "swiglu_clamp": 3}


def _load():
    if not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    lib = C.CDLL(_SO)
    lib.kq_oracle_codec_id.argtypes = [C.c_char_p]
    lib.kq_oracle_f16_to_f32.restype = C.c_float
    lib.kq_oracle_f16_to_f32.argtypes = [C.c_uint16]
    lib.kq_oracle_f32_to_f16.restype = C.c_uint16
    lib.kq_oracle_f32_to_f16.argtypes = [C.c_float]
    lib.kq_oracle_f32_to_bf16.restype = C.c_uint16
    lib.kq_oracle_f32_to_bf16.argtypes = [C.c_float]
    lib.kq_oracle_glu_epilogue.restype = C.c_float
    lib.kq_oracle_glu_epilogue.argtypes = [C.c_int, C.c_float, C.c_float, C.c_float, C.c_float]
    vp, i, i64, u64, f = C.c_void_p, C.c_int, C.c_int64, C.c_uint64, C.c_float
    lib.kq_oracle_dequantize.argtypes = [i, vp, vp, u64, i]
    lib.kq_oracle_qmm.argtypes = [i, vp, vp, vp, i, i, i, i, i]
    lib.kq_oracle_gather_qmm.argtypes = [i, vp, vp, vp, vp, vp, i, i, i, i, i64, i64, i, i]
    lib.kq_oracle_moe_glu_gather.argtypes = [i, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, f, f, i]
    lib.kq_oracle_gather_qmv.argtypes = [i, vp, vp, vp, vp, vp, i, i, i, i, i]
    lib.kq_oracle_moe_glu_gather_shexp.argtypes = [i, i, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, i]
    lib.kq_oracle_gather_qmv_mix.argtypes = [i, i, vp, vp, vp, vp, vp, vp, i, i, i, i, i]
    lib.kq_oracle_router_topk.argtypes = [vp, i, i, i, i, i, i, vp, vp, i, f, vp, vp]
    return lib


lib = _load()


class Codec(C.Structure):
    _fields_ = [("name", C.c_char_p), ("wpb", C.c_int), ("bpb", C.c_int), ("bits", C.c_int),
                ("has_matmul", C.c_int), ("has_encode", C.c_int), ("has_nax", C.c_int),
                ("requires_imatrix", C.c_int)]


lib.kq_oracle_codec.restype = C.POINTER(Codec)
lib.kq_oracle_codec.argtypes = [C.c_int]


def codec_id(name):
    cid = lib.kq_oracle_codec_id(name.encode())
    if cid < 0:
        raise ValueError(name)
    return cid


def geometry(name):
    c = lib.kq_oracle_codec(codec_id(name)).contents
    return c.wpb, c.bpb


ALL_CODECS = [lib.kq_oracle_codec(i).contents.name.decode() for i in range(21)]


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _np_dtype(dtype):
    return np.float32 if dtype == "float32" else np.uint16


def f32_to_bits(a, dtype):
    """float32 array -> storage of `dtype` (f32 itself, or uint16 bit patterns, RNE)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    if dtype == "float32":
        return a
    if dtype == "float16":
        return a.astype(np.float16).view(np.uint16)
    u = a.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r


def bits_to_f32(a, dtype):
    if dtype == "float32":
        return np.asarray(a, dtype=np.float32)
    if dtype == "float16":
        return np.asarray(a, dtype=np.uint16).view(np.float16).astype(np.float32)
    return (np.asarray(a, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def dequantize(wire, codec, dtype="float32"):
    wire = np.ascontiguousarray(wire, dtype=np.uint8)
    wpb, bpb = geometry(codec)
    assert wire.shape[-1] % bpb == 0
    shape = wire.shape[:-1] + (wire.shape[-1] // bpb * wpb,)
    out = np.empty(shape, dtype=_np_dtype(dtype))
    rc = lib.kq_oracle_dequantize(codec_id(codec), _ptr(wire), _ptr(out), out.size, DT[dtype])
    assert rc == 0
    return out


def qmm(x, wire, codec, transpose=True, dtype="float32"):
    """x: storage array [M, K] of `dtype`; wire uint8 [rows, bpr]."""
    x = np.ascontiguousarray(x)
    wire = np.ascontiguousarray(wire, dtype=np.uint8)
    wpb, bpb = geometry(codec)
    M, K = x.shape
    wpr = wire.shape[1] // bpb * wpb
    N = wire.shape[0] if transpose else wpr
    out = np.empty((M, N), dtype=_np_dtype(dtype))
    rc = lib.kq_oracle_qmm(codec_id(codec), _ptr(out), _ptr(x), _ptr(wire), M, N, K, int(transpose), DT[dtype])
    assert rc == 0, rc
    return out


def gather_qmm(x, wire, codec, lhs, rhs, transpose=True, dtype="float32"):
    """x [Bx, M, K] storage, wire [E, rows, bpr], lhs/rhs flat uint32 [B] -> [B, M, N]."""
    x = np.ascontiguousarray(x)
    wire = np.ascontiguousarray(wire, dtype=np.uint8)
    lhs = np.ascontiguousarray(lhs, dtype=np.uint32)
    rhs = np.ascontiguousarray(rhs, dtype=np.uint32)
    wpb, bpb = geometry(codec)
    _, M, K = x.shape
    wpr = wire.shape[2] // bpb * wpb
    N = wire.shape[1] if transpose else wpr
    B = lhs.size
    out = np.empty((B, M, N), dtype=_np_dtype(dtype))
    rc = lib.kq_oracle_gather_qmm(codec_id(codec), _ptr(out), _ptr(x), _ptr(wire), _ptr(lhs), _ptr(rhs), B, M, N, K,
                                  M * K, wire.shape[1] * wire.shape[2], int(transpose), DT[dtype])
    assert rc == 0, rc
    return out


def moe_glu_gather(x, gate, up, codec, idx, act="silu", limit=0.0, gate_bias=None, up_bias=None, alpha=0.0,
                   dtype="bfloat16"):
    x = np.ascontiguousarray(x)
    gate = np.ascontiguousarray(gate, dtype=np.uint8)
    up = np.ascontiguousarray(up, dtype=np.uint8)
    idx = np.ascontiguousarray(idx, dtype=np.uint32)
    T, K = x.shape
    R = idx.shape[1]
    N = gate.shape[1]
    gb = None if gate_bias is None else np.ascontiguousarray(gate_bias, dtype=np.float32)
    ub = None if up_bias is None else np.ascontiguousarray(up_bias, dtype=np.float32)
    out = np.empty((T, R, N), dtype=np.uint16)
    rc = lib.kq_oracle_moe_glu_gather(codec_id(codec), _ptr(out), _ptr(x), _ptr(gate), _ptr(up), _ptr(idx), _ptr(gb),
                                      _ptr(ub), T, R, N, K, ACT[act], limit, alpha, DT[dtype])
    assert rc == 0, rc
    return out


def gather_qmv(x, wire, codec, idx, bias=None, dtype="bfloat16"):
    x = np.ascontiguousarray(x)
    wire = np.ascontiguousarray(wire, dtype=np.uint8)
    idx = np.ascontiguousarray(idx, dtype=np.uint32)
    T, R, K = x.shape
    N = wire.shape[1]
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    out = np.empty((T, R, N), dtype=np.uint16)
    rc = lib.kq_oracle_gather_qmv(codec_id(codec), _ptr(out), _ptr(x), _ptr(wire), _ptr(idx), _ptr(b), T, R, N, K,
                                  DT[dtype])
    assert rc == 0, rc
    return out


def moe_glu_gather_shexp(x, gate, up, sgate, sup, codec, shexp_codec, idx, act="silu", dtype="bfloat16"):
    x = np.ascontiguousarray(x)
    idx = np.ascontiguousarray(idx, dtype=np.uint32)
    T, K = x.shape
    R, N = idx.shape[1], gate.shape[1]
    out = np.empty((T, R + 1, N), dtype=np.uint16)
    arrs = [np.ascontiguousarray(a, dtype=np.uint8) for a in (gate, up, sgate, sup)]
    rc = lib.kq_oracle_moe_glu_gather_shexp(codec_id(codec), codec_id(shexp_codec), _ptr(out), _ptr(x), *map(_ptr, arrs),
                                            _ptr(idx), T, R, N, K, {"silu": 0, "gelu": 1}[act], DT[dtype])
    assert rc == 0, rc
    return out


def gather_qmv_mix(x, wire, shexp_wire, codec, shexp_codec, idx, scores, dtype="bfloat16"):
    x = np.ascontiguousarray(x)
    wire = np.ascontiguousarray(wire, dtype=np.uint8)
    sw = None if shexp_wire is None else np.ascontiguousarray(shexp_wire, dtype=np.uint8)
    idx = np.ascontiguousarray(idx, dtype=np.uint32)
    sc = np.ascontiguousarray(scores, dtype=np.float32)
    T, S, K = x.shape
    N = wire.shape[1]
    out = np.empty((T, N), dtype=np.uint16)
    rc = lib.kq_oracle_gather_qmv_mix(codec_id(codec), codec_id(shexp_codec or codec), _ptr(out), _ptr(x), _ptr(wire),
                                      _ptr(sw), _ptr(idx), _ptr(sc), T, S, N, K, DT[dtype])
    assert rc == 0, rc
    return out


def router_topk(logits, dtype, top_k, norm, shared, pes=None, bias=None, scoring=0, scale=1.0):
    """logits: numpy storage ([T, E + shared] f32, or uint16 bits for the half types)."""
    logits = np.ascontiguousarray(logits)
    T, E = logits.shape[0], logits.shape[1] - (1 if shared else 0)
    p = None if pes is None else np.ascontiguousarray(pes, dtype=np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    idx = np.empty((T, top_k), dtype=np.uint32)
    sc = np.empty((T, top_k + (1 if shared else 0)), dtype=np.float32)
    rc = lib.kq_oracle_router_topk(_ptr(logits), DT[dtype], T, E, top_k, int(norm), int(shared), _ptr(p), _ptr(b),
                                   scoring, scale, _ptr(idx), _ptr(sc))
    assert rc == 0, rc
    return idx, sc


def synth_wire(codec, n_blocks, seed):
    """Structurally valid random wire: random bytes with sane scale fields so that
    decode stays finite (the recipe of the reference's tests/test_codecs.py:74-95 and
    benchmarks/bench_native_fp_ab.py:58-70, extended to every codec)."""
    rng = np.random.default_rng(seed)
    wpb, bpb = geometry(codec)
    wire = rng.integers(0, 256, size=(n_blocks, bpb), dtype=np.uint8)
    d = rng.uniform(0.004, 0.01, n_blocks).astype(np.float16)
    d2 = rng.uniform(0.004, 0.01, n_blocks).astype(np.float16)

    def put16(off, v):
        wire[:, off:off + 2] = v.view(np.uint8).reshape(n_blocks, 2)

    if codec == "nvfp4":
        wire[:, 0:4] = rng.integers(0x08, 0x19, (n_blocks, 4), dtype=np.uint8)
    elif codec == "mxfp4":
        wire[:, 0] = rng.integers(121, 130, n_blocks, dtype=np.uint8)
    elif codec == "iq1_m":
        dbits = d.view(np.uint16)
        for k, byteidx in enumerate((49, 51, 53, 55)):
            nib = ((dbits >> (4 * k)) & 0xF).astype(np.uint8)
            wire[:, byteidx] = (wire[:, byteidx] & 0x0F) | (nib << 4)
    elif codec in ("q4_k", "q5_k"):
        put16(0, d)
        put16(2, d2)
    elif codec == "q6_k":
        put16(208, d)
    elif codec == "q3_k":
        put16(108, d)
    elif codec == "q2_k":
        put16(80, d)
        put16(82, d2)
    elif codec in ("q4_1", "q5_1"):
        put16(0, d)
        put16(2, d2)
    else:
        put16(0, d)
    return wire
