"""Minimal GGUF reader (and a writer for small files): tensor wire bytes straight from a memory map, plus the
key/value metadata -- the data the reference's C++ loader returns (src/kquant_gguf.h:32-65): quantized tensors
as uint8 in row-major axis order with the last dim byte-packed and a `<name>.scales` placeholder each, float /
integer tensors in their native dtype, the tensor -> codec list, the decoded metadata and the logical shapes in
GGUF (innermost-first) order.

File layout (GGUF v2 / v3, little-endian): magic "GGUF", u32 version, u64 tensor count, u64 kv count; kv pairs
(string key, u32 value type, value); tensor infos (string name, u32 n_dims, u64 dims innermost-first, u32 ggml
type, u64 offset into the data section); padding to `general.alignment` (default 32); tensor data.
"""
from __future__ import annotations

import mmap
import struct
from typing import Dict, List, NamedTuple, Tuple

import numpy as np
import torch

from .codec_geometry import CODEC_GEOMETRY

MAGIC = b"GGUF"
# ggml tensor type id -> codec name (quantized) / numpy dtype (plain)
GGML_QUANT = {2: "q4_0", 3: "q4_1", 6: "q5_0", 7: "q5_1", 8: "q8_0", 10: "q2_k", 11: "q3_k", 12: "q4_k", 13: "q5_k",
              14: "q6_k", 16: "iq2_xxs", 17: "iq2_xs", 18: "iq3_xxs", 19: "iq1_s", 20: "iq4_nl", 21: "iq3_s",
              22: "iq2_s", 23: "iq4_xs", 29: "iq1_m", 39: "mxfp4", 40: "nvfp4"}
GGML_PLAIN = {0: np.float32, 1: np.float16, 24: np.int8, 25: np.int16, 26: np.int32, 27: np.int64, 28: np.float64,
              30: "bfloat16"}
_CODEC_TO_GGML = {v: k for k, v in GGML_QUANT.items()}
_SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
T_STRING, T_ARRAY = 8, 9


class GgufFile(NamedTuple):
    arrays: Dict[str, torch.Tensor]
    codecs: List[Tuple[str, str]]               # quantized tensor name -> codec, file order
    metadata: Dict[str, object]                 # file order
    tensor_shapes: Dict[str, Tuple[int, ...]]   # logical dims, innermost first


class _Cursor:
    def __init__(self, buf):
        self.buf, self.pos = buf, 0

    def take(self, fmt):
        v = struct.unpack_from(fmt, self.buf, self.pos)[0]
        self.pos += struct.calcsize(fmt)
        return v

    def string(self):
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise ValueError("GGUF: string runs past the end of the file")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8", errors="replace")
        self.pos += n
        return s

    def value(self, vtype):
        if vtype in _SCALAR:
            v = self.take(_SCALAR[vtype])
            return bool(v) if vtype == 7 else (float(v) if vtype in (6, 12) else int(v))
        if vtype == T_STRING:
            return self.string()
        if vtype == T_ARRAY:
            etype, count = self.take("<I"), self.take("<Q")
            if etype == T_ARRAY:
                raise ValueError("GGUF: nested arrays are not allowed")
            return [self.value(etype) for _ in range(count)]
        raise ValueError(f"GGUF: unknown metadata value type {vtype}")


def load_gguf(path: str, device=None) -> GgufFile:
    """Parse `path`.  Tensor data is copied out of the memory map once (to `device` when given)."""
    with open(path, "rb") as f:
        mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
    try:
        cur = _Cursor(memoryview(mm))
        if bytes(cur.buf[:4]) != MAGIC:
            raise ValueError(f"{path}: not a GGUF file")
        cur.pos = 4
        version = cur.take("<I")
        if version not in (2, 3):
            raise ValueError(f"{path}: unsupported GGUF version {version}")
        n_tensors, n_kv = cur.take("<Q"), cur.take("<Q")
        metadata: Dict[str, object] = {}
        for _ in range(n_kv):
            key = cur.string()
            metadata[key] = cur.value(cur.take("<I"))
        infos = []
        for _ in range(n_tensors):
            name = cur.string()
            nd = cur.take("<I")
            dims = tuple(cur.take("<Q") for _ in range(nd))
            infos.append((name, dims, cur.take("<I"), cur.take("<Q")))
        align = int(metadata.get("general.alignment", 32))
        data0 = (cur.pos + align - 1) // align * align
        arrays, codecs, shapes = {}, [], {}
        for name, dims, gtype, off in infos:
            shapes[name] = dims
            count = int(np.prod(dims)) if dims else 1
            if gtype in GGML_QUANT:
                codec = GGML_QUANT[gtype]
                _, _, bpb, wpb = CODEC_GEOMETRY[codec]
                if not dims or dims[0] % wpb:
                    raise ValueError(f"{name}: row length {dims[:1]} is not a multiple of {wpb} ({codec})")
                nbytes = count // wpb * bpb
                shape = tuple(reversed(dims[1:])) + (dims[0] // wpb * bpb,)
                np_dtype = np.uint8
            elif gtype in GGML_PLAIN:
                np_dtype = np.uint16 if GGML_PLAIN[gtype] == "bfloat16" else GGML_PLAIN[gtype]
                nbytes = count * np.dtype(np_dtype).itemsize
                shape = tuple(reversed(dims))
            else:
                raise ValueError(f"{name}: unsupported ggml tensor type {gtype}")
            if data0 + off + nbytes > len(mm):
                raise ValueError(f"{name}: tensor data runs past the end of the file")
            a = np.frombuffer(mm, dtype=np_dtype, count=nbytes // np.dtype(np_dtype).itemsize, offset=data0 + off)
            t = torch.from_numpy(a.reshape(shape).copy())
            del a  # no view of the map may outlive this function
            if gtype in GGML_PLAIN and GGML_PLAIN[gtype] == "bfloat16":
                t = t.view(torch.bfloat16)
            arrays[name] = t if device is None else t.to(device)
            if gtype in GGML_QUANT:
                codecs.append((name, GGML_QUANT[gtype]))
                prefix = name[:-len(".weight")] if name.endswith(".weight") else name
                sc = torch.zeros(1, dtype=torch.uint8)
                arrays[prefix + ".scales"] = sc if device is None else sc.to(device)
        return GgufFile(arrays, codecs, metadata, shapes)
    finally:
        if "cur" in locals():
            cur.buf.release()
        try:
            mm.close()
        except BufferError:  # an exception left a view of the map alive: the map goes with it
            pass


def _put_string(out: bytearray, s: str):
    b = s.encode("utf-8")
    out += struct.pack("<Q", len(b)) + b


def _put_value(out: bytearray, v):
    if isinstance(v, bool):
        out += struct.pack("<I?", 7, v)
    elif isinstance(v, int):
        out += struct.pack("<Iq", 11, v) if v < 0 else struct.pack("<IQ", 10, v)
    elif isinstance(v, float):
        out += struct.pack("<If", 6, v)
    elif isinstance(v, str):
        out += struct.pack("<I", T_STRING)
        _put_string(out, v)
    elif isinstance(v, (list, tuple)):
        et = T_STRING if v and isinstance(v[0], str) else (6 if v and isinstance(v[0], float) else 11)
        out += struct.pack("<IIQ", T_ARRAY, et, len(v))
        for e in v:
            if et == T_STRING:
                _put_string(out, e)
            else:
                out += struct.pack("<f" if et == 6 else "<q", e)
    else:
        raise TypeError(f"unsupported metadata value {v!r}")


def save_gguf(path: str, tensors: Dict[str, torch.Tensor], codecs: Dict[str, str], metadata: Dict[str, object] = None,
              alignment: int = 32):
    """Write a GGUF v3 file.  `tensors[name]` is either wire bytes (uint8, row-major, last dim byte-packed; its
    codec in `codecs[name]`) or a float32 / float16 / bfloat16 / int tensor."""
    plain = {torch.float32: 0, torch.float16: 1, torch.int8: 24, torch.int16: 25, torch.int32: 26, torch.int64: 27,
             torch.float64: 28, torch.bfloat16: 30}
    meta = dict(metadata or {})
    meta.setdefault("general.alignment", alignment)
    head = bytearray(MAGIC + struct.pack("<IQQ", 3, len(tensors), len(meta)))
    for k, v in meta.items():
        _put_string(head, k)
        _put_value(head, v)
    blobs, off = [], 0
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if name in codecs:
            _, _, bpb, wpb = CODEC_GEOMETRY[codecs[name]]
            dims = (t.shape[-1] // bpb * wpb,) + tuple(reversed(t.shape[:-1]))
            gtype = _CODEC_TO_GGML[codecs[name]]
        else:
            dims, gtype = tuple(reversed(t.shape)), plain[t.dtype]
        raw = (t.view(torch.uint16) if t.dtype == torch.bfloat16 else t).numpy().tobytes()
        _put_string(head, name)
        head += struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", gtype, off)
        blobs.append((off, raw))
        off = (off + len(raw) + alignment - 1) // alignment * alignment
    data0 = (len(head) + alignment - 1) // alignment * alignment
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (data0 - len(head)))
        for o, raw in blobs:
            f.seek(data0 + o)
            f.write(raw)
        f.truncate(data0 + off if blobs else data0)
