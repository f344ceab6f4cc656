"""kq -- the reference's `kq.*` quantized-weight ops on PyTorch-ROCm tensors, backed by libkq
(hand-written HIP for gfx950 behind a C ABI, include/kq.h).

Mirrors the Python op boundary of the reference (bindings.cpp:94-141, 885-952, 1349-1461 and the
validation in src/kquant_ops.cpp / src/kquant_moe_glu.cpp): same names, argument order and
meaning, dtype rules and error types.  Wire tensors are uint8 GGUF block bytes, unchanged.

There is no CPU execution path here: tensors must live on a ROCm device, and a missing or
unloadable libkq raises at import / first call instead of falling back.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch

from . import codec_geometry
from .codec_geometry import CODEC_GEOMETRY, bytes_per_row, weights_per_row

# codec -> (weights_per_block, bytes_per_block)
_GEOM = {k: (v[3], v[2]) for k, v in CODEC_GEOMETRY.items()}

__all__ = [
    "codecs", "codec_has_matmul", "codec_has_moe_glu", "dequantize", "quantized_matmul", "quantized_matmul_qmv_bias",
    "gather_qmm", "expert_tile_map", "gather_qmm_seg",
    "moe_glu_gather_kq", "gather_qmv_kq", "moe_glu_gather_shexp_kq", "gather_qmv_mix_kq", "gather_qmv_mix_ns_kq",
    "moe_router_topk", "mxfp4_packed_to_wire", "mxfp4_wire_to_packed", "set_packed_cache", "invalidate_packed_cache", "moe_glu_gather", "gather_qmv_bias",
    "gather_qmv_mix_bias", "quantize", "codec_geometry", "CODEC_GEOMETRY", "bytes_per_row",
    "weights_per_row", "lib_path",
]

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libkq.so")
_lib = None

KQ_F32, KQ_F16, KQ_BF16 = 0, 1, 2
_ACTS = {"silu": 0, "gelu": 1, "silu_limit": 2, "swiglu_clamp": 3}
_DT = {torch.float32: KQ_F32, torch.float16: KQ_F16, torch.bfloat16: KQ_BF16}


class _CodecInfo(C.Structure):
    _fields_ = [("name", C.c_char * 16), ("weights_per_block", C.c_int), ("bytes_per_block", C.c_int),
                ("bits", C.c_int), ("has_matmul_kernel", C.c_int), ("has_encode", C.c_int),
                ("has_nax_kernel", C.c_int), ("requires_imatrix", C.c_int)]


def lib_path() -> str:
    return _LIB_PATH


def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"[kq] {_LIB_PATH} is missing: build it with `python mlx-kquant_amd/build.py` "
            "(there is no fallback implementation)")
    lib = C.CDLL(_LIB_PATH)
    vp, i, i64, u64, f, sz = C.c_void_p, C.c_int, C.c_int64, C.c_uint64, C.c_float, C.c_size_t
    lib.kq_last_error.restype = C.c_char_p
    lib.kq_version.restype = C.c_char_p
    lib.kq_codec_id.argtypes = [C.c_char_p]
    lib.kq_codec_get.argtypes = [i, C.POINTER(_CodecInfo)]
    lib.kq_codec_has_moe_glu.argtypes = [i]
    lib.kq_dequantize.argtypes = [vp, vp, u64, i, i, vp]
    lib.kq_qmm_workspace_size.restype = sz
    lib.kq_qmm_workspace_size.argtypes = [i, i, i, i, i, i]
    lib.kq_qmm.argtypes = [vp, vp, vp, i, i, i, i, i, i, vp, sz, vp]
    lib.kq_qmm_noalloc.argtypes = [vp, vp, vp, i, i, i, i, i, vp]
    lib.kq_qmv_bias.argtypes = [vp, vp, vp, vp, i, i, i, i, vp]
    lib.kq_moe_glu_gather_shexp_workspace_size.restype = sz
    lib.kq_moe_glu_gather_shexp_workspace_size.argtypes = [i, i, i, i, i, i, i, i]
    lib.kq_moe_glu_gather_shexp.argtypes = [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, i, i, vp, sz, vp]
    lib.kq_gather_qmv_mix_workspace_size.restype = sz
    lib.kq_gather_qmv_mix_workspace_size.argtypes = [i, i, i, i, i, i, i, i]
    lib.kq_gather_qmv_mix.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, i, vp, sz, vp]
    lib.kq_moe_router_topk.argtypes = [vp, i, i, i, i, i, i, vp, vp, i, C.c_float, vp, vp, vp]
    lib.kq_gather_qmm_workspace_size.restype = sz
    lib.kq_gather_qmm_workspace_size.argtypes = [i, i, i, i, i, i, i, i]
    lib.kq_gather_qmm.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, i, i64, i64, i, i, i, i, vp, sz, vp]
    lib.kq_moe_workspace_size.restype = sz
    lib.kq_moe_workspace_size.argtypes = [i, i, i, i, i, i, i, i]
    lib.kq_moe_glu_gather.argtypes = [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, f, f, i, i, vp, sz, vp]
    lib.kq_gather_qmv.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, i, i, i, vp, sz, vp]
    lib.kq_quantize.argtypes = [vp, vp, vp, i64, i64, i]
    lib.kq_quantize_dev_supported.argtypes = [i]
    lib.kq_quantize_dev.argtypes = [vp, i, vp, vp, i64, i64, i, vp]
    lib.kq_gather_qmv_mix_bias.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, vp, sz, vp]
    lib.kq_mxfp4_packed_to_wire.argtypes = [vp, vp, vp, i64, vp]
    lib.kq_mxfp4_wire_to_packed.argtypes = [vp, vp, vp, i64, vp]
    lib.kq_expert_tile_map_cap.restype = i64
    lib.kq_expert_tile_map_cap.argtypes = [i64, i]
    lib.kq_expert_tile_map.argtypes = [vp, i64, i, vp, i64, vp, vp]
    lib.kq_gather_qmm_seg_workspace_size.restype = sz
    lib.kq_gather_qmm_seg_workspace_size.argtypes = [i64, i, i, i, i, i]
    lib.kq_gather_qmm_seg.argtypes = [vp, vp, vp, vp, vp, i64, i64, i, i, i, i, i, vp, sz, vp]
    _lib = lib
    return lib


def _check(rc: int):
    if rc == 0:
        return
    msg = _load().kq_last_error().decode(errors="replace")
    if rc == -1:
        raise ValueError("[kq] " + msg)
    raise RuntimeError("[kq] " + msg)


def _codec(op: str, name: str):
    cid = _load().kq_codec_id(str(name).encode())
    if cid < 0:
        raise ValueError(f"[kq.{op}] Unknown kquant_type: '{name}'.")
    return cid, _GEOM[name]


def _stream_ptr(op: str, t: torch.Tensor, stream) -> int:
    if isinstance(stream, str) and stream == "cpu" or isinstance(stream, torch.device) and stream.type == "cpu":
        raise RuntimeError(f"[kq.{op}] this build has no CPU execution path; tensors must be on a ROCm device")
    if t.device.type != "cuda":
        raise RuntimeError(f"[kq.{op}] tensors must live on a ROCm device (got {t.device}); there is no CPU path")
    if isinstance(stream, torch.cuda.Stream):
        return stream.cuda_stream
    return torch.cuda.current_stream(t.device).cuda_stream


def _on_stream(fn):
    """`stream=` handling shared by every op: a torch.cuda.Stream other than the current one first waits for the
    current stream (the producers of the inputs), then the whole op -- its temporaries, its workspace, its output
    and its launches -- runs with that stream current, so the caching allocator ties every buffer to the stream
    the kernels run on.  Inputs are marked as used on that stream.  As with any torch side stream, whoever reads
    the result on another stream waits for this one first (`other.wait_stream(stream)`)."""
    import functools

    @functools.wraps(fn)
    def wrapper(*args, stream=None, **kw):
        if isinstance(stream, torch.cuda.Stream) and stream != torch.cuda.current_stream(stream.device):
            stream.wait_stream(torch.cuda.current_stream(stream.device))
            for a in list(args) + list(kw.values()):
                if isinstance(a, torch.Tensor) and a.is_cuda:
                    a.record_stream(stream)
            with torch.cuda.stream(stream):
                return fn(*args, stream=None, **kw)
        return fn(*args, stream=stream, **kw)

    return wrapper


def _same_device(op, ref, *ts):
    for t in ts:
        if t is not None and t.device != ref.device:
            raise ValueError(f"[kq.{op}] all tensors must be on the same device")


# ------------------------------------------------------------------ introspection
def codecs():
    """Canonical ordered codec names (bindings.cpp:40-60)."""
    lib = _load()
    out, info = [], _CodecInfo()
    for i in range(lib.kq_codec_count()):
        lib.kq_codec_get(i, C.byref(info))
        out.append(info.name.decode())
    return out


def codec_has_matmul(kquant_type: str) -> bool:
    lib = _load()
    cid = lib.kq_codec_id(str(kquant_type).encode())
    if cid < 0:
        return False
    info = _CodecInfo()
    lib.kq_codec_get(cid, C.byref(info))
    return bool(info.has_matmul_kernel)


def codec_has_moe_glu(kquant_type: str) -> bool:
    lib = _load()
    cid = lib.kq_codec_id(str(kquant_type).encode())
    return cid >= 0 and bool(lib.kq_codec_has_moe_glu(cid))


# ------------------------------------------------------------------ ops
def dequantize(w, scales, kquant_type, dtype=None, *, stream=None):
    """Decode wire bytes `w` (uint8 [..., bytes_per_row]) to `dtype` (default float16).
    Mirrors dequantize, reference src/kquant_ops.cpp:55-110."""
    op = "dequantize"
    if w.dtype != torch.uint8:
        raise ValueError("[kq.dequantize] w must be uint8 (raw GGUF wire bytes).")
    if w.ndim < 1:
        raise ValueError("[kq.dequantize] w must have at least 1 dimension.")
    cid, (wpb, bpb) = _codec(op, kquant_type)
    if w.shape[-1] % bpb != 0:
        raise ValueError(f"[kq.dequantize] Last dim ({w.shape[-1]}) must be a multiple of bytes_per_block "
                         f"({bpb}) for codec '{kquant_type}'.")
    out_type = dtype if dtype is not None else torch.float16
    if out_type not in _DT:
        raise ValueError("[kq.dequantize] Only real floating output dtypes are supported.")
    sp = _stream_ptr(op, w, stream)
    w_c = w.contiguous()
    out_shape = list(w.shape)
    out_shape[-1] = w.shape[-1] // bpb * wpb
    out = torch.empty(out_shape, dtype=out_type, device=w.device)
    with torch.cuda.device(w.device):
        _check(_load().kq_dequantize(w_c.data_ptr(), out.data_ptr(), out.numel(), cid, _DT[out_type], sp))
    return out


def _out_dtype(op, x):
    if not x.dtype.is_floating_point or x.dtype not in _DT:
        raise ValueError(f"[kq.{op}] Only real floating x dtypes are supported.")
    return torch.bfloat16 if x.dtype == torch.float32 else x.dtype


def _expand_geometry(op, x, w, kquant_type, transpose):
    cid, (wpb, bpb) = _codec(op, kquant_type)
    bpr = w.shape[-1]
    if bpr % bpb != 0:
        raise ValueError(f"[kq.{op}] KQuant weight last dim ({bpr} bytes) is not a whole number of "
                         f"{bpb}-byte {kquant_type} blocks.")
    wpr = bpr // bpb * wpb
    inner = wpr if transpose else w.shape[-2]
    outer = w.shape[-2] if transpose else wpr
    if inner != x.shape[-1]:
        raise ValueError(f"[kq.{op}] x last dim ({x.shape[-1]}) does not match the expanded quantized matrix inner "
                         f"dim ({inner}) for codec '{kquant_type}' with transpose={str(bool(transpose)).lower()}.")
    return cid, inner, outer


class _QuantizedMatmulFn(torch.autograd.Function):
    """Gradient with respect to the activations only (the wire bytes are a frozen base): d/dx (x @ W.T) =
    dy @ W, the same op with `transpose` flipped.  Mirrors KQuantMatmul::vjp, src/kquant_matmul.cpp:1166-1195."""

    @staticmethod
    def forward(ctx, x, w, kquant_type, transpose, stream):
        ctx.save_for_backward(w)
        ctx.meta = (kquant_type, bool(transpose), stream, x.dtype)
        return _quantized_matmul_impl(x, w, kquant_type, transpose, stream)

    @staticmethod
    def backward(ctx, dy):
        (w,) = ctx.saved_tensors
        kquant_type, transpose, stream, x_dtype = ctx.meta
        dx = _quantized_matmul_impl(dy, w, kquant_type, not transpose, stream)
        return dx.to(x_dtype), None, None, None, None


def quantized_matmul(x, w, scales, kquant_type, transpose=True, *, stream=None):
    """y = x @ W.T (transpose) or x @ W.  Output dtype = x dtype, float32 promoted to bfloat16 (the
    activations themselves are cast first).  Differentiable with respect to x (a frozen quantized layer passes
    gradients to what sits upstream of it, e.g. a LoRA adapter).  Mirrors quantized_matmul,
    src/kquant_ops.cpp:112-183."""
    if torch.is_grad_enabled() and x.requires_grad:
        return _QuantizedMatmulFn.apply(x, w, kquant_type, transpose, stream)
    return _quantized_matmul_impl(x, w, kquant_type, transpose, stream)


def _quantized_matmul_impl(x, w, kquant_type, transpose, stream):
    op = "quantized_matmul"
    if w.dtype != torch.uint8:
        raise ValueError("[kq.quantized_matmul] w must be uint8 (raw GGUF wire bytes).")
    if x.ndim > 2 and w.ndim > 2:
        raise ValueError("[kq.quantized_matmul] batched (>2D) weights are not supported; use gather_qmm for "
                         "mixture-of-experts.")
    if w.ndim != 2:
        raise ValueError("[kq.quantized_matmul] w must be 2-D [rows, bytes_per_row].")
    if x.ndim < 1:
        raise ValueError("[kq.quantized_matmul] x must have at least 1 dimension.")
    cid, K, N = _expand_geometry(op, x, w, kquant_type, transpose)
    out_type = _out_dtype(op, x)
    _same_device(op, x, w)
    sp = _stream_ptr(op, x, stream)
    x_c = x.to(out_type).contiguous()
    w_c = w.contiguous()
    M = x_c.numel() // K if K else 0
    out = torch.empty(list(x.shape[:-1]) + [N], dtype=out_type, device=x.device)
    lib = _load()
    with torch.cuda.device(x.device):
        ws_bytes = lib.kq_qmm_workspace_size(M, N, K, int(bool(transpose)), cid, _DT[out_type])
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
        _check(lib.kq_qmm(x_c.data_ptr(), w_c.data_ptr(), out.data_ptr(), M, N, K, int(bool(transpose)), cid,
                          _DT[out_type], ws.data_ptr() if ws is not None else None, ws_bytes, sp))
    return out


def quantized_matmul_qmv_bias(x, w, scales, bias, kquant_type, *, stream=None):
    """Decode-only y = x @ W.T + bias with the add fused into the matvec (f32 sum, one rounding): exactly one
    activation row, q8_0 only.  Mirrors quantized_matmul_qmv_bias, src/kquant_ops.cpp:185-270."""
    op = "quantized_matmul_qmv_bias"
    if kquant_type != "q8_0":
        raise ValueError(f"[kq.quantized_matmul_qmv_bias] only kquant_type 'q8_0' is wired so far, got '{kquant_type}'.")
    if w.dtype != torch.uint8:
        raise ValueError("[kq.quantized_matmul_qmv_bias] w must be uint8 (raw GGUF wire bytes).")
    if w.ndim != 2:
        raise ValueError("[kq.quantized_matmul_qmv_bias] w must be 2D (this op is not batched); use gather_qmm for "
                         "mixture-of-experts.")
    cid, K, N = _expand_geometry(op, x, w, kquant_type, True)
    if bias.ndim != 1 or bias.shape[0] != N:
        raise ValueError(f"[kq.quantized_matmul_qmv_bias] bias must be 1D with length {N} (the output dim), got shape "
                         f"{tuple(bias.shape)}.")
    if x.numel() // x.shape[-1] != 1:
        raise ValueError(f"[kq.quantized_matmul_qmv_bias] decode-only: x must carry exactly one row (got "
                         f"{x.numel() // x.shape[-1]}). Use quantized_matmul() + a separate add for prefill/verify shapes.")
    out_type = _out_dtype(op, x)
    _same_device(op, x, w, bias)
    sp = _stream_ptr(op, x, stream)
    x_c = x.to(out_type).contiguous()
    w_c = w.contiguous()
    b_c = bias.to(out_type).contiguous()
    out = torch.empty(list(x.shape[:-1]) + [N], dtype=out_type, device=x.device)
    with torch.cuda.device(x.device):
        _check(_load().kq_qmv_bias(x_c.data_ptr(), w_c.data_ptr(), b_c.data_ptr(), out.data_ptr(), N, K, cid,
                                   _DT[out_type], sp))
    return out


_ARANGE = {}


def _default_indices(t):
    """0 .. (batch entries - 1) in the batch shape of t; the tensors are constants and are kept per (device, count)."""
    shape = t.shape[:-2]
    total = 1
    for d in shape:
        total *= d
    key = (str(t.device), total)
    a = _ARANGE.get(key)
    if a is None:
        if len(_ARANGE) > 64:
            _ARANGE.clear()
        a = _ARANGE[key] = torch.arange(total, dtype=torch.int32, device=t.device)
    return a.reshape(shape)


class _GatherQmmFn(torch.autograd.Function):
    """Gradient with respect to x only: every entry's dy[i] @ W[rhs[i]] (the op with `transpose` flipped, one
    cotangent batch per entry) is scatter-added, in float32, into the batch of x that lhs[i] names.
    Mirrors KQuantGatherQMM::vjp, src/kquant_gather.cpp:748-812."""

    @staticmethod
    def forward(ctx, x, w, kquant_type, lhs_indices, rhs_indices, transpose, sorted_indices, stream):
        ctx.save_for_backward(w, lhs_indices, rhs_indices)
        ctx.meta = (kquant_type, bool(transpose), stream, x.dtype, tuple(x.shape))
        return _gather_qmm_impl(x, w, kquant_type, lhs_indices, rhs_indices, transpose, sorted_indices, stream)

    @staticmethod
    def backward(ctx, dy):
        w, lhs_indices, rhs_indices = ctx.saved_tensors
        kquant_type, transpose, stream, x_dtype, x_shape = ctx.meta
        M, K = x_shape[-2], x_shape[-1]
        nb = 1
        for d in x_shape[:-2]:
            nb *= d
        lhs = lhs_indices if lhs_indices is not None else \
            torch.arange(nb, dtype=torch.int64, device=dy.device).reshape(x_shape[:-2])
        rhs = rhs_indices if rhs_indices is not None else _default_indices(w)
        lhs, rhs = torch.broadcast_tensors(lhs, rhs)
        B = lhs.numel()
        g = _gather_qmm_impl(dy.reshape(B, M, dy.shape[-1]), w, kquant_type, None, rhs.reshape(B), not transpose, False,
                             stream)
        dx = torch.zeros((nb, M, K), dtype=torch.float32, device=dy.device)
        dx.index_add_(0, lhs.reshape(B).to(torch.int64), g.to(torch.float32))
        return dx.reshape(x_shape).to(x_dtype), None, None, None, None, None, None, None


def gather_qmm(x, w, scales, kquant_type, lhs_indices=None, rhs_indices=None, transpose=True,
               sorted_indices=False, *, stream=None):
    """out[i] = x[lhs[i]] @ W[rhs[i]].T; out shape = broadcast(lhs, rhs).shape + [M, N].  Differentiable with
    respect to x.  Mirrors gather_qmm, src/kquant_ops.cpp:293-420."""
    if lhs_indices is None and rhs_indices is None:
        return quantized_matmul(x, w, scales, kquant_type, transpose, stream=stream)
    if torch.is_grad_enabled() and x.requires_grad:
        return _GatherQmmFn.apply(x, w, kquant_type, lhs_indices, rhs_indices, transpose, sorted_indices, stream)
    return _gather_qmm_impl(x, w, kquant_type, lhs_indices, rhs_indices, transpose, sorted_indices, stream)


def _gather_qmm_impl(x, w, kquant_type, lhs_indices, rhs_indices, transpose, sorted_indices, stream):
    op = "gather_qmm"
    if w.dtype != torch.uint8:
        raise ValueError("[kq.gather_qmm] w must be uint8 (raw GGUF wire bytes).")
    _codec(op, kquant_type)
    if x.ndim < 2:
        raise ValueError(f"[kq.gather_qmm] x must have at least two dimensions but got shape {tuple(x.shape)}.")
    if w.ndim < 2:
        raise ValueError("[kq.gather_qmm] w must have at least two dimensions.")
    cid, K, N = _expand_geometry(op, x, w, kquant_type, transpose)
    out_type = _out_dtype(op, x)
    _same_device(op, x, w, lhs_indices, rhs_indices)
    sp = _stream_ptr(op, x, stream)
    lhs = lhs_indices if lhs_indices is not None else _default_indices(x)
    rhs = rhs_indices if rhs_indices is not None else _default_indices(w)
    lhs, rhs = torch.broadcast_tensors(lhs, rhs)
    idx_shape = list(lhs.shape)
    lhs = _prep_idx(lhs).reshape(-1)  # uint32 bit pattern
    rhs = _prep_idx(rhs).reshape(-1)
    M = x.shape[-2]
    x_c = x.to(out_type).reshape(-1, M, K).contiguous()
    # the expert (leading) dim of w may be strided; rows inside one expert must be packed
    if w.ndim == 3 and w.stride(-1) == 1 and w.stride(-2) == w.shape[-1]:
        w3 = w
    else:
        w3 = w.contiguous().reshape(-1, w.shape[-2], w.shape[-1])
    estride = w3.stride(0) if w3.shape[0] > 1 else w3.shape[1] * w3.shape[2]
    B = lhs.numel()
    E = w3.shape[0]
    out = torch.empty(idx_shape + [M, N], dtype=out_type, device=x.device)
    right_sorted = bool(sorted_indices) and lhs_indices is None
    lib = _load()
    with torch.cuda.device(x.device):
        ws_bytes = lib.kq_gather_qmm_workspace_size(B, M, E, N, K, int(bool(transpose)), cid, _DT[out_type])
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
        _check(lib.kq_gather_qmm(x_c.data_ptr(), w3.data_ptr(), lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(), B, M, E,
                                 N, K, M * K, estride, int(bool(transpose)), int(right_sorted), cid, _DT[out_type],
                                 ws.data_ptr() if ws is not None else None, ws_bytes, sp))
    return out


def expert_tile_map(indices, n_experts, *, stream=None):
    """Tile map of expert-sorted routing indices, built on the device: (map int32 [cap, 3] rows of
    (expert, first row, rows <= 64), counts int32 [1] = number of valid tiles); cap = rows // 64 +
    min(n_experts, rows) is a shape-only bound and slots past counts are uninitialised.
    Mirrors expert_tile_map, src/kquant_ops.cpp:422-447 (uint32 there; torch has int32)."""
    op = "expert_tile_map"
    if indices.ndim != 1 or indices.dtype not in (torch.int32, torch.int64, torch.uint32):
        raise ValueError(f"[kq.expert_tile_map] indices must be 1-D integer but got shape {tuple(indices.shape)} "
                         f"dtype {indices.dtype}.")
    rows = indices.shape[0]
    if rows < 1 or n_experts < 1:
        raise ValueError("[kq.expert_tile_map] indices must be non-empty and n_experts positive.")
    if not indices.is_cuda:
        raise RuntimeError("[kq.expert_tile_map] the indices must live on the GPU (there is no CPU implementation).")
    sp = _stream_ptr(op, indices, stream)
    idx = _prep_idx(indices)
    lib = _load()
    cap = lib.kq_expert_tile_map_cap(rows, n_experts)
    tiles = torch.empty((cap, 3), dtype=torch.int32, device=indices.device)
    counts = torch.empty((1,), dtype=torch.int32, device=indices.device)
    with torch.cuda.device(indices.device):
        _check(lib.kq_expert_tile_map(idx.data_ptr(), rows, n_experts, tiles.data_ptr(), cap, counts.data_ptr(), sp))
    return tiles, counts


def gather_qmm_seg(x, w, scales, kquant_type, map, counts, *, stream=None):
    """Sorted-segment GEMM for MoE prefill: x [rows, K] sorted by expert, w [E, N, bytes_per_row]; for every valid
    tile (expert e, first row r, n <= 64 rows) of `map` ([n_tiles, 3]; counts [1] = valid tiles) the rows
    out[r : r + n] = x[r : r + n] @ W_e.T.  Rows no tile covers are unspecified.
    Mirrors gather_qmm_seg, src/kquant_ops.cpp:466-548."""
    op = "gather_qmm_seg"
    if w.dtype != torch.uint8:
        raise ValueError("[kq.gather_qmm_seg] w must be uint8 (raw GGUF wire bytes).")
    cid, (wpb, bpb) = _codec(op, kquant_type)
    if x.ndim != 2:
        raise ValueError(f"[kq.gather_qmm_seg] x must be [rows, K] but got shape {tuple(x.shape)}.")
    if w.ndim != 3:
        raise ValueError(f"[kq.gather_qmm_seg] w must be (n_experts, N, bytes_per_row) but got shape {tuple(w.shape)}.")
    ints = (torch.int32, torch.uint32)
    if map.ndim != 2 or map.shape[1] != 3 or map.dtype not in ints or map.shape[0] < 1:
        raise ValueError("[kq.gather_qmm_seg] map must be 32-bit integer [n_tiles >= 1, 3] (expert, row_start, num_rows) "
                         f"but got shape {tuple(map.shape)} dtype {map.dtype}.")
    if counts.ndim != 1 or counts.shape[0] != 1 or counts.dtype not in ints:
        raise ValueError(f"[kq.gather_qmm_seg] counts must be 32-bit integer [1] but got shape {tuple(counts.shape)} "
                         f"dtype {counts.dtype}.")
    if w.shape[-1] % bpb != 0:
        raise ValueError(f"[kq.gather_qmm_seg] KQuant weight last dim ({w.shape[-1]} bytes) is not a whole number of "
                         f"{bpb}-byte {kquant_type} blocks.")
    K = w.shape[-1] // bpb * wpb
    if K != x.shape[-1]:
        raise ValueError(f"[kq.gather_qmm_seg] x last dim ({x.shape[-1]}) does not match the expanded quantized row "
                         f"width ({K}) for codec '{kquant_type}'.")
    if not x.dtype.is_floating_point:
        raise ValueError("[kq.gather_qmm_seg] Only real floating x dtypes are supported.")
    if w.shape[1] % 8 != 0:
        raise ValueError("[kq.gather_qmm_seg] N must be a multiple of 8.")
    _same_device(op, x, w, map, counts)
    sp = _stream_ptr(op, x, stream)
    x_c = (x.to(torch.bfloat16) if x.dtype not in (torch.float16, torch.bfloat16) else x).contiguous()
    w_c, map_c, cnt_c = w.contiguous(), map.contiguous(), counts.contiguous()
    rows, (E, N) = x.shape[0], w.shape[:2]
    out = torch.empty((rows, N), dtype=x_c.dtype, device=x.device)
    if rows == 0 or N == 0:
        return out
    lib = _load()
    with torch.cuda.device(x.device):
        ws_bytes = lib.kq_gather_qmm_seg_workspace_size(rows, E, N, K, cid, _DT[x_c.dtype])
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=x.device)
        _check(lib.kq_gather_qmm_seg(x_c.data_ptr(), w_c.data_ptr(), map_c.data_ptr(), cnt_c.data_ptr(), out.data_ptr(),
                                     rows, map_c.shape[0], E, N, K, cid, _DT[x_c.dtype], ws.data_ptr(), ws_bytes, sp))
    return out


def _check_kq_expert_stack(op, w, kquant_type, K):
    """check_kq_expert_stack, src/kquant_moe_glu.cpp:861-896."""
    if kquant_type not in CODEC_GEOMETRY or not codec_has_moe_glu(kquant_type):
        raise ValueError(f"[kq.{op}] codec '{kquant_type}' has no fused MoE kernel.")
    wpb, bpb = _GEOM[kquant_type]
    if w.ndim != 3 or w.dtype != torch.uint8:
        raise ValueError(f"[kq.{op}] expert weights must be uint8 [E, N, bytes_per_row].")
    if K % wpb != 0 or w.shape[2] != K // wpb * bpb:
        raise ValueError(f"[kq.{op}] weight trailing dim does not match K for '{kquant_type}'.")
    if w.shape[1] % 8 != 0:
        raise ValueError(f"[kq.{op}] N must be a multiple of 8.")
    if not w.is_contiguous():
        raise ValueError(f"[kq.{op}] weights must be row-contiguous.")


def _prep_idx(idx):
    """Index tensor as the contiguous uint32 bit pattern the ABI reads; int32 / uint32 inputs cost no kernel."""
    if idx.dtype == torch.int32:
        return idx.contiguous()
    if idx.dtype == torch.uint32:
        return idx.contiguous().view(torch.int32)
    return idx.to(torch.int64).to(torch.int32).contiguous()


def moe_glu_gather_kq(x, gate_w, up_w, kquant_type, indices, act="silu", limit=0.0, gate_bias=None, up_bias=None,
                      alpha=0.0, *, stream=None):
    """out[t, r] = act(x[t] @ G_e.T, x[t] @ U_e.T), e = indices[t, r]; [T, R, N] in x's dtype.
    Mirrors moe_glu_gather_kq, src/kquant_moe_glu.cpp:1070-1157."""
    op = "moe_glu_gather_kq"
    if x.ndim != 2:
        raise ValueError("[kq.moe_glu_gather_kq] x must be 2-D [T, K].")
    if indices.ndim != 2 or indices.shape[0] != x.shape[0]:
        raise ValueError("[kq.moe_glu_gather_kq] indices must be [T, R].")
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("[kq.moe_glu_gather_kq] x must be float16 or bfloat16.")
    if act not in _ACTS:
        raise ValueError("[kq.moe_glu_gather_kq] act must be 'silu', 'gelu', 'silu_limit' or 'swiglu_clamp'.")
    if act == "silu_limit" and not (limit > 0.0):
        raise ValueError("[kq.moe_glu_gather_kq] act 'silu_limit' requires limit > 0.")
    biased = gate_bias is not None or up_bias is not None
    if act == "swiglu_clamp":
        if gate_bias is None or up_bias is None or not (limit > 0.0) or not (alpha > 0.0):
            raise ValueError("[kq.moe_glu_gather_kq] act 'swiglu_clamp' requires gate_bias, up_bias, limit > 0 and "
                             "alpha > 0.")
        if kquant_type not in ("mxfp4", "nvfp4"):
            raise ValueError("[kq.moe_glu_gather_kq] biased kernels are instantiated for mxfp4/nvfp4 only.")
    elif biased:
        raise ValueError("[kq.moe_glu_gather_kq] gate_bias/up_bias require act 'swiglu_clamp'.")
    K = x.shape[1]
    _check_kq_expert_stack(op, gate_w, kquant_type, K)
    _check_kq_expert_stack(op, up_w, kquant_type, K)
    if gate_w.shape[0] != up_w.shape[0] or gate_w.shape[1] != up_w.shape[1]:
        raise ValueError("[kq.moe_glu_gather_kq] gate/up expert shapes must match.")
    if biased:
        for b in (gate_bias, up_bias):
            if b.ndim != 2 or b.shape[0] != gate_w.shape[0] or b.shape[1] != gate_w.shape[1]:
                raise ValueError("[kq.moe_glu_gather_kq] biases must be [E, N] matching the expert stacks.")
    _same_device(op, x, gate_w, up_w, indices, gate_bias, up_bias)
    sp = _stream_ptr(op, x, stream)
    cid, _ = _codec(op, kquant_type)
    x_c = x.contiguous()
    idx = _prep_idx(indices)
    gb = gate_bias.to(torch.float32).contiguous() if biased else None
    ub = up_bias.to(torch.float32).contiguous() if biased else None
    T, R = idx.shape
    E, N = gate_w.shape[0], gate_w.shape[1]
    out = torch.empty((T, R, N), dtype=x.dtype, device=x.device)
    lib = _load()
    with torch.cuda.device(x.device):
        ws_bytes = lib.kq_moe_workspace_size(T, R, E, N, K, 1, cid, _DT[x.dtype])
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
        _check(lib.kq_moe_glu_gather(x_c.data_ptr(), gate_w.data_ptr(), up_w.data_ptr(), idx.data_ptr(),
                                     gb.data_ptr() if biased else None, ub.data_ptr() if biased else None,
                                     out.data_ptr(), T, R, E, N, K, _ACTS[act], float(limit), float(alpha), cid,
                                     _DT[x.dtype], ws.data_ptr() if ws is not None else None, ws_bytes, sp))
    return out


def gather_qmv_kq(x, w, kquant_type, indices, bias=None, *, stream=None):
    """out[t, r] = x[t, r] @ W_e.T (+ bias_e), e = indices[t, r]; x [T, R, K] -> [T, R, N].
    Mirrors gather_qmv_kq, src/kquant_moe_glu.cpp:1159-1210."""
    op = "gather_qmv_kq"
    if x.ndim != 3:
        raise ValueError("[kq.gather_qmv_kq] x must be 3-D [T, R, K].")
    if indices.ndim != 2 or indices.shape[0] != x.shape[0] or indices.shape[1] != x.shape[1]:
        raise ValueError("[kq.gather_qmv_kq] indices must be [T, R] matching x.")
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("[kq.gather_qmv_kq] x must be float16 or bfloat16.")
    K = x.shape[2]
    _check_kq_expert_stack(op, w, kquant_type, K)
    if bias is not None:
        if kquant_type not in ("mxfp4", "nvfp4"):
            raise ValueError("[kq.gather_qmv_kq] biased kernels are instantiated for mxfp4/nvfp4 only.")
        if bias.ndim != 2 or bias.shape[0] != w.shape[0] or bias.shape[1] != w.shape[1]:
            raise ValueError("[kq.gather_qmv_kq] bias must be [E, N] matching the expert stack.")
    _same_device(op, x, w, indices, bias)
    sp = _stream_ptr(op, x, stream)
    cid, _ = _codec(op, kquant_type)
    x_c = x.contiguous()
    idx = _prep_idx(indices)
    b = bias.to(torch.float32).contiguous() if bias is not None else None
    T, R = idx.shape
    E, N = w.shape[0], w.shape[1]
    out = torch.empty((T, R, N), dtype=x.dtype, device=x.device)
    lib = _load()
    with torch.cuda.device(x.device):
        ws_bytes = lib.kq_moe_workspace_size(T, R, E, N, K, 0, cid, _DT[x.dtype])
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
        _check(lib.kq_gather_qmv(x_c.data_ptr(), w.data_ptr(), idx.data_ptr(),
                                 b.data_ptr() if b is not None else None, out.data_ptr(), T, R, E, N, K, cid,
                                 _DT[x.dtype], ws.data_ptr() if ws is not None else None, ws_bytes, sp))
    return out


def _shexp_codec(op, kquant_type, shexp_kquant_type):
    """shexp_combo_has_kernel, src/kquant_moe_glu.cpp:852-858."""
    st = shexp_kquant_type or kquant_type
    if not (kquant_type in CODEC_GEOMETRY and st in CODEC_GEOMETRY and codec_has_moe_glu(kquant_type)
            and codec_has_moe_glu(st) and (st == kquant_type or st in ("q6_k", "q8_0"))):
        raise ValueError(f"[kq.{op}] no fused kernel for expert codec '{kquant_type}' with shared-expert codec '{st}'.")
    return st


def _check_shexp_row(op, w, kquant_type, K, N):
    """check_kq_shexp_row, src/kquant_moe_glu.cpp:900-925."""
    wpb, bpb = _GEOM[kquant_type]
    if w.ndim != 2 or w.dtype != torch.uint8:
        raise ValueError(f"[kq.{op}] shared-expert weights must be uint8 [N, bytes_per_row].")
    if K % wpb != 0 or w.shape[0] != N or w.shape[1] != K // wpb * bpb:
        raise ValueError(f"[kq.{op}] shared-expert weights must match the expert stack row shape.")
    if not w.is_contiguous():
        raise ValueError(f"[kq.{op}] weights must be row-contiguous.")


def moe_glu_gather_shexp_kq(x, gate_w, up_w, shexp_gate_w, shexp_up_w, kquant_type, indices, act="silu",
                            shexp_kquant_type="", *, stream=None):
    """moe_glu_gather_kq with the block's shared expert folded in as one extra slot: [T, R + 1, N], the last
    slot is the shared expert.  Mirrors moe_glu_gather_shexp_kq, src/kquant_moe_glu.cpp:1212-1272."""
    op = "moe_glu_gather_shexp_kq"
    st = _shexp_codec(op, kquant_type, shexp_kquant_type)
    if x.ndim != 2:
        raise ValueError("[kq.moe_glu_gather_shexp_kq] x must be 2-D [T, K].")
    if indices.ndim != 2 or indices.shape[0] != x.shape[0]:
        raise ValueError("[kq.moe_glu_gather_shexp_kq] indices must be [T, R].")
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("[kq.moe_glu_gather_shexp_kq] x must be float16 or bfloat16.")
    if act not in ("silu", "gelu"):
        raise ValueError("[kq.moe_glu_gather_shexp_kq] act must be 'silu' or 'gelu'.")
    K = x.shape[1]
    _check_kq_expert_stack(op, gate_w, kquant_type, K)
    _check_kq_expert_stack(op, up_w, kquant_type, K)
    if gate_w.shape[0] != up_w.shape[0] or gate_w.shape[1] != up_w.shape[1]:
        raise ValueError("[kq.moe_glu_gather_shexp_kq] gate/up expert shapes must match.")
    E, N = gate_w.shape[0], gate_w.shape[1]
    _check_shexp_row(op, shexp_gate_w, st, K, N)
    _check_shexp_row(op, shexp_up_w, st, K, N)
    _same_device(op, x, gate_w, up_w, shexp_gate_w, shexp_up_w, indices)
    sp = _stream_ptr(op, x, stream)
    cid, _ = _codec(op, kquant_type)
    sid, _ = _codec(op, st)
    x_c = x.contiguous()
    idx = _prep_idx(indices)
    T, R = idx.shape
    out = torch.empty((T, R + 1, N), dtype=x.dtype, device=x.device)
    lib = _load()
    with torch.cuda.device(x.device):
        ws_bytes = lib.kq_moe_glu_gather_shexp_workspace_size(T, R, E, N, K, cid, sid, _DT[x.dtype])
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=x.device)
        _check(lib.kq_moe_glu_gather_shexp(x_c.data_ptr(), gate_w.data_ptr(), up_w.data_ptr(), shexp_gate_w.data_ptr(),
                                           shexp_up_w.data_ptr(), idx.data_ptr(), out.data_ptr(), T, R, E, N, K,
                                           _ACTS[act], cid, sid, _DT[x.dtype], ws.data_ptr(), ws_bytes, sp))
    return out


def _gather_qmv_mix(op, x, w, shexp_w, kquant_type, st, indices, scores, stream):
    if x.ndim != 3:
        raise ValueError(f"[kq.{op}] x must be 3-D [T, S, K].")
    T, S, K = x.shape
    want = S - 1 if shexp_w is not None else S
    if indices.ndim != 2 or indices.shape[0] != T or indices.shape[1] != want:
        raise ValueError(f"[kq.{op}] indices must be [T, {'S - 1' if shexp_w is not None else 'S'}].")
    if scores.ndim != 2 or scores.shape[0] != T or scores.shape[1] != S:
        raise ValueError(f"[kq.{op}] scores must be [T, S].")
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError(f"[kq.{op}] x must be float16 or bfloat16.")
    _check_kq_expert_stack(op, w, kquant_type, K)
    E, N = w.shape[0], w.shape[1]
    if shexp_w is not None:
        _check_shexp_row(op, shexp_w, st, K, N)
    _same_device(op, x, w, shexp_w, indices, scores)
    sp = _stream_ptr(op, x, stream)
    cid, _ = _codec(op, kquant_type)
    sid = _codec(op, st)[0] if shexp_w is not None else -1
    x_c = x.contiguous()
    idx = _prep_idx(indices)
    sc = scores.to(torch.float32).contiguous()
    out = torch.empty((T, N), dtype=x.dtype, device=x.device)
    lib = _load()
    with torch.cuda.device(x.device):
        ws_bytes = lib.kq_gather_qmv_mix_workspace_size(T, S, E, N, K, cid, sid, _DT[x.dtype])
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=x.device)
        _check(lib.kq_gather_qmv_mix(x_c.data_ptr(), w.data_ptr(), shexp_w.data_ptr() if shexp_w is not None else None,
                                     idx.data_ptr(), sc.data_ptr(), out.data_ptr(), T, S, E, N, K, cid, sid,
                                     _DT[x.dtype], ws.data_ptr(), ws_bytes, sp))
    return out


def gather_qmv_mix_kq(x, w, shexp_w, kquant_type, indices, scores, shexp_kquant_type="", *, stream=None):
    """Down projection with the routing mix folded in: x [T, S, K] (slot S-1 = shared expert), indices
    [T, S-1], scores [T, S]; f32 accumulation over the S slots, returns [T, N].
    Mirrors gather_qmv_mix_kq, src/kquant_moe_glu.cpp:1274-1323."""
    op = "gather_qmv_mix_kq"
    st = _shexp_codec(op, kquant_type, shexp_kquant_type)
    if shexp_w is None:
        raise ValueError("[kq.gather_qmv_mix_kq] shexp_w is required (use gather_qmv_mix_ns_kq without a shared expert).")
    return _gather_qmv_mix(op, x, w, shexp_w, kquant_type, st, indices, scores, stream)


def gather_qmv_mix_ns_kq(x, w, kquant_type, indices, scores, *, stream=None):
    """No-shared-expert routing mix: x [T, S, K], indices [T, S], scores [T, S]; returns [T, N].
    Mirrors gather_qmv_mix_ns_kq, src/kquant_moe_glu.cpp:1325-1364."""
    return _gather_qmv_mix("gather_qmv_mix_ns_kq", x, w, None, kquant_type, kquant_type, indices, scores, stream)


# ------------------------------------------------------------------ MLX packed mxfp4 layout
_PACKED_INTS = (torch.int32, torch.uint32)


def _check_packed_stack(op, w, sc, b, K):
    """check_expert_stack, src/kquant_moe_glu.cpp:802-841 (uint32 there; torch callers may hold int32)."""
    if w.ndim != 3 or w.dtype not in _PACKED_INTS:
        raise ValueError(f"[kq.{op}] expert weights must be uint32 [E, N, K/8].")
    if sc.ndim != 3 or sc.dtype != torch.uint8:
        raise ValueError(f"[kq.{op}] expert scales must be uint8 [E, N, K/32].")
    if w.shape[2] * 8 != K or sc.shape[2] * 32 != K:
        raise ValueError(f"[kq.{op}] weight/scale trailing dims do not match K.")
    if w.shape[0] != sc.shape[0] or w.shape[1] != sc.shape[1]:
        raise ValueError(f"[kq.{op}] weight/scale expert dims do not match.")
    if b is not None and (b.ndim != 2 or b.shape[0] != w.shape[0] or b.shape[1] != w.shape[1]):
        raise ValueError(f"[kq.{op}] bias must be [E, N].")
    if w.shape[1] % 8 != 0:
        raise ValueError(f"[kq.{op}] N must be a multiple of 8.")
    if K % 32 != 0:
        raise ValueError(f"[kq.{op}] K must be a multiple of 32.")
    if not w.is_contiguous() or not sc.is_contiguous():
        raise ValueError(f"[kq.{op}] weights/scales must be row-contiguous.")


def mxfp4_packed_to_wire(w, scales, *, stream=None):
    """MLX packed mxfp4 (codes uint32 / int32 [..., K/8], e8m0 scales uint8 [..., K/32]) -> GGUF wire uint8
    [..., K/32 * 17] (the two-halves nibble order of src/kquant_cpu_decode.cpp:403-418).  A device kernel; convert a
    stack once at load time and call the wire-form ops on the result."""
    op = "mxfp4_packed_to_wire"
    if w.dtype not in _PACKED_INTS or scales.dtype != torch.uint8 or w.ndim < 1 or w.shape[:-1] != scales.shape[:-1] \
            or w.shape[-1] != 4 * scales.shape[-1]:
        raise ValueError("[kq.mxfp4_packed_to_wire] expects codes [..., K/8] (32-bit words) and uint8 scales [..., K/32].")
    _same_device(op, w, scales)
    sp = _stream_ptr(op, w, stream)
    w_c, s_c = w.contiguous(), scales.contiguous()
    wire = torch.empty(tuple(scales.shape[:-1]) + (scales.shape[-1] * 17,), dtype=torch.uint8, device=w.device)
    with torch.cuda.device(w.device):
        _check(_load().kq_mxfp4_packed_to_wire(w_c.data_ptr(), s_c.data_ptr(), wire.data_ptr(), s_c.numel(), sp))
    return wire


# Wire forms of packed stacks.  The reference's kernels read the packed layout directly on every call
# (src/kquant_moe_glu.cpp:149-275); here a stack is rewritten to wire form on the device before the wire-form
# kernels run, once per call by default.  set_packed_cache(n) lets the three packed-layout ops below keep the wire
# form of up to n stacks between calls (17/16 of a stack's bytes of device memory each).  A kept wire form is used
# again only while the same two tensor objects are passed and their torch version counters stand still; writes that
# bypass those counters (w.data.copy_(), set_(), a kernel writing through data_ptr()) are not seen, so a caller who
# reloads weights that way calls invalidate_packed_cache(w) afterwards.  That is why the cache is off by default.
_PACKED_CACHE = {}
_PACKED_CACHE_MAX = 0


def set_packed_cache(max_entries: int) -> None:
    """Number of packed mxfp4 stacks whose wire form is kept between calls (0, the default: convert on every call).
    A kept wire form follows in-place changes made through torch ops on the tensor itself; after a write torch's
    version counters do not see (w.data.copy_(), set_(), raw-pointer writes) call invalidate_packed_cache."""
    global _PACKED_CACHE_MAX
    _PACKED_CACHE_MAX = max(0, int(max_entries))
    _drop_packed(list(_PACKED_CACHE))


def invalidate_packed_cache(w=None) -> None:
    """Forget the kept wire form of the packed stack whose codes tensor is w (every stack when w is None)."""
    _drop_packed([k for k, v in _PACKED_CACHE.items() if w is None or v[0]() is w or v[1]() is w])


def _drop_packed(keys):
    # A dropped wire form may still be read by kernels in flight: every stream other than the allocating one that
    # used it was named to the caching allocator with record_stream, so the block is not handed out again before
    # those streams pass the point of release.
    for k in keys:
        _PACKED_CACHE.pop(k, None)


def _consumer_stream(t, stream):
    return stream if isinstance(stream, torch.cuda.Stream) else torch.cuda.current_stream(t.device)


def _wire_of_packed(w, scales, stream):
    import weakref
    if _PACKED_CACHE_MAX == 0:
        return mxfp4_packed_to_wire(w, scales, stream=stream)
    key = (w.data_ptr(), scales.data_ptr(), tuple(w.shape), str(w.device))
    cs = _consumer_stream(w, stream)
    hit = _PACKED_CACHE.get(key)
    if hit is not None:
        wref, sref, ver, wire, ev, made_on = hit
        if wref() is w and sref() is scales and ver == (w._version, scales._version):
            if cs != made_on:
                cs.wait_event(ev)          # order this stream after the conversion
                wire.record_stream(cs)     # and keep the block from reuse while this stream reads it
            return wire
        _drop_packed([key])
    wire = mxfp4_packed_to_wire(w, scales, stream=stream)
    ev = torch.cuda.Event()
    ev.record(cs)
    if cs != torch.cuda.current_stream(w.device):
        wire.record_stream(cs)             # allocated on the current stream, written and read on cs
    while len(_PACKED_CACHE) >= _PACKED_CACHE_MAX:
        _drop_packed([next(iter(_PACKED_CACHE))])
    _PACKED_CACHE[key] = (weakref.ref(w), weakref.ref(scales), (w._version, scales._version), wire, ev, cs)
    weakref.finalize(w, _PACKED_CACHE.pop, key, None)
    return wire


def mxfp4_wire_to_packed(wire, *, stream=None):
    """The inverse of mxfp4_packed_to_wire: (codes int32 [..., K/8], scales uint8 [..., K/32])."""
    op = "mxfp4_wire_to_packed"
    if wire.dtype != torch.uint8 or wire.ndim < 1 or wire.shape[-1] % 17 != 0:
        raise ValueError("[kq.mxfp4_wire_to_packed] expects uint8 wire [..., K/32 * 17].")
    sp = _stream_ptr(op, wire, stream)
    nb = wire.shape[-1] // 17
    w_c = wire.contiguous()
    packed = torch.empty(tuple(wire.shape[:-1]) + (nb * 4,), dtype=torch.int32, device=wire.device)
    scales = torch.empty(tuple(wire.shape[:-1]) + (nb,), dtype=torch.uint8, device=wire.device)
    with torch.cuda.device(wire.device):
        _check(_load().kq_mxfp4_wire_to_packed(w_c.data_ptr(), packed.data_ptr(), scales.data_ptr(), scales.numel(), sp))
    return packed, scales


def moe_glu_gather(x, gate_w, gate_scales, gate_bias, up_w, up_scales, up_bias, indices, alpha=1.702, limit=7.0, *,
                   stream=None):
    """Fused gate / up expert products with expert biases and the clamped SwiGLU epilogue on MLX packed mxfp4
    stacks: x [T, K], indices [T, R] -> [T, R, N].  The stacks are brought to wire form on the device (one pass
    over their bytes per call; convert once with mxfp4_packed_to_wire and call moe_glu_gather_kq to avoid it).
    Mirrors moe_glu_gather, src/kquant_moe_glu.cpp:936-986."""
    op = "moe_glu_gather"
    if x.ndim != 2:
        raise ValueError("[kq.moe_glu_gather] x must be 2-D [T, K].")
    if indices.ndim != 2 or indices.shape[0] != x.shape[0]:
        raise ValueError("[kq.moe_glu_gather] indices must be [T, R] matching x.")
    K = x.shape[1]
    _check_packed_stack(op, gate_w, gate_scales, gate_bias, K)
    _check_packed_stack(op, up_w, up_scales, up_bias, K)
    if gate_w.shape != up_w.shape:
        raise ValueError("[kq.moe_glu_gather] gate and up stacks must have the same shape.")
    return moe_glu_gather_kq(x, _wire_of_packed(gate_w, gate_scales, stream),
                             _wire_of_packed(up_w, up_scales, stream), "mxfp4", indices, act="swiglu_clamp",
                             limit=limit, gate_bias=gate_bias, up_bias=up_bias, alpha=alpha, stream=stream)


def gather_qmv_bias(x, w, scales, bias, indices, *, stream=None):
    """out[t, r] = x[t, r] @ W_e.T + bias_e on an MLX packed mxfp4 stack: x [T, R, K] -> [T, R, N].
    Mirrors gather_qmv_bias, src/kquant_moe_glu.cpp:988-1024."""
    op = "gather_qmv_bias"
    if x.ndim != 3:
        raise ValueError("[kq.gather_qmv_bias] x must be 3-D [T, R, K].")
    if indices.ndim != 2 or tuple(indices.shape) != tuple(x.shape[:2]):
        raise ValueError("[kq.gather_qmv_bias] indices must be [T, R] matching x.")
    _check_packed_stack(op, w, scales, bias, x.shape[2])
    return gather_qmv_kq(x, _wire_of_packed(w, scales, stream), "mxfp4", indices, bias=bias, stream=stream)


def gather_qmv_mix_bias(x, w, scales, bias, indices, scores, *, stream=None):
    """gather_qmv_bias with the routing mix folded in: out[t] = sum_s scores[t, s] * (x[t, s] @ W_e.T + bias_e),
    f32 accumulation, one rounding; x [T, S, K], indices / scores [T, S] -> [T, N].
    Mirrors gather_qmv_mix_bias, src/kquant_moe_glu.cpp:1026-1068."""
    op = "gather_qmv_mix_bias"
    if x.ndim != 3:
        raise ValueError("[kq.gather_qmv_mix_bias] x must be 3-D [T, S, K].")
    T, S, K = x.shape
    if indices.ndim != 2 or tuple(indices.shape) != (T, S):
        raise ValueError("[kq.gather_qmv_mix_bias] indices must be [T, S].")
    if scores.ndim != 2 or tuple(scores.shape) != (T, S):
        raise ValueError("[kq.gather_qmv_mix_bias] scores must be [T, S].")
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("[kq.gather_qmv_mix_bias] x must be float16 or bfloat16.")
    _check_packed_stack(op, w, scales, bias, K)
    _same_device(op, x, w, scales, bias, indices, scores)
    sp = _stream_ptr(op, x, stream)
    wire = _wire_of_packed(w, scales, stream)
    cid, _ = _codec(op, "mxfp4")
    E, N = w.shape[0], w.shape[1]
    x_c, idx = x.contiguous(), _prep_idx(indices)
    sc, b = scores.to(torch.float32).contiguous(), bias.to(torch.float32).contiguous()
    out = torch.empty((T, N), dtype=x.dtype, device=x.device)
    lib = _load()
    with torch.cuda.device(x.device):
        ws_bytes = lib.kq_gather_qmv_mix_workspace_size(T, S, E, N, K, cid, -1, _DT[x.dtype])
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=x.device)
        _check(lib.kq_gather_qmv_mix_bias(x_c.data_ptr(), wire.data_ptr(), b.data_ptr(), idx.data_ptr(), sc.data_ptr(),
                                          out.data_ptr(), T, S, E, N, K, cid, _DT[x.dtype], ws.data_ptr(), ws_bytes, sp))
    return out


def moe_router_topk(logits, top_k, norm_topk_prob, shared_gate=True, per_expert_scale=None, bias=None,
                    scoring="softmax", scale=1.0, *, stream=None):
    """Router scoring + top-k + mixing weights in one launch: returns (indices int32 [T, top_k] holding the
    uint32 expert ids, scores float32 [T, top_k + shared_gate]) -- the inputs of the fused MoE ops.
    Mirrors moe_router_topk, src/kquant_moe_glu.cpp:1366-1441."""
    op = "moe_router_topk"
    if scoring not in ("softmax", "sqrtsoftplus"):
        raise ValueError("[kq.moe_router_topk] scoring must be softmax or sqrtsoftplus.")
    if scoring == "sqrtsoftplus" and not norm_topk_prob:
        raise ValueError("[kq.moe_router_topk] sqrtsoftplus requires norm_topk_prob.")
    if logits.ndim != 2:
        raise ValueError("[kq.moe_router_topk] logits must be 2-D [T, E + shared_gate].")
    if logits.dtype not in _DT:
        raise ValueError("[kq.moe_router_topk] logits must be float32/float16/bfloat16.")
    shared = 1 if shared_gate else 0
    T, E = logits.shape[0], logits.shape[1] - shared
    if top_k < 1 or top_k > 16 or top_k > E:
        raise ValueError("[kq.moe_router_topk] top_k must be in [1, min(E, 16)].")
    if E > 1024:
        raise ValueError("[kq.moe_router_topk] requires E <= 1024.")
    for name, v in (("per_expert_scale", per_expert_scale), ("bias", bias)):
        if v is not None and (v.ndim != 1 or v.shape[0] != E):
            raise ValueError(f"[kq.moe_router_topk] {name} must be 1-D [E].")
    _same_device(op, logits, per_expert_scale, bias)
    sp = _stream_ptr(op, logits, stream)
    l_c = logits.contiguous()
    pes = per_expert_scale.to(torch.float32).contiguous() if per_expert_scale is not None else None
    bs = bias.to(torch.float32).contiguous() if bias is not None else None
    indices = torch.empty((T, top_k), dtype=torch.int32, device=logits.device)
    scores = torch.empty((T, top_k + shared), dtype=torch.float32, device=logits.device)
    with torch.cuda.device(logits.device):
        _check(_load().kq_moe_router_topk(l_c.data_ptr(), _DT[logits.dtype], T, E, int(top_k), int(bool(norm_topk_prob)),
                                          shared, pes.data_ptr() if pes is not None else None,
                                          bs.data_ptr() if bs is not None else None,
                                          1 if scoring == "sqrtsoftplus" else 0, float(scale), indices.data_ptr(),
                                          scores.data_ptr(), sp))
    return indices, scores


def quantize(w, kquant_type, imatrix=None, *, stream=None):
    """Encode float weights [..., K] to wire bytes; returns (wq uint8 [..., bytes_per_row], scales uint8 [1]) on w's
    device.  A tensor on the GPU is encoded there for the legacy and K-quant codecs (one thread per block running
    the host encoder's code: same bytes); the IQ codecs, CPU tensors and stream="cpu" take the host encoder, as the
    reference keeps its IQ encoders on the CPU.  Mirrors quantize, src/kquant_ops.cpp:550-631."""
    op = "quantize"
    cid, (wpb, bpb) = _codec(op, kquant_type)
    if not w.dtype.is_floating_point:
        raise ValueError("[kq.quantize] w must be a real floating tensor.")
    if w.ndim < 1:
        raise ValueError("[kq.quantize] w must have at least 1 dimension.")
    K = w.shape[-1]
    if K % wpb != 0:
        raise ValueError(f"[kq.quantize] Last dim ({K}) must be a multiple of weights_per_block ({wpb}) for codec "
                         f"'{kquant_type}'.")
    info = _CodecInfo()
    lib = _load()
    lib.kq_codec_get(cid, C.byref(info))
    if not info.has_encode:
        raise ValueError(f"[kq.quantize] codec '{kquant_type}' has no encoder.")
    if imatrix is not None:
        if imatrix.ndim != 1 or imatrix.shape[0] != K:
            raise ValueError(f"[kq.quantize] imatrix must be 1-D with length {K}.")
    elif info.requires_imatrix:
        raise ValueError(f"[kq.quantize] codec '{kquant_type}' requires an importance matrix (imatrix).")
    rows = w.numel() // K if K else 0
    on_host = isinstance(stream, str) and stream == "cpu" or isinstance(stream, torch.device) and stream.type == "cpu"
    if w.is_cuda and not on_host and lib.kq_quantize_dev_supported(cid):
        sp = _stream_ptr(op, w, stream)
        w_c = (w if w.dtype in _DT else w.to(torch.float32)).contiguous()
        im = None if imatrix is None else imatrix.detach().to(w.device, torch.float32).contiguous()
        wire = torch.empty(list(w.shape[:-1]) + [K // wpb * bpb], dtype=torch.uint8, device=w.device)
        with torch.cuda.device(w.device):
            _check(lib.kq_quantize_dev(w_c.data_ptr(), _DT[w_c.dtype], im.data_ptr() if im is not None else None,
                                       wire.data_ptr(), rows, K, cid, sp))
        return wire, torch.zeros(1, dtype=torch.uint8, device=w.device)
    im = None if imatrix is None else imatrix.detach().to("cpu", torch.float32).contiguous()
    w_h = w.detach().to("cpu", torch.float32).contiguous()
    wire = torch.empty(list(w.shape[:-1]) + [K // wpb * bpb], dtype=torch.uint8)
    _check(lib.kq_quantize(w_h.data_ptr(), im.data_ptr() if im is not None else None, wire.data_ptr(), rows, K, cid))
    return wire.to(w.device), torch.zeros(1, dtype=torch.uint8, device=w.device)


# every op that takes `stream=` gets the shared stream handling
for _name in ("dequantize", "quantized_matmul", "quantized_matmul_qmv_bias", "gather_qmm", "expert_tile_map",
              "gather_qmm_seg", "moe_glu_gather_kq", "gather_qmv_kq", "moe_glu_gather_shexp_kq", "gather_qmv_mix_kq",
              "gather_qmv_mix_ns_kq", "mxfp4_packed_to_wire", "mxfp4_wire_to_packed", "moe_glu_gather",
              "gather_qmv_bias", "gather_qmv_mix_bias", "moe_router_topk", "quantize"):
    globals()[_name] = _on_stream(globals()[_name])
del _name
