"""torch.nn modules that keep GGUF wire bytes as their weight and call the kq ops: the counterparts of
the reference's mlx_kquant/nn.py (KQuantEmbedding :50-101, KQuantLinear :104-160, KQuantSwitchLinear
:163-269, KQuantMultiLinear :272-368).  Same constructor arguments, attribute names (`mode`,
`kquant_type`, `group_size`, `bits`, `biases`, `weight`, `scales`, `bias`) and call conventions:
`transpose=True` everywhere, expert ids go in as `rhs_indices`, the layer bias is added after the op
(`bias[indices]` expanded on axis -2 for expert stacks), an embedding gathers wire rows and decodes only
those.

KQuantSwitchLinear keeps the reference's sorted prefill arm (:191-261): a prefill-shaped sorted call
(x [B, 1, K], ascending 1-D indices, at least KQ_SWITCH_GEMM_MIN_ROWS rows, 512 by default, 0 disables)
builds the tile map on the device (kq.expert_tile_map) and runs kq.gather_qmm_seg, with no host sync on the
routing indices.  Every other call goes to kq.gather_qmm, which itself groups its entries by expert on the
device whenever there are more than 16 output rows, so here the two arms differ in bookkeeping, not in the
GEMM kernels behind them.
"""
from __future__ import annotations

import os

import numpy as np
import torch

import kq

from .codec_geometry import CODEC_GEOMETRY, bytes_per_row

__all__ = ["KQuantEmbedding", "KQuantLinear", "KQuantSwitchLinear", "KQuantMultiLinear"]


# kq.gather_qmm_seg tile height
_SEG_TILE_ROWS = 64


def _host_tile_maps(counts, device=None):
    """Host-built equivalent of kq.expert_tile_map from per-expert row counts: (map int32 [n_tiles, 3] rows of
    (expert, first row, rows <= 64), counts int32 [1]); only the last tile of an expert's run is partial
    (reference :33-47)."""
    counts = np.asarray(counts, dtype=np.int64)
    tiles, row = [], 0
    for e in np.flatnonzero(counts):
        c = int(counts[e])
        tiles += [(int(e), row + off, min(_SEG_TILE_ROWS, c - off)) for off in range(0, c, _SEG_TILE_ROWS)]
        row += c
    m = torch.tensor(tiles or [(0, 0, 0)], dtype=torch.int32, device=device)
    return m, torch.tensor([len(tiles)], dtype=torch.int32, device=device)


class _KQuantBase(torch.nn.Module):
    def _init_codec(self, codec: str):
        if codec not in CODEC_GEOMETRY:
            raise ValueError("unknown codec %r; known codecs: %s" % (codec, ", ".join(sorted(CODEC_GEOMETRY))))
        gs, bits, _, _ = CODEC_GEOMETRY[codec]
        self.mode = "kquant"
        self.group_size = gs
        self.bits = bits
        self.kquant_type = codec
        self.biases = None

    def _wire_buffers(self, shape, device):
        # placeholders, overwritten by load_state_dict / load_wire with the GGUF wire bytes
        self.register_buffer("weight", torch.zeros(shape, dtype=torch.uint8, device=device))
        self.register_buffer("scales", torch.zeros((1,), dtype=torch.uint8, device=device))

    def load_wire(self, wire: torch.Tensor, bias: torch.Tensor | None = None):
        """Install wire bytes (uint8, the module's weight shape) and optionally the bias."""
        if wire.dtype != torch.uint8 or tuple(wire.shape) != tuple(self.weight.shape):
            raise ValueError("wire bytes must be uint8 of shape %s, got %s %s"
                             % (tuple(self.weight.shape), wire.dtype, tuple(wire.shape)))
        self.weight = wire.to(self.weight.device).contiguous()
        if bias is not None:
            if getattr(self, "bias", None) is None:
                raise ValueError("this layer was built without a bias")
            if tuple(bias.shape) != tuple(self.bias.shape):
                raise ValueError("bias must have shape %s" % (tuple(self.bias.shape),))
            self.bias = bias.to(self.bias.device)
        return self


class KQuantEmbedding(_KQuantBase):
    """Embedding table kept as wire bytes [num_embeddings, bytes_per_row]: a lookup gathers the wire
    rows of the requested tokens and decodes only those; `as_linear` is the tied lm_head projection."""

    def __init__(self, num_embeddings: int, dims: int, codec: str, out_dtype: torch.dtype = torch.bfloat16,
                 device=None):
        super().__init__()
        self._init_codec(codec)
        self.num_embeddings = num_embeddings
        self.dims = dims
        self.out_dtype = out_dtype
        self._wire_buffers((num_embeddings, bytes_per_row(codec, dims)), device)

    def forward(self, x):
        gathered = self.weight[x]  # [*, bytes_per_row]
        flat = gathered.reshape(-1, gathered.shape[-1])
        deq = kq.dequantize(flat, self.scales, self.kquant_type)  # float16, then the compute dtype (reference :93-95)
        return deq.reshape(*gathered.shape[:-1], self.dims).to(self.out_dtype)

    def as_linear(self, x):
        return kq.quantized_matmul(x, self.weight, self.scales, self.kquant_type, transpose=True)

    def extra_repr(self):
        return f"{self.num_embeddings}, {self.dims}, kquant_type={self.kquant_type}"


class KQuantLinear(_KQuantBase):
    """y = x @ W.T (+ bias) with W stored as wire bytes [out_dims, bytes_per_row]."""

    def __init__(self, in_dims: int, out_dims: int, bias: bool, codec: str, device=None):
        super().__init__()
        self._init_codec(codec)
        self._wire_buffers((out_dims, bytes_per_row(codec, in_dims)), device)
        if bias:
            self.register_buffer("bias", torch.zeros((out_dims,), device=device))
        else:
            self.bias = None

    def forward(self, x):
        # decode (one row) with a real bias on q8_0: the add is fused into the matvec (reference :122-140)
        if self.bias is not None and self.kquant_type == "q8_0" and x.numel() // x.shape[-1] == 1:
            return kq.quantized_matmul_qmv_bias(x, self.weight, self.scales, self.bias, self.kquant_type)
        y = kq.quantized_matmul(x, self.weight, self.scales, self.kquant_type, transpose=True)
        if self.bias is not None:
            y = y + self.bias
        return y

    def extra_repr(self):
        out_dims, bpr = self.weight.shape
        return f"output_dims={out_dims}, bytes_per_row={bpr}, kquant_type={self.kquant_type}"


class KQuantSwitchLinear(_KQuantBase):
    """Expert stack [num_experts, output_dims, bytes_per_row]; forward(x, indices) multiplies every
    x[..., M, K] entry by the expert its index names (kq.gather_qmm with rhs_indices=indices)."""

    def __init__(self, num_experts: int, output_dims: int, input_dims: int, bias: bool, codec: str, device=None):
        super().__init__()
        self._init_codec(codec)
        self._wire_buffers((num_experts, output_dims, bytes_per_row(codec, input_dims)), device)
        if bias:
            self.register_buffer("bias", torch.zeros((num_experts, output_dims), device=device))
        else:
            self.bias = None

    def forward(self, x, indices, sorted_indices=False):
        if sorted_indices and indices.ndim == 1 and x.ndim == 3 and x.shape[0] == indices.numel() and x.shape[1] == 1:
            min_rows = int(os.environ.get("KQ_SWITCH_GEMM_MIN_ROWS", "512"))  # read live, as the reference does
            if min_rows > 0 and indices.numel() >= min_rows and self.weight.shape[1] % 8 == 0:
                y = self._sorted_expert_gemm(x, indices)
                if self.bias is not None:
                    y = y + self.bias[indices.to(torch.int64)].unsqueeze(-2)
                return y
        y = kq.gather_qmm(x, self.weight, self.scales, self.kquant_type, rhs_indices=indices, transpose=True,
                          sorted_indices=sorted_indices)
        if self.bias is not None:
            y = y + self.bias[indices.to(torch.int64)].unsqueeze(-2)
        return y

    def _sorted_expert_gemm(self, x, indices):
        xf = x.reshape(indices.numel(), -1)
        maps = kq.expert_tile_map(indices, self.weight.shape[0])
        return kq.gather_qmm_seg(xf, self.weight, self.scales, self.kquant_type, *maps)[:, None, :]

    def extra_repr(self):
        n, m, b = self.weight.shape
        return f"num_experts={n}, output_dims={m}, bytes_per_row={b}, kquant_type={self.kquant_type}"


class KQuantMultiLinear(_KQuantBase):
    """Per-head batched linear [num_heads, output_dims, bytes_per_row] (absorbed-MLA up-projections).
    x is [B, Hx, L, D] with Hx = num_heads, or 1 for an activation shared by every head;
    transpose=True contracts over the quantized axis (x @ W[h].T), transpose=False over the other
    (x @ W[h])."""

    def __init__(self, input_dims: int, output_dims: int, num_heads: int, codec: str, device=None):
        super().__init__()
        self._init_codec(codec)
        self.num_heads = num_heads
        self._wire_buffers((num_heads, output_dims, bytes_per_row(codec, input_dims)), device)
        self._gather_idx = None

    def forward(self, x, transpose: bool = True):
        nh = self.num_heads
        B, Hx = x.shape[0], x.shape[1]
        cached = self._gather_idx
        if cached is not None and cached[0] == (B, Hx, x.device):
            lhs, rhs = cached[1], cached[2]
        else:
            rhs = torch.arange(nh, dtype=torch.int64, device=x.device).reshape(1, nh).expand(B, nh)
            if Hx == nh:
                lhs = torch.arange(B * nh, dtype=torch.int64, device=x.device).reshape(B, nh)
            elif Hx == 1:
                lhs = torch.arange(B, dtype=torch.int64, device=x.device).reshape(B, 1).expand(B, nh)
            else:
                raise ValueError(f"KQuantMultiLinear: head axis {Hx} is neither 1 nor num_heads={nh} "
                                 f"(x.shape={tuple(x.shape)})")
            self._gather_idx = ((B, Hx, x.device), lhs, rhs)
        return kq.gather_qmm(x, self.weight, self.scales, self.kquant_type, lhs_indices=lhs, rhs_indices=rhs,
                             transpose=transpose)

    def extra_repr(self):
        nh, out_dims, bpr = self.weight.shape
        return f"num_heads={nh}, output_dims={out_dims}, bytes_per_row={bpr}, kquant_type={self.kquant_type}"
