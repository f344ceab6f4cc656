"""Block geometry of every wire codec, for Python callers (same helper names and tuple order as
the reference's mlx_kquant/codec_geometry.py:16-98).  The numbers are those of the library's own
registry (kq.codecs() / kq_codec_get); tests assert the two agree."""
from __future__ import annotations

_SUPER = 256
_FLAT = 32


def _entry(group_size, bits, bytes_per_block, weights_per_block):
    return (group_size, bits, bytes_per_block, weights_per_block)


# codec -> (group_size, bits, bytes_per_block, weights_per_block)
CODEC_GEOMETRY = {
    # K-quant superblocks
    "q2_k": _entry(_SUPER, 2, 84, _SUPER),
    "q3_k": _entry(_SUPER, 3, 110, _SUPER),
    "q4_k": _entry(_SUPER, 4, 144, _SUPER),
    "q5_k": _entry(_SUPER, 5, 176, _SUPER),
    "q6_k": _entry(_SUPER, 6, 210, _SUPER),
    # legacy 32-weight blocks
    "q4_0": _entry(_FLAT, 4, 18, _FLAT),
    "q4_1": _entry(_FLAT, 4, 20, _FLAT),
    "q5_0": _entry(_FLAT, 5, 22, _FLAT),
    "q5_1": _entry(_FLAT, 5, 24, _FLAT),
    "q8_0": _entry(_FLAT, 8, 34, _FLAT),
    # IQ grid / LUT codecs
    "iq4_nl": _entry(_FLAT, 4, 18, _FLAT),
    "iq4_xs": _entry(_SUPER, 4, 136, _SUPER),
    "iq3_s": _entry(_SUPER, 3, 110, _SUPER),
    "iq3_xxs": _entry(_SUPER, 3, 98, _SUPER),
    "iq2_xxs": _entry(_SUPER, 2, 66, _SUPER),
    "iq2_xs": _entry(_SUPER, 2, 74, _SUPER),
    "iq2_s": _entry(_SUPER, 2, 82, _SUPER),
    "iq1_s": _entry(_SUPER, 1, 50, _SUPER),
    "iq1_m": _entry(_SUPER, 1, 56, _SUPER),
    # OCP micro-scaled fp4: nvfp4 scales every 16 values but packs 64 per block
    "mxfp4": _entry(_FLAT, 4, 17, _FLAT),
    "nvfp4": _entry(16, 4, 36, 64),
}

DECODE_ONLY_CODECS = frozenset({"mxfp4", "nvfp4"})
ENCODER_CODECS = frozenset(CODEC_GEOMETRY) - DECODE_ONLY_CODECS
IMATRIX_CODECS = frozenset({"q2_k", "q3_k", "q4_k", "q5_k", "q6_k"})


def geometry(codec):
    """(group_size, bits, bytes_per_block, weights_per_block) of `codec`."""
    if codec not in CODEC_GEOMETRY:
        raise ValueError("unknown codec %r; known codecs: %s" % (codec, ", ".join(sorted(CODEC_GEOMETRY))))
    return CODEC_GEOMETRY[codec]


def bytes_per_row(codec, in_dims):
    """Wire bytes of one quantized row holding `in_dims` weights."""
    _, _, bpb, wpb = geometry(codec)
    if in_dims % wpb:
        raise ValueError("codec %r packs %d weights/block; row width %d is not a multiple of %d"
                         % (codec, wpb, in_dims, wpb))
    return in_dims // wpb * bpb


def in_features(codec, row_bytes):
    """Inverse of bytes_per_row."""
    _, _, bpb, wpb = geometry(codec)
    if row_bytes % bpb:
        raise ValueError("codec %r uses %d-byte blocks; row width %d is not a multiple of %d"
                         % (codec, bpb, row_bytes, bpb))
    return row_bytes // bpb * wpb


weights_per_row = in_features
