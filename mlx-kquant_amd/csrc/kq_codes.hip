// Skinny-M matmul (M <= 8) on the matrix cores for the legacy, IQ and fp4 codecs:
// y[m, n] = sum_k x[m, k] W[n, k] with W in q8_0, q4_0/1, q5_0/1, iq4_nl, iq4_xs, iq3_s, iq3_xxs,
// iq2_xxs, iq2_xs, iq2_s, iq1_s, iq1_m, mxfp4 or nvfp4 wire form.
//
// Numerics.  Every one of these codecs stores a weight as (block scale) x (small code): an int8, a
// nibble minus a zero point, an entry of a 16-value table, a codebook magnitude with a sign, or a
// ternary value +- 1/8.  The codes are exact in f16, so they go into v_mfma_f32_32x32x16_f16 as they
// are, one scale block (16 or 32 weights) per accumulator set, and the block scale multiplies the f32
// partial sum afterwards: products are exact and everything else is f32, so the result differs from
// the f32 reference (src/kquant_cpu_decode.cpp:1010-1065) by summation order only.  q4_1 / q5_1 add
// their block minimum times the block's activation sum.  bf16 activations are converted to f16 per
// (row, 256-wide K step) with an exact power-of-two scale so that they cannot overflow.
//
// Tiling.  Workgroup = 8 waves that share 32 weight rows (the MFMA's 32 columns) and split K: wave w
// takes the 256-weight steps w, w + 8, ... entirely on its own -- wire bytes and activations of a step
// are fetched one step ahead with 16-byte loads and parked in wave-private LDS, so no workgroup
// barrier sits in the weight stream -- and the eight partial sums meet in LDS at the end.  Codebooks
// live in LDS as f16 tables built once per workgroup.  A lane copies its row's step bytes into
// registers with conflict-free 16-byte LDS reads and picks exactly the 8 codes its MFMA B operand
// needs (row l % 32, K half l / 32) at compile-time offsets, so nothing decoded is shared or stored.
//
// The batched MoE ops (more than 16 (token, expert) pairs) use the same decode in a workgroup-tiled
// grouped kernel (further down): 32 gathered pairs of one expert x 128 weight rows per workgroup.
#include "kq_epilogue.h"
#include "kq_mma.h"

namespace {

using namespace kqmma;

typedef u32x4 u32x4_a1 __attribute__((aligned(1)));  // the hardware serves unaligned vector loads
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int CK_WAVES = 8;          // waves per workgroup: they share 32 weight rows and split K
constexpr int CK_STEP = 256;         // weights of K per step
constexpr int XA_STRIDE = 512 + 32;  // bytes per activation row of one step in LDS (rows 8 banks apart)
constexpr int CK_MAXM = 8;

// ------------------------------------------------------------------ codec traits
template <int C>
struct CodeGeom {
  static constexpr int WPB = kq_geom(C).wpb, BPB = kq_geom(C).bpb;
  static constexpr int BLOCKS = CK_STEP / WPB;      // blocks per step and row
  static constexpr int BYTES = BLOCKS * BPB;        // wire bytes per step and row
  static constexpr int PIECES = (BYTES + 15) / 16;  // 16-byte pieces (the last may read past the step)
  static constexpr int LROW = (PIECES | 1) * 16;    // LDS row stride: an odd number of pieces
  // scale granularity: one MFMA (16 weights) or two (32 weights) per scale
  static constexpr int SB = (C == KQ_NVFP4 || C == KQ_IQ2_XS || C == KQ_IQ2_S || C == KQ_IQ1_M) ? 16 : 32;
  static constexpr bool HAS_MIN = C == KQ_Q4_1 || C == KQ_Q5_1;
  // f16 codebook in LDS: entries of 8 weights (16 bytes) or 4 weights (8 bytes)
  static constexpr int GRID_N = C == KQ_IQ2_XXS ? 256 : C == KQ_IQ2_XS ? 512 : C == KQ_IQ2_S ? 1024
                               : (C == KQ_IQ1_S || C == KQ_IQ1_M) ? 2048 : C == KQ_IQ3_XXS ? 256 : C == KQ_IQ3_S ? 512 : 0;
  static constexpr int GRID_W = (C == KQ_IQ3_XXS || C == KQ_IQ3_S) ? 4 : 8;
  static constexpr int GRID_OFF = C == KQ_IQ2_XXS ? KQ_GRID_IQ2XXS : C == KQ_IQ2_XS ? KQ_GRID_IQ2XS
                                 : C == KQ_IQ2_S ? KQ_GRID_IQ2S : (C == KQ_IQ1_S || C == KQ_IQ1_M) ? KQ_GRID_IQ1S
                                 : C == KQ_IQ3_XXS ? KQ_GRID_IQ3XXS : KQ_GRID_IQ3S;
  static constexpr bool GRID_SIGNED = C == KQ_IQ1_S || C == KQ_IQ1_M;  // int8 entries
  // 32-weight blocks whose byte j holds weights j and j + 16 as indices of a 16-value table (iq4_nl, mxfp4): the
  // table in LDS maps a byte to the f16 pair of its two values, and the activations of a block are staged as
  // x[j], x[j + 16] interleaved, so four table reads are the B operand of an MFMA with no further arithmetic
  static constexpr bool PAIR_LUT = C == KQ_IQ4_NL || C == KQ_MXFP4;
  // pair table: 256 entries of 4 bytes.  The grouped kernel keeps one copy per LDS bank (entry b copy c at
  // 128 b + 4 c, lane l reads copy l % 32: the 64 data-dependent reads of an instruction never meet in a bank),
  // + 1 KiB for the plain table the copies are made from; the per-entry kernel, whose launches are too short to
  // earn the 32 KiB build back, keeps the plain table.
  static constexpr int GRID_BYTES = PAIR_LUT ? 1024 : GRID_N * GRID_W * 2;
  static constexpr int GROUPED_GRID_BYTES = PAIR_LUT ? 32768 + 1024 : GRID_BYTES;
  // 256-entry table spreading 8 bits over the 8 halves of a B operand: sign bits (bit 15) for the
  // signed codebooks, the fifth code bit (bit 4) for q5_0 / q5_1
  static constexpr bool SIGNS = C == KQ_IQ2_XXS || C == KQ_IQ2_XS || C == KQ_IQ2_S || C == KQ_IQ3_XXS || C == KQ_IQ3_S;
  static constexpr bool FIFTH = C == KQ_Q5_0 || C == KQ_Q5_1;
  static constexpr int SPREAD_BYTES = (SIGNS || FIFTH) ? 4096 : 0;
  static constexpr int SPREAD_BIT = SIGNS ? 15 : 4;
};

// LDS of one wave: wire bytes of a step (32 rows), f16 activations (mb rows), row scales, block sums
template <int C>
constexpr int wave_lds_bytes(int mb) {
  return 32 * CodeGeom<C>::LROW + mb * XA_STRIDE + CK_MAXM * 4 + 8 * CK_MAXM * 4;
}

// ------------------------------------------------------------------ small helpers
__device__ __forceinline__ uint32_t pk_sub(uint32_t v, float bias) {
  const f16x2 b = {(_Float16)bias, (_Float16)bias};
  return __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, v) - b);
}
// bytes (c0 c1 c2 c3) of `b`, each below 256 -> f16 pairs (c0, c2) and (c1, c3), less `bias`:
// 0x6400 | c is the f16 1024 + c, and the subtraction is exact
__device__ __forceinline__ void bytes_to_f16(uint32_t b, float bias, uint32_t& e, uint32_t& o) {
  const uint32_t m = opaque_sgpr(0x00ff00ffu), k = opaque_sgpr(0x64006400u);
  e = pk_sub((b & m) | k, 1024.f + bias);
  o = pk_sub(((b >> 8) & m) | k, 1024.f + bias);
}
// two dwords of 8 bytes -> B operand in the fragment order k0 k2 k1 k3 k4 k6 k5 k7
__device__ __forceinline__ f16x8 bytes8_to_frag(uint32_t lo, uint32_t hi, float bias) {
  u32x4 r;
  uint32_t e, o;
  bytes_to_f16(lo, bias, e, o);
  r[0] = e;
  r[1] = o;
  bytes_to_f16(hi, bias, e, o);
  r[2] = e;
  r[3] = o;
  return __builtin_bit_cast(f16x8, r);
}
// 16-entry byte table lookup on the four nibble-valued bytes of n: two 8-entry byte permutes and a
// per-byte select on bit 3 (the select mask is a third permute)
__device__ __forceinline__ uint32_t lut16(uint32_t n, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
  const uint32_t sel = n & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel);
  const uint32_t hi = __builtin_amdgcn_perm(t3, t2, sel);
  // selector bytes 0x0c / 0x0d read as 0x00 / 0xff: 0xff in every byte whose bit 3 is set
  const uint32_t mask = __builtin_amdgcn_perm(n, n, ((n >> 3) & 0x01010101u) | 0x0c0c0c0cu);
  return (hi & mask) | (lo & ~mask);
}
// One lane's eight consecutive activations h[0..7] (8-group `pc` of a row) to the row's staging area: in the fragment
// order k0 k2 k1 k3 inside the group, or (PAIR) with x[j], x[j + 16] interleaved over each 32: lanes pc and pc ^ 2 of a
// quad hold x[8 a ..] and x[16 + 8 a ..] and write one half each of the 16 interleaved values.
template <bool PAIR>
__device__ __forceinline__ void stage_group(uint8_t* row_lds, int pc, const _Float16* h) {
  if constexpr (!PAIR) {
    const f16x8 v8 = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
    *reinterpret_cast<f16x8*>(row_lds + 16 * pc) = v8;
  } else {
    uint32_t own[4], par[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      own[e] = (uint32_t)__builtin_bit_cast(uint16_t, h[2 * e]) | ((uint32_t)__builtin_bit_cast(uint16_t, h[2 * e + 1]) << 16);
      par[e] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)own[e], 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
    }
    const bool high = (pc & 2) != 0;
    const uint32_t a0 = high ? par[2] : own[0], a1 = high ? par[3] : own[1];
    const uint32_t b0 = high ? own[2] : par[0], b1 = high ? own[3] : par[1];
    const u32x4 o = {(a0 & 0xffffu) | (b0 << 16), (a0 >> 16) | (b0 & 0xffff0000u), (a1 & 0xffffu) | (b1 << 16),
                     (a1 >> 16) | (b1 & 0xffff0000u)};
    *reinterpret_cast<u32x4*>(row_lds + 64 * (pc >> 2) + 32 * (pc & 1) + (high ? 16 : 0)) = o;
  }
}
__device__ __forceinline__ float f16bits(uint32_t h) { return (float)__builtin_bit_cast(_Float16, (uint16_t)h); }

// 128-bit value >> 8 k bits (k >= 1 bytes)
__device__ __forceinline__ u32x4 shr_bytes(u32x4 v, uint32_t k) {
  if (k >= 16) return u32x4{0, 0, 0, 0};
  uint64_t lo = (uint64_t)v[0] | ((uint64_t)v[1] << 32), hi = (uint64_t)v[2] | ((uint64_t)v[3] << 32);
  if (k & 8) {
    lo = hi;
    hi = 0;
  }
  const uint32_t sh = 8 * (k & 7);
  if (sh) {
    lo = (lo >> sh) | (hi << (64 - sh));
    hi >>= sh;
  }
  return u32x4{(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
}

// The wire bytes of one (row, step) in registers: the lane fetches them from LDS with 16-byte reads
// (row stride an odd number of 16-byte pieces: conflict-free) and every field is then picked at a
// compile-time byte offset, so that the decode issues no narrow, bank-conflicting LDS reads.
template <int NDW>
struct RowRegs {
  uint32_t d[NDW];
  template <int OFF>
  __device__ __forceinline__ uint32_t u32() const {
    static_assert(OFF >= 0 && OFF / 4 < NDW, "offset outside the row");
    if constexpr (OFF % 4 == 0)
      return d[OFF / 4];
    else
      return __builtin_amdgcn_alignbyte(d[OFF / 4 + 1 < NDW ? OFF / 4 + 1 : OFF / 4], d[OFF / 4], OFF % 4);
  }
  template <int OFF>
  __device__ __forceinline__ uint32_t u16() const {
    if constexpr (OFF % 4 <= 2)
      return (d[OFF / 4] >> (8 * (OFF % 4))) & 0xffffu;
    else
      return u32<OFF>() & 0xffffu;
  }
  template <int OFF>
  __device__ __forceinline__ uint32_t u8() const {
    return (d[OFF / 4] >> (8 * (OFF % 4))) & 0xffu;
  }
};
__device__ __forceinline__ uint32_t pick(int kg, uint32_t a, uint32_t b) { return kg ? b : a; }

struct Tables {
  const uint8_t* grid;    // f16 codebook (LDS)
  const uint8_t* spread;  // 256 x 16-byte bit-spread table (LDS)
  int pair_shift;         // log2 of the byte distance between pair-table entries (2, or 7 with a copy per bank)
};

// The B operand of MFMA J (weights 16 J + 8 kg .. + 7 of the step) of the row whose step bytes are in
// `row`.  J is a compile-time constant.
template <int C, int J, class R>
__device__ __forceinline__ f16x8 codes(const R& row, int kg, const Tables& t) {
  using G = CodeGeom<C>;
  if constexpr (C == KQ_Q8_0) {
    constexpr int off = (J / 2) * 34 + 2 + 16 * (J & 1);
    const uint32_t lo = pick(kg, row.template u32<off>(), row.template u32<off + 8>());
    const uint32_t hi = pick(kg, row.template u32<off + 4>(), row.template u32<off + 12>());
    return bytes8_to_frag(lo ^ 0x80808080u, hi ^ 0x80808080u, 128.f);
  } else if constexpr (C == KQ_Q4_0 || C == KQ_Q4_1 || C == KQ_Q5_0 || C == KQ_Q5_1 || C == KQ_IQ4_NL ||
                       C == KQ_MXFP4) {
    // 32-weight blocks: weights 0..15 = low nibbles of q[0..15], 16..31 = high nibbles
    constexpr int QOFF = C == KQ_Q4_0 || C == KQ_IQ4_NL ? 2 : C == KQ_Q4_1 ? 4 : C == KQ_Q5_0 ? 6 : C == KQ_Q5_1 ? 8 : 1;
    constexpr int boff = (J / 2) * G::BPB, off = boff + QOFF;
    if constexpr (G::PAIR_LUT) {
      // staged positions 16 J + 8 kg .. + 7 = bytes 8 (J % 2) + 4 kg .. + 3 of block J / 2, both nibbles of each
      const uint32_t w = pick(kg, row.template u32<off + 8 * (J & 1)>(), row.template u32<off + 8 * (J & 1) + 4>());
      u32x4 r;
#pragma unroll
      for (int e = 0; e < 4; e++)
        r[e] = *reinterpret_cast<const uint32_t*>(t.grid + (((w >> (8 * e)) & 0xffu) << t.pair_shift));
      return __builtin_bit_cast(f16x8, r);
    }
    uint32_t lo = pick(kg, row.template u32<off>(), row.template u32<off + 8>());
    uint32_t hi = pick(kg, row.template u32<off + 4>(), row.template u32<off + 12>());
    if constexpr (J & 1) {
      lo >>= 4;
      hi >>= 4;
    }
    lo &= 0x0f0f0f0fu;
    hi &= 0x0f0f0f0fu;
    if constexpr (C == KQ_IQ4_NL) {
      return bytes8_to_frag(lut16(lo, 0x3f2d1801u, 0x766a5d4fu, 0xa6998d81u, 0xf1d9c5b5u),
                            lut16(hi, 0x3f2d1801u, 0x766a5d4fu, 0xa6998d81u, 0xf1d9c5b5u), 128.f);
    } else if constexpr (C == KQ_MXFP4) {
      return bytes8_to_frag(lut16(lo, 0x83828180u, 0x8c888684u, 0x7d7e7f80u, 0x74787a7cu),
                            lut16(hi, 0x83828180u, 0x8c888684u, 0x7d7e7f80u, 0x74787a7cu), 128.f);
    } else if constexpr (C == KQ_Q5_0 || C == KQ_Q5_1) {
      // fifth bits of weights 16 (J & 1) + 8 kg .. + 7: one byte of qh, spread to bit 4 of every half
      constexpr int hoff = boff + (C == KQ_Q5_0 ? 2 : 4) + 2 * (J & 1);
      const uint32_t hb = pick(kg, row.template u8<hoff>(), row.template u8<hoff + 1>());
      const u32x4 sp = *reinterpret_cast<const u32x4*>(t.spread + 16 * hb);
      u32x4 r = __builtin_bit_cast(u32x4, bytes8_to_frag(lo, hi, -1024.f));  // keep the 1024 + q form
      r |= sp;
      const float bias = C == KQ_Q5_0 ? 1024.f + 16.f : 1024.f;
      r[0] = pk_sub(r[0], bias);
      r[1] = pk_sub(r[1], bias);
      r[2] = pk_sub(r[2], bias);
      r[3] = pk_sub(r[3], bias);
      return __builtin_bit_cast(f16x8, r);
    } else {
      return bytes8_to_frag(lo, hi, C == KQ_Q4_0 ? 8.f : 0.f);
    }
  } else if constexpr (C == KQ_NVFP4) {
    // 64-weight blocks, 16-weight groups: weights 0..7 = low nibbles of q[0..7], 8..15 = high nibbles
    constexpr int off = (J / 4) * 36 + 4 + 8 * (J & 3);
    const int sh = 4 * kg;
    const uint32_t lo = (row.template u32<off>() >> sh) & 0x0f0f0f0fu;
    const uint32_t hi = (row.template u32<off + 4>() >> sh) & 0x0f0f0f0fu;
    return bytes8_to_frag(lut16(lo, 0x83828180u, 0x8c888684u, 0x7d7e7f80u, 0x74787a7cu),
                          lut16(hi, 0x83828180u, 0x8c888684u, 0x7d7e7f80u, 0x74787a7cu), 128.f);
  } else if constexpr (C == KQ_IQ4_XS) {
    constexpr int off = 8 + 16 * (J / 2);
    uint32_t lo = pick(kg, row.template u32<off>(), row.template u32<off + 8>());
    uint32_t hi = pick(kg, row.template u32<off + 4>(), row.template u32<off + 12>());
    if constexpr (J & 1) {
      lo >>= 4;
      hi >>= 4;
    }
    lo &= 0x0f0f0f0fu;
    hi &= 0x0f0f0f0fu;
    return bytes8_to_frag(lut16(lo, 0x3f2d1801u, 0x766a5d4fu, 0xa6998d81u, 0xf1d9c5b5u),
                          lut16(hi, 0x3f2d1801u, 0x766a5d4fu, 0xa6998d81u, 0xf1d9c5b5u), 128.f);
  } else {
    // codebook codecs: 8-weight group l = 2 (J & 1) + kg of 32-weight sub-block ib = J / 2
    constexpr int ib = J / 2, l0 = 2 * (J & 1);
    const int l = l0 + kg;
    u32x4 r;
    uint32_t sbits = 0;
    if constexpr (C == KQ_IQ2_XXS) {
      const uint32_t aux = row.template u32<2 + 8 * ib + 4>();
      const uint32_t gi = pick(kg, row.template u8<2 + 8 * ib + l0>(), row.template u8<2 + 8 * ib + l0 + 1>());
      r = *reinterpret_cast<const u32x4*>(t.grid + 16 * gi);
      sbits = (aux >> (7 * l)) & 127u;
      sbits |= (uint32_t)(__builtin_popcount(sbits) & 1) << 7;
    } else if constexpr (C == KQ_IQ2_XS) {
      const uint32_t q = pick(kg, row.template u16<2 + 8 * ib + 2 * l0>(), row.template u16<2 + 8 * ib + 2 * l0 + 2>());
      r = *reinterpret_cast<const u32x4*>(t.grid + 16 * (q & 511u));
      sbits = q >> 9;
      sbits |= (uint32_t)(__builtin_popcount(sbits) & 1) << 7;
    } else if constexpr (C == KQ_IQ2_S) {
      const uint32_t qb = pick(kg, row.template u8<2 + 4 * ib + l0>(), row.template u8<2 + 4 * ib + l0 + 1>());
      const uint32_t gi = qb | ((row.template u8<66 + ib>() << (8 - 2 * l)) & 0x300u);
      r = *reinterpret_cast<const u32x4*>(t.grid + 16 * gi);
      sbits = pick(kg, row.template u8<34 + 4 * ib + l0>(), row.template u8<34 + 4 * ib + l0 + 1>());
    } else if constexpr (C == KQ_IQ3_XXS) {
      const uint32_t aux = row.template u32<66 + 4 * ib>();
      const uint32_t qq = pick(kg, row.template u16<2 + 8 * ib + 2 * l0>(), row.template u16<2 + 8 * ib + 2 * l0 + 2>());
      const u32x2 g1 = *reinterpret_cast<const u32x2*>(t.grid + 8 * (qq & 0xffu));
      const u32x2 g2 = *reinterpret_cast<const u32x2*>(t.grid + 8 * (qq >> 8));
      r = u32x4{g1[0], g1[1], g2[0], g2[1]};
      sbits = (aux >> (7 * l)) & 127u;
      sbits |= (uint32_t)(__builtin_popcount(sbits) & 1) << 7;
    } else if constexpr (C == KQ_IQ3_S) {
      const uint32_t h = row.template u8<66 + ib>();
      const uint32_t qq = pick(kg, row.template u16<2 + 8 * ib + 2 * l0>(), row.template u16<2 + 8 * ib + 2 * l0 + 2>());
      const uint32_t i1 = (qq & 0xffu) | ((h << (8 - 2 * l)) & 256u);
      const uint32_t i2 = (qq >> 8) | ((h << (7 - 2 * l)) & 256u);
      const u32x2 g1 = *reinterpret_cast<const u32x2*>(t.grid + 8 * i1);
      const u32x2 g2 = *reinterpret_cast<const u32x2*>(t.grid + 8 * i2);
      r = u32x4{g1[0], g1[1], g2[0], g2[1]};
      sbits = pick(kg, row.template u8<74 + 4 * ib + l0>(), row.template u8<74 + 4 * ib + l0 + 1>());
    } else if constexpr (C == KQ_IQ1_S) {
      const uint32_t qh = row.template u16<34 + 2 * ib>();
      const uint32_t qb = pick(kg, row.template u8<2 + 4 * ib + l0>(), row.template u8<2 + 4 * ib + l0 + 1>());
      r = *reinterpret_cast<const u32x4*>(t.grid + 16 * (qb | (((qh >> (3 * l)) & 7u) << 8)));
      const float delta = (qh & 0x8000u) ? 0.125f : -0.125f;  // subtracted below
      r[0] = pk_sub(r[0], delta);
      r[1] = pk_sub(r[1], delta);
      r[2] = pk_sub(r[2], delta);
      r[3] = pk_sub(r[3], delta);
    } else {  // KQ_IQ1_M
      const uint32_t hb = row.template u8<32 + 2 * ib + (J & 1)>();
      const uint32_t nib = kg ? (hb >> 4) : (hb & 15u);
      const uint32_t qb = pick(kg, row.template u8<4 * ib + l0>(), row.template u8<4 * ib + l0 + 1>());
      r = *reinterpret_cast<const u32x4*>(t.grid + 16 * (qb | ((nib & 7u) << 8)));
      const float delta = (nib & 8u) ? 0.125f : -0.125f;  // subtracted below
      r[0] = pk_sub(r[0], delta);
      r[1] = pk_sub(r[1], delta);
      r[2] = pk_sub(r[2], delta);
      r[3] = pk_sub(r[3], delta);
    }
    if constexpr (G::SIGNS) {
      const u32x4 sp = *reinterpret_cast<const u32x4*>(t.spread + 16 * sbits);
      r ^= sp;
    }
    return __builtin_bit_cast(f16x8, r);
  }
}

// f32 scale of scale block SBI of the step (SBI counts G::SB-weight blocks); mn = block minimum (q4_1 / q5_1)
template <int C, int SBI, class R>
__device__ __forceinline__ float block_scale(const R& row, float& mn) {
  constexpr int BPB = CodeGeom<C>::BPB;
  mn = 0.f;
  if constexpr (C == KQ_Q8_0 || C == KQ_Q4_0 || C == KQ_Q5_0 || C == KQ_IQ4_NL) {
    return f16bits(row.template u16<SBI * BPB>());
  } else if constexpr (C == KQ_Q4_1 || C == KQ_Q5_1) {
    const uint32_t dm = row.template u32<SBI * BPB>();
    mn = f16bits(dm >> 16);
    return f16bits(dm & 0xffffu);
  } else if constexpr (C == KQ_MXFP4) {
    return kq::e8m0_half(row.template u8<SBI * 17>());
  } else if constexpr (C == KQ_NVFP4) {
    return kq::ue4m3_half(row.template u8<(SBI / 4) * 36 + (SBI & 3)>());
  } else if constexpr (C == KQ_IQ4_XS) {
    const float d = f16bits(row.template u16<0>());
    const uint32_t sh = row.template u16<2>();
    const int ls = (int)((row.template u8<4 + (SBI >> 1)>() >> (4 * (SBI & 1))) & 15u) | (int)(((sh >> (2 * SBI)) & 3u) << 4);
    return d * (float)(ls - 32);
  } else if constexpr (C == KQ_IQ2_XXS) {
    const float d = f16bits(row.template u16<0>());
    const uint32_t aux = row.template u32<2 + 8 * SBI + 4>();
    return d * (0.5f + (float)(aux >> 28)) * 0.25f;
  } else if constexpr (C == KQ_IQ2_XS || C == KQ_IQ2_S) {  // 16-weight blocks
    const float d = f16bits(row.template u16<0>());
    const uint32_t scb = row.template u8<(C == KQ_IQ2_XS ? 66 : 74) + (SBI >> 1)>();
    return d * (0.5f + (float)((SBI & 1) ? (scb >> 4) : (scb & 15u))) * 0.25f;
  } else if constexpr (C == KQ_IQ3_XXS) {
    const float d = f16bits(row.template u16<0>());
    const uint32_t aux = row.template u32<66 + 4 * SBI>();
    return d * (0.5f + (float)(aux >> 28)) * 0.5f;
  } else if constexpr (C == KQ_IQ3_S) {
    const float d = f16bits(row.template u16<0>());
    const uint32_t sb = row.template u8<106 + (SBI >> 1)>();
    return d * (float)(1 + 2 * (int)((SBI & 1) ? (sb >> 4) : (sb & 15u)));
  } else if constexpr (C == KQ_IQ1_S) {
    const float d = f16bits(row.template u16<0>());
    const uint32_t qh = row.template u16<34 + 2 * SBI>();
    return d * (float)(2 * (int)((qh >> 12) & 7u) + 1);
  } else {  // KQ_IQ1_M, 16-weight blocks
    const uint32_t s0 = row.template u16<48>(), s1 = row.template u16<50>(), s2 = row.template u16<52>(),
                   s3 = row.template u16<54>();
    const float d = f16bits((s0 >> 12) | ((s1 >> 8) & 0x00f0u) | ((s2 >> 4) & 0x0f00u) | (s3 & 0xf000u));
    constexpr int ib = SBI >> 1;
    const uint32_t scw = ib < 2 ? s0 : ib < 4 ? s1 : ib < 6 ? s2 : s3;
    const int sc3 = (scw >> (6 * (ib & 1) + 3 * (SBI & 1))) & 7;
    return d * (float)(2 * sc3 + 1);
  }
}

// ------------------------------------------------------------------ kernel
struct CkArgs {
  const void* x;  // [M][K]
  const uint8_t* w;
  void* y;        // [M][N]
  const uint16_t* bias;  // [N] in the activation dtype, added in f32 before the rounding; or null
  const uint8_t* grids;
  int M, N, K;
  // gathered calls (GMODE 1 / 2), one item per blockIdx.y: activation row x + (lhs ? lhs[item] : item / x_div) *
  // x_item_stride, matrix w (+ w2 for the GLU) + rhs[item] * w_expert_stride, f32 biases [E][N], output row
  // through the out map
  const uint8_t* w2;
  const uint32_t* lhs;
  const uint32_t* rhs;
  const float* fbias;
  const float* fbias2;
  int x_div, act;
  int64_t x_item_stride, w_expert_stride;
  float limit, alpha;
  KqOutMap om;
  int E;  // gathered calls: items whose expert id is >= E are skipped (output rows left untouched)
};

__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroup = CK_WAVES waves that share 32 weight rows and split K: wave w takes the 256-weight steps
// w, w + CK_WAVES, ... on its own (wave-private LDS buffers, no workgroup barrier in the stream), and
// the partial sums meet in LDS at the end.  MB = activation rows the LDS buffers are sized for.
// GMODE 0: one dense matrix.  GMODE 1: gathered, one (activation row, expert matrix) item per blockIdx.y.
// GMODE 2: gathered GLU: the tile's 32 rows are 16 gate rows and the same 16 up rows, the epilogue act(g) * u runs
// on the reduced sums before the single rounding.
// WV = waves per workgroup.  Gathered launches (many small workgroups, short K) need the whole grid resident at
// once: the codecs whose kernel stays under 128 registers get there with 8 waves (two workgroups per CU), the
// others use 4-wave workgroups (iq4_xs 11.9 + 8.9 -> 10.3 + 6.3 us for the GLU + down of 8 experts of 768 x 2048;
// iq1_s went the other way, 6.8 + 5.0 -> 8.1 + 5.8 us, hence the split).  Dense launches use 8 waves, except
// single-row calls of those larger kernels with more row tiles than CUs, where 4-wave workgroups measured 7 - 15 %
// faster (iq4_xs 128256 x 4096: 127 -> 110 us) and 20 - 40 % slower with fewer tiles.
template <int C>
constexpr bool ck_small() {
  return C == KQ_IQ2_XXS || C == KQ_IQ2_XS || C == KQ_IQ2_S || C == KQ_IQ1_S || C == KQ_IQ1_M;
}
template <int C, int GMODE>
constexpr int ck_waves() {
  return (GMODE && !ck_small<C>()) ? 4 : CK_WAVES;
}

template <int C, int DT, int MB, int GMODE, int WV>
__global__ __launch_bounds__((64 * WV), (WV == 4 ? 2 : 1)) void codes_skinny_kernel(CkArgs a) {
  constexpr int NWAVES = WV, NTHREADS = 64 * NWAVES;
  using G = CodeGeom<C>;
  constexpr int TILE_N = GMODE == 2 ? 16 : 32;  // output columns per workgroup
  constexpr int WPT = (32 * G::PIECES + 63) / 64;  // wire pieces per lane and step
  constexpr int XPT = MB >= 2 ? MB / 2 : 1;        // activation pieces per lane and step (rows lane / 32 + 2 t)
  constexpr int WAVE_LDS = wave_lds_bytes<C>(MB);
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* grid_lds = smem;
  uint8_t* spread_lds = grid_lds + G::GRID_BYTES;
  uint8_t* wave_base = spread_lds + G::SPREAD_BYTES;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, kg = lane >> 5;
  const int M = a.M, N = a.N, K = a.K;
  const int nsteps = (K + CK_STEP - 1) / CK_STEP;
  const size_t row_bytes = (size_t)(K / G::WPB) * G::BPB;
  const int n0 = blockIdx.x * TILE_N;
  const int ncols = N - n0 < TILE_N ? N - n0 : TILE_N;
  const int item = GMODE ? (int)blockIdx.y : 0;
  const uint32_t expert = GMODE ? a.rhs[item] : 0u;
  if (GMODE && expert >= (uint32_t)a.E) return;  // uniform over the workgroup, ahead of every barrier
  const uint8_t* wmat = a.w + (GMODE ? (size_t)expert * (size_t)a.w_expert_stride : 0);
  const uint8_t* wmat2 = GMODE == 2 ? a.w2 + (size_t)expert * (size_t)a.w_expert_stride : wmat;
  const uint8_t* w_last = wmat + (size_t)N * row_bytes - 16;    // the last 16 bytes of the matrix
  const uint8_t* w_last2 = wmat2 + (size_t)N * row_bytes - 16;

  uint8_t* b_lds = wave_base + wave * WAVE_LDS;                                    // [32][LROW] wire bytes of the step
  uint8_t* a_lds = b_lds + 32 * G::LROW;                                           // [MB][XA_STRIDE] f16 activations
  float* xs_lds = reinterpret_cast<float*>(a_lds + MB * XA_STRIDE);                // [8] activation scale per row
  float* xsum_lds = xs_lds + CK_MAXM;                                              // [8 blocks][8 rows] (HAS_MIN)

  // ---- tables (whole workgroup)
  if constexpr (G::GRID_N > 0) {
    const uint8_t* src = a.grids + G::GRID_OFF;
    if constexpr (G::GRID_W == 8) {
      for (int e = tid; e < G::GRID_N; e += NTHREADS) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(src + 8 * e);
        f16x8 f;
        if constexpr (G::GRID_SIGNED)
          f = bytes8_to_frag(v[0] ^ 0x80808080u, v[1] ^ 0x80808080u, 128.f);
        else
          f = bytes8_to_frag(v[0], v[1], 0.f);
        *reinterpret_cast<f16x8*>(grid_lds + 16 * e) = f;
      }
    } else {
      for (int e = tid; e < G::GRID_N; e += NTHREADS) {
        const uint32_t v = *reinterpret_cast<const uint32_t*>(src + 4 * e);
        uint32_t ev, od;
        bytes_to_f16(v, 0.f, ev, od);
        *reinterpret_cast<u32x2*>(grid_lds + 8 * e) = u32x2{ev, od};
      }
    }
  }
  if constexpr (G::PAIR_LUT) {
    if (tid < 256) {
      const f16x2 e = C == KQ_MXFP4 ? f16x2{(_Float16)kq::kv_mxfp4(tid & 15), (_Float16)kq::kv_mxfp4(tid >> 4)}
                                    : f16x2{(_Float16)kq::kv_iq4nl(tid & 15), (_Float16)kq::kv_iq4nl(tid >> 4)};
      reinterpret_cast<uint32_t*>(grid_lds)[tid] = __builtin_bit_cast(uint32_t, e);
    }
  }
  if constexpr (G::SPREAD_BYTES > 0) {
    if (tid < 256) {
      const uint32_t b = tid;
      auto bit = [&](int i) { return (b >> i) & 1u; };
      constexpr int P = G::SPREAD_BIT;
      *reinterpret_cast<u32x4*>(spread_lds + 16 * tid) =
          u32x4{(bit(0) << P) | (bit(2) << (P + 16)), (bit(1) << P) | (bit(3) << (P + 16)),
                (bit(4) << P) | (bit(6) << (P + 16)), (bit(5) << P) | (bit(7) << (P + 16))};
    }
  }
  if constexpr (G::GRID_N > 0 || G::SPREAD_BYTES > 0 || G::PAIR_LUT) lds_barrier();
  const Tables tabs{grid_lds, spread_lds, 2};

  // ---- piece maps of this wave.  Wire: piece i = lane + 64 t -> (row i / PIECES, piece i % PIECES).
  // Activations: lane -> (row lane / 32 + 2 t, 16-byte piece lane % 32).
  const uint8_t* w_src[WPT];
  uint32_t w_loff[WPT];
  bool w_up[WPT];
#pragma unroll
  for (int t = 0; t < WPT; t++) {
    const int i = lane + 64 * t;
    const int r = i / G::PIECES, pc = i % G::PIECES;
    const int col = GMODE == 2 ? (r & 15) : r;  // GLU: LDS rows 0..15 gate, 16..31 up
    w_up[t] = GMODE == 2 && (r & 16);
    const bool ok = col < ncols;  // rows past N (and pieces past the tile) re-read the tile's first row
    w_src[t] = (w_up[t] ? wmat2 : wmat) + (size_t)(n0 + (ok ? col : 0)) * row_bytes + 16 * pc;
    w_loff[t] = r < 32 ? (uint32_t)r * G::LROW + 16 * pc : 0xffffffffu;
  }
  const int a_row0 = lane >> 5, a_pc = lane & 31;
  const uint16_t* a_src = static_cast<const uint16_t*>(a.x) + 8 * a_pc +
                          (GMODE ? (size_t)(a.lhs ? a.lhs[item] : (uint32_t)(item / a.x_div)) * (size_t)a.x_item_stride : 0);

  u32x4 areg[XPT], wreg[WPT];
  auto issue = [&](int st) {
    const int kvalid = K - CK_STEP * st;  // weights of this step that exist (>= 256 except in the last step)
#pragma unroll
    for (int t = 0; t < XPT; t++) {
      const int row = a_row0 + 2 * t;
      u32x4 av = {0, 0, 0, 0};
      if (row < M && row < MB && 8 * a_pc < kvalid)
        av = *reinterpret_cast<const u32x4*>(a_src + (size_t)row * K + (size_t)CK_STEP * st);
      areg[t] = av;
    }
#pragma unroll
    for (int t = 0; t < WPT; t++) {
      // Pieces past the step's valid bytes (last step of a ragged K, last piece of a row) carry bytes
      // that no MFMA reads; only the end of the matrix needs care: there the 16 bytes ending at the
      // matrix end are loaded instead and shifted down, so nothing past the end is ever read.
      const uint8_t* p = w_src[t] + (size_t)st * G::BYTES;
      const uint8_t* end = (GMODE == 2 && w_up[t]) ? w_last2 : w_last;
      const uint8_t* q = p <= end ? p : end;
      u32x4 v = *reinterpret_cast<const u32x4_a1*>(q);
      if (q != p) v = shr_bytes(v, (uint32_t)(p - q));
      wreg[t] = v;
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int t = 0; t < XPT; t++) {
      const int row = a_row0 + 2 * t;
      if (MB == 1 && lane >= 32) break;
      // activations: f16 as given, bf16 scaled into f16 range by a power of two per (row, step)
      float xscale = 1.f;
      _Float16 h[8];
      if constexpr (DT == KQ_BF16) {
        float amax = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, areg[t][e] << 16)));
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, areg[t][e] & 0xffff0000u)));
        }
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));  // the row's 32 lanes
        float inv = 1.f;
        const uint32_t eb = (__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff;
        if (eb != 0 && eb != 0xff) {
          int e = (int)eb - 127 - 14;  // the largest magnitude lands in [2^14, 2^15)
          if (e < -100) e = -100;
          xscale = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
          inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
        }
#pragma unroll
        for (int e = 0; e < 4; e++) {
          h[2 * e] = (_Float16)(__builtin_bit_cast(float, areg[t][e] << 16) * inv);
          h[2 * e + 1] = (_Float16)(__builtin_bit_cast(float, areg[t][e] & 0xffff0000u) * inv);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          h[2 * e] = __builtin_bit_cast(_Float16, (uint16_t)(areg[t][e] & 0xffff));
          h[2 * e + 1] = __builtin_bit_cast(_Float16, (uint16_t)(areg[t][e] >> 16));
        }
      }
      stage_group<G::PAIR_LUT>(a_lds + row * XA_STRIDE, a_pc, h);
      if (a_pc == 0) xs_lds[row] = xscale;
      if constexpr (G::HAS_MIN) {
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) sum += (float)h[e];
        sum += __shfl_xor(sum, 1);
        sum += __shfl_xor(sum, 2);  // 4 lanes = one 32-weight block
        if ((a_pc & 3) == 0) xsum_lds[(a_pc >> 2) * CK_MAXM + row] = sum;
      }
    }
#pragma unroll
    for (int t = 0; t < WPT; t++)
      if (w_loff[t] != 0xffffffffu) *reinterpret_cast<u32x4*>(b_lds + w_loff[t]) = wreg[t];
  };

  float acc[4] = {0.f, 0.f, 0.f, 0.f};  // output rows 4 kg + i of weight row n0 + l32
  const uint8_t* b_lane = b_lds + l32 * G::LROW;
  const uint8_t* a_lane = a_lds + (l32 & (MB - 1)) * XA_STRIDE + 16 * kg;
  if (lane < CK_MAXM) xs_lds[lane] = 0.f;  // rows past MB keep a zero scale

  if (wave < nsteps) issue(wave);
  for (int st = wave; st < nsteps; st += NWAVES) {
    park();
    wave_sync();
    if (st + NWAVES < nsteps) issue(st + NWAVES);
    const int kvalid = K - CK_STEP * st;
    float sacc[4] = {0.f, 0.f, 0.f, 0.f};
    constexpr int MPS = G::SB / 16;  // MFMAs per scale block
    // FULL: all 16 MFMAs of the step, branch-free so that decode, MFMA and scaling of neighbouring
    // blocks overlap; otherwise (the last step of a K that is not a multiple of 256) MFMA by MFMA.
    auto run_step = [&](auto full_c) {
      constexpr bool FULL = decltype(full_c)::value;
      f32x16 part[2];
      RowRegs<4 * G::PIECES> row;
      StaticFor<G::PIECES>::run([&](auto pc) {
        constexpr int P = decltype(pc)::value;
        const u32x4 v = *reinterpret_cast<const u32x4*>(b_lane + 16 * P);
        row.d[4 * P] = v[0];
        row.d[4 * P + 1] = v[1];
        row.d[4 * P + 2] = v[2];
        row.d[4 * P + 3] = v[3];
      });
      StaticFor<16>::run([&](auto jc) {
        constexpr int J = decltype(jc)::value;
        if (FULL || 16 * J < kvalid) {  // uniform
          const f16x8 bv = codes<C, J>(row, kg, tabs);
          // activation rows past M hold zeros or another row's values: they only reach output rows that
          // are never stored
          const f16x8 av = *reinterpret_cast<const f16x8*>(a_lane + 32 * J);
          constexpr int sbi = J / MPS, slot = sbi & 1;
          if constexpr (J % MPS == 0)
            part[slot] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, f32x16{0}, 0, 0, 0);
          else
            part[slot] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, part[slot], 0, 0, 0);
          if constexpr (J % MPS == MPS - 1) {
            float mn;
            const float sc = block_scale<C, sbi>(row, mn);
#pragma unroll
            for (int i = 0; i < 4; i++) sacc[i] = fmaf(sc, part[slot][i], sacc[i]);
            if constexpr (G::HAS_MIN) {
              const float4 xm = *reinterpret_cast<const float4*>(xsum_lds + sbi * CK_MAXM + 4 * kg);
              sacc[0] = fmaf(mn, xm.x, sacc[0]);
              sacc[1] = fmaf(mn, xm.y, sacc[1]);
              sacc[2] = fmaf(mn, xm.z, sacc[2]);
              sacc[3] = fmaf(mn, xm.w, sacc[3]);
            }
          }
        }
      });
    };
    if (kvalid >= CK_STEP)
      run_step(std::true_type{});
    else
      run_step(std::false_type{});
    const float4 xs4 = *reinterpret_cast<const float4*>(xs_lds + 4 * kg);
    acc[0] = fmaf(xs4.x, sacc[0], acc[0]);
    acc[1] = fmaf(xs4.y, sacc[1], acc[1]);
    acc[2] = fmaf(xs4.z, sacc[2], acc[2]);
    acc[3] = fmaf(xs4.w, sacc[3], acc[3]);
    wave_sync();  // this wave's reads of the step are done before the next park overwrites it
  }

  // ---- the waves' partial sums meet in LDS (the step buffers are free now)
  lds_barrier();
  float* red = reinterpret_cast<float*>(wave_base);  // [NWAVES][4][64]
#pragma unroll
  for (int i = 0; i < 4; i++) red[(wave * 4 + i) * 64 + lane] = acc[i];
  lds_barrier();
  if (wave == 0) {
    const int n = n0 + l32;
    uint16_t* y = static_cast<uint16_t*>(a.y);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < NWAVES; w++) v += red[(w * 4 + i) * 64 + lane];
      const int m = 4 * kg + i;
      if constexpr (GMODE == 0) {
        if (m < M && n < N) {
          if (a.bias) v += DT == KQ_F16 ? kq::h2f(a.bias[n]) : kq::bf162f(a.bias[n]);
          y[(size_t)m * N + n] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
        }
      } else if constexpr (GMODE == 1) {
        if (m < M && n < N) {
          if (a.fbias) v += a.fbias[(size_t)expert * N + n];
          kq::store_result<DT>(a.y, a.om, ((size_t)kq::out_row(a.om, item) * M + m) * N + n, v);
        }
      } else {
        float u = 0.f;  // the up row of this column sits 16 lanes further on
#pragma unroll
        for (int w = 0; w < NWAVES; w++) u += red[(w * 4 + i) * 64 + (lane ^ 16)];
        if (l32 < 16 && m < M && l32 < ncols) {
          if (a.fbias) v += a.fbias[(size_t)expert * N + n];
          if (a.fbias2) u += a.fbias2[(size_t)expert * N + n];
          v = kq::glu_epilogue(a.act, v, u, a.limit, a.alpha);
          kq::store_result<DT>(a.y, a.om, ((size_t)kq::out_row(a.om, item) * M + m) * N + n, v);
        }
      }
    }
  }
}

template <int C, int DT, int MB, int GMODE, int NWAVES>
int launch_codes_wv(const CkArgs& a, hipStream_t s, int items) {
  using G = CodeGeom<C>;
  size_t lds = (size_t)G::GRID_BYTES + G::SPREAD_BYTES + (size_t)NWAVES * wave_lds_bytes<C>(MB);
  const size_t red = (size_t)G::GRID_BYTES + G::SPREAD_BYTES + NWAVES * 4 * 64 * 4;
  if (lds < red) lds = red;
  auto kern = codes_skinny_kernel<C, DT, MB, GMODE, NWAVES>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  constexpr int TILE_N = GMODE == 2 ? 16 : 32;
  hipLaunchKernelGGL(kern, dim3((a.N + TILE_N - 1) / TILE_N, items), dim3(64 * NWAVES), lds, s, a);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

template <int C, int DT, int MB, int GMODE = 0>
int launch_codes(const CkArgs& a, hipStream_t s, int items = 1) {
  if constexpr (GMODE == 0 && MB == 1 && !ck_small<C>()) {
    if ((a.N + 31) / 32 > 256) return launch_codes_wv<C, DT, MB, GMODE, 4>(a, s, items);
  }
  return launch_codes_wv<C, DT, MB, GMODE, ck_waves<C, GMODE>()>(a, s, items);
}

template <int C>
int launch_codes_dt(const CkArgs& a, int dtype, hipStream_t s) {
  const int mb = a.M <= 1 ? 1 : a.M <= 2 ? 2 : a.M <= 4 ? 4 : 8;
#define KQ_MB(m)                                                                               \
  if (mb == m)                                                                                 \
    return dtype == KQ_F16 ? launch_codes<C, KQ_F16, m>(a, s) : launch_codes<C, KQ_BF16, m>(a, s);
  KQ_MB(1) KQ_MB(2) KQ_MB(4) KQ_MB(8)
#undef KQ_MB
  return KQ_ERR_UNSUPPORTED;
}

// ------------------------------------------------------------------ grouped kernel (batched MoE)
// Pairs sorted by expert and cut into segments of at most 32 pairs of one expert (moe_sort_kernel).  A
// workgroup multiplies a segment's gathered activation rows (the MFMA's 32 rows) by a 128-row slab of that
// expert's wire: 4 waves x 32 weight rows, one 256-weight step at a time, wire bytes and activations
// fetched one step ahead and parked in LDS.  GLU: the slab is 64 gate rows + the same 64 up rows (waves
// 0 / 2 gate, 1 / 3 up); the up waves hand their sums to the gate waves through LDS and the epilogue runs
// before the single rounding.  Same code extraction and block-scale-after-the-MFMA numerics as above.
struct Segment {
  int expert, start, count, pad;
};

struct CgArgs {
  const void* x;        // [rows][K], pair p reads row p / x_div
  const uint8_t* w;
  const uint8_t* w2;    // up stack (GLU) or null
  void* y;              // [P][N]
  const float* bias;    // f32 [E][N] or null
  const float* bias2;
  const int* order;     // pair ids sorted by expert
  const Segment* segs;
  const int* nseg;
  const uint8_t* grids;
  int N, K, x_div, act;
  int64_t w_expert_stride;
  float limit, alpha;
  KqOutMap om;
  // outputs of codes_prepass_kernel: per activation row and 256-wide step the f16 values in staging order (512 bytes),
  // their power-of-two scale and (codecs with a block minimum) the sums of the eight 32-wide blocks
  const uint8_t* xh;
  const float* xsc;
  const float* xsum;
};

constexpr int CG_THREADS = 256;

// Activation prepass of the grouped kernel: what every workgroup used to redo for its 32 slots at every step (bf16 ->
// f16 with an exact power-of-two scale per (row, step), staging order, block sums) is done once per row.  One
// workgroup per row; 32 threads per step, eight steps at a time.  Steps are zero-filled past K.
template <int DT, bool PAIR, bool SUMS>
__global__ __launch_bounds__(256) void codes_prepass_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ xh,
                                                            float* __restrict__ xsc, float* __restrict__ xsum, int K,
                                                            int nsteps) {
  const int row = blockIdx.x, tid = threadIdx.x, pc = tid & 31;
  for (int st = tid >> 5; st < nsteps; st += 8) {
    const int k0 = CK_STEP * st + 8 * pc;
    u32x4 v = {0, 0, 0, 0};
    if (k0 < K) v = *reinterpret_cast<const u32x4*>(x + (size_t)row * K + k0);
    float xscale = 1.f;
    _Float16 h[8];
    if constexpr (DT == KQ_BF16) {
      float amax = 0.f;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] << 16)));
        amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] & 0xffff0000u)));
      }
#pragma unroll
      for (int off = 16; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));  // the step's 32 lanes
      float inv = 1.f;
      const uint32_t eb = (__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff;
      if (eb != 0 && eb != 0xff) {
        int e = (int)eb - 127 - 14;  // the largest magnitude lands in [2^14, 2^15)
        if (e < -100) e = -100;
        xscale = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
        inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
      }
#pragma unroll
      for (int e = 0; e < 4; e++) {
        h[2 * e] = (_Float16)(__builtin_bit_cast(float, v[e] << 16) * inv);
        h[2 * e + 1] = (_Float16)(__builtin_bit_cast(float, v[e] & 0xffff0000u) * inv);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; e++) {
        h[2 * e] = __builtin_bit_cast(_Float16, (uint16_t)(v[e] & 0xffff));
        h[2 * e + 1] = __builtin_bit_cast(_Float16, (uint16_t)(v[e] >> 16));
      }
    }
    const size_t rs = (size_t)row * nsteps + st;
    stage_group<PAIR>(xh + rs * 512, pc, h);
    if (pc == 0) xsc[rs] = xscale;
    if constexpr (SUMS) {
      float sum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) sum += (float)h[e];
      sum += __shfl_xor(sum, 1);
      sum += __shfl_xor(sum, 2);  // 4 lanes = one 32-weight block
      if ((pc & 3) == 0) xsum[rs * 8 + (pc >> 2)] = sum;
    }
  }
}

constexpr int CG_BN = 128;

template <int C>
constexpr int grouped_lds_bytes() {
  return 32 * XA_STRIDE + 32 * 4 + 8 * 32 * 4 + CG_BN * CodeGeom<C>::LROW + 32 * 4 + CodeGeom<C>::GROUPED_GRID_BYTES +
         CodeGeom<C>::SPREAD_BYTES;
}

template <int C, int DT, bool GLU>
__global__ __launch_bounds__(CG_THREADS, 2) void codes_grouped_kernel(CgArgs a) {
  using G = CodeGeom<C>;
  constexpr int WPT = (CG_BN * G::PIECES + CG_THREADS - 1) / CG_THREADS;
  constexpr int NCOLS = GLU ? CG_BN / 2 : CG_BN;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* a_lds = smem;                                                  // [32][XA_STRIDE] f16 activations of the step
  float* xs_lds = reinterpret_cast<float*>(a_lds + 32 * XA_STRIDE);       // [32] activation scale per slot
  float* xsum_lds = xs_lds + 32;                                          // [8 blocks][32 slots] (HAS_MIN)
  uint8_t* b_lds = reinterpret_cast<uint8_t*>(xsum_lds + 8 * 32);         // [128][LROW]
  int* pair_lds = reinterpret_cast<int*>(b_lds + CG_BN * G::LROW);        // [32] output row per slot, -1 = none
  uint8_t* grid_lds = reinterpret_cast<uint8_t*>(pair_lds + 32);
  uint8_t* spread_lds = grid_lds + G::GROUPED_GRID_BYTES;

  if ((int)blockIdx.y >= *a.nseg) return;  // uniform: the grid is sized for the worst case
  const Segment seg = a.segs[blockIdx.y];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, kg = lane >> 5;
  const int N = a.N, K = a.K;
  const int nsteps = (K + CK_STEP - 1) / CK_STEP;
  const size_t row_bytes = (size_t)(K / G::WPB) * G::BPB;
  const int n0 = blockIdx.x * NCOLS;
  const int ncols = N - n0 < NCOLS ? N - n0 : NCOLS;
  const uint8_t* wbase = a.w + (size_t)seg.expert * (size_t)a.w_expert_stride;
  const uint8_t* wbase2 = GLU ? a.w2 + (size_t)seg.expert * (size_t)a.w_expert_stride : wbase;
  const uint8_t* w_last = wbase + (size_t)N * row_bytes - 16;  // the last 16 bytes of the expert's matrix
  const uint8_t* w_last2 = wbase2 + (size_t)N * row_bytes - 16;

  // slab row rr (= wave * 32 + l32 in the compute phase) -> (matrix, column)
  auto slab_col = [&](int rr, bool& up) {
    if constexpr (GLU) {
      const int wv = rr >> 5;
      up = wv & 1;
      return (wv >> 1) * 32 + (rr & 31);
    } else {
      up = false;
      return rr;
    }
  };

  if (tid < 32) pair_lds[tid] = tid < seg.count ? a.order[seg.start + tid] : -1;

  // ---- tables
  if constexpr (G::GRID_N > 0) {
    const uint8_t* src = a.grids + G::GRID_OFF;
    if constexpr (G::GRID_W == 8) {
      for (int e = tid; e < G::GRID_N; e += CG_THREADS) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(src + 8 * e);
        f16x8 f;
        if constexpr (G::GRID_SIGNED)
          f = bytes8_to_frag(v[0] ^ 0x80808080u, v[1] ^ 0x80808080u, 128.f);
        else
          f = bytes8_to_frag(v[0], v[1], 0.f);
        *reinterpret_cast<f16x8*>(grid_lds + 16 * e) = f;
      }
    } else {
      for (int e = tid; e < G::GRID_N; e += CG_THREADS) {
        const uint32_t v = *reinterpret_cast<const uint32_t*>(src + 4 * e);
        uint32_t ev, od;
        bytes_to_f16(v, 0.f, ev, od);
        *reinterpret_cast<u32x2*>(grid_lds + 8 * e) = u32x2{ev, od};
      }
    }
  }
  if constexpr (G::PAIR_LUT) {
    // one entry per thread into a plain table, then eight lanes write the 128 bytes of an entry's copies: a wave
    // store covers consecutive LDS
    uint32_t* plain = reinterpret_cast<uint32_t*>(grid_lds + 32768);
    if (tid < 256) {
      const f16x2 e = C == KQ_MXFP4 ? f16x2{(_Float16)kq::kv_mxfp4(tid & 15), (_Float16)kq::kv_mxfp4(tid >> 4)}
                                    : f16x2{(_Float16)kq::kv_iq4nl(tid & 15), (_Float16)kq::kv_iq4nl(tid >> 4)};
      plain[tid] = __builtin_bit_cast(uint32_t, e);
    }
    lds_barrier();
    for (int i = tid; i < 256 * 8; i += CG_THREADS) {
      const uint32_t ev = plain[i >> 3];
      *reinterpret_cast<u32x4*>(grid_lds + 16 * i) = u32x4{ev, ev, ev, ev};
    }
  }
  if constexpr (G::SPREAD_BYTES > 0) {
    const uint32_t b = tid;  // 256 threads, 256 entries
    auto bit = [&](int i) { return (b >> i) & 1u; };
    constexpr int P = G::SPREAD_BIT;
    *reinterpret_cast<u32x4*>(spread_lds + 16 * tid) =
        u32x4{(bit(0) << P) | (bit(2) << (P + 16)), (bit(1) << P) | (bit(3) << (P + 16)),
              (bit(4) << P) | (bit(6) << (P + 16)), (bit(5) << P) | (bit(7) << (P + 16))};
  }
  const Tables tabs{G::PAIR_LUT ? grid_lds + 4 * (tid & 31) : grid_lds, spread_lds, 7};

  // ---- piece maps.  Activations: piece i = tid + 256 t -> (slot i / 32, 16-byte piece i % 32).
  const int a_slot0 = tid >> 5, a_pc = tid & 31;
  size_t a_rs[4];  // (row, step 0) index of the slot's activation row in the prepass outputs
  bool a_live[4];
#pragma unroll
  for (int t = 0; t < 4; t++) {
    const int slot = a_slot0 + 8 * t;
    a_live[t] = slot < seg.count;
    a_rs[t] = (size_t)(a.order[seg.start + (a_live[t] ? slot : 0)] / a.x_div) * nsteps;
  }
  const uint8_t* w_src[WPT];
  uint32_t w_loff[WPT];
  bool w_up[WPT];
#pragma unroll
  for (int t = 0; t < WPT; t++) {
    const int i = tid + CG_THREADS * t;
    const int r = i / G::PIECES, pc = i % G::PIECES;
    bool up;
    const int col = slab_col(r < CG_BN ? r : 0, up);
    const bool ok = r < CG_BN && col < ncols;  // rows past N re-read the slab's first row
    w_up[t] = up;
    w_src[t] = (up ? wbase2 : wbase) + (size_t)(n0 + (ok ? col : 0)) * row_bytes + 16 * pc;
    w_loff[t] = r < CG_BN ? (uint32_t)r * G::LROW + 16 * pc : 0xffffffffu;
  }

  u32x4 areg[4], wreg[WPT];
  float sreg[4] = {0.f, 0.f, 0.f, 0.f};  // a_pc == 0: the slot's scale; a_pc 8 .. 15 (HAS_MIN): block sum a_pc - 8
  auto issue = [&](int st) {
#pragma unroll
    for (int t = 0; t < 4; t++) {
      u32x4 av = {0, 0, 0, 0};
      float sv = 0.f;
      if (a_live[t]) {
        av = *reinterpret_cast<const u32x4*>(a.xh + (a_rs[t] + st) * 512 + 16 * a_pc);
        if (a_pc == 0) sv = a.xsc[a_rs[t] + st];
        if constexpr (G::HAS_MIN) {
          if (a_pc >= 8 && a_pc < 16) sv = a.xsum[(a_rs[t] + st) * 8 + (a_pc - 8)];
        }
      }
      areg[t] = av;
      sreg[t] = sv;
    }
#pragma unroll
    for (int t = 0; t < WPT; t++) {
      const uint8_t* p = w_src[t] + (size_t)st * G::BYTES;
      const uint8_t* last = w_up[t] ? w_last2 : w_last;
      const uint8_t* q = p <= last ? p : last;  // never read past the end of the expert's matrix
      u32x4 v = *reinterpret_cast<const u32x4_a1*>(q);
      if (q != p) v = shr_bytes(v, (uint32_t)(p - q));
      wreg[t] = v;
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const int slot = a_slot0 + 8 * t;
      *reinterpret_cast<u32x4*>(a_lds + slot * XA_STRIDE + 16 * a_pc) = areg[t];
      if (a_pc == 0) xs_lds[slot] = sreg[t];
      if constexpr (G::HAS_MIN) {
        if (a_pc >= 8 && a_pc < 16) xsum_lds[(a_pc - 8) * 32 + slot] = sreg[t];
      }
    }
#pragma unroll
    for (int t = 0; t < WPT; t++)
      if (w_loff[t] != 0xffffffffu) *reinterpret_cast<u32x4*>(b_lds + w_loff[t]) = wreg[t];
  };

  float acc[16];  // output slots 8 (i / 4) + 4 kg + i % 4 of slab row wave * 32 + l32
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = 0.f;
  const uint8_t* b_lane = b_lds + (wave * 32 + l32) * G::LROW;
  const uint8_t* a_lane = a_lds + l32 * XA_STRIDE + 16 * kg;

  issue(0);
  for (int st = 0; st < nsteps; st++) {
    lds_barrier();  // tables built / everyone is done reading the previous step
    park();
    if (st + 1 < nsteps) issue(st + 1);
    lds_barrier();
    const int kvalid = K - CK_STEP * st;
    float sacc[16];
#pragma unroll
    for (int i = 0; i < 16; i++) sacc[i] = 0.f;
    constexpr int MPS = G::SB / 16;
    auto run_step = [&](auto full_c) {
      constexpr bool FULL = decltype(full_c)::value;
      f32x16 part[2];
      RowRegs<4 * G::PIECES> row;
      StaticFor<G::PIECES>::run([&](auto pc) {
        constexpr int P = decltype(pc)::value;
        const u32x4 v = *reinterpret_cast<const u32x4*>(b_lane + 16 * P);
        row.d[4 * P] = v[0];
        row.d[4 * P + 1] = v[1];
        row.d[4 * P + 2] = v[2];
        row.d[4 * P + 3] = v[3];
      });
      StaticFor<16>::run([&](auto jc) {
        constexpr int J = decltype(jc)::value;
        if (FULL || 16 * J < kvalid) {  // uniform
          const f16x8 bv = codes<C, J>(row, kg, tabs);
          const f16x8 av = *reinterpret_cast<const f16x8*>(a_lane + 32 * J);
          constexpr int sbi = J / MPS, slot = sbi & 1;
          if constexpr (J % MPS == 0)
            part[slot] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, f32x16{0}, 0, 0, 0);
          else
            part[slot] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, part[slot], 0, 0, 0);
          if constexpr (J % MPS == MPS - 1) {
            float mn;
            const float sc = block_scale<C, sbi>(row, mn);
#pragma unroll
            for (int i = 0; i < 16; i++) sacc[i] = fmaf(sc, part[slot][i], sacc[i]);
            if constexpr (G::HAS_MIN) {
#pragma unroll
              for (int q = 0; q < 4; q++) {
                const float4 xm = *reinterpret_cast<const float4*>(xsum_lds + sbi * 32 + 8 * q + 4 * kg);
                sacc[4 * q + 0] = fmaf(mn, xm.x, sacc[4 * q + 0]);
                sacc[4 * q + 1] = fmaf(mn, xm.y, sacc[4 * q + 1]);
                sacc[4 * q + 2] = fmaf(mn, xm.z, sacc[4 * q + 2]);
                sacc[4 * q + 3] = fmaf(mn, xm.w, sacc[4 * q + 3]);
              }
            }
          }
        }
      });
    };
    if (kvalid >= CK_STEP)
      run_step(std::true_type{});
    else
      run_step(std::false_type{});
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const float4 xs4 = *reinterpret_cast<const float4*>(xs_lds + 8 * q + 4 * kg);
      acc[4 * q + 0] = fmaf(xs4.x, sacc[4 * q + 0], acc[4 * q + 0]);
      acc[4 * q + 1] = fmaf(xs4.y, sacc[4 * q + 1], acc[4 * q + 1]);
      acc[4 * q + 2] = fmaf(xs4.z, sacc[4 * q + 2], acc[4 * q + 2]);
      acc[4 * q + 3] = fmaf(xs4.w, sacc[4 * q + 3], acc[4 * q + 3]);
    }
  }

  // ---- epilogue
  if constexpr (!GLU) {
    const int col = wave * 32 + l32;
    const float bv = (a.bias && col < ncols) ? a.bias[(size_t)seg.expert * N + n0 + col] : 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int pr = pair_lds[8 * (i >> 2) + 4 * kg + (i & 3)];
      if (pr >= 0 && col < ncols)
        kq::store_result<DT>(a.y, a.om, (size_t)kq::out_row(a.om, pr) * N + n0 + col, acc[i] + bv);
    }
  } else {
    lds_barrier();  // the step buffers are free: reuse them for the up sums
    float* ex = reinterpret_cast<float*>(smem);  // [2 column blocks][16][64]
    const int nb = wave >> 1;
    if (wave & 1) {
#pragma unroll
      for (int i = 0; i < 16; i++) ex[(nb * 16 + i) * 64 + lane] = acc[i];
    }
    lds_barrier();
    if (!(wave & 1)) {
      const int col = nb * 32 + l32;
      const bool live = col < ncols;
      const float gb = (a.bias && live) ? a.bias[(size_t)seg.expert * N + n0 + col] : 0.f;
      const float ub = (a.bias2 && live) ? a.bias2[(size_t)seg.expert * N + n0 + col] : 0.f;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int pr = pair_lds[8 * (i >> 2) + 4 * kg + (i & 3)];
        if (pr >= 0 && live) {
          const float v = kq::glu_epilogue_fast(a.act, acc[i] + gb, ex[(nb * 16 + i) * 64 + lane] + ub, a.limit, a.alpha);
          kq::store_result<DT>(a.y, a.om, (size_t)kq::out_row(a.om, pr) * N + n0 + col, v);
        }
      }
    }
  }
}

template <int C, int DT, bool GLU>
int launch_grouped(const CgArgs& a, int P, int E, hipStream_t s) {
  constexpr int NCOLS = GLU ? CG_BN / 2 : CG_BN;
  int maxseg = E + P / 32;  // sum over experts of ceil(c_e / 32) <= E + P / 32
  if (maxseg > P) maxseg = P;
  const size_t lds = grouped_lds_bytes<C>();
  auto kern = codes_grouped_kernel<C, DT, GLU>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  hipLaunchKernelGGL(kern, dim3((a.N + NCOLS - 1) / NCOLS, maxseg), dim3(CG_THREADS), lds, s, a);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

template <int C>
int launch_grouped_any(const CgArgs& a, int P, int E, int glu, int dtype, hipStream_t s) {
  if (glu) return dtype == KQ_F16 ? launch_grouped<C, KQ_F16, true>(a, P, E, s) : launch_grouped<C, KQ_BF16, true>(a, P, E, s);
  return dtype == KQ_F16 ? launch_grouped<C, KQ_F16, false>(a, P, E, s) : launch_grouped<C, KQ_BF16, false>(a, P, E, s);
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

// kq_moe.hip
// The three launcher groups below can be compiled into separate objects (KQ_CODES_PART = 1 dense, 2 gathered,
// 3 grouped; unset = all) so that the build instantiates their kernels in parallel.
#if !defined(KQ_CODES_PART) || KQ_CODES_PART == 3
int kq_launch_moe_sort(const uint32_t* idx, int P, int E, void* order, void* segs, void* nseg, hipStream_t s);

bool kq_codes_moe_supported(int P, int E, int N, int K, int codec) {
  // nvfp4 (a scale per 16 weights: 16 x 16 scalings per step) does not fit the register file here and
  // stays on the any-codec path
  if (codec < KQ_Q4_0 || codec >= KQ_NUM_CODECS || codec == KQ_NVFP4) return false;
  return P > 16 && E > 0 && E <= 4096 && (int64_t)E + P / 32 < 65535 && N > 0 && K > 0 && (K & 7) == 0 &&
         K % kq_geom(codec).wpb == 0;
}

// Workspace: sorted pair list, segment table, segment count, then the prepass outputs for `rows` activation rows:
// f16 steps (512 bytes each), step scales, block sums.
size_t kq_codes_moe_workspace_bytes(int P, int E, int rows, int K) {
  const size_t rs = (size_t)rows * ((K + CK_STEP - 1) / CK_STEP);
  return align256((size_t)P * 4) + align256(((size_t)E + P / 32 + 1) * sizeof(Segment)) + 256 + align256(rs * 512) +
         align256(rs * 4) + align256(rs * 32);
}

// x: [rows][K]; pair p reads row p / x_div and expert idx[p]; out [P][N].
int kq_launch_codes_moe(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* idx, const float* bias,
                        const float* bias2, void* out, int P, int E, int N, int K, int x_div, int64_t w_expert_stride,
                        int glu, int act, float limit, float alpha, int codec, int dtype, void* ws, KqOutMap om,
                        hipStream_t s) {
  if (!kq_codes_moe_supported(P, E, N, K, codec) || (reinterpret_cast<uintptr_t>(x) & 15) ||
      (reinterpret_cast<uintptr_t>(ws) & 255))
    return KQ_ERR_UNSUPPORTED;
  uint8_t* p = static_cast<uint8_t*>(ws);
  int* order = reinterpret_cast<int*>(p);
  Segment* segs = reinterpret_cast<Segment*>(p + align256((size_t)P * 4));
  int* nseg = reinterpret_cast<int*>(p + align256((size_t)P * 4) + align256(((size_t)E + P / 32 + 1) * sizeof(Segment)));
  int rc = kq_launch_moe_sort(idx, P, E, order, segs, nseg, s);
  if (rc) return rc;
  const int rows = glu ? P / (x_div < 1 ? 1 : x_div) : P, nsteps = (K + CK_STEP - 1) / CK_STEP;
  const size_t rs = (size_t)rows * nsteps;
  uint8_t* xh = reinterpret_cast<uint8_t*>(nseg) + 256;
  float* xsc = reinterpret_cast<float*>(xh + align256(rs * 512));
  float* xsum = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(xsc) + align256(rs * 4));
  {
    const bool pair = codec == KQ_IQ4_NL || codec == KQ_MXFP4, sums = codec == KQ_Q4_1 || codec == KQ_Q5_1;
    const uint16_t* xi = static_cast<const uint16_t*>(x);
#define KQ_PRE(DTV, PV, SV) \
  hipLaunchKernelGGL((codes_prepass_kernel<DTV, PV, SV>), dim3(rows), dim3(256), 0, s, xi, xh, xsc, xsum, K, nsteps)
    if (dtype == KQ_F16) {
      if (pair) KQ_PRE(KQ_F16, true, false);
      else if (sums) KQ_PRE(KQ_F16, false, true);
      else KQ_PRE(KQ_F16, false, false);
    } else {
      if (pair) KQ_PRE(KQ_BF16, true, false);
      else if (sums) KQ_PRE(KQ_BF16, false, true);
      else KQ_PRE(KQ_BF16, false, false);
    }
#undef KQ_PRE
    KQ_HIP_CHECK(hipGetLastError());
  }
  CgArgs a{};
  a.xh = xh;
  a.xsc = xsc;
  a.xsum = xsum;
  a.x = x;
  a.w = w;
  a.w2 = w2;
  a.y = out;
  a.bias = bias;
  a.bias2 = bias2;
  a.order = order;
  a.segs = segs;
  a.nseg = nseg;
  a.grids = kq_device_grids();
  if (!a.grids) return KQ_ERR_HIP;
  a.N = N;
  a.K = K;
  a.x_div = x_div < 1 ? 1 : x_div;
  a.act = act;
  a.w_expert_stride = w_expert_stride;
  a.limit = limit;
  a.alpha = alpha;
  a.om = om;
  switch (codec) {
#define KQ_CASE(c) \
  case c:          \
    return launch_grouped_any<c>(a, P, E, glu, dtype, s);
    KQ_CASE(KQ_Q4_0) KQ_CASE(KQ_Q4_1) KQ_CASE(KQ_Q5_0) KQ_CASE(KQ_Q5_1) KQ_CASE(KQ_Q8_0) KQ_CASE(KQ_IQ4_NL)
    KQ_CASE(KQ_IQ4_XS) KQ_CASE(KQ_IQ3_S) KQ_CASE(KQ_IQ3_XXS) KQ_CASE(KQ_IQ2_XXS) KQ_CASE(KQ_IQ2_XS) KQ_CASE(KQ_IQ2_S)
    KQ_CASE(KQ_IQ1_S) KQ_CASE(KQ_IQ1_M) KQ_CASE(KQ_MXFP4) KQ_CASE(KQ_NVFP4)
#undef KQ_CASE
  }
  return KQ_ERR_UNSUPPORTED;
}

#endif  // grouped

#if !defined(KQ_CODES_PART) || KQ_CODES_PART == 1
bool kq_codes_supported(int M, int N, int K, int codec) {
  if (codec < KQ_Q4_0 || codec >= KQ_NUM_CODECS) return false;  // the K-quants have their own kernels
  return M > 0 && M <= CK_MAXM && N > 0 && K > 0 && K % kq_geom(codec).wpb == 0;
}

int kq_launch_codes_skinny(const void* x, const uint8_t* w, const void* bias, void* y, int M, int N, int K, int codec,
                           int dtype, hipStream_t s) {
  if (!kq_codes_supported(M, N, K, codec) || (reinterpret_cast<uintptr_t>(x) & 15) || (K & 7)) return KQ_ERR_UNSUPPORTED;
  CkArgs a{};
  a.x = x;
  a.w = w;
  a.y = y;
  a.bias = static_cast<const uint16_t*>(bias);
  a.grids = kq_device_grids();
  if (!a.grids) return KQ_ERR_HIP;
  a.M = M;
  a.N = N;
  a.K = K;
  switch (codec) {
#define KQ_CASE(c) \
  case c:          \
    return launch_codes_dt<c>(a, dtype, s);
    KQ_CASE(KQ_Q4_0) KQ_CASE(KQ_Q4_1) KQ_CASE(KQ_Q5_0) KQ_CASE(KQ_Q5_1) KQ_CASE(KQ_Q8_0) KQ_CASE(KQ_IQ4_NL)
    KQ_CASE(KQ_IQ4_XS) KQ_CASE(KQ_IQ3_S) KQ_CASE(KQ_IQ3_XXS) KQ_CASE(KQ_IQ2_XXS) KQ_CASE(KQ_IQ2_XS) KQ_CASE(KQ_IQ2_S)
    KQ_CASE(KQ_IQ1_S) KQ_CASE(KQ_IQ1_M) KQ_CASE(KQ_MXFP4) KQ_CASE(KQ_NVFP4)
#undef KQ_CASE
  }
  return KQ_ERR_UNSUPPORTED;
}

#endif  // dense

#if !defined(KQ_CODES_PART) || KQ_CODES_PART == 2
// Gathered calls of up to a few entries (MoE decode): one activation row per entry (M = 1), the entry's expert
// matrix, optional f32 biases; glu != 0 runs gate and up stacks and the fused epilogue.
// (iq4_nl / q4_0 / mxfp4 / nvfp4 entries come here only when the streamed kernel declines them: a K that is no
// multiple of 256, more than 16 (32) superblocks.)
// (q8_0 entries are not taken here: the streamed kernel has a q8_0 unit, and where that declines - a K that is no
// multiple of 256 - the plain vector kernel measured 9.1 / 8.4 us against 12.7 / 9.0 us here for the GLU / down ops
// of 8 experts of 768 x 2048.)
bool kq_codes_gather_supported(int M, int N, int K, int codec) {
  return M == 1 && codec != KQ_Q8_0 && kq_codes_supported(M, N, K, codec);
}

int kq_launch_codes_gather(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* lhs, const uint32_t* rhs,
                           const float* bias, const float* bias2, void* out, int B, int M, int N, int K, int x_div,
                           int64_t x_batch_stride, int64_t w_expert_stride, int glu, int act, float limit, float alpha,
                           int codec, int dtype, int E, KqOutMap om, hipStream_t s) {
  if (!kq_codes_gather_supported(M, N, K, codec) || !rhs || B <= 0 || B > 65535 || (reinterpret_cast<uintptr_t>(x) & 15) ||
      (K & 7) || (x_batch_stride & 7) || (glu && !w2))
    return KQ_ERR_UNSUPPORTED;
  CkArgs a{};
  a.x = x;
  a.w = w;
  a.w2 = w2;
  a.y = out;
  a.lhs = lhs;
  a.rhs = rhs;
  a.fbias = bias;
  a.fbias2 = bias2;
  a.grids = kq_device_grids();
  if (!a.grids) return KQ_ERR_HIP;
  a.M = M;
  a.N = N;
  a.K = K;
  a.x_div = x_div < 1 ? 1 : x_div;
  a.act = act;
  a.x_item_stride = x_batch_stride;
  a.w_expert_stride = w_expert_stride;
  a.limit = limit;
  a.alpha = alpha;
  a.om = om;
  a.E = E;
  switch (codec) {
#define KQ_CASE(c)                                                                                               \
  case c:                                                                                                        \
    if (glu) return dtype == KQ_F16 ? launch_codes<c, KQ_F16, 1, 2>(a, s, B) : launch_codes<c, KQ_BF16, 1, 2>(a, s, B); \
    return dtype == KQ_F16 ? launch_codes<c, KQ_F16, 1, 1>(a, s, B) : launch_codes<c, KQ_BF16, 1, 1>(a, s, B);
    KQ_CASE(KQ_Q4_0) KQ_CASE(KQ_Q4_1) KQ_CASE(KQ_Q5_0) KQ_CASE(KQ_Q5_1) KQ_CASE(KQ_Q8_0) KQ_CASE(KQ_IQ4_NL)
    KQ_CASE(KQ_IQ4_XS) KQ_CASE(KQ_IQ3_S) KQ_CASE(KQ_IQ3_XXS) KQ_CASE(KQ_IQ2_XXS) KQ_CASE(KQ_IQ2_XS) KQ_CASE(KQ_IQ2_S)
    KQ_CASE(KQ_IQ1_S) KQ_CASE(KQ_IQ1_M) KQ_CASE(KQ_MXFP4) KQ_CASE(KQ_NVFP4)
#undef KQ_CASE
  }
  return KQ_ERR_UNSUPPORTED;
}
#endif  // gathered
