// Device-side reference decoders: kq_decode8<CODEC>() returns weights [8g, 8g+8) of one wire
// block as f32, with exactly the operation order of the reference's scalar decoders
// (src/kquant_cpu_decode.cpp:49-735), so results are bit-identical as long as the including
// translation unit is compiled with -ffp-contract=off.  These are the ground-truth device
// decoders: the dequantize kernel and the generic matmul kernels are built on them; the tuned
// MFMA kernels use their own integer-code paths and are tested against these.
#pragma once

#include "kq_common.h"

namespace kq {

__device__ __forceinline__ float h2f(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t ld16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }
__device__ __forceinline__ uint32_t ld32(const uint8_t* p) {
  return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}
__device__ __forceinline__ float ldh(const uint8_t* p) { return h2f(ld16(p)); }
// the same loads where the caller vouches for a 2-byte aligned address (A2), else byte by byte
template <bool A2>
__device__ __forceinline__ uint32_t ld16a(const uint8_t* p) {
  if constexpr (A2) return *reinterpret_cast<const uint16_t*>(p);
  else return ld16(p);
}
template <bool A2>
__device__ __forceinline__ uint32_t ld32a(const uint8_t* p) {
  if constexpr (A2) return (uint32_t) * reinterpret_cast<const uint16_t*>(p) | ((uint32_t) * reinterpret_cast<const uint16_t*>(p + 2) << 16);
  else return ld32(p);
}

// src/kquant_iq_tables.h:10
__device__ __forceinline__ float kv_iq4nl(int i) {
  // packed as bytes to stay in registers / scalar constants
  const uint64_t lo = 0xF6EADDCFBFAD9881ull;  // -127,-104,-83,-65,-49,-35,-22,-10
  const uint64_t hi = 0x7159453526190D01ull;  // 1,13,25,38,53,69,89,113
  uint64_t v = (i & 8) ? hi : lo;
  return (float)(int8_t)(v >> (8 * (i & 7)));
}
// src/kquant_fp_tables.h:16 (2x OCP E2M1)
__device__ __forceinline__ float kv_mxfp4(int i) {
  const uint64_t mag = 0x0C08060403020100ull;  // 0,1,2,3,4,6,8,12
  int m = (int)((mag >> (8 * (i & 7))) & 0xff);
  return (float)((i & 8) ? -m : m);
}
// src/kquant_iq_tables.h:1458: 7-bit index -> 8 sign bits, bit 7 = parity
__device__ __forceinline__ uint32_t ksigns(uint32_t i) {
  i &= 127u;
  return i | ((uint32_t)(__builtin_popcount(i) & 1) << 7);
}
// src/kquant_fp_tables.h:21-27
__device__ __forceinline__ float e8m0_half(uint32_t e) {
  uint32_t bits = e < 2 ? (0x00200000u << e) : ((e - 1) << 23);
  return __builtin_bit_cast(float, bits);
}
// src/kquant_fp_tables.h:32-41 (all steps exact power-of-two scalings)
__device__ __forceinline__ float ue4m3_half(uint32_t x) {
  if (x == 0 || x == 0x7f) return 0.0f;
  int ex = (x >> 3) & 15;
  float man = (float)(x & 7);
  float raw = ex == 0 ? man * 0x1p-9f : ldexpf(1.0f + man * 0.125f, ex - 7);
  return raw * 0.5f;
}
__device__ __forceinline__ float sgn(uint32_t signs, int j) { return (signs >> j) & 1 ? -1.f : 1.f; }

// 6-bit (scale, min) pair j of a q4_k / q5_k block (src/kquant_cpu_decode.cpp:155-174)
__device__ __forceinline__ void q4k_scale_min(const uint8_t* s, int j, int& sc, int& mn) {
  if (j < 4) {
    sc = s[j] & 63;
    mn = s[j + 4] & 63;
  } else {
    sc = (s[j + 4] & 15) | ((s[j - 4] >> 6) << 4);
    mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
  }
}

// A codebook entry read as whole words (the codebook blob is 16-byte aligned wherever it lies, its tables start on
// multiples of 1024 and their entries are 4 or 8 bytes long) and byte j of it.
__device__ __forceinline__ uint32_t grid4(const uint8_t* p) { return *reinterpret_cast<const uint32_t*>(p); }
__device__ __forceinline__ uint2 grid8(const uint8_t* p) { return *reinterpret_cast<const uint2*>(p); }
__device__ __forceinline__ uint32_t byte_of(uint32_t w, int j) { return (w >> (8 * j)) & 0xffu; }
__device__ __forceinline__ uint32_t byte_of(uint2 w, int j) { return byte_of(j < 4 ? w.x : w.y, j & 3); }

// The codecs whose groups of 8 weights are a codebook entry of 8 magnitudes, 8 sign bits and a scale.
__host__ __device__ constexpr bool is_sign_grid_codec(int c) {
  return c == KQ_IQ3_XXS || c == KQ_IQ3_S || c == KQ_IQ2_XXS || c == KQ_IQ2_XS || c == KQ_IQ2_S;
}

// Group g (weights 8 g .. 8 g + 7) of a block of such a codec: the magnitudes are the bytes of lo (weights 0-3) and hi
// (4-7), bit j of s is the sign of weight j, db the scale in the reference's order of operations; UNIT takes the
// superblock scale d as 1 (the caller applies d; db times a magnitude is then an integer multiple of 1/8 below 512,
// i.e. an f16 number), A2 vouches for a 2-byte aligned block.
template <int C, bool UNIT, bool A2 = false>
__device__ __forceinline__ void iq_group(const uint8_t* __restrict__ b, int g, const uint8_t* __restrict__ grids,
                                         uint32_t& lo, uint32_t& hi, uint32_t& s, float& db) {
  const float d = UNIT ? 1.0f : ldh(b);
  const int ib = g >> 2, l = g & 3;
  if constexpr (C == KQ_IQ3_XXS) {  // :467-500
    const uint32_t aux = ld32a<A2>(b + 66 + 4 * ib);
    db = d * (0.5f + (float)(aux >> 28)) * 0.5f;
    s = ksigns(aux >> (7 * l));
    const uint32_t two = ld16a<A2>(b + 2 + 8 * ib + 2 * l);
    lo = grid4(grids + KQ_GRID_IQ3XXS + 4 * (two & 255u));
    hi = grid4(grids + KQ_GRID_IQ3XXS + 4 * (two >> 8));
  } else if constexpr (C == KQ_IQ3_S) {  // :502-551
    const int nib = (ib & 1) ? (b[106 + (ib >> 1)] >> 4) : (b[106 + (ib >> 1)] & 15);
    db = d * (float)(1 + 2 * nib);
    const uint32_t h = b[66 + ib];
    const uint32_t two = ld16a<A2>(b + 2 + 8 * ib + 2 * l);
    const uint32_t i1 = (two & 255u) | ((h << (8 - 2 * l)) & 256u);
    const uint32_t i2 = (two >> 8) | ((h << (7 - 2 * l)) & 256u);
    s = b[74 + 4 * ib + l];
    lo = grid4(grids + KQ_GRID_IQ3S + 4 * i1);
    hi = grid4(grids + KQ_GRID_IQ3S + 4 * i2);
  } else if constexpr (C == KQ_IQ2_XXS) {  // :556-584
    const uint32_t a1 = ld32a<A2>(b + 2 + 8 * ib + 4);
    db = d * (0.5f + (float)(a1 >> 28)) * 0.25f;
    const uint2 gr = grid8(grids + KQ_GRID_IQ2XXS + 8 * b[2 + 8 * ib + l]);
    s = ksigns(a1 >> (7 * l));
    lo = gr.x;
    hi = gr.y;
  } else if constexpr (C == KQ_IQ2_XS) {  // :586-617
    const uint32_t scb = b[66 + ib];
    db = d * (0.5f + (float)((l < 2) ? (scb & 15) : (scb >> 4))) * 0.25f;
    const uint32_t q = ld16a<A2>(b + 2 + 2 * (4 * ib + l));
    const uint2 gr = grid8(grids + KQ_GRID_IQ2XS + 8 * (q & 511u));
    s = ksigns(q >> 9);
    lo = gr.x;
    hi = gr.y;
  } else {  // iq2_s :619-650
    static_assert(C == KQ_IQ2_S, "not a sign-and-grid codec");
    const uint32_t scb = b[74 + ib];
    db = d * (0.5f + (float)((l < 2) ? (scb & 15) : (scb >> 4))) * 0.25f;
    const uint32_t gi = b[2 + 4 * ib + l] | (((uint32_t)b[66 + ib] << (8 - 2 * l)) & 0x300u);
    const uint2 gr = grid8(grids + KQ_GRID_IQ2S + 8 * gi);
    s = b[34 + 4 * ib + l];
    lo = gr.x;
    hi = gr.y;
  }
}

// Group g of a block of the ternary codecs iq1_s / iq1_m: the codebook entry's 8 signed bytes (-1, 0, 1) in lo and hi,
// the group's scale dl and its shift delta = +-1/8: weight j = dl * (entry[j] + delta).  A2 as above.
template <int C, bool UNIT, bool A2 = false>
__device__ __forceinline__ void iq1_group(const uint8_t* __restrict__ b, int g, const uint8_t* __restrict__ grids,
                                          uint32_t& lo, uint32_t& hi, float& dl, float& delta) {
  const int ib = g >> 2, l = g & 3;
  uint2 gr;
  if constexpr (C == KQ_IQ1_S) {  // :658-685
    const float d = UNIT ? 1.0f : ldh(b);
    const uint32_t qh = ld16a<A2>(b + 34 + 2 * ib);
    dl = d * (float)(2 * (int)((qh >> 12) & 7) + 1);
    delta = (qh & 0x8000u) ? -0.125f : 0.125f;
    gr = grid8(grids + KQ_GRID_IQ1S + 8 * (b[2 + 4 * ib + l] | (((qh >> (3 * l)) & 7) << 8)));
  } else {  // iq1_m :687-735
    static_assert(C == KQ_IQ1_M, "not a ternary codec");
    float d = 1.0f;
    if constexpr (!UNIT) {
      const uint32_t s0 = ld16(b + 48), s1 = ld16(b + 50), s2 = ld16(b + 52), s3 = ld16(b + 54);
      d = h2f((uint16_t)((s0 >> 12) | ((s1 >> 8) & 0x00f0u) | ((s2 >> 4) & 0x0f00u) | (s3 & 0xf000u)));
    }
    const uint32_t scw = ld16a<A2>(b + 48 + 2 * (ib >> 1));
    const int sc3 = (scw >> (6 * (ib & 1) + 3 * (l >> 1))) & 7;
    dl = d * (float)(2 * sc3 + 1);
    const uint32_t hb = b[32 + 2 * ib + (l >> 1)];
    const uint32_t nib = (l & 1) ? (hb >> 4) : (hb & 15);
    delta = (nib & 8) ? -0.125f : 0.125f;
    gr = grid8(grids + KQ_GRID_IQ1S + 8 * (b[4 * ib + l] | ((nib & 7) << 8)));
  }
  lo = gr.x;
  hi = gr.y;
}

template <int C>
__device__ __forceinline__ void decode8(const uint8_t* __restrict__ b, int g, const uint8_t* __restrict__ grids,
                                        float* __restrict__ o) {
  if constexpr (C == KQ_Q8_0) {  // :49-63
    float d = ldh(b);
    for (int t = 0; t < 8; t++) o[t] = d * (float)(int8_t)b[2 + 8 * g + t];
  } else if constexpr (C == KQ_Q4_0) {  // :65-82
    float d = ldh(b);
    const uint8_t* q = b + 2 + 8 * (g & 1);
    for (int t = 0; t < 8; t++) o[t] = d * (float)((int)((g < 2) ? (q[t] & 15) : (q[t] >> 4)) - 8);
  } else if constexpr (C == KQ_Q4_1) {  // :84-102
    float d = ldh(b), m = ldh(b + 2);
    const uint8_t* q = b + 4 + 8 * (g & 1);
    for (int t = 0; t < 8; t++) o[t] = d * (float)((g < 2) ? (q[t] & 15) : (q[t] >> 4)) + m;
  } else if constexpr (C == KQ_Q5_0) {  // :104-128
    float d = ldh(b);
    uint32_t qh = ld32(b + 2);
    const uint8_t* q = b + 6 + 8 * (g & 1);
    for (int t = 0; t < 8; t++) {
      int hb = (qh >> (8 * g + t)) & 1;
      int v = (int)((g < 2) ? (q[t] & 15) : (q[t] >> 4)) | (hb << 4);
      o[t] = d * (float)(v - 16);
    }
  } else if constexpr (C == KQ_Q5_1) {  // :130-153
    float d = ldh(b), m = ldh(b + 2);
    uint32_t qh = ld32(b + 4);
    const uint8_t* q = b + 8 + 8 * (g & 1);
    for (int t = 0; t < 8; t++) {
      int hb = (qh >> (8 * g + t)) & 1;
      int v = (int)((g < 2) ? (q[t] & 15) : (q[t] >> 4)) | (hb << 4);
      o[t] = d * (float)v + m;
    }
  } else if constexpr (C == KQ_Q4_K || C == KQ_Q5_K) {  // :176-235
    float d = ldh(b), dmin = ldh(b + 2);
    int j = g >> 2, i0 = 8 * (g & 3), isc, imn;
    q4k_scale_min(b + 4, j, isc, imn);
    float sc = d * (float)isc, mn = dmin * (float)imn;
    const uint8_t* qs = b + (C == KQ_Q4_K ? 16 : 48) + 32 * (j >> 1) + i0;
    for (int t = 0; t < 8; t++) {
      int v = (j & 1) ? (qs[t] >> 4) : (qs[t] & 15);
      if constexpr (C == KQ_Q5_K) v |= ((b[16 + i0 + t] >> j) & 1) << 4;
      o[t] = sc * (float)v - mn;
    }
  } else if constexpr (C == KQ_Q6_K) {  // :237-280
    float d = ldh(b + 208);
    int w = 8 * g, h = w >> 7, r = w & 127, qd = r >> 5, l0 = r & 31;
    const uint8_t* ql = b + 64 * h + ((qd & 1) ? 32 : 0) + l0;
    const uint8_t* qh = b + 128 + 32 * h + l0;
    float dsc = d * (float)(int8_t)b[192 + (w >> 4)];
    for (int t = 0; t < 8; t++) {
      int lo = (qd & 2) ? (ql[t] >> 4) : (ql[t] & 15);
      int v = (lo | (((qh[t] >> (2 * qd)) & 3) << 4)) - 32;
      o[t] = dsc * (float)v;  // (d * sc) * q, left to right
    }
  } else if constexpr (C == KQ_Q3_K) {  // :282-337
    float d = ldh(b + 108);
    int w = 8 * g, half = w >> 7, r = w & 127, si = r >> 5, l0 = r & 31, is = w >> 4;
    const uint8_t* s = b + 96;
    int k = is & 3, grp = is >> 2, sc;  // sc[k + 4*grp]
    int lo4 = (grp & 1) ? s[k + 4] : s[k];
    lo4 = (grp & 2) ? (lo4 >> 4) : (lo4 & 15);
    sc = lo4 | (((s[8 + k] >> (2 * grp)) & 3) << 4);
    float dl = d * (float)(sc - 32);
    const uint8_t* q = b + 32 + 32 * half + l0;
    const uint8_t* hm = b + l0;
    for (int t = 0; t < 8; t++) {
      int q2 = (q[t] >> (2 * si)) & 3;
      int hh = ((hm[t] >> (4 * half + si)) & 1) ? 0 : 4;
      o[t] = dl * (float)(q2 - hh);
    }
  } else if constexpr (C == KQ_Q2_K) {  // :339-377
    float d = ldh(b + 80), dmin = ldh(b + 82);
    int w = 8 * g, half = w >> 7, r = w & 127, si = r >> 5, l0 = r & 31;
    uint8_t sb = b[w >> 4];
    float dl = d * (float)(sb & 15), ml = dmin * (float)(sb >> 4);
    const uint8_t* q = b + 16 + 32 * half + l0;
    for (int t = 0; t < 8; t++) o[t] = dl * (float)((q[t] >> (2 * si)) & 3) - ml;
  } else if constexpr (C == KQ_IQ4_NL) {  // :382-397
    float d = ldh(b);
    const uint8_t* q = b + 2 + 8 * (g & 1);
    for (int t = 0; t < 8; t++) o[t] = d * kv_iq4nl((g < 2) ? (q[t] & 15) : (q[t] >> 4));
  } else if constexpr (C == KQ_MXFP4) {  // :403-418
    float d = e8m0_half(b[0]);
    const uint8_t* q = b + 1 + 8 * (g & 1);
    for (int t = 0; t < 8; t++) o[t] = d * kv_mxfp4((g < 2) ? (q[t] & 15) : (q[t] >> 4));
  } else if constexpr (C == KQ_NVFP4) {  // :420-438
    int grp = g >> 1;
    float d = ue4m3_half(b[grp]);
    const uint8_t* q = b + 4 + 8 * grp;
    for (int t = 0; t < 8; t++) o[t] = d * kv_mxfp4((g & 1) ? (q[t] >> 4) : (q[t] & 15));
  } else if constexpr (C == KQ_IQ4_XS) {  // :440-465
    float d = ldh(b);
    uint32_t sh = ld16(b + 2);
    int ib = g >> 2, r = g & 3;
    int ls = ((b[4 + (ib >> 1)] >> (4 * (ib & 1))) & 15) | (int)(((sh >> (2 * ib)) & 3) << 4);
    float dl = d * (float)(ls - 32);
    const uint8_t* q = b + 8 + 16 * ib + 8 * (r & 1);
    for (int t = 0; t < 8; t++) o[t] = dl * kv_iq4nl((r < 2) ? (q[t] & 15) : (q[t] >> 4));
  } else if constexpr (is_sign_grid_codec(C)) {  // iq3_xxs, iq3_s, iq2_xxs, iq2_xs, iq2_s
    uint32_t lo, hi, s;
    float db;
    iq_group<C, false>(b, g, grids, lo, hi, s, db);
    for (int j = 0; j < 4; j++) {
      o[j] = db * (float)byte_of(lo, j) * sgn(s, j);
      o[j + 4] = db * (float)byte_of(hi, j) * sgn(s, j + 4);
    }
  } else if constexpr (C == KQ_IQ1_S || C == KQ_IQ1_M) {
    uint32_t lo, hi;
    float dl, delta;
    iq1_group<C, false>(b, g, grids, lo, hi, dl, delta);
    for (int j = 0; j < 4; j++) {
      o[j] = dl * ((float)(int8_t)byte_of(lo, j) + delta);
      o[j + 4] = dl * ((float)(int8_t)byte_of(hi, j) + delta);
    }
  }
}

// superblock scale d of an IQ block (iq1_m keeps it in the top nibbles of its four scale words)
template <int C>
__device__ __forceinline__ float iq_block_d(const uint8_t* __restrict__ b) {
  if constexpr (C == KQ_IQ1_M) {
    const uint32_t s0 = ld16(b + 48), s1 = ld16(b + 50), s2 = ld16(b + 52), s3 = ld16(b + 54);
    return h2f((uint16_t)((s0 >> 12) | ((s1 >> 8) & 0x00f0u) | ((s2 >> 4) & 0x0f00u) | (s3 & 0xf000u)));
  } else {
    return ldh(b);
  }
}

// f32 -> storage dtype, one round-to-nearest-even
__device__ __forceinline__ uint16_t f2bf16(float f) {
  uint32_t x = __builtin_bit_cast(uint32_t, f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}
__device__ __forceinline__ uint16_t f2f16(float f) {
  // Keep the f32 value in a register of its own: otherwise the compiler may fold the producing
  // multiply into a mixed-precision fma with a +0 addend, which turns -0.0 into +0.0.
  asm volatile("" : "+v"(f));
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}
__device__ __forceinline__ float bf162f(uint16_t h) { return __builtin_bit_cast(float, (uint32_t)h << 16); }

}  // namespace kq
