/*
 * kq_oracle.c -- CPU restatement of the reference's scalar `eval_cpu` path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are compared
 * against (and the "port" CPU baseline timed next to them).  Nothing in the shipped
 * library or its Python front end may link, import or call it.
 *
 * Every function cites the reference file:line whose arithmetic (operation order
 * included -- f32 results must be bit-identical) it restates.  Built with
 * -ffp-contract=off so no multiply/add pair is ever fused.
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   block decoders  : pinned by hand-built known-answer blocks, brute-force closed
 *                     forms for the 32-weight codecs, an independent numpy decoder
 *                     for the K-quants, and the reference's own wire fixtures
 *                     (round-trip error against the regenerated pre-image).
 *   half rounding   : pinned against numpy's IEEE float16 conversion (all 2^16
 *                     patterns + random f32) and a closed-form bf16 RNE.
 *   qmm / gather    : pinned against numpy float64 `x @ deq(W).T`.
 *   GLU epilogue    : pinned against the numpy formulas the reference tests use.
 *   shexp / mix ops : compositions of the pinned matvec and epilogue; checked against the numpy
 *                     compositions of the reference's tests (tests/test_moe_glu.py:234-310).
 *   router top-k    : pinned against the numpy formulas of the reference's router test
 *                     (tests/test_moe_glu.py:453-551: softmax / sqrt-softplus, stable argsort, renorm).
 */
#include "kq_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ tables */

/* The IQ codebooks are opaque ggml constants; they live in a binary data file that
 * is linked in with .incbin (path given by -DKQ_GRID_BLOB=...). Layout, little
 * endian: iq2xxs u64[256] | iq2xs u64[512] | iq2s u64[1024] | iq1s u64[2048] |
 * iq3xxs u32[256] | iq3s u32[512]. */
__asm__(".section .rodata\n"
        ".balign 16\n"
        "kq_oracle_grid_blob:\n"
        ".incbin \"" KQ_GRID_BLOB "\"\n"
        ".previous\n");
extern const uint8_t kq_oracle_grid_blob[];

#define GRID_IQ2XXS (kq_oracle_grid_blob + 0)
#define GRID_IQ2XS (kq_oracle_grid_blob + 2048)
#define GRID_IQ2S (kq_oracle_grid_blob + 6144)
#define GRID_IQ1S (kq_oracle_grid_blob + 14336)
#define GRID_IQ3XXS (kq_oracle_grid_blob + 30720)
#define GRID_IQ3S (kq_oracle_grid_blob + 31744)

/* src/kquant_iq_tables.h:10 */
static const int8_t KV_IQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10,
                                    1,    13,   25,  38,  53,  69,  89,  113};
/* src/kquant_fp_tables.h:16 (2x OCP E2M1) */
static const int8_t KV_MXFP4[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};

/* src/kquant_iq_tables.h:1458 -- entry i is i with bit 7 set to make the popcount even. */
static inline uint8_t ksigns(uint32_t i) {
  i &= 127u;
  return (uint8_t)(i | ((uint32_t)(__builtin_popcount(i) & 1) << 7));
}

/* ---------------------------------------------------- half-precision casts */

float kq_oracle_f16_to_f32(uint16_t h) {
  /* src/kquant_cpu_decode.cpp:43-47 (`_Float16` -> float, exact). */
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        e++;
      } while (!(man & 0x400u));
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t kq_oracle_f32_to_f16(float f) {
  /* IEEE round-to-nearest-even, the conversion `static_cast<float16_t>(float)` performs
   * at src/kquant_cpu_decode.cpp:60,194,1128. */
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0));
  }
  if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x33000001u) { /* < 2^-25 (or == 2^-25 tie -> even = 0) */
    return (uint16_t)sign;
  }
  int e = (int)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u;
  int shift = (e < -14) ? (13 + (-14 - e)) : 13; /* bits dropped from the 24-bit significand */
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) q++;
  uint32_t out;
  if (e < -14) {
    out = q; /* subnormal (q may carry into the smallest normal: bit pattern is still right) */
  } else {
    out = ((uint32_t)(e + 15) << 10) + (q - 0x400u); /* carry in q bumps the exponent */
  }
  return (uint16_t)(sign | out);
}

float kq_oracle_bf16_to_f32(uint16_t h) {
  uint32_t bits = (uint32_t)h << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t kq_oracle_f32_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

static inline float rd_f16(const uint8_t* p) {
  uint16_t h = (uint16_t)(p[0] | (p[1] << 8));
  return kq_oracle_f16_to_f32(h);
}
static inline uint16_t rd_u16(const uint8_t* p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static inline uint32_t rd_u32(const uint8_t* p) {
  return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

/* ---------------------------------------------------------- codec registry */

/* src/kquant_codec.cpp:12-37 */
static const kq_oracle_codec_t CODECS[KQ_ORACLE_NUM_CODECS] = {
    {"q2_k", 256, 84, 2, 1, 1, 1, 0},    {"q3_k", 256, 110, 3, 1, 1, 1, 0},
    {"q4_k", 256, 144, 4, 1, 1, 1, 0},   {"q5_k", 256, 176, 5, 1, 1, 1, 0},
    {"q6_k", 256, 210, 6, 1, 1, 1, 0},   {"q4_0", 32, 18, 4, 1, 1, 1, 0},
    {"q4_1", 32, 20, 4, 1, 1, 1, 0},     {"q5_0", 32, 22, 5, 1, 1, 1, 0},
    {"q5_1", 32, 24, 5, 1, 1, 1, 0},     {"q8_0", 32, 34, 8, 1, 1, 1, 0},
    {"iq4_nl", 32, 18, 4, 1, 1, 1, 0},   {"iq4_xs", 256, 136, 4, 1, 1, 1, 0},
    {"iq3_s", 256, 110, 3, 1, 1, 1, 0},  {"iq3_xxs", 256, 98, 3, 1, 1, 1, 0},
    {"iq2_xxs", 256, 66, 2, 1, 1, 1, 1}, {"iq2_xs", 256, 74, 2, 1, 1, 1, 1},
    {"iq2_s", 256, 82, 2, 1, 1, 1, 0},   {"iq1_s", 256, 50, 1, 1, 1, 1, 1},
    {"iq1_m", 256, 56, 1, 1, 1, 1, 0},   {"mxfp4", 32, 17, 4, 1, 0, 0, 0},
    {"nvfp4", 64, 36, 4, 1, 0, 0, 0},
};

enum {
  C_Q2_K, C_Q3_K, C_Q4_K, C_Q5_K, C_Q6_K, C_Q4_0, C_Q4_1, C_Q5_0, C_Q5_1, C_Q8_0, C_IQ4_NL,
  C_IQ4_XS, C_IQ3_S, C_IQ3_XXS, C_IQ2_XXS, C_IQ2_XS, C_IQ2_S, C_IQ1_S, C_IQ1_M, C_MXFP4, C_NVFP4
};

int kq_oracle_codec_id(const char* name) {
  /* src/kquant_codec.cpp:39-46 */
  for (int i = 0; i < KQ_ORACLE_NUM_CODECS; i++)
    if (strcmp(CODECS[i].name, name) == 0) return i;
  return -1;
}
const kq_oracle_codec_t* kq_oracle_codec(int id) {
  return (id >= 0 && id < KQ_ORACLE_NUM_CODECS) ? &CODECS[id] : NULL;
}

/* ------------------------------------------------------ per-block decoders */
/* Each decodes ONE block to f32.  Operation order follows the cited lines. */

static void blk_q8_0(const uint8_t* b, float* o) { /* src/kquant_cpu_decode.cpp:49-63 */
  float d = rd_f16(b);
  const int8_t* q = (const int8_t*)(b + 2);
  for (int i = 0; i < 32; i++) o[i] = d * (float)q[i];
}
static void blk_q4_0(const uint8_t* b, float* o) { /* :65-82 */
  float d = rd_f16(b);
  for (int j = 0; j < 16; j++) {
    o[j] = d * (float)((b[2 + j] & 15) - 8);
    o[j + 16] = d * (float)((b[2 + j] >> 4) - 8);
  }
}
static void blk_q4_1(const uint8_t* b, float* o) { /* :84-102 */
  float d = rd_f16(b), m = rd_f16(b + 2);
  for (int j = 0; j < 16; j++) {
    o[j] = d * (float)(b[4 + j] & 15) + m;
    o[j + 16] = d * (float)(b[4 + j] >> 4) + m;
  }
}
static void blk_q5_0(const uint8_t* b, float* o) { /* :104-128 */
  float d = rd_f16(b);
  uint32_t qh = rd_u32(b + 2);
  for (int j = 0; j < 16; j++) {
    int h0 = (int)(((qh >> j) << 4) & 0x10u);
    int h1 = (int)((qh >> (j + 12)) & 0x10u);
    o[j] = d * (float)(((b[6 + j] & 15) | h0) - 16);
    o[j + 16] = d * (float)(((b[6 + j] >> 4) | h1) - 16);
  }
}
static void blk_q5_1(const uint8_t* b, float* o) { /* :130-153 */
  float d = rd_f16(b), m = rd_f16(b + 2);
  uint32_t qh = rd_u32(b + 4);
  for (int j = 0; j < 16; j++) {
    int h0 = (int)(((qh >> j) << 4) & 0x10u);
    int h1 = (int)((qh >> (j + 12)) & 0x10u);
    o[j] = d * (float)((b[8 + j] & 15) | h0) + m;
    o[j + 16] = d * (float)((b[8 + j] >> 4) | h1) + m;
  }
}

/* :155-174 -- 12 packed bytes -> 8 (scale, min) pairs, pre-multiplied by d / dmin. */
static void q4k_scales(const uint8_t* s, float d, float dmin, float* sc, float* mn) {
  for (int j = 0; j < 8; j++) {
    int rs, rm;
    if (j < 4) {
      rs = s[j] & 63;
      rm = s[j + 4] & 63;
    } else {
      rs = (s[j + 4] & 15) | ((s[j - 4] >> 6) << 4);
      rm = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
    sc[j] = d * (float)rs;
    mn[j] = dmin * (float)rm;
  }
}
static void blk_q4_k(const uint8_t* b, float* o) { /* :176-202 */
  float sc[8], mn[8];
  q4k_scales(b + 4, rd_f16(b), rd_f16(b + 2), sc, mn);
  const uint8_t* qs = b + 16;
  for (int g = 0; g < 4; g++)
    for (int i = 0; i < 32; i++) {
      o[64 * g + i] = sc[2 * g] * (float)(qs[32 * g + i] & 15) - mn[2 * g];
      o[64 * g + 32 + i] = sc[2 * g + 1] * (float)(qs[32 * g + i] >> 4) - mn[2 * g + 1];
    }
}
static void blk_q5_k(const uint8_t* b, float* o) { /* :204-235 */
  float sc[8], mn[8];
  q4k_scales(b + 4, rd_f16(b), rd_f16(b + 2), sc, mn);
  const uint8_t* qh = b + 16;
  const uint8_t* qs = b + 48;
  for (int g = 0; g < 4; g++)
    for (int i = 0; i < 32; i++) {
      int lo = (qs[32 * g + i] & 15) | (((qh[i] >> (2 * g)) & 1) << 4);
      int hi = (qs[32 * g + i] >> 4) | (((qh[i] >> (2 * g + 1)) & 1) << 4);
      o[64 * g + i] = sc[2 * g] * (float)lo - mn[2 * g];
      o[64 * g + 32 + i] = sc[2 * g + 1] * (float)hi - mn[2 * g + 1];
    }
}
static void blk_q6_k(const uint8_t* b, float* o) { /* :237-280 */
  const int8_t* scales = (const int8_t*)(b + 192);
  float d = rd_f16(b + 208);
  for (int h = 0; h < 2; h++) {
    const uint8_t* ql = b + 64 * h;
    const uint8_t* qh = b + 128 + 32 * h;
    const int8_t* sc = scales + 8 * h;
    float* y = o + 128 * h;
    for (int l = 0; l < 32; l++) {
      int is = l / 16;
      int8_t q1 = (int8_t)(((ql[l] & 15) | (((qh[l] >> 0) & 3) << 4)) - 32);
      int8_t q2 = (int8_t)(((ql[l + 32] & 15) | (((qh[l] >> 2) & 3) << 4)) - 32);
      int8_t q3 = (int8_t)(((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
      int8_t q4 = (int8_t)(((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
      /* left-associative: (d * sc) * q */
      y[l] = d * (float)sc[is] * (float)q1;
      y[l + 32] = d * (float)sc[is + 2] * (float)q2;
      y[l + 64] = d * (float)sc[is + 4] * (float)q3;
      y[l + 96] = d * (float)sc[is + 6] * (float)q4;
    }
  }
}
static void blk_q3_k(const uint8_t* b, float* o) { /* :282-337 */
  const uint8_t* hm = b;
  const uint8_t* qs = b + 32;
  const uint8_t* s = b + 96;
  float d = rd_f16(b + 108);
  int sc[16];
  for (int k = 0; k < 4; k++) {
    sc[k] = (s[k] & 15) | ((s[8 + k] & 3) << 4);
    sc[k + 4] = (s[k + 4] & 15) | (((s[8 + k] >> 2) & 3) << 4);
    sc[k + 8] = (s[k] >> 4) | (((s[8 + k] >> 4) & 3) << 4);
    sc[k + 12] = (s[k + 4] >> 4) | (((s[8 + k] >> 6) & 3) << 4);
  }
  int idx = 0;
  for (int half = 0; half < 2; half++) {
    const uint8_t* q = qs + 32 * half;
    for (int si = 0; si < 4; si++) {
      int shift = 2 * si;
      uint8_t m = (uint8_t)(1u << (4 * half + si));
      int is = 8 * half + 2 * si;
      for (int side = 0; side < 2; side++) {
        float dl = d * (float)(sc[is + side] - 32);
        for (int l = 0; l < 16; l++) {
          int q2 = (q[l + 16 * side] >> shift) & 3;
          int h = (hm[l + 16 * side] & m) ? 0 : 4;
          o[idx++] = dl * (float)(q2 - h);
        }
      }
    }
  }
}
static void blk_q2_k(const uint8_t* b, float* o) { /* :339-377 */
  const uint8_t* scales = b;
  const uint8_t* qs = b + 16;
  float d = rd_f16(b + 80), dmin = rd_f16(b + 82);
  int idx = 0, is = 0;
  for (int half = 0; half < 2; half++) {
    const uint8_t* q = qs + 32 * half;
    for (int si = 0; si < 4; si++) {
      int shift = 2 * si;
      for (int side = 0; side < 2; side++) {
        uint8_t sb = scales[is++];
        float dl = d * (float)(sb & 15);
        float ml = dmin * (float)(sb >> 4);
        for (int l = 0; l < 16; l++) o[idx++] = dl * (float)((q[l + 16 * side] >> shift) & 3) - ml;
      }
    }
  }
}
static void blk_iq4_nl(const uint8_t* b, float* o) { /* :382-397 */
  float d = rd_f16(b);
  for (int j = 0; j < 16; j++) {
    o[j] = d * (float)KV_IQ4NL[b[2 + j] & 15];
    o[j + 16] = d * (float)KV_IQ4NL[b[2 + j] >> 4];
  }
}
/* src/kquant_fp_tables.h:21-27 */
static float e8m0_half(uint8_t e) {
  uint32_t bits = e < 2 ? (0x00200000u << e) : ((uint32_t)(e - 1) << 23);
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
/* src/kquant_fp_tables.h:32-41 */
static float ue4m3_half(uint8_t x) {
  if (x == 0 || x == 0x7f) return 0.0f;
  int ex = (x >> 3) & 15;
  float man = (float)(x & 7);
  float raw = ex == 0 ? man * 0x1p-9f : ldexpf(1.0f + man * 0.125f, ex - 7);
  return raw * 0.5f;
}
static void blk_mxfp4(const uint8_t* b, float* o) { /* src/kquant_cpu_decode.cpp:403-418 */
  float d = e8m0_half(b[0]);
  for (int j = 0; j < 16; j++) {
    o[j] = d * (float)KV_MXFP4[b[1 + j] & 15];
    o[j + 16] = d * (float)KV_MXFP4[b[1 + j] >> 4];
  }
}
static void blk_nvfp4(const uint8_t* b, float* o) { /* :420-438 */
  for (int g = 0; g < 4; g++) {
    float d = ue4m3_half(b[g]);
    const uint8_t* q = b + 4 + 8 * g;
    for (int j = 0; j < 8; j++) {
      o[16 * g + j] = d * (float)KV_MXFP4[q[j] & 15];
      o[16 * g + j + 8] = d * (float)KV_MXFP4[q[j] >> 4];
    }
  }
}
static void blk_iq4_xs(const uint8_t* b, float* o) { /* :440-465 */
  float d = rd_f16(b);
  uint32_t sh = rd_u16(b + 2);
  const uint8_t* sl = b + 4;
  const uint8_t* qs = b + 8;
  for (int ib = 0; ib < 8; ib++) {
    int ls = ((sl[ib / 2] >> (4 * (ib % 2))) & 15) | (int)(((sh >> (2 * ib)) & 3) << 4);
    float dl = d * (float)(ls - 32);
    for (int j = 0; j < 16; j++) {
      o[32 * ib + j] = dl * (float)KV_IQ4NL[qs[16 * ib + j] & 15];
      o[32 * ib + j + 16] = dl * (float)KV_IQ4NL[qs[16 * ib + j] >> 4];
    }
  }
}
static inline float sgn(uint8_t signs, int j) { return (signs & (1u << j)) ? -1.f : 1.f; }

static void blk_iq3_xxs(const uint8_t* b, float* o) { /* :467-500 */
  float d = rd_f16(b);
  const uint8_t* qs = b + 2;
  const uint8_t* gas = b + 66;
  for (int ib = 0; ib < 8; ib++) {
    uint32_t aux = rd_u32(gas + 4 * ib);
    float db = d * (0.5f + (float)(aux >> 28)) * 0.5f;
    for (int l = 0; l < 4; l++) {
      uint8_t s = ksigns(aux >> (7 * l));
      const uint8_t* g1 = GRID_IQ3XXS + 4 * qs[8 * ib + 2 * l];
      const uint8_t* g2 = GRID_IQ3XXS + 4 * qs[8 * ib + 2 * l + 1];
      float* y = o + 32 * ib + 8 * l;
      for (int j = 0; j < 4; j++) {
        y[j] = db * (float)g1[j] * sgn(s, j);
        y[j + 4] = db * (float)g2[j] * sgn(s, j + 4);
      }
    }
  }
}
static void blk_iq3_s(const uint8_t* b, float* o) { /* :502-551 */
  float d = rd_f16(b);
  const uint8_t* qs = b + 2;
  const uint8_t* qh = b + 66;
  const uint8_t* signs = b + 74;
  const uint8_t* scales = b + 106;
  for (int ib = 0; ib < 8; ib++) { /* ib = 32-weight group; pairs share a scale byte */
    int nib = (ib & 1) ? (scales[ib / 2] >> 4) : (scales[ib / 2] & 15);
    float db = d * (float)(1 + 2 * nib);
    uint32_t h = qh[ib];
    for (int l = 0; l < 4; l++) {
      uint32_t i1 = qs[8 * ib + 2 * l] | ((h << (8 - 2 * l)) & 256u);
      uint32_t i2 = qs[8 * ib + 2 * l + 1] | ((h << (7 - 2 * l)) & 256u);
      const uint8_t* g1 = GRID_IQ3S + 4 * i1;
      const uint8_t* g2 = GRID_IQ3S + 4 * i2;
      uint8_t s = signs[4 * ib + l];
      float* y = o + 32 * ib + 8 * l;
      for (int j = 0; j < 4; j++) {
        y[j] = db * (float)g1[j] * sgn(s, j);
        y[j + 4] = db * (float)g2[j] * sgn(s, j + 4);
      }
    }
  }
}
static void blk_iq2_xxs(const uint8_t* b, float* o) { /* :556-584 */
  float d = rd_f16(b);
  const uint8_t* qs = b + 2;
  for (int ib = 0; ib < 8; ib++) {
    const uint8_t* a8 = qs + 8 * ib;
    uint32_t a1 = rd_u32(a8 + 4);
    float db = d * (0.5f + (float)(a1 >> 28)) * 0.25f;
    for (int l = 0; l < 4; l++) {
      const uint8_t* g = GRID_IQ2XXS + 8 * a8[l];
      uint8_t s = ksigns(a1 >> (7 * l));
      for (int j = 0; j < 8; j++) o[32 * ib + 8 * l + j] = db * (float)g[j] * sgn(s, j);
    }
  }
}
static void blk_iq2_xs(const uint8_t* b, float* o) { /* :586-617 */
  float d = rd_f16(b);
  const uint8_t* qs = b + 2;
  const uint8_t* scales = b + 66;
  for (int ib = 0; ib < 8; ib++) {
    float db[2];
    db[0] = d * (0.5f + (float)(scales[ib] & 15)) * 0.25f;
    db[1] = d * (0.5f + (float)(scales[ib] >> 4)) * 0.25f;
    for (int l = 0; l < 4; l++) {
      uint32_t q = rd_u16(qs + 2 * (4 * ib + l));
      const uint8_t* g = GRID_IQ2XS + 8 * (q & 511u);
      uint8_t s = ksigns(q >> 9);
      float dl = db[l / 2];
      for (int j = 0; j < 8; j++) o[32 * ib + 8 * l + j] = dl * (float)g[j] * sgn(s, j);
    }
  }
}
static void blk_iq2_s(const uint8_t* b, float* o) { /* :619-650 */
  float d = rd_f16(b);
  const uint8_t* qs = b + 2;
  const uint8_t* signs = b + 34;
  const uint8_t* qh = b + 66;
  const uint8_t* scales = b + 74;
  for (int ib = 0; ib < 8; ib++) {
    float db[2];
    db[0] = d * (0.5f + (float)(scales[ib] & 15)) * 0.25f;
    db[1] = d * (0.5f + (float)(scales[ib] >> 4)) * 0.25f;
    for (int l = 0; l < 4; l++) {
      float dl = db[l / 2];
      uint32_t gi = qs[4 * ib + l] | (((uint32_t)qh[ib] << (8 - 2 * l)) & 0x300u);
      const uint8_t* g = GRID_IQ2S + 8 * gi;
      uint8_t s = signs[4 * ib + l];
      for (int j = 0; j < 8; j++) o[32 * ib + 8 * l + j] = dl * (float)g[j] * sgn(s, j);
    }
  }
}
static void blk_iq1_s(const uint8_t* b, float* o) { /* :658-685 */
  float d = rd_f16(b);
  const uint8_t* qs = b + 2;
  for (int ib = 0; ib < 8; ib++) {
    uint32_t qh = rd_u16(b + 34 + 2 * ib);
    float dl = d * (float)(2 * (int)((qh >> 12) & 7) + 1);
    float delta = (qh & 0x8000u) ? -0.125f : 0.125f;
    for (int l = 0; l < 4; l++) {
      const int8_t* g = (const int8_t*)(GRID_IQ1S + 8 * (qs[4 * ib + l] | (((qh >> (3 * l)) & 7) << 8)));
      for (int j = 0; j < 8; j++) o[32 * ib + 8 * l + j] = dl * ((float)g[j] + delta);
    }
  }
}
static void blk_iq1_m(const uint8_t* b, float* o) { /* :687-735 */
  const uint8_t* qs = b;
  const uint8_t* qh = b + 32;
  uint32_t sc[4];
  for (int i = 0; i < 4; i++) sc[i] = rd_u16(b + 48 + 2 * i);
  uint16_t du = (uint16_t)((sc[0] >> 12) | ((sc[1] >> 8) & 0x00f0u) | ((sc[2] >> 4) & 0x0f00u) |
                           (sc[3] & 0xf000u));
  float d = kq_oracle_f16_to_f32(du);
  for (int ib = 0; ib < 8; ib++) {
    float dl1 = d * (float)(2 * (int)((sc[ib / 2] >> (6 * (ib % 2) + 0)) & 7) + 1);
    float dl2 = d * (float)(2 * (int)((sc[ib / 2] >> (6 * (ib % 2) + 3)) & 7) + 1);
    const uint8_t* q = qs + 4 * ib;
    const uint8_t* h = qh + 2 * ib;
    uint32_t idx[4] = {q[0] | (((uint32_t)h[0] << 8) & 0x700u), q[1] | (((uint32_t)h[0] << 4) & 0x700u),
                       q[2] | (((uint32_t)h[1] << 8) & 0x700u), q[3] | (((uint32_t)h[1] << 4) & 0x700u)};
    float delta[4] = {(h[0] & 0x08) ? -0.125f : 0.125f, (h[0] & 0x80) ? -0.125f : 0.125f,
                      (h[1] & 0x08) ? -0.125f : 0.125f, (h[1] & 0x80) ? -0.125f : 0.125f};
    for (int l = 0; l < 4; l++) {
      const int8_t* g = (const int8_t*)(GRID_IQ1S + 8 * idx[l]);
      float dl = l < 2 ? dl1 : dl2;
      for (int j = 0; j < 8; j++) o[32 * ib + 8 * l + j] = dl * ((float)g[j] + delta[l]);
    }
  }
}

typedef void (*blk_fn)(const uint8_t*, float*);
static const blk_fn BLK[KQ_ORACLE_NUM_CODECS] = {
    blk_q2_k,   blk_q3_k,   blk_q4_k,  blk_q5_k,    blk_q6_k,    blk_q4_0,   blk_q4_1,
    blk_q5_0,   blk_q5_1,   blk_q8_0,  blk_iq4_nl,  blk_iq4_xs,  blk_iq3_s,  blk_iq3_xxs,
    blk_iq2_xxs, blk_iq2_xs, blk_iq2_s, blk_iq1_s,  blk_iq1_m,   blk_mxfp4,  blk_nvfp4,
};

/* -------------------------------------------------------------- dequantize */

static int g_threads = 0;
void kq_oracle_set_threads(int n) { g_threads = n; }
#ifdef _OPENMP
#include <omp.h>
int kq_oracle_threads(void) {
  /* src/kquant_cpu_decode.cpp:797-810: hardware concurrency, KQ_CPU_THREADS override, cap 64 */
  int n = g_threads > 0 ? g_threads : omp_get_num_procs();
  const char* env = getenv("KQ_CPU_THREADS");
  if (g_threads <= 0 && env && atoi(env) > 0) n = atoi(env);
  if (n < 1) n = 1;
  if (n > 64) n = 64;
  return n;
}
#else
int kq_oracle_threads(void) { return 1; }
#endif

/* out_dtype: 0 = f32, 1 = f16, 2 = bf16 (single RNE rounding of the f32 value). */
static inline void store_out(void* out, size_t i, float v, int dt) {
  if (dt == 0)
    ((float*)out)[i] = v;
  else if (dt == 1)
    ((uint16_t*)out)[i] = kq_oracle_f32_to_f16(v);
  else
    ((uint16_t*)out)[i] = kq_oracle_f32_to_bf16(v);
}
static inline float load_in(const void* p, size_t i, int dt) {
  if (dt == 0) return ((const float*)p)[i];
  if (dt == 1) return kq_oracle_f16_to_f32(((const uint16_t*)p)[i]);
  return kq_oracle_bf16_to_f32(((const uint16_t*)p)[i]);
}

int kq_oracle_dequantize(int codec, const uint8_t* w, void* out, uint64_t num_weights, int out_dtype) {
  /* src/kquant_cpu_decode.cpp:1135-1207: whole blocks, split over the worker pool. */
  const kq_oracle_codec_t* c = kq_oracle_codec(codec);
  if (!c || out_dtype < 0 || out_dtype > 2) return -1;
  const int64_t nb = (int64_t)(num_weights / (uint64_t)c->weights_per_block);
  const int wpb = c->weights_per_block, bpb = c->bytes_per_block;
  blk_fn fn = BLK[codec];
  int nt = kq_oracle_threads();
  (void)nt;
#pragma omp parallel for schedule(static) num_threads(nt)
  for (int64_t b = 0; b < nb; b++) {
    float buf[256];
    fn(w + (size_t)b * bpb, buf);
    for (int i = 0; i < wpb; i++) store_out(out, (size_t)b * wpb + i, buf[i], out_dtype);
  }
  return 0;
}

/* ------------------------------------------------------------------- qmm */

/* src/kquant_cpu_decode.cpp:1010-1024 */
static inline float dot8(const float* a, const float* b, int n) {
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f, s4 = 0.f, s5 = 0.f, s6 = 0.f, s7 = 0.f;
  for (int i = 0; i < n; i += 8) {
    s0 += a[i] * b[i];
    s1 += a[i + 1] * b[i + 1];
    s2 += a[i + 2] * b[i + 2];
    s3 += a[i + 3] * b[i + 3];
    s4 += a[i + 4] * b[i + 4];
    s5 += a[i + 5] * b[i + 5];
    s6 += a[i + 6] * b[i + 6];
    s7 += a[i + 7] * b[i + 7];
  }
  return ((s0 + s1) + (s2 + s3)) + ((s4 + s5) + (s6 + s7));
}

#define KQ_FUSED_MAX_M 16 /* kQmvFusedMaxM, src/kquant_cpu_decode.h */

/* src/kquant_cpu_decode.cpp:1032-1065: decode one block, dot it against every x row. */
static void fused_rows(float* outf, const float* xf, const uint8_t* w, int M, int N, int K,
                       const kq_oracle_codec_t* c, blk_fn fn, int64_t n0, int64_t n1) {
  float buf[256], acc[KQ_FUSED_MAX_M];
  const int wpb = c->weights_per_block, nblk = K / wpb;
  const size_t row_bytes = (size_t)nblk * c->bytes_per_block;
  for (int64_t n = n0; n < n1; n++) {
    const uint8_t* wr = w + (size_t)n * row_bytes;
    for (int m = 0; m < M; m++) acc[m] = 0.f;
    for (int b = 0; b < nblk; b++) {
      fn(wr + (size_t)b * c->bytes_per_block, buf);
      const float* xb = xf + (size_t)b * wpb;
      for (int m = 0; m < M; m++) acc[m] += dot8(xb + (size_t)m * K, buf, wpb);
    }
    for (int m = 0; m < M; m++) outf[(size_t)m * N + n] = acc[m];
  }
}

int kq_oracle_qmm_f32(int codec, float* out, const float* xf, const uint8_t* w, int M, int N, int K,
                      int transpose) {
  /* src/kquant_cpu_decode.cpp:1209-1359 with T = float. */
  const kq_oracle_codec_t* c = kq_oracle_codec(codec);
  if (!c) return -1;
  blk_fn fn = BLK[codec];
  const int w_rows = transpose ? N : K, w_cols = transpose ? K : N;
  if (w_cols % c->weights_per_block) return -2;
  const size_t row_bytes = (size_t)(w_cols / c->weights_per_block) * c->bytes_per_block;
  int nt = kq_oracle_threads();
  (void)nt;
  if (transpose && M <= KQ_FUSED_MAX_M) {
    /* decode shape: parallel over output rows (parts pulled dynamically, :934) */
    const int64_t chunk = 16;
    const int64_t nch = (N + chunk - 1) / chunk;
#pragma omp parallel for schedule(dynamic, 1) num_threads(nt)
    for (int64_t ch = 0; ch < nch; ch++) {
      int64_t a = ch * chunk, b = a + chunk < N ? a + chunk : N;
      fused_rows(out, xf, w, M, N, K, c, fn, a, b);
    }
    return 0;
  }
  /* prefill shape: dequantize once to f32 scratch, then sequential-k scalar GEMM (:1301-1352) */
  float* wd = (float*)malloc((size_t)w_rows * w_cols * sizeof(float));
  if (!wd) return -3;
  const int nblk_row = w_cols / c->weights_per_block;
#pragma omp parallel for schedule(static) num_threads(nt)
  for (int64_t r = 0; r < w_rows; r++)
    for (int b = 0; b < nblk_row; b++)
      fn(w + (size_t)r * row_bytes + (size_t)b * c->bytes_per_block,
         wd + (size_t)r * w_cols + (size_t)b * c->weights_per_block);
#pragma omp parallel for schedule(dynamic, 8) num_threads(nt)
  for (int64_t n = 0; n < N; n++) {
    for (int m = 0; m < M; m++) {
      const float* xm = xf + (size_t)m * K;
      float acc = 0.f;
      if (transpose) {
        const float* wn = wd + (size_t)n * K;
        for (int k = 0; k < K; k++) acc += xm[k] * wn[k];
      } else {
        for (int k = 0; k < K; k++) acc += xm[k] * wd[(size_t)k * N + n];
      }
      out[(size_t)m * N + n] = acc;
    }
  }
  free(wd);
  return 0;
}

int kq_oracle_qmm(int codec, void* out, const void* x, const uint8_t* w, int M, int N, int K,
                  int transpose, int dtype) {
  /* src/kquant_cpu_decode.cpp:1231-1252,1356-1358: stage x (and y) in f32, one rounding to T. */
  if (dtype == 0) return kq_oracle_qmm_f32(codec, (float*)out, (const float*)x, w, M, N, K, transpose);
  size_t xe = (size_t)M * K, oe = (size_t)M * N;
  float* xf = (float*)malloc(xe * sizeof(float));
  float* of = (float*)malloc(oe * sizeof(float));
  if (!xf || !of) return -3;
  for (size_t i = 0; i < xe; i++) xf[i] = load_in(x, i, dtype);
  int rc = kq_oracle_qmm_f32(codec, of, xf, w, M, N, K, transpose);
  for (size_t i = 0; i < oe; i++) store_out(out, i, of[i], dtype);
  free(xf);
  free(of);
  return rc;
}

/* ---------------------------------------------------------------- gather */

typedef struct {
  int i, x_idx, w_idx;
} entry_t;

static int entry_cmp(const void* a, const void* b) {
  const entry_t* ea = (const entry_t*)a;
  const entry_t* eb = (const entry_t*)b;
  if (ea->w_idx != eb->w_idx) return ea->w_idx < eb->w_idx ? -1 : 1;
  return ea->i < eb->i ? -1 : (ea->i > eb->i); /* stable: original order within an expert */
}

int kq_oracle_gather_qmm(int codec, void* out, const void* x, const uint8_t* w, const uint32_t* lhs,
                         const uint32_t* rhs, int B, int M, int N, int K, int64_t x_batch_stride,
                         int64_t w_expert_stride_bytes, int transpose, int dtype) {
  /* src/kquant_gather.cpp:470-746.  One [M, N] output per index pair; entries are
   * stable-sorted by expert and each group runs as one qmm of (rows * M) activation
   * rows, so the fused-vs-GEMM accumulation order is chosen per group exactly as the
   * reference chooses it (:584-593 -- all groups small -> fused path for every group;
   * otherwise per-group M decides, :681-731). */
  const kq_oracle_codec_t* c = kq_oracle_codec(codec);
  if (!c) return -1;
  const size_t esz = dtype == 0 ? 4 : 2;
  entry_t* e = (entry_t*)malloc(sizeof(entry_t) * (size_t)(B > 0 ? B : 1));
  for (int i = 0; i < B; i++) {
    e[i].i = i;
    e[i].x_idx = (int)lhs[i];
    e[i].w_idx = (int)rhs[i];
  }
  qsort(e, (size_t)B, sizeof(entry_t), entry_cmp);
  const size_t row_els = (size_t)M * K, out_els = (size_t)M * N;
  int rc = 0;
  for (int a = 0; a < B && rc == 0;) {
    int b = a;
    while (b < B && e[b].w_idx == e[a].w_idx) b++;
    const int rg = b - a;
    const uint8_t* wp = w + (int64_t)e[a].w_idx * w_expert_stride_bytes;
    uint8_t* xg = (uint8_t*)malloc((size_t)rg * row_els * esz);
    uint8_t* og = (uint8_t*)malloc((size_t)rg * out_els * esz);
    for (int r = 0; r < rg; r++)
      memcpy(xg + (size_t)r * row_els * esz,
             (const uint8_t*)x + (size_t)((int64_t)e[a + r].x_idx * x_batch_stride) * esz, row_els * esz);
    /* Duplicate (x, expert) entries are computed once by the reference and fanned out
     * (:571-612); row results do not depend on their neighbours in either path, so
     * computing them again gives the same bits. */
    rc = kq_oracle_qmm(codec, og, xg, wp, rg * M, N, K, transpose, dtype);
    for (int r = 0; r < rg; r++)
      memcpy((uint8_t*)out + (size_t)e[a + r].i * out_els * esz, og + (size_t)r * out_els * esz,
             out_els * esz);
    free(xg);
    free(og);
    a = b;
  }
  free(e);
  return rc;
}

/* ------------------------------------------------------------- fused MoE */

/* metal/mlx/backend/metal/kernels/kq_moe_glu_kq.h:34-60 */
float kq_oracle_glu_epilogue(int act, float g, float u, float limit, float alpha) {
  if (act == KQ_ORACLE_ACT_GELU) {
    const float g3 = 0.044715f * g * g * g;
    const float t = tanhf(0.7978845608028654f * (g + g3));
    return (0.5f * g * (1.0f + t)) * u;
  }
  if (act == KQ_ORACLE_ACT_SWIGLU_CLAMP) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    const float sig = 1.0f / (1.0f + expf(-alpha * g));
    return (g * sig) * (u + 1.0f);
  }
  if (act == KQ_ORACLE_ACT_SILU_LIMIT) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  const float sig = 1.0f / (1.0f + expf(-g));
  return (g * sig) * u;
}

int kq_oracle_moe_glu_gather(int codec, void* out, const void* x, const uint8_t* gate_w,
                             const uint8_t* up_w, const uint32_t* idx, const float* gate_bias,
                             const float* up_bias, int T, int R, int N, int K, int act, float limit,
                             float alpha, int dtype) {
  /* Op contract src/kquant_moe_glu.cpp:1070-1157; the reference has no CPU kernel for
   * it (eval_cpu throws, :662-667).  Truth = the composition its tests use
   * (tests/test_moe_glu.py:196-216): g = x . G_e^T, u = x . U_e^T in f32 on the
   * upcast activations with unrounded g/u, biases added in f32, epilogue in f32, one
   * rounding to x's dtype (kq_moe_glu_kq.h:153-158,874-880). */
  const kq_oracle_codec_t* c = kq_oracle_codec(codec);
  if (!c || K % c->weights_per_block || dtype == 0) return -1;
  const size_t ebytes = (size_t)N * (K / c->weights_per_block) * c->bytes_per_block;
  float* xf = (float*)malloc((size_t)K * sizeof(float));
  float* g = (float*)malloc((size_t)N * sizeof(float));
  float* u = (float*)malloc((size_t)N * sizeof(float));
  int rc = 0;
  for (int t = 0; t < T && rc == 0; t++) {
    for (int k = 0; k < K; k++) xf[k] = load_in(x, (size_t)t * K + k, dtype);
    for (int r = 0; r < R && rc == 0; r++) {
      uint32_t ex = idx[(size_t)t * R + r];
      rc = kq_oracle_qmm_f32(codec, g, xf, gate_w + ex * ebytes, 1, N, K, 1);
      if (rc == 0) rc = kq_oracle_qmm_f32(codec, u, xf, up_w + ex * ebytes, 1, N, K, 1);
      for (int n = 0; n < N && rc == 0; n++) {
        float gv = g[n], uv = u[n];
        if (gate_bias) gv += gate_bias[(size_t)ex * N + n];
        if (up_bias) uv += up_bias[(size_t)ex * N + n];
        store_out(out, ((size_t)t * R + r) * N + n, kq_oracle_glu_epilogue(act, gv, uv, limit, alpha),
                  dtype);
      }
    }
  }
  free(xf);
  free(g);
  free(u);
  return rc;
}

int kq_oracle_gather_qmv(int codec, void* out, const void* x, const uint8_t* w, const uint32_t* idx,
                         const float* bias, int T, int R, int N, int K, int dtype) {
  /* Op contract src/kquant_moe_glu.cpp:1159-1210; kernel semantics
   * kq_moe_glu_kq.h:933-999: out[t,r,:] = T(x[t,r,:] . W_e^T (+ bias_e)), f32 throughout. */
  const kq_oracle_codec_t* c = kq_oracle_codec(codec);
  if (!c || K % c->weights_per_block || dtype == 0) return -1;
  const size_t ebytes = (size_t)N * (K / c->weights_per_block) * c->bytes_per_block;
  float* xf = (float*)malloc((size_t)K * sizeof(float));
  float* y = (float*)malloc((size_t)N * sizeof(float));
  int rc = 0;
  for (int64_t p = 0; p < (int64_t)T * R && rc == 0; p++) {
    for (int k = 0; k < K; k++) xf[k] = load_in(x, (size_t)p * K + k, dtype);
    uint32_t ex = idx[p];
    rc = kq_oracle_qmm_f32(codec, y, xf, w + ex * ebytes, 1, N, K, 1);
    for (int n = 0; n < N && rc == 0; n++)
      store_out(out, (size_t)p * N + n, bias ? y[n] + bias[(size_t)ex * N + n] : y[n], dtype);
  }
  free(xf);
  free(y);
  return rc;
}

int kq_oracle_moe_glu_gather_shexp(int codec, int shexp_codec, void* out, const void* x, const uint8_t* gate_w,
                                   const uint8_t* up_w, const uint8_t* shexp_gate_w, const uint8_t* shexp_up_w,
                                   const uint32_t* idx, int T, int R, int N, int K, int act, int dtype) {
  /* Op contract src/kquant_moe_glu.cpp:1212-1272: slots r < R as moe_glu_gather_kq, slot R = the same GLU
   * against the shared expert's two matrices (f32 throughout, one rounding). */
  const kq_oracle_codec_t* c = kq_oracle_codec(codec);
  const kq_oracle_codec_t* sc = kq_oracle_codec(shexp_codec);
  if (!c || !sc || K % c->weights_per_block || K % sc->weights_per_block || dtype == 0) return -1;
  const size_t ebytes = (size_t)N * (K / c->weights_per_block) * c->bytes_per_block;
  float* xf = (float*)malloc((size_t)K * sizeof(float));
  float* g = (float*)malloc((size_t)N * sizeof(float));
  float* u = (float*)malloc((size_t)N * sizeof(float));
  int rc = 0;
  for (int t = 0; t < T && rc == 0; t++) {
    for (int k = 0; k < K; k++) xf[k] = load_in(x, (size_t)t * K + k, dtype);
    for (int r = 0; r <= R && rc == 0; r++) {
      if (r < R) {
        const uint32_t e = idx[(size_t)t * R + r];
        rc = kq_oracle_qmm_f32(codec, g, xf, gate_w + e * ebytes, 1, N, K, 1);
        if (!rc) rc = kq_oracle_qmm_f32(codec, u, xf, up_w + e * ebytes, 1, N, K, 1);
      } else {
        rc = kq_oracle_qmm_f32(shexp_codec, g, xf, shexp_gate_w, 1, N, K, 1);
        if (!rc) rc = kq_oracle_qmm_f32(shexp_codec, u, xf, shexp_up_w, 1, N, K, 1);
      }
      for (int n = 0; n < N && rc == 0; n++)
        store_out(out, ((size_t)t * (R + 1) + r) * N + n, kq_oracle_glu_epilogue(act, g[n], u[n], 0.f, 0.f), dtype);
    }
  }
  free(xf);
  free(g);
  free(u);
  return rc;
}

int kq_oracle_gather_qmv_mix(int codec, int shexp_codec, void* out, const void* x, const uint8_t* w,
                             const uint8_t* shexp_w, const uint32_t* idx, const float* scores, int T, int S, int N,
                             int K, int dtype) {
  /* Op contracts src/kquant_moe_glu.cpp:1274-1364: every slot's matvec in f32, the score-weighted sum
   * accumulates in f32 in slot order, one rounding to the activation dtype. */
  const kq_oracle_codec_t* c = kq_oracle_codec(codec);
  if (!c || K % c->weights_per_block || dtype == 0 || S < 1) return -1;
  const size_t ebytes = (size_t)N * (K / c->weights_per_block) * c->bytes_per_block;
  const int routed = shexp_w ? S - 1 : S;
  float* xf = (float*)malloc((size_t)K * sizeof(float));
  float* y = (float*)malloc((size_t)N * sizeof(float));
  float* acc = (float*)malloc((size_t)N * sizeof(float));
  int rc = 0;
  for (int t = 0; t < T && rc == 0; t++) {
    for (int n = 0; n < N; n++) acc[n] = 0.f;
    for (int s = 0; s < S && rc == 0; s++) {
      for (int k = 0; k < K; k++) xf[k] = load_in(x, ((size_t)t * S + s) * K + k, dtype);
      if (s < routed)
        rc = kq_oracle_qmm_f32(codec, y, xf, w + idx[(size_t)t * routed + s] * ebytes, 1, N, K, 1);
      else
        rc = kq_oracle_qmm_f32(shexp_codec, y, xf, shexp_w, 1, N, K, 1);
      const float sc = scores[(size_t)t * S + s];
      for (int n = 0; n < N; n++) acc[n] = fmaf(sc, y[n], acc[n]);
    }
    for (int n = 0; n < N && rc == 0; n++) store_out(out, (size_t)t * N + n, acc[n], dtype);
  }
  free(xf);
  free(y);
  free(acc);
  return rc;
}

int kq_oracle_router_topk(const void* logits, int dtype, int T, int E, int top_k, int norm, int shared,
                          const float* per_expert_scale, const float* bias, int scoring, float scale,
                          uint32_t* indices, float* scores) {
  /* Op contract src/kquant_moe_glu.cpp:1366-1441; kernel semantics kq_moe_glu_kq.h:1215-1358: all math
   * in f32; top_k rounds of arg-max over p (+ bias), smallest index first on ties, the winner leaves the
   * pool; emitted scores are the unbiased p, divided by the picked sum (norm; + 1e-20 for sqrt-softplus)
   * or by the softmax sum, times per_expert_scale[e] and scale; shared: sigmoid of column E last. */
  if (T < 0 || E < 1 || E > 1024 || top_k < 1 || top_k > 16 || top_k > E) return -1;
  if (scoring != 0 && scoring != 1) return -1;
  if (scoring == 1 && !norm) return -1;
  float* p = (float*)malloc((size_t)E * sizeof(float));
  for (int t = 0; t < T; t++) {
    const size_t row = (size_t)t * (E + (shared ? 1 : 0));
    float gsum = 1.0f;
    if (scoring == 1) {
      for (int e = 0; e < E; e++) {
        const float x = load_in(logits, row + e, dtype);
        const float z = expf(-fabsf(x));
        const float l1p = z < 1e-4f ? fmaf(-0.5f * z, z, z) : logf(1.0f + z);
        p[e] = sqrtf(fmaxf(x, 0.0f) + l1p);
      }
    } else {
      float m = -INFINITY;
      for (int e = 0; e < E; e++) m = fmaxf(m, load_in(logits, row + e, dtype));
      float s = 0.f;
      for (int e = 0; e < E; e++) {
        p[e] = expf(load_in(logits, row + e, dtype) - m);
        s += p[e];
      }
      gsum = s;
    }
    float win_v[16];
    uint32_t win_i[16];
    for (int r = 0; r < top_k; r++) {
      float bv = -INFINITY;
      uint32_t bi = 0xffffffffu;
      for (int e = 0; e < E; e++) {
        const float v = bias ? p[e] + bias[e] : p[e];
        if (v > bv || (v == bv && (uint32_t)e < bi)) {
          bv = v;
          bi = (uint32_t)e;
        }
      }
      if (bi == 0xffffffffu) bi = 0; /* every value NaN: keep the index in range */
      indices[(size_t)t * top_k + r] = bi;
      win_v[r] = p[bi];
      win_i[r] = bi;
      p[bi] = -INFINITY;
    }
    float ps = 0.f;
    for (int r = 0; r < top_k; r++) ps += win_v[r];
    const float denom = norm ? (scoring == 1 ? ps + 1e-20f : ps) : gsum;
    float* srow = scores + (size_t)t * (top_k + (shared ? 1 : 0));
    for (int r = 0; r < top_k; r++) {
      float sv = win_v[r] / denom;
      if (per_expert_scale) sv *= per_expert_scale[win_i[r]];
      srow[r] = sv * scale;
    }
    if (shared) srow[top_k] = 1.0f / (1.0f + expf(-load_in(logits, row + E, dtype)));
  }
  free(p);
  return 0;
}
