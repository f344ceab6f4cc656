// Host-side wire encoders behind kq_quantize: float rows -> GGUF block bytes for the five legacy
// 32-weight codecs, the five K-quant superblock codecs and the two non-linear 4-bit codecs
// (iq4_nl, iq4_xs).  Like the reference's encoder
// (src/kquant_cpu_encode.cpp:38-859, ggml's search heuristics) this runs on the CPU; unlike it,
// blocks are encoded in parallel (blocks are independent).  Operation order inside a block
// follows the cited reference lines so that, on the same x86 host arithmetic, the bytes agree.
//
//   legacy  : q8_0 :38-61, q4_0 :63-91, q4_1 :93-125, q5_0 :136-169, q5_1 :171-208
//             (round-half-away-from-zero, scale written as fp16)
//   K-quant : q4_k/q5_k :445-540, q6_k :542-628, q3_k :630-734, q2_k :736-820
//             (round-half-to-even; super-scales written as fp16 and read back before the
//             final re-quantisation of every weight)
//   iq4     : iq4_nl / iq4_xs, src/kquant_iq_encode.cpp:49-214 (ggml quantize_row_iq4_nl_impl: nearest
//             codebook entry, weighted least-squares scale, 15 trial scales around max / -127)
#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include "kq_common.h"

namespace {

inline void put_f16(uint8_t* p, float v) {
  _Float16 h = static_cast<_Float16>(v);
  std::memcpy(p, &h, 2);
}
inline float get_f16(const uint8_t* p) {
  _Float16 h;
  std::memcpy(&h, p, 2);
  return static_cast<float>(h);
}
inline int rne(float v) { return static_cast<int>(std::rint(v)); }  // kq_nearest_int, encode_util.h:41-43
inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// ------------------------------------------------------------------ legacy 32-weight codecs
void enc_q8_0(const float* x, uint8_t* b) {
  float amax = 0.f;
  for (int j = 0; j < 32; j++) amax = std::max(amax, std::fabs(x[j]));
  const float d = amax / 127.0f, id = d != 0.f ? 1.0f / d : 0.f;
  put_f16(b, d);
  for (int j = 0; j < 32; j++)
    reinterpret_cast<int8_t*>(b + 2)[j] = static_cast<int8_t>(std::clamp(std::round(x[j] * id), -127.0f, 127.0f));
}

template <bool kHasMin, int kBits>
void enc_legacy(const float* x, uint8_t* b) {
  constexpr int top = (1 << kBits) - 1;       // 15 or 31
  constexpr float bias = kHasMin ? 0.f : float(1 << (kBits - 1));
  float lo = x[0], hi = x[0], amax = 0.f;
  for (int j = 0; j < 32; j++) {
    lo = std::min(lo, x[j]);
    hi = std::max(hi, x[j]);
    amax = std::max(amax, std::fabs(x[j]));
  }
  // symmetric codecs divide |x|max by 7 / 15; min codecs spread (max - min) over all levels
  const float d = kHasMin ? (hi - lo) / float(top) : amax / float((1 << (kBits - 1)) - 1);
  const float id = d != 0.f ? 1.0f / d : 0.f;
  uint8_t* p = b;
  put_f16(p, d);
  p += 2;
  if (kHasMin) {
    put_f16(p, lo);
    p += 2;
  }
  uint8_t* qh_p = p;
  if (kBits == 5) p += 4;
  uint32_t qh = 0;
  for (int j = 0; j < 16; j++) {
    const float v0 = kHasMin ? (x[j] - lo) * id : x[j] * id;
    const float v1 = kHasMin ? (x[j + 16] - lo) * id : x[j + 16] * id;
    const uint8_t q0 = static_cast<uint8_t>(std::clamp(std::round(v0) + bias, 0.0f, float(top)));
    const uint8_t q1 = static_cast<uint8_t>(std::clamp(std::round(v1) + bias, 0.0f, float(top)));
    p[j] = (q0 & 15) | ((q1 & 15) << 4);
    if (kBits == 5) {
      qh |= uint32_t(q0 >> 4) << j;
      qh |= uint32_t(q1 >> 4) << (j + 16);
    }
  }
  if (kBits == 5)
    for (int i = 0; i < 4; i++) qh_p[i] = uint8_t(qh >> (8 * i));
}

// ------------------------------------------------------------------ K-quant fitting helpers

// Weighted fit of (scale, min) to n values with levels 0..nmax: start from the min/max grid and
// scan 37 candidate inverse scales around it, solving the 2x2 least-squares system for each
// (ggml make_qkx3_quants; reference :250-334).  Returns the scale, *neg_min receives -min.
float fit_scale_min(const float* x, const float* wt, int n, int nmax, float* neg_min) {
  float vmin = x[0], vmax = x[0], sw = wt[0], swx = sw * x[0];
  for (int i = 1; i < n; i++) {
    if (x[i] < vmin) vmin = x[i];
    if (x[i] > vmax) vmax = x[i];
    sw += wt[i];
    swx += wt[i] * x[i];
  }
  if (vmin > 0.f) vmin = 0.f;
  if (vmax <= vmin) {
    *neg_min = -vmin;
    return 0.f;
  }
  float inv = float(nmax) / (vmax - vmin), scale = 1.0f / inv, best_min = vmin, best_err = 0.f;
  for (int i = 0; i < n; i++) {
    const int l = clampi(rne(inv * (x[i] - vmin)), 0, nmax);
    const float e = scale * float(l) + vmin - x[i];
    best_err += wt[i] * e * e;
  }
  uint8_t lv[32];
  for (int step = 0; step <= 36; step++) {
    const float inv_s = (-0.9f + 0.05f * float(step) + float(nmax)) / (vmax - vmin);
    float sl = 0.f, sl2 = 0.f, sxl = 0.f;
    for (int i = 0; i < n; i++) {
      const int l = clampi(rne(inv_s * (x[i] - vmin)), 0, nmax);
      lv[i] = uint8_t(l);
      sl += wt[i] * float(l);
      sl2 += wt[i] * float(l) * float(l);
      sxl += wt[i] * float(l) * x[i];
    }
    const float det = sw * sl2 - sl * sl;
    if (det > 0.f) {
      float s = (sw * sxl - swx * sl) / det, m = (sl2 * swx - sl * sxl) / det;
      if (m > 0.f) {
        m = 0.f;
        s = sxl / sl2;
      }
      float err = 0.f;
      for (int i = 0; i < n; i++) {
        const float e = s * float(lv[i]) + m - x[i];
        err += wt[i] * e * e;
      }
      if (err < best_err) {
        best_err = err;
        scale = s;
        best_min = m;
      }
    }
  }
  *neg_min = -best_min;
  return scale;
}

// Weighted fit of one non-negative scale to n values with levels 0..nmax, 9-point scan plus up to
// five rounds of coordinate refinement (ggml make_qp_quants; kquant_cpu_encode_util.h:50-136).
float fit_positive(const float* x, const float* wt, int n, int nmax, uint8_t* out) {
  float vmax = 0.f;
  for (int i = 0; i < n; i++)
    if (x[i] > vmax) vmax = x[i];
  if (vmax < 1e-30f) {
    for (int i = 0; i < n; i++) out[i] = 0;
    return 0.f;
  }
  float inv = float(nmax) / vmax;
  uint8_t lv[16];
  float best = 0.f;
  {
    const float s = 1.0f / inv;
    for (int i = 0; i < n; i++) {
      lv[i] = uint8_t(clampi(rne(inv * x[i]), 0, nmax));
      const float e = x[i] - s * float(lv[i]);
      best += wt[i] * e * e;
    }
  }
  for (int k = -4; k <= 4; k++) {
    if (k == 0) continue;
    const float inv_k = (0.1f * float(k) + float(nmax)) / vmax, s_k = 1.0f / inv_k;
    float err = 0.f;
    for (int i = 0; i < n; i++) {
      const int l = std::min(nmax, rne(inv_k * x[i]));
      const float e = x[i] - s_k * float(l);
      err += wt[i] * e * e;
    }
    if (err < best) {
      best = err;
      inv = inv_k;
    }
  }
  float slx = 0.f, sl2 = 0.f;
  for (int i = 0; i < n; i++) {
    const int l = std::min(nmax, rne(inv * x[i]));
    lv[i] = uint8_t(l);
    slx += wt[i] * x[i] * float(l);
    sl2 += wt[i] * float(l) * float(l);
  }
  for (int round = 0; round < 5; round++) {
    int changed = 0;
    for (int i = 0; i < n; i++) {
      const float w = wt[i];
      float a = slx - w * x[i] * float(lv[i]);
      float b = sl2 - w * float(lv[i]) * float(lv[i]);
      if (a > 0.f && b > 0.f) {
        const int nl = std::min(nmax, rne(x[i] * b / a));
        if (nl != int(lv[i])) {
          a += w * x[i] * float(nl);
          b += w * float(nl) * float(nl);
          if (a * a * sl2 > slx * slx * b) {
            lv[i] = uint8_t(nl);
            slx = a;
            sl2 = b;
            changed++;
          }
        }
      }
    }
    if (!changed) break;
  }
  for (int i = 0; i < n; i++) out[i] = lv[i];
  return sl2 > 0.f ? slx / sl2 : 0.f;
}

// Weighted fit of one signed scale to 16 values with levels -nmax..nmax-1, 19-point scan (ggml
// make_qx_quants; reference :338-395).  wt == nullptr weights by x^2.
float fit_signed16(const float* x, const float* wt, int nmax) {
  float peak = 0.f, apeak = 0.f;
  for (int i = 0; i < 16; i++) {
    const float a = std::fabs(x[i]);
    if (a > apeak) {
      apeak = a;
      peak = x[i];
    }
  }
  if (apeak < 1e-30f) return 0.f;
  auto sums = [&](float inv, float& slx, float& sl2) {
    slx = sl2 = 0.f;
    for (int i = 0; i < 16; i++) {
      const int l = clampi(rne(inv * x[i]), -nmax, nmax - 1);
      const float w = wt ? wt[i] : x[i] * x[i];
      slx += w * x[i] * float(l);
      sl2 += w * float(l) * float(l);
    }
  };
  float slx, sl2;
  sums(-float(nmax) / peak, slx, sl2);
  float scale = sl2 > 0.f ? slx / sl2 : 0.f, best = scale * slx;
  for (int k = -9; k <= 9; k++) {
    if (k == 0) continue;
    sums(-(float(nmax) + 0.1f * float(k)) / peak, slx, sl2);
    if (sl2 > 0.f && slx * slx > best * sl2) {
      scale = slx / sl2;
      best = scale * slx;
    }
  }
  return scale;
}

// importance weights of a superblock (reference :237-245 and the per-codec prologues)
void importance(const float* x, const float* imatrix_blk, float sigma_factor, float* wt) {
  float total = 0.f;
  for (int i = 0; i < 256; i++) total += x[i] * x[i];
  const float sigma2 = sigma_factor * total / 256.0f, av = std::sqrt(sigma2);
  if (imatrix_blk) {
    for (int i = 0; i < 256; i++) wt[i] = imatrix_blk[i] * std::sqrt(sigma2 + x[i] * x[i]);
  } else {
    for (int i = 0; i < 256; i++) wt[i] = av + std::fabs(x[i]);
  }
}

// 2-bit plane packing shared by q2_k and q3_k: weight 128 h + 32 s + l sits in byte 32 h + l at bits 2 s
void pack_2bit(const uint8_t* lv, uint8_t* qs) {
  for (int i = 0; i < 64; i++) {
    const int h = i >> 5, l = i & 31;
    uint8_t byte = 0;
    for (int s = 0; s < 4; s++) byte |= uint8_t((lv[128 * h + 32 * s + l] & 3) << (2 * s));
    qs[i] = byte;
  }
}

template <int kBits>  // 4 or 5
void enc_q45_k(const float* x, const float* im, uint8_t* b) {
  constexpr int nmax = (1 << kBits) - 1;
  constexpr int QS = kBits == 4 ? 16 : 48;
  float wt[256], sc[8], mn[8], sw[8];
  importance(x, im, 2.0f, wt);
  for (int j = 0; j < 8; j++) {
    float s = 0.f;
    for (int l = 0; l < 32; l++) s += wt[32 * j + l];
    sw[j] = s;
    sc[j] = fit_scale_min(x + 32 * j, wt + 32 * j, 32, nmax, &mn[j]);
  }
  uint8_t ls[8], lm[8];
  put_f16(b, fit_positive(sc, sw, 8, 63, ls));
  put_f16(b + 2, fit_positive(mn, sw, 8, 63, lm));
  uint8_t* s12 = b + 4;
  std::memset(s12, 0, 12);
  for (int j = 0; j < 8; j++) {
    if (j < 4) {
      s12[j] |= ls[j];
      s12[j + 4] |= lm[j];
    } else {
      s12[j + 4] = (ls[j] & 15) | ((lm[j] & 15) << 4);
      s12[j - 4] |= (ls[j] >> 4) << 6;
      s12[j] |= (lm[j] >> 4) << 6;
    }
  }
  const float d = get_f16(b), dmin = get_f16(b + 2);
  uint8_t lv[256];
  for (int i = 0; i < 256; i++) {
    const int j = i >> 5;
    const float ds = d * float(ls[j]), dm = dmin * float(lm[j]);
    lv[i] = ds == 0.f ? 0 : uint8_t(clampi(rne((x[i] + dm) / ds), 0, nmax));
  }
  for (int g = 0; g < 4; g++)
    for (int l = 0; l < 32; l++) b[QS + 32 * g + l] = (lv[64 * g + l] & 15) | ((lv[64 * g + 32 + l] & 15) << 4);
  if (kBits == 5) {
    for (int l = 0; l < 32; l++) {
      uint8_t bits = 0;
      for (int j = 0; j < 8; j++) bits |= uint8_t((lv[32 * j + l] > 15) << j);
      b[16 + l] = bits;
    }
  }
}

void enc_q6_k(const float* x, const float* im, uint8_t* b) {
  float sc[16], peak = 0.f, apeak = 0.f;
  for (int j = 0; j < 16; j++) {
    sc[j] = fit_signed16(x + 16 * j, im ? im + 16 * j : nullptr, 32);
    if (std::fabs(sc[j]) > apeak) {
      apeak = std::fabs(sc[j]);
      peak = sc[j];
    }
  }
  if (apeak < 1e-30f) {
    std::memset(b, 0, 210);
    return;
  }
  const float inv = -128.0f / peak;
  put_f16(b + 208, 1.0f / inv);
  int8_t* so = reinterpret_cast<int8_t*>(b + 192);
  for (int j = 0; j < 16; j++) so[j] = int8_t(std::min(127, rne(inv * sc[j])));
  const float d = get_f16(b + 208);
  uint8_t lv[256];
  for (int i = 0; i < 256; i++) {
    const float de = d * float(so[i >> 4]);
    lv[i] = de == 0.f ? 32 : uint8_t(clampi(rne(x[i] / de), -32, 31) + 32);
  }
  for (int h = 0; h < 2; h++)
    for (int l = 0; l < 32; l++) {
      const uint8_t a = lv[128 * h + l], bb = lv[128 * h + l + 32], c = lv[128 * h + l + 64], e = lv[128 * h + l + 96];
      b[64 * h + l] = (a & 15) | ((c & 15) << 4);
      b[64 * h + l + 32] = (bb & 15) | ((e & 15) << 4);
      b[128 + 32 * h + l] = (a >> 4) | ((bb >> 4) << 2) | ((c >> 4) << 4) | ((e >> 4) << 6);
    }
}

void enc_q3_k(const float* x, const float* im, uint8_t* b) {
  float wt[256], sc[16], peak = 0.f, apeak = 0.f;
  if (im) importance(x, im, 2.0f, wt);
  for (int j = 0; j < 16; j++) {
    sc[j] = fit_signed16(x + 16 * j, im ? wt + 16 * j : nullptr, 4);
    if (std::fabs(sc[j]) > apeak) {
      apeak = std::fabs(sc[j]);
      peak = sc[j];
    }
  }
  uint8_t* s12 = b + 96;
  std::memset(s12, 0, 12);
  int lsc[16];
  for (int j = 0; j < 16; j++) lsc[j] = 0;  // biased code 0 <-> scale -32 when the block is empty
  float dblk = 0.f;
  if (peak != 0.f) {
    const float inv = -32.0f / peak;
    for (int j = 0; j < 16; j++) {
      const int l = clampi(rne(inv * sc[j]), -32, 31) + 32;
      lsc[j] = l;
      if (j < 8)
        s12[j] = uint8_t(l & 15);
      else
        s12[j - 8] |= uint8_t((l & 15) << 4);
      s12[8 + (j & 3)] |= uint8_t(((l >> 4) & 3) << (2 * (j >> 2)));
    }
    dblk = 1.0f / inv;
  }
  put_f16(b + 108, dblk);
  const float d = get_f16(b + 108);
  uint8_t lv[256];
  for (int i = 0; i < 256; i++) {
    const float de = d * float(lsc[i >> 4] - 32);
    lv[i] = de == 0.f ? 4 : uint8_t(clampi(rne(x[i] / de), -4, 3) + 4);
  }
  pack_2bit(lv, b + 32);
  for (int l = 0; l < 32; l++) {
    uint8_t byte = 0;
    for (int bit = 0; bit < 8; bit++) byte |= uint8_t(((lv[128 * (bit >> 2) + 32 * (bit & 3) + l] >> 2) & 1) << bit);
    b[l] = byte;
  }
}

void enc_q2_k(const float* x, const float* im, uint8_t* b) {
  float wt[256], sc[16], mn[16], sw[16];
  importance(x, im, 1.0f, wt);
  for (int j = 0; j < 16; j++) {
    float s = 0.f;
    for (int l = 0; l < 16; l++) s += wt[16 * j + l];
    sw[j] = s;
    sc[j] = fit_scale_min(x + 16 * j, wt + 16 * j, 16, 3, &mn[j]);
  }
  uint8_t ls[16], lm[16];
  put_f16(b + 80, fit_positive(sc, sw, 16, 15, ls));
  put_f16(b + 82, fit_positive(mn, sw, 16, 15, lm));
  for (int j = 0; j < 16; j++) b[j] = (ls[j] & 15) | ((lm[j] & 15) << 4);
  const float d = get_f16(b + 80), dmin = get_f16(b + 82);
  uint8_t lv[256];
  for (int i = 0; i < 256; i++) {
    const float de = d * float(ls[i >> 4]), me = dmin * float(lm[i >> 4]);
    lv[i] = de == 0.f ? 0 : uint8_t(clampi(rne((x[i] + me) / de), 0, 3));
  }
  pack_2bit(lv, b + 16);
}

// ------------------------------------------------------------------ iq4_nl / iq4_xs
// Codebook kvalues_iq4nl (src/kquant_iq_tables.h:10), ascending.
const int8_t kIq4Values[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

// Index of the codebook entry nearest to v; a tie goes to the upper entry (the comparison is strict).
inline int iq4_nearest(float v) {
  if (v <= (float)kIq4Values[0]) return 0;
  if (v >= (float)kIq4Values[15]) return 15;
  int lo = 0, hi = 15;
  while (hi - lo > 1) {
    const int mid = (lo + hi) / 2;
    if (v < (float)kIq4Values[mid]) hi = mid; else lo = mid;
  }
  return v - (float)kIq4Values[hi - 1] < (float)kIq4Values[hi] - v ? hi - 1 : hi;
}

// Weighted least-squares fit of one 32-weight block: levels for inverse scale `inv`, returns sum w q x
// and sum w q^2 through the references.
inline void iq4_fit(const float* x, const float* wt, float inv, uint8_t* lv, float& sqx, float& sq2) {
  sqx = sq2 = 0.f;
  for (int j = 0; j < 32; j++) {
    const int l = iq4_nearest(inv * x[j]);
    if (lv) lv[j] = (uint8_t)l;
    const float q = (float)kIq4Values[l];
    sqx += wt[j] * q * x[j];
    sq2 += wt[j] * q * q;
  }
}

// kSuper = 32 (iq4_nl: [f16 d][qs 16]) or 256 (iq4_xs: [f16 d][u16 scales_h][scales_l 4][qs 128]).
template <int kSuper>
void enc_iq4(const float* x, const float* im, uint8_t* b) {
  constexpr int kBlocks = kSuper / 32, kTrials = 7;
  float sigma2 = 0.f;
  for (int j = 0; j < kSuper; j++) sigma2 += x[j] * x[j];
  sigma2 *= 2.f / (float)kSuper;

  uint8_t lv[kSuper];
  float scale[kBlocks];
  float top = 0.f, top_abs = 0.f;  // block scale of largest magnitude, signed
  for (int ib = 0; ib < kBlocks; ib++) {
    const float* xb = x + 32 * ib;
    float wt[32];
    for (int j = 0; j < 32; j++) wt[j] = im ? im[32 * ib + j] * std::sqrt(sigma2 + xb[j] * xb[j]) : xb[j] * xb[j];
    float amax = 0.f, vmax = 0.f;
    for (int j = 0; j < 32; j++) {
      const float ax = std::fabs(xb[j]);
      if (ax > amax) {
        amax = ax;
        vmax = xb[j];
      }
    }
    if (amax < 1e-15f) {
      scale[ib] = 0.f;
      std::memset(lv + 32 * ib, 0, 32);
      continue;
    }
    // first guess: the extreme weight maps to the codebook's -127 end (sign flipped)
    float d = -vmax / (float)kIq4Values[0];
    float sqx, sq2;
    iq4_fit(xb, wt, 1.f / d, lv + 32 * ib, sqx, sq2);
    d = sq2 > 0.f ? sqx / sq2 : 0.f;
    float best = d * sqx;
    for (int t = -kTrials; t <= kTrials; t++) {
      iq4_fit(xb, wt, ((float)t + (float)kIq4Values[0]) / vmax, nullptr, sqx, sq2);
      if (sq2 > 0.f && sqx * sqx > best * sq2) {
        d = sqx / sq2;
        best = d * sqx;
      }
    }
    scale[ib] = d;
    if (std::fabs(d) > top_abs) {
      top_abs = std::fabs(d);
      top = d;
    }
  }

  uint8_t* qs;
  if constexpr (kBlocks == 1) {
    qs = b + 2;
    put_f16(b, scale[0]);
    const float inv = scale[0] ? 1.f / scale[0] : 0.f;
    for (int j = 0; j < 32; j++) lv[j] = (uint8_t)iq4_nearest(inv * x[j]);
  } else {
    // super-scale d = -top / 32, 6-bit block scales (low nibbles in scales_l, high 2 bits in scales_h),
    // then every weight is re-quantised against its rounded block scale
    qs = b + 8;
    const float d = -top / 32.f;
    put_f16(b, d);
    const float inv = d ? 1.f / d : 0.f;
    uint32_t sh = 0;
    uint8_t sl[4] = {0, 0, 0, 0};
    for (int ib = 0; ib < kBlocks; ib++) {
      const int l = clampi(rne(inv * scale[ib]), -32, 31);
      const float dl = d * (float)l;
      const float invl = dl ? 1.f / dl : 0.f;
      for (int j = 0; j < 32; j++) lv[32 * ib + j] = (uint8_t)iq4_nearest(invl * x[32 * ib + j]);
      const int u = l + 32;
      sl[ib / 2] |= (uint8_t)((u & 15) << (4 * (ib & 1)));
      sh |= (uint32_t)(u >> 4) << (2 * ib);
    }
    b[2] = (uint8_t)(sh & 0xff);
    b[3] = (uint8_t)(sh >> 8);
    std::memcpy(b + 4, sl, 4);
  }
  for (int i = 0; i < kBlocks; i++)
    for (int j = 0; j < 16; j++) qs[16 * i + j] = (uint8_t)(lv[32 * i + j] | (lv[32 * i + 16 + j] << 4));
}

typedef void (*BlockEnc)(const float*, const float*, uint8_t*);
void legacy_q8_0(const float* x, const float*, uint8_t* b) { enc_q8_0(x, b); }
void legacy_q4_0(const float* x, const float*, uint8_t* b) { enc_legacy<false, 4>(x, b); }
void legacy_q4_1(const float* x, const float*, uint8_t* b) { enc_legacy<true, 4>(x, b); }
void legacy_q5_0(const float* x, const float*, uint8_t* b) { enc_legacy<false, 5>(x, b); }
void legacy_q5_1(const float* x, const float*, uint8_t* b) { enc_legacy<true, 5>(x, b); }

BlockEnc encoder_for(int codec) {
  switch (codec) {
    case KQ_Q8_0: return legacy_q8_0;
    case KQ_Q4_0: return legacy_q4_0;
    case KQ_Q4_1: return legacy_q4_1;
    case KQ_Q5_0: return legacy_q5_0;
    case KQ_Q5_1: return legacy_q5_1;
    case KQ_Q2_K: return enc_q2_k;
    case KQ_Q3_K: return enc_q3_k;
    case KQ_Q4_K: return enc_q45_k<4>;
    case KQ_Q5_K: return enc_q45_k<5>;
    case KQ_Q6_K: return enc_q6_k;
    case KQ_IQ4_NL: return enc_iq4<32>;
    case KQ_IQ4_XS: return enc_iq4<256>;
  }
  return nullptr;
}

}  // namespace

extern "C" int kq_quantize(const float* w_host, const float* imatrix_host, uint8_t* wire_host, int64_t rows, int64_t K,
                           int codec) {
  if (codec < 0 || codec >= KQ_NUM_CODECS) return kq_set_error(KQ_ERR_INVALID, "quantize: unknown codec id %d", codec);
  BlockEnc enc = encoder_for(codec);
  if (!enc) return kq_set_error(KQ_ERR_UNSUPPORTED, "quantize: no encoder for codec id %d in this build", codec);
  const KqGeom g = kq_geom(codec);
  if (rows < 0 || K < 0 || K % g.wpb) return kq_set_error(KQ_ERR_INVALID, "quantize: K (%lld) is not a multiple of %d",
                                                         (long long)K, g.wpb);
  if (rows == 0 || K == 0) return KQ_OK;
  if (!w_host || !wire_host) return kq_set_error(KQ_ERR_INVALID, "quantize: null buffer");
  const int64_t bpr = K / g.wpb, nblocks = rows * bpr;
  // the importance matrix steers the K-quants and the IQ codecs (flat-32 iq4_nl included); the legacy codecs ignore it
  const bool weighted = g.wpb == 256 || codec == KQ_IQ4_NL;
  auto work = [&](int64_t b0, int64_t b1) {
    for (int64_t b = b0; b < b1; b++) {
      const float* im = (imatrix_host && weighted) ? imatrix_host + (b % bpr) * g.wpb : nullptr;
      enc(w_host + b * g.wpb, im, wire_host + b * g.bpb);
    }
  };
  int nt = (int)std::thread::hardware_concurrency();
  if (nt > 32) nt = 32;
  if (nt < 1 || nblocks < 64) nt = 1;
  if (nt == 1) {
    work(0, nblocks);
    return KQ_OK;
  }
  std::vector<std::thread> pool;
  for (int t = 0; t < nt; t++) pool.emplace_back(work, nblocks * t / nt, nblocks * (t + 1) / nt);
  for (auto& th : pool) th.join();
  return KQ_OK;
}
