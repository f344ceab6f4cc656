// Block encoders of the legacy 32-weight codecs and the K-quant superblock codecs, float values of one
// block -> wire bytes, compiled for the host (kq_quantize, kq_encode.cpp) and for the device
// (kq_quantize_dev, kq_encode_dev.hip) from this one source.  Plain float arithmetic in the reference's
// operation order (src/kquant_cpu_encode.cpp:38-859, ggml's search heuristics); both builds keep
// multiplies and adds unfused, so host and device write the same bytes.
#pragma once

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstring>

#if defined(__HIP__) || defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define KQ_HD __host__ __device__
#else
#define KQ_HD
#endif

namespace kqenc {

KQ_HD inline void put_f16(uint8_t* p, float v) {
  _Float16 h = static_cast<_Float16>(v);
  std::memcpy(p, &h, 2);
}
KQ_HD inline float get_f16(const uint8_t* p) {
  _Float16 h;
  std::memcpy(&h, p, 2);
  return static_cast<float>(h);
}
KQ_HD inline int rne(float v) { return static_cast<int>(std::rint(v)); }  // kq_nearest_int, encode_util.h:41-43
KQ_HD inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// ------------------------------------------------------------------ legacy 32-weight codecs
KQ_HD inline void enc_q8_0(const float* x, uint8_t* b) {
  float amax = 0.f;
  for (int j = 0; j < 32; j++) amax = std::max(amax, std::fabs(x[j]));
  const float d = amax / 127.0f, id = d != 0.f ? 1.0f / d : 0.f;
  put_f16(b, d);
  for (int j = 0; j < 32; j++)
    reinterpret_cast<int8_t*>(b + 2)[j] = static_cast<int8_t>(std::clamp(std::round(x[j] * id), -127.0f, 127.0f));
}

template <bool kHasMin, int kBits>
KQ_HD inline void enc_legacy(const float* x, uint8_t* b) {
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
KQ_HD inline float fit_scale_min(const float* x, const float* wt, int n, int nmax, float* neg_min) {
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
KQ_HD inline float fit_positive(const float* x, const float* wt, int n, int nmax, uint8_t* out) {
  float vmax = 0.f;
  for (int i = 0; i < n; i++)
    if (x[i] > vmax) vmax = x[i];
  if (vmax < 1e-30f) {
    for (int i = 0; i < n; i++) out[i] = 0;
    return 0.f;
  }
  float inv = float(nmax) / vmax;
  uint8_t lv[32];
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
KQ_HD inline float fit_signed16(const float* x, const float* wt, int nmax) {
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
KQ_HD inline void importance(const float* x, const float* imatrix_blk, float sigma_factor, float* wt) {
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
KQ_HD inline void pack_2bit(const uint8_t* lv, uint8_t* qs) {
  for (int i = 0; i < 64; i++) {
    const int h = i >> 5, l = i & 31;
    uint8_t byte = 0;
    for (int s = 0; s < 4; s++) byte |= uint8_t((lv[128 * h + 32 * s + l] & 3) << (2 * s));
    qs[i] = byte;
  }
}

template <int kBits>  // 4 or 5
KQ_HD inline void enc_q45_k(const float* x, const float* im, uint8_t* b) {
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

KQ_HD inline void enc_q6_k(const float* x, const float* im, uint8_t* b) {
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

KQ_HD inline void enc_q3_k(const float* x, const float* im, uint8_t* b) {
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

KQ_HD inline void enc_q2_k(const float* x, const float* im, uint8_t* b) {
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

}  // namespace kqenc
