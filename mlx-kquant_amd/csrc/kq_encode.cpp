// Host-side wire encoders behind kq_quantize: float rows -> GGUF block bytes for the five legacy
// 32-weight codecs, the five K-quant superblock codecs, the two non-linear 4-bit codecs
// (iq4_nl, iq4_xs) and seven codebook codecs (iq2_xxs, iq2_xs, iq2_s, iq3_xxs, iq3_s, iq1_s, iq1_m).  Like the reference's encoder
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
//   codebook: iq2_xxs :392-598, iq2_xs :600-818, iq2_s :821-1029, iq3_xxs :1087-1310, iq3_s :1319-1544 (lattice search over the codebook
//             with its neighbour index :228-331; one shared implementation driven by a traits table)
//   ternary : iq1_s :1546-1798, iq1_m :1806-2098 (two-boundary search over the sorted sub-block, codebook snap)
#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstring>
#include <mutex>
#include <thread>
#include <utility>
#include <vector>

#include "kq_common.h"
#include "kq_encode_blocks.h"

namespace {

using namespace kqenc;

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

// ------------------------------------------------------------------ codebook codecs (iq2_xxs, iq2_xs, iq2_s, iq3_xxs, iq3_s)
// A 32-weight sub-block is a scale times odd lattice points 2 l + 1 that must belong to a codebook
// of 8-value (iq2) or 4-value (iq3) groups, plus one sign per weight.  The search representation
// is derived from the decode codebooks linked into the library: the level of a value is its rank
// among the distinct values of the codebook.  For every lattice point that is not in the codebook
// the entries at the `rings` smallest distinct distances are kept as candidates (ties ordered by
// entry number), as ggml's iq2xs_init_impl / iq3xs_init_impl do (reference :228-331).
extern "C" const uint8_t kq_grid_blob_host[];

struct Codebook {
  int dim = 0, bits = 0, size = 0;
  std::vector<int8_t> pts;     // [size][dim] coordinates 2 l + 1
  std::vector<int32_t> slot;   // packed levels -> entry, or -(offset into near) - 1
  std::vector<uint16_t> near;  // per off-codebook point: count, entries...
};

void build_codebook(Codebook& cb, const uint8_t* values, int size, int dim, int bits, int rings, bool is_signed = false) {
  cb.dim = dim;
  cb.bits = bits;
  cb.size = size;
  bool seen[256] = {};
  for (int i = 0; i < size * dim; i++) seen[values[i]] = true;
  int level_of[256], nlevels = 0;
  // levels by rank of the value (int8 values for the ternary codebook: -1, 0, 1)
  for (int r = 0; r < 256; r++) {
    const int v = is_signed ? ((r + 128) & 255) : r;  // -128 .. 127 in order, as bytes
    level_of[v] = seen[v] ? nlevels++ : -1;
  }
  cb.pts.resize((size_t)size * dim);
  const int npacked = 1 << (bits * dim), mask = (1 << bits) - 1;
  cb.slot.assign(npacked, 0);
  std::vector<char> member(npacked, 0);
  for (int e = 0; e < size; e++) {
    int packed = 0;
    for (int i = 0; i < dim; i++) {
      const int l = level_of[values[e * dim + i]];
      cb.pts[(size_t)e * dim + i] = int8_t(2 * l + 1);
      packed |= l << (bits * i);
    }
    cb.slot[packed] = e;
    member[packed] = 1;
  }
  std::vector<std::pair<int, int>> order(size);
  for (int p = 0; p < npacked; p++) {
    if (member[p]) continue;
    int8_t pos[8];
    bool reachable = true;
    for (int i = 0; i < dim; i++) {
      const int l = (p >> (bits * i)) & mask;
      if (l >= nlevels) reachable = false;  // the encoder clamps levels below nlevels
      pos[i] = int8_t(2 * l + 1);
    }
    if (!reachable) {
      cb.slot[p] = 0;
      continue;
    }
    for (int e = 0; e < size; e++) {
      int d2 = 0;
      for (int i = 0; i < dim; i++) {
        const int df = cb.pts[(size_t)e * dim + i] - pos[i];
        d2 += df * df;
      }
      order[e] = {d2, e};
    }
    std::sort(order.begin(), order.end());
    const int32_t off = (int32_t)cb.near.size();
    cb.near.push_back(0);
    int ring = 1, cur = order[0].first, count = 0;
    for (int e = 0; e < size; e++) {
      if (order[e].first > cur) {
        if (ring == rings) break;
        cur = order[e].first;
        ring++;
      }
      cb.near.push_back(uint16_t(order[e].second));
      count++;
    }
    cb.near[off] = uint16_t(count);
    cb.slot[p] = -off - 1;
  }
}

enum { CB_IQ2XXS = 0, CB_IQ2XS, CB_IQ2S, CB_IQ3XXS, CB_IQ3S, CB_IQ1, CB_COUNT };
const Codebook& codebook(int which) {
  static Codebook books[CB_COUNT];
  static std::once_flag once[CB_COUNT];
  std::call_once(once[which], [which] {
    if (which == CB_IQ2XXS) build_codebook(books[which], kq_grid_blob_host + KQ_GRID_IQ2XXS, 256, 8, 2, 2);
    if (which == CB_IQ2XS) build_codebook(books[which], kq_grid_blob_host + KQ_GRID_IQ2XS, 512, 8, 2, 2);
    if (which == CB_IQ2S) build_codebook(books[which], kq_grid_blob_host + KQ_GRID_IQ2S, 1024, 8, 2, 1);
    if (which == CB_IQ3XXS) build_codebook(books[which], kq_grid_blob_host + KQ_GRID_IQ3XXS, 256, 4, 3, 2);
    if (which == CB_IQ3S) build_codebook(books[which], kq_grid_blob_host + KQ_GRID_IQ3S, 512, 4, 3, 3);
    if (which == CB_IQ1) build_codebook(books[which], kq_grid_blob_host + KQ_GRID_IQ1S, 2048, 8, 2, 3, true);
  });
  return books[which];
}

// Levels of one group at inverse scale `inv`, snapped to the codebook: the rounded lattice point if it is
// an entry, else the candidate with the least weighted error (weights sw = sqrt of the importance).
// Returns the entry; *exact tells whether no snapping was needed.
int snap_group(const Codebook& cb, const float* xv, const float* sw, float inv, int maxq, int8_t* lv, bool* exact) {
  int packed = 0;
  for (int i = 0; i < cb.dim; i++) {
    const int l = clampi(rne(0.5f * (inv * xv[i] - 1.0f)), 0, maxq - 1);
    lv[i] = int8_t(l);
    packed |= l << (cb.bits * i);
  }
  const int32_t s = cb.slot[packed];
  if (s >= 0) {
    *exact = true;
    return s;
  }
  *exact = false;
  const uint16_t* cand = cb.near.data() + (-s - 1);
  const float scale = 1.0f / inv;
  float best = FLT_MAX;
  int pick = -1;
  for (int c = 1; c <= int(cand[0]); c++) {
    const int8_t* pt = cb.pts.data() + (size_t)cand[c] * cb.dim;
    float err = 0.f;
    for (int i = 0; i < cb.dim; i++) {
      const float df = scale * float(pt[i]) - xv[i];
      err += sw[i] * df * df;
    }
    if (err < best) {
      best = err;
      pick = cand[c];
    }
  }
  const int8_t* pt = cb.pts.data() + (size_t)pick * cb.dim;
  for (int i = 0; i < cb.dim; i++) lv[i] = int8_t((pt[i] - 1) / 2);
  return pick;
}

struct CbTraits {
  int nw;               // weights per sub-block (one scale): 32 or 16
  float fallback_sigma; // importance without an imatrix: fallback_sigma * sigma2 + x^2
  int book, maxq;       // codebook, levels per coordinate
  float sigma_factor;   // importance prologue
  bool parity_signs;    // 7 stored sign bits per 8 weights (even parity enforced) vs 8
  float zero_eps;       // sub-blocks whose largest magnitude is below this encode as zero
  bool qp_start;        // starting scale from the positive-scale fit (iq2_xxs) vs max / (2 maxq - 1)
  int scan;             // candidate scales -scan..scan
  float scan_step;
  int refine;           // 0: refit every sub-block; 1: only sub-blocks with a snapped group, all groups;
                        // 2: only the snapped groups
  float d_fudge;
};
constexpr CbTraits kIq2xxs{32, 0.f, CB_IQ2XXS, 3, 1.0f, true, 1e-15f, true, 6, 0.1f, 0, 1.0f};
constexpr CbTraits kIq2xs{16, 0.f, CB_IQ2XS, 3, 1.0f, true, 1e-15f, false, 9, 0.1f, 2, 1.0f};
constexpr CbTraits kIq2s{16, 0.25f, CB_IQ2S, 3, 2.0f, false, 1e-8f, false, 9, 0.1f, 2, 0.9875f};
constexpr CbTraits kIq3xxs{32, 0.f, CB_IQ3XXS, 8, 2.0f, true, 1e-8f, false, 15, 0.2f, 2, 1.0125f};
constexpr CbTraits kIq3s{32, 0.f, CB_IQ3S, 8, 2.0f, false, 0.0f, false, 9, 0.2f, 1, 1.033f};

// One 32-weight sub-block: magnitudes, signs, weights in; levels, codebook entries, sign bytes and the
// scale out (ggml quantize_row_iq2_xxs_impl / iq3_xxs_impl / iq3_s_impl; reference :392-598, :1087-1310,
// :1319-1544).
float fit_codebook_subblock(const CbTraits& t, const float* xb, const float* imat, float sigma2, uint8_t* signs,
                            int* entries) {
  const Codebook& cb = codebook(t.book);
  const int nw = t.nw, ngroups = nw / cb.dim;
  float wt[32], sw[32], xv[32];
  for (int i = 0; i < nw; i++) {
    wt[i] = imat ? imat[i] * std::sqrt(sigma2 + xb[i] * xb[i]) : t.fallback_sigma * sigma2 + xb[i] * xb[i];
    sw[i] = std::sqrt(wt[i]);
  }
  for (int k = 0; k < nw / 8; k++) {
    uint8_t s = 0;
    int flips = 0;
    for (int i = 0; i < 8; i++) {
      const float v = xb[8 * k + i];
      xv[8 * k + i] = v >= 0.f ? v : -v;
      if (v < 0.f) {
        s |= uint8_t(1u << i);
        flips++;
      }
    }
    if (t.parity_signs) {
      if (flips & 1) {  // an odd group cannot be stored: give up the sign of the least important weight
        int imin = 0;
        float least = wt[8 * k] * xb[8 * k] * xb[8 * k];
        for (int i = 1; i < 8; i++) {
          const float a = wt[8 * k + i] * xb[8 * k + i] * xb[8 * k + i];
          if (a < least) {
            least = a;
            imin = i;
          }
        }
        xv[8 * k + imin] = -xv[8 * k + imin];
        s ^= uint8_t(1u << imin);
      }
      s &= 127;
    }
    signs[k] = s;
  }
  for (int g = 0; g < ngroups; g++) entries[g] = 0;
  float vmax = xv[0];
  for (int i = 1; i < nw; i++) vmax = std::max(vmax, xv[i]);
  if (t.zero_eps > 0.f ? vmax < t.zero_eps : !(vmax != 0.f)) return 0.f;

  int8_t lv[32] = {}, trial[32] = {};
  bool exact[8], trial_exact[8];
  float scale, span;
  if (t.qp_start) {
    uint8_t tmp[32];
    scale = fit_positive(xv, wt, nw, t.maxq + 1, tmp);
    span = scale * float(t.maxq);
    if (span <= 0.f) return 0.f;
    for (int g = 0; g < ngroups; g++) exact[g] = true;
  } else {
    span = vmax;
    scale = vmax / float(2 * t.maxq - 1);
    for (int g = 0; g < ngroups; g++) exact[g] = t.refine == 2;
  }
  auto sums = [&](const int8_t* l, float& sqx, float& sq2) {
    sqx = sq2 = 0.f;
    for (int i = 0; i < nw; i++) {
      const float q = float(2 * l[i] + 1);
      sqx += wt[i] * xv[i] * q;
      sq2 += wt[i] * q * q;
    }
  };
  float best = 0.f;
  for (int is = -t.scan; is <= t.scan; is++) {
    const float inv = (float(2 * t.maxq - 1) + float(is) * t.scan_step) / span;
    for (int g = 0; g < ngroups; g++)
      snap_group(cb, xv + cb.dim * g, sw + cb.dim * g, inv, t.maxq, trial + cb.dim * g, &trial_exact[g]);
    float sqx, sq2;
    sums(trial, sqx, sq2);
    if (sq2 > 0.f && sqx * sqx > best * sq2) {
      scale = sqx / sq2;
      best = scale * sqx;
      std::memcpy(lv, trial, 32);
      std::memcpy(exact, trial_exact, sizeof(exact));
    }
  }
  bool any_snapped = false;
  for (int g = 0; g < ngroups; g++) any_snapped |= !exact[g];
  if (scale > 0.f && (t.refine == 0 || any_snapped)) {
    const float inv = 1.0f / scale;
    for (int g = 0; g < ngroups; g++) {
      if (t.refine == 2 && exact[g]) continue;
      bool e;
      const int entry = snap_group(cb, xv + cb.dim * g, sw + cb.dim * g, inv, t.maxq, lv + cb.dim * g, &e);
      const int8_t* pt = cb.pts.data() + (size_t)entry * cb.dim;
      for (int i = 0; i < cb.dim; i++) lv[cb.dim * g + i] = int8_t((pt[i] - 1) / 2);
    }
    float sqx, sq2;
    sums(lv, sqx, sq2);
    if (sq2 > 0.f) scale = sqx / sq2;
  }
  if (scale < 0.f) {  // cannot happen with non-negative magnitudes; keep the wire's unsigned scale valid anyway
    scale = -scale;
    for (int k = 0; k < nw / 8; k++) signs[k] = uint8_t(~signs[k]) & (t.parity_signs ? 127 : 255);
  }
  for (int g = 0; g < ngroups; g++) {
    int packed = 0;
    for (int i = 0; i < cb.dim; i++) packed |= int(lv[cb.dim * g + i]) << (cb.bits * i);
    const int32_t s = cb.slot[packed];
    entries[g] = s >= 0 ? s : 0;  // always an entry: every group was snapped above
  }
  return scale;
}

// 4-bit sub-block scale: scale ~ d (2 l + 1)
inline int scale_level(float inv_d, float scale) { return clampi(rne(0.5f * (inv_d * scale - 1.0f)), 0, 15); }

template <int kWhich>  // KQ_IQ2_XXS, KQ_IQ3_XXS, KQ_IQ3_S
void enc_codebook(const float* x, const float* im, uint8_t* b) {
  const CbTraits& t = kWhich == KQ_IQ2_XXS ? kIq2xxs : kWhich == KQ_IQ3_XXS ? kIq3xxs : kIq3s;
  constexpr int kBytes = kWhich == KQ_IQ2_XXS ? 66 : kWhich == KQ_IQ3_XXS ? 98 : 110;
  float total = 0.f;
  for (int i = 0; i < 256; i++) total += x[i] * x[i];
  const float sigma2 = t.sigma_factor * total / 256.0f;
  float scales[8], top = 0.f;
  uint8_t signs[8][4];
  int entries[8][8];
  for (int ib = 0; ib < 8; ib++) {
    scales[ib] = fit_codebook_subblock(t, x + 32 * ib, im ? im + 32 * ib : nullptr, sigma2, signs[ib], entries[ib]);
    top = std::max(top, scales[ib]);
  }
  std::memset(b, 0, kBytes);
  if (!(top > 0.f)) return;
  const float d = top / 31.0f, inv_d = 1.0f / d;
  put_f16(b, d * t.d_fudge);
  if constexpr (kWhich == KQ_IQ2_XXS) {
    // per sub-block: four codebook bytes, then 4 x 7 sign bits and the 4-bit scale in one word
    for (int ib = 0; ib < 8; ib++) {
      uint8_t* q = b + 2 + 8 * ib;
      uint32_t word = uint32_t(scale_level(inv_d, scales[ib])) << 28;
      for (int k = 0; k < 4; k++) {
        q[k] = uint8_t(scales[ib] > 0.f ? entries[ib][k] : 0);
        if (scales[ib] > 0.f) word |= uint32_t(signs[ib][k]) << (7 * k);
      }
      std::memcpy(q + 4, &word, 4);
    }
  } else if constexpr (kWhich == KQ_IQ3_XXS) {
    // 64 codebook bytes, then per sub-block 4 x 7 sign bits and the 4-bit scale in one word
    for (int ib = 0; ib < 8; ib++) {
      uint32_t word = uint32_t(scale_level(inv_d, scales[ib])) << 28;
      for (int g = 0; g < 8; g++) b[2 + 8 * ib + g] = uint8_t(scales[ib] > 0.f ? entries[ib][g] : 0);
      if (scales[ib] > 0.f)
        for (int k = 0; k < 4; k++) word |= uint32_t(signs[ib][k]) << (7 * k);
      std::memcpy(b + 66 + 4 * ib, &word, 4);
    }
  } else {
    // qs[64] low entry bytes | qh[8] ninth bits | signs[32] | scales[4] (two nibbles each).  The qs and
    // sign cursors advance only over non-zero sub-blocks while qh uses the absolute group number
    // (reference :1329-1330, :1497-1508).
    int qpos = 0, spos = 0;
    for (int ib = 0; ib < 8; ib++) {
      if (!(scales[ib] > 0.f) && !std::any_of(x + 32 * ib, x + 32 * ib + 32, [](float v) { return v != 0.f; })) continue;
      for (int g = 0; g < 8; g++) {
        b[2 + qpos + g] = uint8_t(entries[ib][g] & 255);
        b[66 + ib] |= uint8_t((entries[ib][g] >> 8) << g);
      }
      qpos += 8;
      for (int k = 0; k < 4; k++) b[74 + spos + k] = signs[ib][k];
      spos += 4;
    }
    for (int ib = 0; ib < 8; ib += 2)
      b[106 + ib / 2] = uint8_t(scale_level(inv_d, scales[ib]) | (scale_level(inv_d, scales[ib + 1]) << 4));
  }
}

// iq2_xs (74 bytes: d | 32 x u16 = 9-bit entry + 7 sign bits | 8 scale bytes) and iq2_s (82 bytes: d | 32 entry
// low bytes | 32 sign bytes | 8 bytes of entry bits 8-9 | 8 scale bytes): sixteen 16-weight sub-blocks of two
// 8-value groups, a 4-bit scale each (reference :600-818, :821-1029).
template <int kWhich>  // KQ_IQ2_XS, KQ_IQ2_S
void enc_codebook16(const float* x, const float* im, uint8_t* b) {
  const CbTraits& t = kWhich == KQ_IQ2_XS ? kIq2xs : kIq2s;
  constexpr int kBytes = kWhich == KQ_IQ2_XS ? 74 : 82;
  float total = 0.f;
  for (int i = 0; i < 256; i++) total += x[i] * x[i];
  const float sigma2 = t.sigma_factor * total / 256.0f;
  float scales[16], top = 0.f;
  uint8_t signs[16][4];
  int entries[16][8];
  for (int ib = 0; ib < 16; ib++) {
    scales[ib] = fit_codebook_subblock(t, x + 16 * ib, im ? im + 16 * ib : nullptr, sigma2, signs[ib], entries[ib]);
    top = std::max(top, scales[ib]);
  }
  std::memset(b, 0, kBytes);
  if (!(top > 0.f)) return;
  const float d = top / 31.0f, inv_d = 1.0f / d;
  put_f16(b, d * t.d_fudge);
  for (int ib = 0; ib < 16; ib++) {
    for (int k = 0; k < 2; k++) {
      const int g = 2 * ib + k;
      const bool live = scales[ib] > 0.f;
      const int entry = live ? entries[ib][k] : 0;
      const int sg = live ? signs[ib][k] : 0;
      if constexpr (kWhich == KQ_IQ2_XS) {
        const uint16_t q = uint16_t(entry | (sg << 9));
        std::memcpy(b + 2 + 2 * g, &q, 2);
      } else {
        b[2 + g] = uint8_t(entry & 255);
        b[34 + g] = uint8_t(sg);
        b[66 + g / 4] |= uint8_t((entry >> 8) << (2 * (g % 4)));
      }
    }
    const int l = scale_level(inv_d, scales[ib]);
    b[(kWhich == KQ_IQ2_XS ? 66 : 74) + ib / 2] |= uint8_t(ib % 2 ? l << 4 : l);
  }
}

// ------------------------------------------------------------------ iq1_s
// Codebook entry for eight ternary levels (0, 1, 2): the entry itself when the group is on the codebook, else
// the neighbour closest to x under the weights at the given scale and level values; `lv` takes the levels of
// the entry picked (reference :1500-1544, iq1_find_best_neighbour2).
int snap_ternary(const Codebook& cb, int8_t* lv, const float* x, const float* wt, float scale, const float* v,
                 bool* exact) {
  int packed = 0;
  for (int i = 0; i < 8; i++) packed |= int(lv[i]) << (2 * i);
  const int32_t slot = cb.slot[packed];
  if (slot >= 0) return slot;
  *exact = false;
  const uint16_t* cand = cb.near.data() + (-slot - 1);
  float least = FLT_MAX;
  int pick = 0;
  for (int c = 1; c <= int(cand[0]); c++) {
    const int8_t* pt = cb.pts.data() + (size_t)cand[c] * 8;
    float err = 0.f;
    for (int i = 0; i < 8; i++) {
      const float df = scale * v[(pt[i] - 1) / 2] - x[i];
      err += wt[i] * df * df;
    }
    if (err < least) {
      least = err;
      pick = cand[c];
    }
  }
  const int8_t* pt = cb.pts.data() + (size_t)pick * 8;
  for (int i = 0; i < 8; i++) lv[i] = int8_t((pt[i] - 1) / 2);
  return pick;
}

// 50 bytes: d | 32 entry low bytes | 8 x u16 (4 x 3 entry high bits, 3-bit scale, shift sign).  A 32-weight
// sub-block is scale * (t + shift / 8) with t in {-1, 0, 1} drawn from the 2048-entry ternary codebook and one
// shift sign per sub-block.  The ternary split comes from an exhaustive search over the two boundaries in the
// sorted values (prefix sums of w x and w), for both shift signs; groups that miss the codebook snap to the
// best of their neighbours (ggml quantize_row_iq1_s_impl; reference :1546-1798).
void enc_iq1_s(const float* x, const float* im, uint8_t* b) {
  const Codebook& cb = codebook(CB_IQ1);
  constexpr float kDelta = 0.125f;
  const float vp[3] = {-1.f + kDelta, kDelta, 1.f + kDelta}, vm[3] = {-1.f - kDelta, -kDelta, 1.f - kDelta};
  float total = 0.f;
  for (int i = 0; i < 256; i++) total += x[i] * x[i];
  const float sigma2 = 2.0f * total / 256.0f;
  float scales[8], top = 0.f;
  int shifts[8], entries[8][4];
  for (int ib = 0; ib < 8; ib++) {
    const float* xb = x + 32 * ib;
    scales[ib] = 0.f;
    shifts[ib] = 1;
    for (int k = 0; k < 4; k++) entries[ib][k] = 0;
    float wt[32], vmax = 0.f;
    for (int i = 0; i < 32; i++) {
      wt[i] = (im ? im[32 * ib + i] : 1.0f) * std::sqrt(sigma2 + xb[i] * xb[i]);
      vmax = std::max(vmax, std::fabs(xb[i]));
    }
    if (vmax < 1e-12f) continue;
    int order[32];
    for (int i = 0; i < 32; i++) order[i] = i;
    std::stable_sort(order, order + 32, [&](int l, int r) { return xb[l] < xb[r]; });
    float sx[33], sw[33];
    sx[0] = sw[0] = 0.f;
    for (int j = 0; j < 32; j++) {
      sx[j + 1] = sx[j] + wt[order[j]] * xb[order[j]];
      sw[j + 1] = sw[j] + wt[order[j]];
    }
    float best = -FLT_MAX, scale = vmax;
    int b1 = -1, b2 = -1, shift = 0;
    for (int i1 = 0; i1 <= 32; i1++)
      for (int i2 = i1; i2 <= 32; i2++)
        for (int sgn = 1; sgn >= -1; sgn -= 2) {
          const float* v = sgn > 0 ? vp : vm;
          const float sqx = (sx[i1] - sx[0]) * v[0] + (sx[i2] - sx[i1]) * v[1] + (sx[32] - sx[i2]) * v[2];
          const float sq2 = (sw[i1] - sw[0]) * v[0] * v[0] + (sw[i2] - sw[i1]) * v[1] * v[1] + (sw[32] - sw[i2]) * v[2] * v[2];
          if (sq2 > 0.f && sqx * sqx > best * sq2) {
            scale = sqx / sq2;
            best = scale * sqx;
            b1 = i1;
            b2 = i2;
            shift = sgn;
          }
        }
    if (b1 < 0 || shift == 0) continue;
    int8_t lv[32];
    for (int j = 0; j < 32; j++) lv[order[j]] = int8_t(j < b1 ? 0 : j < b2 ? 1 : 2);
    if (scale < 0.f) {
      for (int j = 0; j < 32; j++) lv[j] = int8_t(2 - lv[j]);
      scale = -scale;
      shift = -shift;
    }
    const float* v = shift > 0 ? vp : vm;
    bool all_exact = true;
    for (int k = 0; k < 4; k++) {
      bool exact = true;
      const int slot = snap_ternary(cb, lv + 8 * k, xb + 8 * k, wt + 8 * k, scale, v, &exact);
      all_exact = all_exact && exact;
      entries[ib][k] = slot;
    }
    if (!all_exact) {
      float sqx = 0.f, sq2 = 0.f;
      for (int i = 0; i < 32; i++) {
        const float q = v[lv[i]];
        sqx += wt[i] * q * xb[i];
        sq2 += wt[i] * q * q;
      }
      if (sqx > 0.f && sq2 > 0.f) scale = sqx / sq2;
    }
    scales[ib] = scale;
    shifts[ib] = shift;
    top = std::max(top, scale);
  }
  std::memset(b, 0, 50);
  if (!(top > 0.f)) return;
  const float d = top / 15.0f, inv_d = 1.0f / d;
  put_f16(b, d * 1.125f);
  for (int ib = 0; ib < 8; ib++) {
    uint16_t h = 0;
    for (int k = 0; k < 4; k++) {
      b[2 + 4 * ib + k] = uint8_t(entries[ib][k] & 255);
      h |= uint16_t((entries[ib][k] >> 8) << (3 * k));
    }
    int l = clampi(rne(0.5f * (inv_d * scales[ib] - 1.0f)), 0, 7);
    if (shifts[ib] == -1) l |= 8;
    h |= uint16_t(l << 12);
    std::memcpy(b + 34 + 2 * ib, &h, 2);
  }
}

// ------------------------------------------------------------------ iq1_m
// 56 bytes: 32 entry low bytes | 16 qh bytes (two 3-bit entry tops + two shift-sign bits) | 4 x u16 (four 3-bit
// scales; the top nibbles spell the f16 block scale).  Sixteen 16-weight sub-blocks of two 8-value groups; the
// ternary split is shared by the sub-block, the shift sign is per group, so the boundary search scores the four
// sign pairs from per-group prefix sums (ggml quantize_row_iq1_m_impl; reference :1806-2098).  Without an
// importance matrix the weights are x^2.
void enc_iq1_m(const float* x, const float* im, uint8_t* b) {
  const Codebook& cb = codebook(CB_IQ1);
  constexpr float kDelta = 0.125f;
  const float vp[3] = {-1.f + kDelta, kDelta, 1.f + kDelta}, vm[3] = {-1.f - kDelta, -kDelta, 1.f - kDelta};
  // sign pair s: group 0 takes vm when s & 2, group 1 when s & 1
  auto values = [&](int s, int g) { return ((g == 0 ? s >> 1 : s) & 1) ? vm : vp; };
  float total = 0.f;
  for (int i = 0; i < 256; i++) total += x[i] * x[i];
  const float sigma2 = 2.0f * total / 256.0f;
  float wt[256];
  for (int i = 0; i < 256; i++) wt[i] = im ? im[i] * std::sqrt(sigma2 + x[i] * x[i]) : x[i] * x[i];
  float scales[16], top = 0.f;
  int pairs[16], entries[16][2];
  for (int ib = 0; ib < 16; ib++) {
    const float* xb = x + 16 * ib;
    const float* wb = wt + 16 * ib;
    scales[ib] = 0.f;
    pairs[ib] = 0;
    entries[ib][0] = entries[ib][1] = std::max(0, cb.slot[0x5555]);  // the all-middle group, when the codebook has it
    float vmax = 0.f;
    for (int i = 0; i < 16; i++) vmax = std::max(vmax, std::fabs(xb[i]));
    if (vmax < 1e-7f) continue;
    int order[16];
    for (int i = 0; i < 16; i++) order[i] = i;
    std::stable_sort(order, order + 16, [&](int l, int r) { return xb[l] < xb[r]; });
    float sx[2][17], sw[2][17];
    sx[0][0] = sx[1][0] = sw[0][0] = sw[1][0] = 0.f;
    for (int j = 0; j < 16; j++) {
      const int i = order[j], g = i / 8;
      sx[g][j + 1] = sx[g][j] + wb[i] * xb[i];
      sw[g][j + 1] = sw[g][j] + wb[i];
      sx[g ^ 1][j + 1] = sx[g ^ 1][j];
      sw[g ^ 1][j + 1] = sw[g ^ 1][j];
    }
    float best = -FLT_MAX, scale = vmax;
    int b1 = -1, b2 = -1, pair = -1;
    for (int i1 = 0; i1 <= 16; i1++)
      for (int i2 = i1; i2 <= 16; i2++)
        for (int s = 0; s < 4; s++) {
          float sqx = 0.f, sq2 = 0.f;
          for (int g = 0; g < 2; g++) {
            const float* v = values(s, g);
            const float x0 = sx[g][i1], x1 = sx[g][i2] - sx[g][i1], x2 = sx[g][16] - sx[g][i2];
            const float w0 = sw[g][i1], w1 = sw[g][i2] - sw[g][i1], w2 = sw[g][16] - sw[g][i2];
            sqx += x0 * v[0] + x1 * v[1] + x2 * v[2];
            sq2 += w0 * v[0] * v[0] + w1 * v[1] * v[1] + w2 * v[2] * v[2];
          }
          if (sq2 > 0.f && sqx * sqx > best * sq2) {
            scale = sqx / sq2;
            best = scale * sqx;
            b1 = i1;
            b2 = i2;
            pair = s;
          }
        }
    if (pair < 0) continue;
    int8_t lv[16];
    for (int j = 0; j < 16; j++) lv[order[j]] = int8_t(j < b1 ? 0 : j < b2 ? 1 : 2);
    if (scale < 0.f) {  // mirror: -(t + delta) = (-t) - delta
      for (int j = 0; j < 16; j++) lv[j] = int8_t(2 - lv[j]);
      scale = -scale;
      pair = 3 - pair;
    }
    bool all_exact = true;
    for (int g = 0; g < 2; g++)
      entries[ib][g] = snap_ternary(cb, lv + 8 * g, xb + 8 * g, wb + 8 * g, scale, values(pair, g), &all_exact);
    if (!all_exact) {
      float sqx = 0.f, sq2 = 0.f;
      for (int i = 0; i < 16; i++) {
        const float q = values(pair, i / 8)[lv[i]];
        sqx += wb[i] * q * xb[i];
        sq2 += wb[i] * q * q;
      }
      if (sqx > 0.f && sq2 > 0.f) scale = sqx / sq2;
    }
    scales[ib] = scale;
    pairs[ib] = pair;
    top = std::max(top, scale);
  }
  std::memset(b, 0, 56);
  if (!(top > 0.f)) return;
  float d = top / 15.0f;
  const float inv_d = 1.0f / d;
  uint16_t sc[4] = {0, 0, 0, 0};
  float sqx = 0.f, sq2 = 0.f;
  for (int ib = 0; ib < 16; ib++) {
    const int l = clampi(rne(0.5f * (inv_d * scales[ib] - 1.0f)), 0, 7);
    sc[ib / 4] |= uint16_t(l << (3 * (ib % 4)));
    uint8_t h = 0;
    for (int g = 0; g < 2; g++) {
      const int e = entries[ib][g];
      b[2 * ib + g] = uint8_t(e & 255);
      h |= uint8_t((e >> 8) << (4 * g));
      if (values(pairs[ib], g) == vm) h |= uint8_t(0x08 << (4 * g));
      const int8_t* pt = cb.pts.data() + (size_t)e * 8;
      for (int i = 0; i < 8; i++) {
        const int at = 16 * ib + 8 * g + i;
        const float q = values(pairs[ib], g)[(pt[i] - 1) / 2] * float(2 * l + 1);
        sqx += wt[at] * q * x[at];
        sq2 += wt[at] * q * q;
      }
    }
    b[32 + ib] = h;
  }
  if (sq2 > 0.f) d = sqx / sq2;  // least-squares block scale for the scale levels just fixed
  const _Float16 hd = (_Float16)(d * 1.1125f);
  uint16_t du;
  std::memcpy(&du, &hd, 2);
  for (int k = 0; k < 4; k++) sc[k] |= uint16_t(((du >> (4 * k)) & 15) << 12);
  std::memcpy(b + 48, sc, 8);
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
    case KQ_IQ2_XXS: return enc_codebook<KQ_IQ2_XXS>;
    case KQ_IQ2_XS: return enc_codebook16<KQ_IQ2_XS>;
    case KQ_IQ2_S: return enc_codebook16<KQ_IQ2_S>;
    case KQ_IQ1_S: return enc_iq1_s;
    case KQ_IQ1_M: return enc_iq1_m;
    case KQ_IQ3_XXS: return enc_codebook<KQ_IQ3_XXS>;
    case KQ_IQ3_S: return enc_codebook<KQ_IQ3_S>;
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
