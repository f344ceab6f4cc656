// Building blocks shared by the matrix-core kernels (prefill GEMM, grouped MoE GEMM): wire
// geometry of the K-quant superblocks as they travel HBM -> registers -> LDS, and the
// per-superblock multiply-accumulate of one wave (32 weight rows x MT*32 activation rows).
//
// Numerics.  The B operand of v_mfma_f32_32x32x16_f16 always holds exact integers:
//   q4_k / q5_k : sc_j*q (<= 63*31 < 2048), from 0x6400 | q = 1024 + q and one v_pk_fma_f16; the
//                 -dmin*m_j term is one extra MFMA per superblock on the sub-block sums of x
//                 (X_j split into two f16 halves);
//   q6_k        : sc*(q - 32) reaches 4096, so a weight is fed as two exact terms, sc*ql (<= 1920)
//                 and 16*sc*(qh - 2) (a multiple of 16 up to 4096): two MFMAs share one activation
//                 fragment.
// One f32 accumulator set collects a whole superblock and is folded into the running sum with one
// multiply by d, so results differ from the f32 reference only by summation order.
#pragma once

#include <type_traits>

#include "kq_decode.h"

namespace kqmma {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 16-byte global load from a 2-byte-aligned address (q6_k blocks are 210 bytes long): the
// hardware serves unaligned vector loads, the type only stops the compiler from assuming more
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));

// Compile-time loop: register arrays indexed by the loop variable are split into scalars.
template <int N>
struct StaticFor {
  template <class F>
  __device__ __forceinline__ static void run(F&& f) {
    StaticFor<N - 1>::run(f);
    f(std::integral_constant<int, N - 1>{});
  }
};
template <>
struct StaticFor<0> {
  template <class F>
  __device__ __forceinline__ static void run(F&&) {}
};

// Workgroup barrier that orders LDS traffic only (__syncthreads() would also drain every
// outstanding global load).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
// Constants routed through registers the compiler cannot see through, so that (a & mask) | magic
// becomes one v_and_or_b32 (VOP3 takes no literal operands on this target).
__device__ __forceinline__ uint32_t opaque_vgpr(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}
__device__ __forceinline__ uint32_t opaque_sgpr(uint32_t v) {
  asm volatile("" : "+s"(v));
  return v;
}

// ------------------------------------------------------------------ activation prepass (one row, 256 threads)
// Outputs for row m (rows >= M are written as zeros):
//   xh   f16 [Mpad][K]            x * 2^-e[m], k permuted inside 8-groups to k0 k2 k1 k3 k4 k6 k5 k7
//   xhl  f16 [Mpad][K/256][16]    per superblock: hi_j (8) then lo_j (8) with X_j = 32 (hi_j + lo_j)
//        S16: [Mpad][K/256][32]   sums of the 16-weight sub-blocks: hi_s (16) then lo_s (16), X_s = 16 (hi_s + lo_s)
//   rs   f32 [Mpad]               2^e[m]
// `red` = 4 floats of LDS; every thread of the workgroup must call (one barrier inside for bf16 input).
constexpr int PP_THREADS = 256;

// IL16: xh keeps x[j], x[j + 16] interleaved over every 32 values instead (a byte of an iq4 block holds weights j
// and j + 16 of its sub-block).
template <int DT, bool S16 = false, bool IL16 = false>
__device__ __forceinline__ void prepass_row(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
                                            _Float16* __restrict__ xhl, float* __restrict__ rs, int M, int K, int m,
                                            int tid, float* red) {
  const int ngroups = K >> 3;
  constexpr int HPS = S16 ? 32 : 16;  // halves per superblock in xhl
  _Float16* xo = xh + (size_t)m * K;
  _Float16* ho = xhl + (size_t)m * (K >> 8) * HPS;
  if (m >= M) {
    for (int g = tid; g < ngroups; g += PP_THREADS) *reinterpret_cast<u32x4*>(xo + 8 * g) = u32x4{0, 0, 0, 0};
    for (int i = tid; i < (K >> 8) * HPS; i += PP_THREADS) ho[i] = (_Float16)0.f;
    if (tid == 0) rs[m] = 0.f;
    return;
  }
  const uint16_t* xi = x + (size_t)m * K;
  float inv = 1.f, scale = 1.f;
  if constexpr (DT == KQ_BF16) {
    float amax = 0.f;
    for (int g = tid; g < ngroups; g += PP_THREADS) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(xi + 8 * g);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] << 16)));
        amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] & 0xffff0000u)));
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const uint32_t eb = (__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff;
    if (eb != 0 && eb != 0xff) {
      int e = (int)eb - 127 - 14;  // largest magnitude lands in [2^14, 2^15)
      if (e < -100) e = -100;
      scale = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
      inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
    }
  }
  if (tid == 0) rs[m] = scale;
  for (int g = tid; g < ngroups; g += PP_THREADS) {  // ngroups is a multiple of 32: whole quads stay together
    const u32x4 v = *reinterpret_cast<const u32x4*>(xi + 8 * g);
    _Float16 h[8];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      if constexpr (DT == KQ_BF16) {
        h[2 * e] = (_Float16)(__builtin_bit_cast(float, v[e] << 16) * inv);
        h[2 * e + 1] = (_Float16)(__builtin_bit_cast(float, v[e] & 0xffff0000u) * inv);
      } else {
        h[2 * e] = __builtin_bit_cast(_Float16, (uint16_t)(v[e] & 0xffff));
        h[2 * e + 1] = __builtin_bit_cast(_Float16, (uint16_t)(v[e] >> 16));
      }
    }
    if constexpr (IL16) {
      // threads g and g ^ 2 hold x[8 a ..] and x[16 + 8 a ..] of a 32-block and write one half each of the 16
      // interleaved values
      uint32_t own[4], par[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        own[e] = (uint32_t)__builtin_bit_cast(uint16_t, h[2 * e]) | ((uint32_t)__builtin_bit_cast(uint16_t, h[2 * e + 1]) << 16);
        par[e] = __shfl_xor(own[e], 2);
      }
      const bool high = (g & 2) != 0;
      const uint32_t a0 = high ? par[2] : own[0], a1 = high ? par[3] : own[1];
      const uint32_t b0 = high ? own[2] : par[0], b1 = high ? own[3] : par[1];
      const u32x4 o = {(a0 & 0xffffu) | (b0 << 16), (a0 >> 16) | (b0 & 0xffff0000u), (a1 & 0xffffu) | (b1 << 16),
                       (a1 >> 16) | (b1 & 0xffff0000u)};
      *reinterpret_cast<u32x4*>(xo + 32 * (g >> 2) + 16 * (g & 1) + (high ? 8 : 0)) = o;
      continue;
    }
    const f16x8 o = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
    *reinterpret_cast<f16x8*>(xo + 8 * g) = o;
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) s += (float)h[e];
    s += __shfl_xor(s, 1);
    if constexpr (S16) {  // 2 threads = one 16-wide sub-block
      if ((tid & 1) == 0) {
        const int j = g >> 1;  // global 16-wide sub-block index
        const _Float16 hi = (_Float16)(s * 0.0625f);
        const _Float16 lo = (_Float16)((s - 16.0f * (float)hi) * 0.0625f);
        ho[(j >> 4) * 32 + (j & 15)] = hi;
        ho[(j >> 4) * 32 + 16 + (j & 15)] = lo;
      }
      continue;
    }
    s += __shfl_xor(s, 2);  // 4 threads = one 32-wide sub-block
    if ((tid & 3) == 0) {
      const int j = g >> 2;  // global sub-block index
      const _Float16 hi = (_Float16)(s * 0.03125f);
      const _Float16 lo = (_Float16)((s - 32.0f * (float)hi) * 0.03125f);
      ho[(j >> 3) * 16 + (j & 7)] = hi;
      ho[(j >> 3) * 16 + 8 + (j & 7)] = lo;
    }
  }
}

// A superblock travels as PP 16-byte pieces (q6_k: its first 208 bytes; the trailing 2-byte d
// goes through a side channel) and is parked in LDS LBPB bytes apart.  LBPB / 16 is odd for all
// three codecs, which keeps the row-per-lane ds_read_b128 of the fragment fetch conflict-free.
template <int C>
struct Wire;
template <>
struct Wire<KQ_Q4_K> {
  static constexpr int BPB = 144, LBPB = 144, PP = 9, QS = 16;
  static constexpr bool SIDE_D = false, MINS = true;
  typedef u32x4 piece_t;
};
template <>
struct Wire<KQ_Q5_K> {
  static constexpr int BPB = 176, LBPB = 176, PP = 11, QS = 48;
  static constexpr bool SIDE_D = false, MINS = true;
  typedef u32x4 piece_t;
};
template <>
struct Wire<KQ_Q6_K> {
  static constexpr int BPB = 210, LBPB = 208, PP = 13, QS = 0;
  static constexpr bool SIDE_D = true, MINS = false;
  typedef u32x4_a2 piece_t;
};

// One superblock of one wave: weight row of this lane at b_lane (LDS), activation fragments at
// a_lane + t*a_tile + 64 j + 16 s bytes (a_lane already includes the lane's row and 32*kg), the X
// halves of m-block t at h_lane + t*h_tile (already including the lane's row and 16*kg).
// acc[t] += (decoded weights) . (activations) for the MT m-blocks.
template <int C, int MT>
__device__ __forceinline__ void superblock_mma(const uint8_t* __restrict__ b_lane, uint16_t d_side, int kg,
                                               const uint8_t* __restrict__ a_lane, int a_tile,
                                               const uint8_t* __restrict__ h_lane, int h_tile, f32x16* acc) {
  using G = Wire<C>;
  const uint32_t magic = opaque_vgpr(0x64006400u);
  f32x16 part[MT];
  if constexpr (C == KQ_Q4_K || C == KQ_Q5_K) {
    const uint32_t mask_lo = opaque_sgpr(0x000f000fu), mask_hi = opaque_sgpr(0x00f000f0u);
    const uint32_t mask5_lo = opaque_sgpr(0x00100010u), mask5_hi = opaque_sgpr(0x01000100u);
    (void)mask5_lo;
    (void)mask5_hi;
    const uint4 hdr = *reinterpret_cast<const uint4*>(b_lane);
    const float d = kq::h2f((uint16_t)(hdr.x & 0xffff));
    const float dmin32 = kq::h2f((uint16_t)(hdr.x >> 16)) * 32.0f;
    const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
    const uint32_t scw[2] = {s0 & 0x3f3f3f3fu, (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u)};
    const uint32_t mnw[2] = {s1 & 0x3f3f3f3fu, ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u)};
    // 16 MFMA groups (sub-block j = it / 2, K-half s = it % 2).  The activation fragments of group
    // it + 1 are requested before group it is decoded, so the LDS latency hides behind the decode
    // and the MFMAs instead of stalling each group.
    f16x8 afr[2][MT], bfr[2];
    uint4 qv[4];
    uint32_t hb[4] = {0, 0, 0, 0};  // q5_k: fifth bits of this lane's 16 weights, positioned per pair
#pragma unroll
    for (int g = 0; g < 4; g++) qv[g] = *reinterpret_cast<const uint4*>(b_lane + G::QS + 32 * g + 16 * kg);
    if constexpr (C == KQ_Q5_K) {
      const uint4 hv = *reinterpret_cast<const uint4*>(b_lane + 16 + 16 * kg);
      hb[0] = hv.x;
      hb[1] = hv.y;
      hb[2] = hv.z;
      hb[3] = hv.w;
    }
#pragma unroll
    for (int t = 0; t < MT; t++) afr[0][t] = *reinterpret_cast<const f16x8*>(a_lane + t * a_tile);
    // B fragment of group it: sub-block j = it / 2, K-half s = it % 2
    auto decode = [&](auto itc) -> f16x8 {
      constexpr int it = decltype(itc)::value;
      constexpr int j = it >> 1, s = it & 1, g = j >> 1, h = j & 1;
      const uint32_t qw[4] = {qv[g].x, qv[g].y, qv[g].z, qv[g].w};
      const float scf = (float)((scw[j >> 2] >> (8 * (j & 3))) & 0xff);
      // low nibbles read 1024 + q, high nibbles (in place) 1024 + 16 q: fold the 16 into the scale
      const _Float16 sch = (_Float16)(h ? scf * 0.0625f : scf);
      const _Float16 off = (_Float16)(-(h ? 64.0f : 1024.0f) * scf);
      const f16x2 scp = {sch, sch}, offp = {off, off};
      const uint32_t mask = h ? mask_hi : mask_lo;
      uint32_t fr[4] = {(qw[2 * s] & mask) | magic, ((qw[2 * s] >> 8) & mask) | magic,
                        (qw[2 * s + 1] & mask) | magic, ((qw[2 * s + 1] >> 8) & mask) | magic};
      if constexpr (C == KQ_Q5_K) {
        // fifth bit of weight (j, i) is bit j of qh[i]; this lane's bytes are qh[16 kg + 8 s + 0..7].  It joins the
        // code before the conversion: bit 4 next to a low nibble (1024 + q + 16 b), bit 8 next to a high nibble
        // held in place (1024 + 16 (q + 16 b)); both stay below 2048, so the operand is still exact.
        constexpr int P = h ? 8 : 4;
        const uint32_t mbit = h ? mask5_hi : mask5_lo;
        auto place = [&](uint32_t word, int from) -> uint32_t {  // bits `from`, `from + 16` -> P, P + 16
          return from >= P ? word >> (from - P) : word << (P - from);
        };
        fr[0] |= place(hb[2 * s], j) & mbit;
        fr[1] |= place(hb[2 * s], j + 8) & mbit;
        fr[2] |= place(hb[2 * s + 1], j) & mbit;
        fr[3] |= place(hb[2 * s + 1], j + 8) & mbit;
      }
      f16x2 bq[4];
#pragma unroll
      for (int e = 0; e < 4; e++)  // one rounding: (1024 + q) * sc - 1024 * sc = sc * q exactly
        bq[e] = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, fr[e]), scp, offp);
      return f16x8{bq[0][0], bq[0][1], bq[1][0], bq[1][1], bq[2][0], bq[2][1], bq[3][0], bq[3][1]};
    };
    // 16 MFMA groups, software-pipelined: while the matrix core runs the MFMAs of group it, the wave decodes
    // the B fragment of group it + 1 and requests its activation fragments.  A wave issues in order and a
    // second MFMA waits for the first to leave the matrix core, so vector work placed AFTER a run of MFMAs
    // would idle behind them; the group barriers below interleave it between them instead.
    constexpr int DEC_VALU = C == KQ_Q5_K ? 22 : 14;  // vector instructions of one decode, roughly
    bfr[0] = decode(std::integral_constant<int, 0>{});
    __builtin_amdgcn_sched_barrier(0);  // group 0's own fragments and decode stay out of the pipelined region
    StaticFor<16>::run([&](auto itc) {
      constexpr int it = decltype(itc)::value;
      if constexpr (it + 1 < 16) {
        constexpr int jn = (it + 1) >> 1, sn = (it + 1) & 1;
#pragma unroll
        for (int t = 0; t < MT; t++)
          afr[(it + 1) & 1][t] = *reinterpret_cast<const f16x8*>(a_lane + t * a_tile + 64 * jn + 16 * sn);
        bfr[(it + 1) & 1] = decode(std::integral_constant<int, it + 1>{});
      }
#pragma unroll
      for (int t = 0; t < MT; t++) {
        if constexpr (it == 0)
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t], bfr[0], f32x16{0}, 0, 0, 0);
        else
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[it & 1][t], bfr[it & 1], part[t], 0, 0, 0);
      }
      if constexpr (it + 1 < 16) {
        __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);  // the next group's fragment requests go first
#pragma unroll
        for (int t = 0; t < MT; t++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                          // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x002, (DEC_VALU + MT - 1) / MT, 0);   // a slice of the decode
        }
      }
    });
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[t][i] = fmaf(d, part[t][i], acc[t][i]);

    // mins: sum_j m_j X_j = 32 sum_j m_j (hi_j + lo_j); K slots 0..7 = hi, 8..15 = lo
    _Float16 mj[8];
#pragma unroll
    for (int j = 0; j < 8; j++) mj[j] = (_Float16)(float)((mnw[j >> 2] >> (8 * (j & 3))) & 0xff);
    const f16x8 bm = {mj[0], mj[1], mj[2], mj[3], mj[4], mj[5], mj[6], mj[7]};
#pragma unroll
    for (int t = 0; t < MT; t++) {
      const f16x8 a = *reinterpret_cast<const f16x8*>(h_lane + t * h_tile);
      part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bm, f32x16{0}, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[t][i] = fmaf(-dmin32, part[t][i], acc[t][i]);
  } else {
    // q6_k.  LDS block: ql[128] | qh[64] | int8 scales[16].  Weight 128 hf + 32 t + l (hf = half,
    // t = 0..3, l = 0..31) has its low nibble in ql[64 hf + 32 (t & 1) + l] (high nibble of the byte
    // when t >= 2), its high bits in bits 2t, 2t+1 of qh[32 hf + l] and scale 8 hf + 2 t + l / 16.
    // Lane (row, kg) takes l = 16 kg .. 16 kg + 15: one scale per lane and sub-block.
    const uint32_t mask_q = opaque_sgpr(0x00f000f0u), mask_h = opaque_sgpr(0x03000300u);
    const uint4 scv = *reinterpret_cast<const uint4*>(b_lane + 192);
    const uint32_t scw[4] = {scv.x, scv.y, scv.z, scv.w};
    // 16 groups in wire order: it = 8 hf + 4 qr + 2 h + s -> sub-block j = 4 hf + qr + 2 h, K-half s.
    // The activation fragments of group it + 1 are requested before group it is decoded.
    uint4 hv[2], qv[4];
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
      hv[hf] = *reinterpret_cast<const uint4*>(b_lane + 128 + 32 * hf + 16 * kg);
#pragma unroll
      for (int qr = 0; qr < 2; qr++)
        qv[2 * hf + qr] = *reinterpret_cast<const uint4*>(b_lane + 64 * hf + 32 * qr + 16 * kg);
    }
    f16x8 afr[2][MT];
#pragma unroll
    for (int t = 0; t < MT; t++) afr[0][t] = *reinterpret_cast<const f16x8*>(a_lane + t * a_tile);
    StaticFor<16>::run([&](auto itc) {
      constexpr int it = decltype(itc)::value;
      constexpr int hf = it >> 3, qr = (it >> 2) & 1, h = (it >> 1) & 1, s = it & 1;
      constexpr int t4 = qr + 2 * h;
      if constexpr (it + 1 < 16) {
        constexpr int n = it + 1;
        constexpr int jn = 4 * (n >> 3) + ((n >> 2) & 1) + 2 * ((n >> 1) & 1), sn = n & 1;
#pragma unroll
        for (int t = 0; t < MT; t++)
          afr[n & 1][t] = *reinterpret_cast<const f16x8*>(a_lane + t * a_tile + 64 * jn + 16 * sn);
        __builtin_amdgcn_sched_barrier(0);  // keep the requests ahead of this group's decode
      }
      const uint32_t hw[4] = {hv[hf].x, hv[hf].y, hv[hf].z, hv[hf].w};
      const uint32_t qw[4] = {qv[2 * hf + qr].x, qv[2 * hf + qr].y, qv[2 * hf + qr].z, qv[2 * hf + qr].w};
      const int sc = __builtin_amdgcn_sbfe((int)scw[2 * hf + (t4 >> 1)], 8 * (2 * (t4 & 1) + kg), 8);
      const float scf = (float)sc;
      const _Float16 sch = (_Float16)(scf * 0.0625f), ofl = (_Float16)(-64.0f * scf), ofh = (_Float16)(-96.0f * scf);
      const f16x2 scp = {sch, sch}, oflp = {ofl, ofl}, ofhp = {ofh, ofh};
      uint32_t fl[4], fh[4];
#pragma unroll
      for (int e = 0; e < 2; e++) {
        const uint32_t q = qw[2 * s + e], hq = hw[2 * s + e];
        const uint32_t qe = h ? q : (q << 4), qo = h ? (q >> 8) : (q >> 4);
        const uint32_t he = hq << (8 - 2 * t4), ho = t4 ? (hq >> (2 * t4)) : hq;
        fl[2 * e] = (qe & mask_q) | magic;      // bytes 0, 2 of the word: 1024 + 16 ql
        fl[2 * e + 1] = (qo & mask_q) | magic;  // bytes 1, 3
        fh[2 * e] = (he & mask_h) | magic;      // 1024 + 256 qh
        fh[2 * e + 1] = (ho & mask_h) | magic;
      }
      f16x2 bl2[4], bh2[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        // (1024 + 16 ql) sc / 16 - 64 sc = sc ql;  (1024 + 256 qh) sc / 16 - 96 sc = 16 sc (qh - 2)
        bl2[e] = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, fl[e]), scp, oflp);
        bh2[e] = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, fh[e]), scp, ofhp);
      }
      const f16x8 blo = {bl2[0][0], bl2[0][1], bl2[1][0], bl2[1][1], bl2[2][0], bl2[2][1], bl2[3][0], bl2[3][1]};
      const f16x8 bhi = {bh2[0][0], bh2[0][1], bh2[1][0], bh2[1][1], bh2[2][0], bh2[2][1], bh2[3][0], bh2[3][1]};
#pragma unroll
      for (int t = 0; t < MT; t++) {
        if constexpr (it == 0)
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t], blo, f32x16{0}, 0, 0, 0);
        else
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[it & 1][t], blo, part[t], 0, 0, 0);
        part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[it & 1][t], bhi, part[t], 0, 0, 0);
      }
    });
    const float d = kq::h2f(d_side);
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[t][i] = fmaf(d, part[t][i], acc[t][i]);
  }
}

}  // namespace kqmma
