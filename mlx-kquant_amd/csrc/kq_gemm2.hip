// Prefill GEMM, 128-row wave tiles (q4_k / q5_k): y[M,N] = x[M,K] . W^T on the f16 matrix cores.
//
// The 64 x 128 kernel of kq_gemm.hip decodes a weight fragment (VALU) for every two MFMAs and is bound by
// that decode.  Here a wave owns 128 activation rows x 32 weight rows, so a decoded fragment feeds four
// MFMAs, and everything that is not arithmetic is taken off the vector ALU:
//   * workgroup = 8 waves = 128 activation rows x 256 weight rows, one workgroup per CU (a second shape, 4 waves =
//     128 x 128 with K steps of 64 and two workgroups per CU, measured the same and is kept selectable);
//   * activations (f16, prepared by the prepass of kq_gemm.hip) and wire bytes travel HBM / L2 -> LDS with
//     direct-to-LDS loads (kq_dma.h): no staging registers, no LDS store instructions;
//   * K advances in steps of 128 (half a superblock): two activation stages of 32 KiB, two wire stages of
//     one superblock each; the loads of step s + 1 are queued right after the barrier that opens step s, the
//     wire bytes of the next superblock one step earlier still;
//   * the activation tile is stored unpadded with the 16-byte pieces of row r XOR-ed by r % 16 (the swizzle is
//     applied on the global side of the load, LDS is written linearly), which keeps the row-per-lane fragment
//     reads free of bank conflicts; the eight per-lane read addresses are loop invariants;
//   * accumulators: 4 x 16 running sums + 4 x 16 for the superblock in hand (exact integer products, folded
//     with d at the end of the superblock), 2 waves per SIMD.
// Numerics are those of kq_mma.h: B operands are the exact integers sc_j * q, the -dmin * m_j term is one extra
// MFMA per superblock on the split sub-block sums of x.
#include "kq_dma.h"
#include "kq_mma.h"

namespace {

using namespace kqmma;
using namespace kqdma;

constexpr int G2_TM = 128, G2_MT = 4;

// Wire geometry of a weight row's superblock in LDS: PP 16-byte pieces, piece p taken from block byte off(p) and
// parked at 16 p; HB = bytes of activation sub-block sums per row and superblock (8 or 16 hi / lo pairs).
//   q2_k (84 B):  pieces 0 .. 4, then the block's last 16 bytes: scales[16] at 0, qs[64] at 16, d at 92, dmin at 94
//   q3_k (110 B): pieces 0 .. 5, then the block's last 16 bytes: hmask[32] at 0, qs[64] at 32, scales[12] at 98, d at 110
template <int C>
struct G2Wire : Wire<C> {
  static constexpr int HB = 32;
  __device__ static uint32_t off(int p) { return 16u * (uint32_t)p; }
};
template <>
struct G2Wire<KQ_Q2_K> {
  static constexpr int BPB = 84, LBPB = 96, PP = 6, QS = 16, HB = 64;
  __device__ static uint32_t off(int p) { return p == 5 ? 68u : 16u * (uint32_t)p; }
};
template <>
struct G2Wire<KQ_Q3_K> {
  static constexpr int BPB = 110, LBPB = 112, PP = 7, QS = 32, HB = 64;
  __device__ static uint32_t off(int p) { return p == 6 ? 94u : 16u * (uint32_t)p; }
};
//   iq4_xs (136 B): piece 0 = bytes 0 .. 15 (d, scales_h, scales_l), piece i = bytes 8 + 16 (i - 1) ..: qs[q] at 16 + q;
//                   no sums of x are needed
template <>
struct G2Wire<KQ_IQ4_XS> {
  static constexpr int BPB = 136, LBPB = 144, PP = 9, QS = 16, HB = 0;
  __device__ static uint32_t off(int p) { return p == 0 ? 0u : 16u * (uint32_t)p - 8u; }
};
template <int C>
constexpr bool g2_low() { return C == KQ_Q2_K || C == KQ_Q3_K; }
constexpr int G2_IQ4_TBL = 1024;  // iq4_xs: [256] byte -> f16 pair (kvalues[low nibble], kvalues[high nibble])

// WAVES = 8 or 4 (tile 128 x 256 or 128 x 128), KS = K per step (128 or 64)
template <int C, int WAVES, int KS>
constexpr int g2_lds_bytes() {
  return 2 * G2_TM * KS * 2 + 2 * 32 * WAVES * G2Wire<C>::LBPB + 2 * G2_TM * G2Wire<C>::HB + (C == KQ_IQ4_XS ? G2_IQ4_TBL : 0);
}

template <int C, int DT, int WAVES, int KS>
__global__ __launch_bounds__(64 * WAVES, WAVES == 8 ? 1 : 2) void kquant_gemm2_kernel(const _Float16* __restrict__ xh,
                                                                     const _Float16* __restrict__ xhl,
                                                                     const float* __restrict__ rs,
                                                                     const uint8_t* __restrict__ w,
                                                                     uint16_t* __restrict__ y, int M, int N, int K,
                                                                     int mtiles, int nt0) {
  using G = G2Wire<C>;
  constexpr bool LOW = g2_low<C>(), IQ4 = C == KQ_IQ4_XS;
  constexpr int G2_H_STAGE = G2_TM * G::HB;
  constexpr int H_INSTR = G2_H_STAGE / 1024;  // load instructions of the sub-block sums per superblock: 0, 4 or 8
  static_assert(!(LOW || IQ4) || (WAVES == 8 && KS == 128), "q2_k / q3_k / iq4_xs: the eight-wave shape only");
  constexpr int MT = G2_MT;
  constexpr int G2_WAVES = WAVES, G2_BN = 32 * WAVES, G2_KS = KS;
  constexpr int G2_A_STAGE = G2_TM * KS * 2;
  constexpr int PR = KS / 8;            // 16-byte activation pieces per row and step
  constexpr int RPI = 64 / PR;          // activation rows one load instruction covers
  constexpr int A_PER_WAVE = G2_TM / (RPI * WAVES);  // activation loads per wave and step
  constexpr int SPS = 256 / KS;         // steps per superblock
  constexpr int GPS = KS / 16;          // MFMA groups per step
  static_assert(RPI * WAVES == 32, "the swizzle of a wave's loads repeats every 32 rows");
  constexpr int W_STAGE = G2_BN * G::LBPB;
  constexpr int W_INSTR = G2_BN * G::PP / 64;            // wire load instructions per superblock (all full waves)
  constexpr int W_PER_WAVE = (W_INSTR + G2_WAVES - 1) / G2_WAVES;
  static_assert(W_PER_WAVE + 1 <= 7 && W_INSTR / G2_WAVES + (H_INSTR >= G2_WAVES ? 1 : 0) >= 4 && H_INSTR <= G2_WAVES,
                "the step wait covers 4 .. 7 loads per wave");
  static_assert(G2_BN * G::PP % 64 == 0, "wire tile is a whole number of 64-piece loads");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // LDS: A[2] | W[2] | H[2]
  constexpr int A_OFF = 0, W_OFF = 2 * G2_A_STAGE, H_OFF = W_OFF + 2 * W_STAGE;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, kg = lane >> 5;
  const int mt = blockIdx.x % mtiles, nt = nt0 + blockIdx.x / mtiles;  // consecutive workgroups share the weight columns
  const int m0 = mt * G2_TM, n0 = nt * G2_BN;
  const int nsb = K >> 8;
  const uint32_t row_bytes = (uint32_t)nsb * G::BPB;
  const int nrows = N - n0 < G2_BN ? N - n0 : G2_BN;
  const uint32_t lds0 = lds_addr(smem);

  // ---- load maps
  // activations: load q of this wave covers rows RPI (wave + WAVES q) + lane / PR, pieces lane % PR of the step;
  // LDS piece p of row r holds global piece p ^ swz(r)
  auto swz = [](int row) { return PR == 16 ? (row & 15) : ((row >> 1) & 7); };
  const int a_r = RPI * wave + lane / PR;
  const uint32_t a_voff = (uint32_t)a_r * (uint32_t)K * 2u + 16u * (uint32_t)((lane % PR) ^ swz(a_r));
  const uint8_t* a_base = reinterpret_cast<const uint8_t*>(xh) + (size_t)m0 * K * 2;
  // wire: load j = wave + 8 q covers pieces 64 j + lane of the tile's 256 x PP; piece i -> (row i / PP, i % PP)
  uint32_t w_voff[W_PER_WAVE];
  StaticFor<W_PER_WAVE>::run([&](auto qq) {
    constexpr int q = decltype(qq)::value;
    const int i = 64 * (wave + G2_WAVES * q) + lane;
    int r = i / G::PP;
    const int p = i - r * G::PP;
    r = r < nrows ? r : nrows - 1;  // rows past N re-read the last row (their columns are not stored)
    w_voff[q] = (uint32_t)r * row_bytes + G::off(p);
  });
  const uint8_t* w_base = w + (size_t)n0 * row_bytes;
  // X halves: 128 rows x HB bytes = H_INSTR loads, waves 0 .. H_INSTR - 1
  constexpr int HPR = G::HB > 0 ? G::HB / 16 : 1;  // pieces per row
  const int h_i = 64 * (wave & (H_INSTR > 0 ? H_INSTR - 1 : 0)) + lane;
  const uint32_t h_voff = (uint32_t)(h_i / HPR) * (uint32_t)nsb * (uint32_t)G::HB + 16u * (h_i % HPR);
  const uint8_t* h_base = reinterpret_cast<const uint8_t*>(xhl) + (size_t)m0 * nsb * G::HB;

  auto issue_a = [&](int step) {  // K step `step` (KS wide) -> A stage step % 2
    const uint8_t* base = a_base + (size_t)step * (G2_KS * 2);
    const uint32_t l = lds0 + A_OFF + (step & 1) * G2_A_STAGE + wave * 1024;
#pragma unroll
    for (int q = 0; q < A_PER_WAVE; q++) dma16(base + (size_t)q * 32 * K * 2, a_voff, l + q * (G2_WAVES * 1024));
  };
  auto issue_w = [&](int sb) {  // superblock sb -> W / H stage sb % 2
    const uint8_t* base = w_base + (size_t)sb * G::BPB;
    const uint32_t l = lds0 + W_OFF + (sb & 1) * W_STAGE + wave * 1024;
    StaticFor<W_PER_WAVE>::run([&](auto qq) {
      constexpr int q = decltype(qq)::value;
      if (wave + G2_WAVES * q < W_INSTR) dma16(base, w_voff[q], l + q * (G2_WAVES * 1024));
    });
    if (wave < H_INSTR) dma16(h_base + (size_t)sb * G::HB, h_voff, lds0 + H_OFF + (sb & 1) * G2_H_STAGE + wave * 1024);
  };
  // load instructions of one issue_w of this wave (wave-uniform)
  int w_count = 0;
#pragma unroll
  for (int q = 0; q < W_PER_WAVE; q++) w_count += (wave + G2_WAVES * q < W_INSTR) ? 1 : 0;
  w_count += wave < H_INSTR ? 1 : 0;

  // ---- fragment addresses
  // A fragment of m-block t, MFMA group g of the step = (sub-block g / 2, K-half s = g % 2): lane half kg holds the
  // weights 16 kg + 8 s .. + 7 of the sub-block, i.e. activation piece 4 (g / 2) + 2 kg + s of the step, stored at
  // piece index ^ swz(row) of row 32 t + l32
  uint32_t a_addr[GPS];
#pragma unroll
  for (int g = 0; g < GPS; g++)
    a_addr[g] = (uint32_t)l32 * (16u * PR) +
                16u * (uint32_t)((LOW || IQ4 ? 2 * g + kg : 4 * (g >> 1) + 2 * kg + (g & 1)) ^ swz(l32));
  const uint8_t* b_lane0 = smem + W_OFF + (wave * 32 + l32) * G::LBPB;
  const uint8_t* h_lane0 = smem + H_OFF + l32 * G::HB + 16 * kg;

  f32x16 acc[MT], part[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) acc[t] = f32x16{0};

  const uint32_t magic = opaque_vgpr(0x64006400u);
  const uint32_t mask_lo = opaque_sgpr(0x000f000fu), mask_hi = opaque_sgpr(0x00f000f0u);
  const uint32_t mask5_lo = opaque_sgpr(0x00100010u), mask5_hi = opaque_sgpr(0x01000100u);
  (void)mask5_lo;
  (void)mask5_hi;

  // per-superblock state shared by the two half steps
  float d = 0.f, dmin32 = 0.f;
  uint32_t scw[2] = {0, 0}, mnw[2] = {0, 0};
  uint32_t lsc[4] = {0, 0, 0, 0};  // q2_k: the 16 scale / min bytes; q3_k: the 16 unpacked 6-bit scales
  const uint32_t mask_f[4] = {opaque_sgpr(0x00030003u), opaque_sgpr(0x000c000cu), opaque_sgpr(0x00300030u),
                              opaque_sgpr(0x00c000c0u)};
  const uint32_t bit_f[4] = {opaque_sgpr(0x00040004u), opaque_sgpr(0x00100010u), opaque_sgpr(0x00400040u),
                             opaque_sgpr(0x01000100u)};
  (void)mask_f;
  (void)bit_f;

  // q2_k / q3_k step: MFMA group g of half n = part (sub-block 8 n + g, one scale): field j = g / 2 of the bytes
  // qs[32 n + 16 (g % 2) + 8 kg .. + 7].  The field is masked in place (1024 + 4^j q; q3_k: its third bit, hmask bit
  // 4 n + j, is moved to bit 2 j + 2 first) and one packed fma turns it into the exact integer sc q.  The rest of the
  // weight, -dmin m_s (q2_k) or -4 d sc_s (q3_k), is two more MFMAs per superblock on the hi / lo sums of x.
  auto k_step_low = [&](auto partc, const uint8_t* a_stage, const uint8_t* b_lane, const uint8_t* h_lane) {
    constexpr int part_i = decltype(partc)::value;
    if constexpr (part_i == 0) {
      if constexpr (C == KQ_Q2_K) {
        const uint4 sv = *reinterpret_cast<const uint4*>(b_lane);
        lsc[0] = sv.x;
        lsc[1] = sv.y;
        lsc[2] = sv.z;
        lsc[3] = sv.w;
        const uint32_t dd = *reinterpret_cast<const uint32_t*>(b_lane + 92);
        d = kq::h2f((uint16_t)(dd & 0xffff));
        dmin32 = kq::h2f((uint16_t)(dd >> 16)) * 16.0f;
      } else {
        const uint4 t = *reinterpret_cast<const uint4*>(b_lane + 96);  // block bytes 94 .. 109
        const uint32_t aux0 = __builtin_amdgcn_alignbyte(t.y, t.x, 2), aux1 = __builtin_amdgcn_alignbyte(t.z, t.y, 2);
        const uint32_t tmp = __builtin_amdgcn_alignbyte(t.w, t.z, 2);
        d = kq::h2f((uint16_t)(t.w >> 16));
        dmin32 = d * 16.0f;
        lsc[0] = (aux0 & 0x0f0f0f0fu) | ((tmp & 0x03030303u) << 4);
        lsc[1] = (aux1 & 0x0f0f0f0fu) | (((tmp >> 2) & 0x03030303u) << 4);
        lsc[2] = ((aux0 >> 4) & 0x0f0f0f0fu) | (((tmp >> 4) & 0x03030303u) << 4);
        lsc[3] = ((aux1 >> 4) & 0x0f0f0f0fu) | (((tmp >> 6) & 0x03030303u) << 4);
      }
    }
    uint2 qv[2], hv[2] = {{0, 0}, {0, 0}};
#pragma unroll
    for (int h = 0; h < 2; h++) {
      qv[h] = *reinterpret_cast<const uint2*>(b_lane + G::QS + 32 * part_i + 16 * h + 8 * kg);
      if constexpr (C == KQ_Q3_K) hv[h] = *reinterpret_cast<const uint2*>(b_lane + 16 * h + 8 * kg);
    }
    f16x8 afr[2][MT], bfr[2];
    auto load_a = [&](auto gc, int buf) {
      constexpr int g = decltype(gc)::value;
#pragma unroll
      for (int t = 0; t < MT; t++) afr[buf][t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[g] + t * (32 * 16 * PR));
    };
    auto decode = [&](auto gc) -> f16x8 {
      constexpr int g = decltype(gc)::value, j = g >> 1, h = g & 1, s = 8 * part_i + g;
      const uint32_t sb8 = (lsc[s >> 2] >> (8 * (s & 3))) & 0xff;
      const float scf = C == KQ_Q2_K ? (float)(sb8 & 15) : (float)(int)sb8 - 32.0f;
      constexpr float f = 1.0f / (float)(1 << (2 * j));  // the field reads 4^j q
      const _Float16 sch = (_Float16)(scf * f);
      const _Float16 off = (_Float16)(-1024.0f * f * scf);
      const f16x2 scp = {sch, sch}, offp = {off, off};
      const uint32_t w0 = h ? qv[1].x : qv[0].x, w1 = h ? qv[1].y : qv[0].y;
      uint32_t fr[4] = {(w0 & mask_f[j]) | magic, ((w0 >> 8) & mask_f[j]) | magic, (w1 & mask_f[j]) | magic,
                        ((w1 >> 8) & mask_f[j]) | magic};
      if constexpr (C == KQ_Q3_K) {
        constexpr int from = 4 * part_i + j, to = 2 * j + 2;
        auto place = [&](uint32_t word, int fr_bit) -> uint32_t {
          return fr_bit >= to ? word >> (fr_bit - to) : word << (to - fr_bit);
        };
        const uint32_t m0 = h ? hv[1].x : hv[0].x, m1 = h ? hv[1].y : hv[0].y;
        fr[0] |= place(m0, from) & bit_f[j];
        fr[1] |= place(m0, from + 8) & bit_f[j];
        fr[2] |= place(m1, from) & bit_f[j];
        fr[3] |= place(m1, from + 8) & bit_f[j];
      }
      f16x2 bq[4];
#pragma unroll
      for (int e = 0; e < 4; e++) bq[e] = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, fr[e]), scp, offp);
      return f16x8{bq[0][0], bq[0][1], bq[1][0], bq[1][1], bq[2][0], bq[2][1], bq[3][0], bq[3][1]};
    };
    constexpr int DEC_VALU = C == KQ_Q3_K ? 26 : 16;
    load_a(std::integral_constant<int, 0>{}, 0);
    bfr[0] = decode(std::integral_constant<int, 0>{});
    __builtin_amdgcn_sched_barrier(0);
    StaticFor<GPS>::run([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      if constexpr (g + 1 < GPS) {
        load_a(std::integral_constant<int, g + 1>{}, (g + 1) & 1);
        bfr[(g + 1) & 1] = decode(std::integral_constant<int, g + 1>{});
      }
#pragma unroll
      for (int t = 0; t < MT; t++) {
        if constexpr (part_i == 0 && g == 0)
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t], bfr[0], f32x16{0}, 0, 0, 0);
        else
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[g & 1][t], bfr[g & 1], part[t], 0, 0, 0);
      }
      if constexpr (g + 1 < GPS) {
        __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);
#pragma unroll
        for (int t = 0; t < MT; t++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, (DEC_VALU + MT - 1) / MT, 0);
        }
      }
    });
    if constexpr (part_i == SPS - 1) {
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = fmaf(d, part[t][i], acc[t][i]);
      // the other term: sum_s c_s X_s with X_s = 16 (hi_s + lo_s); c_s = m_s (q2_k) or 4 sc_s (q3_k), s = 8 kg .. + 7
      _Float16 cj[8];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const uint32_t b = (lsc[2 * kg + (j >> 2)] >> (8 * (j & 3))) & 0xff;
        cj[j] = C == KQ_Q2_K ? (_Float16)(float)(b >> 4) : (_Float16)(4.0f * ((float)(int)b - 32.0f));
      }
      const f16x8 bm = {cj[0], cj[1], cj[2], cj[3], cj[4], cj[5], cj[6], cj[7]};
#pragma unroll
      for (int t = 0; t < MT; t++) {
        const f16x8 ahi = *reinterpret_cast<const f16x8*>(h_lane + t * (32 * G::HB));
        const f16x8 alo = *reinterpret_cast<const f16x8*>(h_lane + t * (32 * G::HB) + 32);
        part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ahi, bm, f32x16{0}, 0, 0, 0);
        part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(alo, bm, part[t], 0, 0, 0);
      }
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = fmaf(-dmin32, part[t][i], acc[t][i]);
    }
  };

  // one step: MFMA groups it = GPS part .. GPS part + GPS - 1 of the superblock (sub-block j = it / 2, K-half s = it % 2)
  // iq4_xs step: MFMA group g of half `part` = bytes 8 (g % 2) + 4 kg .. + 3 of sub-block 4 part + g / 2.  One table
  // read turns a byte into the f16 pair of its two codebook values (weights j and j + 16; the activations are staged in
  // that order).  (ls - 32) kv reaches 4064 and is not always an f16 number (feeding its rounded value cost 8e-4
  // rel-L2 on bf16 outputs), so a weight goes in as two exact terms, the even part of the scale times kv (twice a
  // product <= 2032) and its parity times kv: two MFMAs per group on one activation fragment.
  const uint8_t* tbl = smem + H_OFF + 2 * G2_H_STAGE;
  if constexpr (IQ4) {
    if (tid < 256) {
      const f16x2 e = {(_Float16)kq::kv_iq4nl(tid & 15), (_Float16)kq::kv_iq4nl(tid >> 4)};
      reinterpret_cast<uint32_t*>(smem + H_OFF + 2 * G2_H_STAGE)[tid] = __builtin_bit_cast(uint32_t, e);
    }
  }
  uint32_t iq_sl = 0, iq_sh = 0;
  auto k_step_iq4 = [&](auto partc, const uint8_t* a_stage, const uint8_t* b_lane) {
    constexpr int part_i = decltype(partc)::value;
    if constexpr (part_i == 0) {
      const uint2 hdr = *reinterpret_cast<const uint2*>(b_lane);
      d = kq::h2f((uint16_t)(hdr.x & 0xffff));
      iq_sh = hdr.x >> 16;
      iq_sl = hdr.y;
    }
    uint32_t qw[GPS];
#pragma unroll
    for (int g = 0; g < GPS; g++)
      qw[g] = *reinterpret_cast<const uint32_t*>(b_lane + 16 + 16 * (4 * part_i + (g >> 1)) + 8 * (g & 1) + 4 * kg);
    f16x8 afr[2][MT], bfr[2][2];
    auto load_a = [&](auto gc, int buf) {
      constexpr int g = decltype(gc)::value;
#pragma unroll
      for (int t = 0; t < MT; t++) afr[buf][t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[g] + t * (32 * 16 * PR));
    };
    auto decode = [&](auto gc, f16x8* out) {
      constexpr int g = decltype(gc)::value, ib = 4 * part_i + (g >> 1);
      const int ls = (int)(((iq_sl >> (4 * ib)) & 15) | (((iq_sh >> (2 * ib)) & 3) << 4)) - 32;
      const int odd = ls & 1;  // ls - odd is even and at most 32 in magnitude
      const _Float16 se = (_Float16)(float)(ls - odd), so = (_Float16)(float)odd;
      const f16x2 sep = {se, se}, sop = {so, so};
      f16x2 be[4], bo[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const uint32_t idx = (qw[g] >> (8 * e)) & 0xff;
        const f16x2 kv = __builtin_bit_cast(f16x2, *reinterpret_cast<const uint32_t*>(tbl + 4 * idx));
        be[e] = kv * sep;
        bo[e] = kv * sop;
      }
      out[0] = f16x8{be[0][0], be[0][1], be[1][0], be[1][1], be[2][0], be[2][1], be[3][0], be[3][1]};
      out[1] = f16x8{bo[0][0], bo[0][1], bo[1][0], bo[1][1], bo[2][0], bo[2][1], bo[3][0], bo[3][1]};
    };
    load_a(std::integral_constant<int, 0>{}, 0);
    decode(std::integral_constant<int, 0>{}, bfr[0]);
    StaticFor<GPS>::run([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      if constexpr (g + 1 < GPS) {
        load_a(std::integral_constant<int, g + 1>{}, (g + 1) & 1);
        decode(std::integral_constant<int, g + 1>{}, bfr[(g + 1) & 1]);
      }
#pragma unroll
      for (int t = 0; t < MT; t++) {
        if constexpr (part_i == 0 && g == 0)
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t], bfr[0][0], f32x16{0}, 0, 0, 0);
        else
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[g & 1][t], bfr[g & 1][0], part[t], 0, 0, 0);
      }
#pragma unroll
      for (int t = 0; t < MT; t++)
        part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[g & 1][t], bfr[g & 1][1], part[t], 0, 0, 0);
    });
    if constexpr (part_i == SPS - 1) {
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = fmaf(d, part[t][i], acc[t][i]);
    }
  };

  auto k_step = [&](auto partc, const uint8_t* a_stage, const uint8_t* b_lane, const uint8_t* h_lane) {
    constexpr int part_i = decltype(partc)::value;
    constexpr int NQ = GPS / 4;  // nibble pairs (32 wire bytes each) of the step
    if constexpr (part_i == 0) {
      const uint4 hdr = *reinterpret_cast<const uint4*>(b_lane);
      d = kq::h2f((uint16_t)(hdr.x & 0xffff));
      dmin32 = kq::h2f((uint16_t)(hdr.x >> 16)) * 32.0f;
      const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
      scw[0] = s0 & 0x3f3f3f3fu;
      scw[1] = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
      mnw[0] = s1 & 0x3f3f3f3fu;
      mnw[1] = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
    }
    uint4 qv[NQ];
#pragma unroll
    for (int g = 0; g < NQ; g++) qv[g] = *reinterpret_cast<const uint4*>(b_lane + G::QS + 32 * (NQ * part_i + g) + 16 * kg);
    uint32_t hb[4] = {0, 0, 0, 0};
    if constexpr (C == KQ_Q5_K) {
      const uint4 hv = *reinterpret_cast<const uint4*>(b_lane + 16 + 16 * kg);
      hb[0] = hv.x;
      hb[1] = hv.y;
      hb[2] = hv.z;
      hb[3] = hv.w;
    }
    f16x8 afr[2][MT], bfr[2];
    auto load_a = [&](auto gc, int buf) {
      constexpr int g = decltype(gc)::value;  // group inside the step
#pragma unroll
      for (int t = 0; t < MT; t++) afr[buf][t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[g] + t * (32 * 16 * PR));
    };
    auto decode = [&](auto itc) -> f16x8 {
      constexpr int it = decltype(itc)::value;  // group inside the superblock
      constexpr int j = it >> 1, s = it & 1, gq = (j >> 1) % NQ, h = j & 1;
      const uint32_t qw[4] = {qv[gq].x, qv[gq].y, qv[gq].z, qv[gq].w};
      const float scf = (float)((scw[j >> 2] >> (8 * (j & 3))) & 0xff);
      // low nibbles read 1024 + q, high nibbles (in place) 1024 + 16 q: the 16 goes into the scale
      const _Float16 sch = (_Float16)(h ? scf * 0.0625f : scf);
      const _Float16 off = (_Float16)(-(h ? 64.0f : 1024.0f) * scf);
      const f16x2 scp = {sch, sch}, offp = {off, off};
      const uint32_t mask = h ? mask_hi : mask_lo;
      uint32_t fr[4] = {(qw[2 * s] & mask) | magic, ((qw[2 * s] >> 8) & mask) | magic,
                        (qw[2 * s + 1] & mask) | magic, ((qw[2 * s + 1] >> 8) & mask) | magic};
      if constexpr (C == KQ_Q5_K) {
        // fifth bit of weight (j, i) is bit j of qh[i]; this lane's bytes are qh[16 kg + 8 s + 0..7]: bit 4 next
        // to a low nibble (1024 + q + 16 b), bit 8 next to a high nibble held in place (1024 + 16 (q + 16 b))
        constexpr int P = h ? 8 : 4;
        const uint32_t mbit = h ? mask5_hi : mask5_lo;
        auto place = [&](uint32_t word, int from) -> uint32_t {
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
    constexpr int DEC_VALU = C == KQ_Q5_K ? 22 : 14;
    load_a(std::integral_constant<int, 0>{}, 0);
    bfr[0] = decode(std::integral_constant<int, GPS * part_i>{});
    __builtin_amdgcn_sched_barrier(0);
    StaticFor<GPS>::run([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      constexpr int it = GPS * part_i + g;
      if constexpr (g + 1 < GPS) {
        load_a(std::integral_constant<int, g + 1>{}, (g + 1) & 1);
        bfr[(g + 1) & 1] = decode(std::integral_constant<int, it + 1>{});
      }
#pragma unroll
      for (int t = 0; t < MT; t++) {
        if constexpr (it == 0)
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[0][t], bfr[0], f32x16{0}, 0, 0, 0);
        else
          part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[g & 1][t], bfr[g & 1], part[t], 0, 0, 0);
      }
      if constexpr (g + 1 < GPS) {
        __builtin_amdgcn_sched_group_barrier(0x100, MT, 0);  // the next group's fragment requests go first
#pragma unroll
        for (int t = 0; t < MT; t++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                         // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x002, (DEC_VALU + MT - 1) / MT, 0);  // a slice of the decode
        }
      }
    });
    if constexpr (part_i == SPS - 1) {
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
        const f16x8 a = *reinterpret_cast<const f16x8*>(h_lane + t * (32 * 32));
        part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bm, f32x16{0}, 0, 0, 0);
      }
#pragma unroll
      for (int t = 0; t < MT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[t][i] = fmaf(-dmin32, part[t][i], acc[t][i]);
    }
  };

  // ---- main loop: step s = SPS sb + part.  Loads of step s + 1 are queued right after the barrier that opens
  // step s (their stage was last read in step s - 1); the wire bytes of superblock sb + 1 follow them in part 0.
  issue_a(0);
  issue_w(0);
  for (int sb = 0; sb < nsb; sb++) {
    const uint8_t* b_lane = b_lane0 + (sb & 1) * W_STAGE;
    const uint8_t* h_lane = h_lane0 + (sb & 1) * G2_H_STAGE;
    StaticFor<SPS>::run([&](auto pc) {
      constexpr int p = decltype(pc)::value;
      const int step = SPS * sb + p;
      // part 1 needs only its activations: the next superblock's wire bytes, queued after them, stay in flight
      if (p == 1 && sb + 1 < nsb) {
        if (w_count >= 7) vmwait<7>();
        else if (w_count == 6) vmwait<6>();
        else if (w_count == 5) vmwait<5>();
        else vmwait<4>();
      } else {
        vmwait<0>();
      }
      lds_barrier();
      if (p + 1 < SPS || sb + 1 < nsb) issue_a(step + 1);
      if (p == 0 && sb + 1 < nsb) issue_w(sb + 1);
      if constexpr (LOW)
        k_step_low(pc, smem + A_OFF + (p & 1) * G2_A_STAGE, b_lane, h_lane);
      else if constexpr (IQ4)
        k_step_iq4(pc, smem + A_OFF + (p & 1) * G2_A_STAGE, b_lane);
      else
        k_step(pc, smem + A_OFF + (p & 1) * G2_A_STAGE, b_lane, h_lane);
    });
  }

  // ---- epilogue: undo the per-row activation scale, round once, store
  const int n = n0 + wave * 32 + l32;
#pragma unroll
  for (int t = 0; t < MT; t++) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int m = m0 + t * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);
      if (m < M && n < N) {
        const float v = acc[t][i] * rs[m];
        y[(size_t)m * N + n] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
      }
    }
  }
}

template <int C, int DT, int WAVES, int KS>
int launch_gemm2(const _Float16* xh, const _Float16* xhl, const float* rs, const uint8_t* w, void* y, int M, int N, int K,
                 hipStream_t s, int nt0 = 0, int ntiles_sel = -1) {
  constexpr int BN = 32 * WAVES;
  const int mtiles = (M + G2_TM - 1) / G2_TM, ntiles = ntiles_sel >= 0 ? ntiles_sel : (N + BN - 1) / BN;
  if (ntiles == 0) return KQ_OK;
  constexpr int lds = g2_lds_bytes<C, WAVES, KS>();
  static_assert(lds <= 160 * 1024, "tile does not fit the LDS of a CU");
  auto kern = kquant_gemm2_kernel<C, DT, WAVES, KS>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  hipLaunchKernelGGL(kern, dim3(mtiles * ntiles), dim3(64 * WAVES), lds, s, xh, xhl, rs, w, static_cast<uint16_t*>(y), M, N,
                     K, mtiles, nt0);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

template <int C, int DT>
int launch_gemm2_shape(const _Float16* xh, const _Float16* xhl, const float* rs, const uint8_t* w, void* y, int M, int N,
                       int K, int shape, hipStream_t s, int nt0, int ntiles) {
  if (shape == 1) return launch_gemm2<C, DT, 4, 64>(xh, xhl, rs, w, y, M, N, K, s);
  return launch_gemm2<C, DT, 8, 128>(xh, xhl, rs, w, y, M, N, K, s, nt0, ntiles);
}

// activation prepass with the sums of the 16-weight sub-blocks (q2_k / q3_k)
template <int DT>
__global__ __launch_bounds__(PP_THREADS) void gemm2_prepass16_kernel(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
                                                                     _Float16* __restrict__ xhl, float* __restrict__ rs,
                                                                     int M, int K) {
  __shared__ float red[PP_THREADS / 64];
  prepass_row<DT, true>(x, xh, xhl, rs, M, K, blockIdx.x, threadIdx.x, red);
}

// activation prepass in the order of the iq4 nibble pairs (x[j], x[j + 16] interleaved)
template <int DT>
__global__ __launch_bounds__(PP_THREADS) void gemm2_prepass_il16_kernel(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
                                                                        _Float16* __restrict__ xhl, float* __restrict__ rs,
                                                                        int M, int K) {
  __shared__ float red[PP_THREADS / 64];
  prepass_row<DT, false, true>(x, xh, xhl, rs, M, K, blockIdx.x, threadIdx.x, red);
}

template <int C, int DT>
int launch_gemm2_low(const void* x, const uint8_t* w, void* y, int M, int N, int K, void* ws, hipStream_t s) {
  const int mpad = ((M + G2_TM - 1) / G2_TM) * G2_TM, nsb = K >> 8;
  _Float16* xh = static_cast<_Float16*>(ws);
  _Float16* xhl = xh + (size_t)mpad * K;
  float* rs = reinterpret_cast<float*>(xhl + (size_t)mpad * nsb * 32);
  if constexpr (C == KQ_IQ4_XS)
    hipLaunchKernelGGL((gemm2_prepass_il16_kernel<DT>), dim3(mpad), dim3(PP_THREADS), 0, s, static_cast<const uint16_t*>(x),
                       xh, xhl, rs, M, K);
  else
    hipLaunchKernelGGL((gemm2_prepass16_kernel<DT>), dim3(mpad), dim3(PP_THREADS), 0, s, static_cast<const uint16_t*>(x), xh,
                       xhl, rs, M, K);
  KQ_HIP_CHECK(hipGetLastError());
  return launch_gemm2<C, DT, 8, 128>(xh, xhl, rs, w, y, M, N, K, s);
}

}  // namespace

// q2_k / q3_k on the 128 x 256 tile kernel: M >= 256 and enough tiles to fill the chip; the any-codec kernel keeps
// the smaller shapes.
bool kq_gemm2_low_supported(int M, int N, int K, int codec) {
  return (codec == KQ_Q2_K || codec == KQ_Q3_K || codec == KQ_IQ4_XS) && M >= 256 && K >= 256 && (K & 255) == 0 && N > 0 &&
         (int64_t)((M + 127) / 128) * ((N + 255) / 256) >= 256 && (int64_t)N * (K >> 8) * 136 < ((int64_t)1 << 32) &&
         (int64_t)K * 2 * 128 < ((int64_t)1 << 32);
}

size_t kq_gemm2_low_workspace_bytes(int M, int K) {
  const size_t mpad = (size_t)((M + G2_TM - 1) / G2_TM) * G2_TM;
  return mpad * K * 2 + mpad * (K >> 8) * 64 + mpad * 4 + 256;
}

int kq_launch_gemm2_low(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                        hipStream_t s) {
  if (!kq_gemm2_low_supported(M, N, K, codec)) return KQ_ERR_UNSUPPORTED;
  // q2_k blocks are 4-byte multiples, q3_k blocks 2-byte ones, iq4_xs blocks 8-byte ones
  if ((reinterpret_cast<uintptr_t>(w) & (codec == KQ_Q2_K ? 3 : codec == KQ_IQ4_XS ? 7 : 1)) || (reinterpret_cast<uintptr_t>(x) & 15) ||
      (reinterpret_cast<uintptr_t>(ws) & 15))
    return KQ_ERR_UNSUPPORTED;
  if (codec == KQ_Q2_K)
    return dtype == KQ_F16 ? launch_gemm2_low<KQ_Q2_K, KQ_F16>(x, w, y, M, N, K, ws, s)
                           : launch_gemm2_low<KQ_Q2_K, KQ_BF16>(x, w, y, M, N, K, ws, s);
  if (codec == KQ_IQ4_XS)
    return dtype == KQ_F16 ? launch_gemm2_low<KQ_IQ4_XS, KQ_F16>(x, w, y, M, N, K, ws, s)
                           : launch_gemm2_low<KQ_IQ4_XS, KQ_BF16>(x, w, y, M, N, K, ws, s);
  return dtype == KQ_F16 ? launch_gemm2_low<KQ_Q3_K, KQ_F16>(x, w, y, M, N, K, ws, s)
                         : launch_gemm2_low<KQ_Q3_K, KQ_BF16>(x, w, y, M, N, K, ws, s);
}

// xh / xhl / rs: outputs of the activation prepass (kq_launch_act_prepass) for rows padded to a multiple of 128.
bool kq_gemm2_supported(int M, int N, int K, int codec) {
  return (codec == KQ_Q4_K || codec == KQ_Q5_K) && M > 8 && K >= 256 && (K & 255) == 0 && N > 0 &&
         (int64_t)N * (K >> 8) * 176 < ((int64_t)1 << 32) && (int64_t)K * 2 * 128 < ((int64_t)1 << 32);
}

// shape 0: 128 x 256 tiles on eight waves, K steps of 128 (column tiles nt0 .. nt0 + ntiles - 1; ntiles < 0: all);
// shape 1: 128 x 128 tiles on four waves, K steps of 64 (two workgroups per CU, always the whole matrix)
int kq_launch_gemm2(const void* xh, const void* xhl, const float* rs, const uint8_t* w, void* y, int M, int N, int K,
                    int codec, int dtype, int shape, hipStream_t s, int nt0, int ntiles) {
  if (!kq_gemm2_supported(M, N, K, codec)) return KQ_ERR_UNSUPPORTED;
  const _Float16* a = static_cast<const _Float16*>(xh);
  const _Float16* h = static_cast<const _Float16*>(xhl);
  if (codec == KQ_Q4_K)
    return dtype == KQ_F16 ? launch_gemm2_shape<KQ_Q4_K, KQ_F16>(a, h, rs, w, y, M, N, K, shape, s, nt0, ntiles)
                           : launch_gemm2_shape<KQ_Q4_K, KQ_BF16>(a, h, rs, w, y, M, N, K, shape, s, nt0, ntiles);
  return dtype == KQ_F16 ? launch_gemm2_shape<KQ_Q5_K, KQ_F16>(a, h, rs, w, y, M, N, K, shape, s, nt0, ntiles)
                         : launch_gemm2_shape<KQ_Q5_K, KQ_BF16>(a, h, rs, w, y, M, N, K, shape, s, nt0, ntiles);
}
