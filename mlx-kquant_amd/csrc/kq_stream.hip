// Streamed skinny-M (decode) kernel: y[M,N] = x[M,K] . W^T for M <= 8, codecs q2_k ... q6_k, iq4_xs, iq3_s, iq2_xxs,
// q8_0, iq4_nl, q4_0, mxfp4, nvfp4 (the 32- and 64-weight-block codecs with K a multiple of 256).
// The weight bytes go HBM -> LDS with direct-to-LDS loads (global_load_lds_dwordx4): no staging
// registers, no LDS store instructions, and a wave keeps its next units in flight while it works.
//
// Mapping.  A workgroup (4 or 8 waves) owns tiles of up to 32 weight rows and a K range of at most 4
// superblocks per wave; wave w takes superblocks w, w + NW, ... of the range, a "unit" being 32 rows x one
// superblock.  Workgroups are persistent: tile t of workgroup b is tile b + t * gridDim.x, so the
// activations are prepared once per workgroup and the weight stream of the next tile is already on
// its way while the current one is multiplied.  Longer K ranges are split over grid z with an f32
// reduction launch behind.
//
// Matrix cores.  v_mfma_f32_4x4x4_16b_f16 is sixteen independent 4 x 4 x 4 products: block b = lanes
// 4 b .. 4 b + 3 multiplies four activation rows (A) by four weight rows (B).  Lane l serves weight
// row l % 32 and the half kg = l / 32 of the superblock (128 weights), so no two lanes share an
// accumulator and every lane folds its own block scales.  The eight blocks of a half-wave share one A
// block (cbsz = 3), picked by the instruction's abid field: one register pair holds the A operands of
// eight MFMAs, lane (kg, a, i) keeping the four activations that row i needs in MFMA number a.  The
// activations of a whole unit are 4 (q4_k / q5_k) or 8 (q6_k) such pairs, loaded once per workgroup.
//
// Codes.  As in the other tuned kernels a K-quant weight enters the matrix core as an exact f16 integer made
// with one AND-OR (0x6400 | field = 1024 + field, fields masked in place); scales, the 1024 offset and
// the block minimum are applied in f32 to the per-lane partial sums.  The codebook codecs read their values as
// ready f16 from tables the workgroup builds in LDS (iq4_xs: byte -> two values; iq2_xxs: grid index -> eight
// magnitudes, sign index -> eight sign masks; iq3_s: 9-bit grid index -> four magnitudes, sign byte -> eight sign
// masks).  These kernels are bound by the LDS once the table reads of a wave meet in a bank, so the one-row
// kernels spend their spare LDS on that: a copy of the table per bank group (iq4_xs, iq2_xxs) or entries with the
// signs already applied (iq3_s).  q8_0 (eight 34-byte blocks per unit row) needs no table: a byte permute and one
// exact packed subtraction turn a quant byte into its f16 value.  iq4_nl, q4_0 and mxfp4 (eight 18- or 17-byte blocks
// per unit row, a quant byte holding weights j and j + 16 of its block) share the iq4_xs table with their own sixteen
// values in it; nvfp4 (a byte = weights j and j + 8 of 16 with a scale of their own) does too.
//
// Waiting.  The compiler cannot see a direct-to-LDS load land, so these loads are issued from inline
// assembly and every wait on them is an explicit s_waitcnt vmcnt(n): loads return in order, n is the
// number of load instructions issued after the unit that is needed.  All other LDS traffic is ordinary
// code.
#include <type_traits>

#include "kq_decode.h"
#include "kq_epilogue.h"
#include "kq_dma.h"

namespace {

using namespace kqdma;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int ST_ROWS = 32;

template <int N>
struct SFor {
  template <class F>
  __device__ __forceinline__ static void run(F&& f) {
    SFor<N - 1>::run(f);
    f(std::integral_constant<int, N - 1>{});
  }
};
template <>
struct SFor<0> {
  template <class F>
  __device__ __forceinline__ static void run(F&&) {}
};

__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) { return (a & mask) | magic; }
__device__ __forceinline__ uint32_t opaque_vgpr(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}
__device__ __forceinline__ uint32_t opaque_sgpr(uint32_t v) {
  asm volatile("" : "+s"(v));
  return v;
}
__device__ __forceinline__ void tie_v(u32x4& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void tie_v2(u32x2& v) { asm volatile("" : "+v"(v)); }

__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ void wg_lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// maximum of a non-negative value over the wave, as a wave-uniform number
__device__ __forceinline__ float wave_max_nonneg(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));   // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp_f<0x4E>(v));   // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp_f<0x141>(v));  // row_half_mirror
  v = fmaxf(v, dpp_f<0x140>(v));  // row_mirror
  const uint32_t b = __builtin_bit_cast(uint32_t, v);
  const uint32_t m0 = __builtin_amdgcn_readlane(b, 0), m1 = __builtin_amdgcn_readlane(b, 16),
                 m2 = __builtin_amdgcn_readlane(b, 32), m3 = __builtin_amdgcn_readlane(b, 48);
  const uint32_t m01 = m0 > m1 ? m0 : m1, m23 = m2 > m3 ? m2 : m3;
  return __builtin_bit_cast(float, m01 > m23 ? m01 : m23);
}

// Per-codec geometry of a unit.  PP 16-byte pieces of every block travel (q6_k: the first 208 bytes, its
// trailing d goes as one 2-byte load per row); LBPB = LDS bytes per row; NAP = A register pairs per unit;
// XSG = activation sums per half superblock (sub-blocks of 32, q6_k: scale groups of 16).
template <int C>
struct StGeom;
template <>
struct StGeom<KQ_Q4_K> {
  static constexpr int BPB = 144, PP = 9, LBPB = 144, NAP = 4, XSG = 4;
  static constexpr bool SIDE_D = false;
};
template <>
struct StGeom<KQ_Q5_K> {
  static constexpr int BPB = 176, PP = 11, LBPB = 176, NAP = 4, XSG = 4;
  static constexpr bool SIDE_D = false;
};
template <>
struct StGeom<KQ_Q6_K> {
  static constexpr int BPB = 210, PP = 13, LBPB = 208, NAP = 8, XSG = 8;
  static constexpr bool SIDE_D = true;
};
// q2_k (84 bytes) and q3_k (110): the last piece of a block starts at BPB - 16, overlapping the one before it,
// so that whole blocks travel as 16-byte pieces.  LDS row of q2_k: scales[16] | qs[64] at 16 | piece 5 =
// block bytes 68 .. 83 at 80 (d at 92, dmin at 94).  q3_k: hmask[32] | qs[64] at 32 | piece 6 = block bytes
// 94 .. 109 at 96 (scales[12] at 98, d at 110).
template <>
struct StGeom<KQ_Q2_K> {
  static constexpr int BPB = 84, PP = 6, LBPB = 96, NAP = 4, XSG = 8;
  static constexpr bool SIDE_D = false;
};
template <>
struct StGeom<KQ_Q3_K> {
  static constexpr int BPB = 110, PP = 7, LBPB = 112, NAP = 4, XSG = 8;
  static constexpr bool SIDE_D = false;
};
// The codebook codecs put their byte arrays on 16-byte LDS boundaries by starting pieces at odd block offsets:
//   iq4_xs  (136): piece 0 = bytes 0 .. 15 (d, scales_h, scales_l), piece i = bytes 8 + 16 (i - 1) ..: qs[q] at 16 + q
//   iq2_xxs  (66): pieces at 0, 2, 18, 34, 50: d at 0, the eight 8-byte groups at 16 + 8 ib
template <>
struct StGeom<KQ_IQ4_XS> {
  static constexpr int BPB = 136, PP = 9, LBPB = 144, NAP = 4, XSG = 8;
  static constexpr bool SIDE_D = false;
};
template <>
struct StGeom<KQ_IQ2_XXS> {
  static constexpr int BPB = 66, PP = 5, LBPB = 80, NAP = 4, XSG = 8;
  static constexpr bool SIDE_D = false;
};
//   iq3_s  (110): pieces at 2, 18, .., 82 and 94; d travels as a 2-byte load per row.  LDS row: qs[64] at 0,
//                 qh[8] at 64, sign words 0..5 at 72 + 4 k, block bytes 94 .. 109 at 96 (sign words 6, 7 at 100,
//                 104; scales[4] at 108)
template <>
struct StGeom<KQ_IQ3_S> {
  static constexpr int BPB = 110, PP = 7, LBPB = 112, NAP = 4, XSG = 8;
  static constexpr bool SIDE_D = true;
};
//   q8_0: a "superblock" is eight 34-byte blocks (272 bytes), copied as they lie
template <>
struct StGeom<KQ_Q8_0> {
  static constexpr int BPB = 272, PP = 17, LBPB = 272, NAP = 4, XSG = 4;
  static constexpr bool SIDE_D = false;
};
//   iq4_nl / q4_0 (eight 18-byte blocks = 144 bytes, copied as they lie) and mxfp4 (eight 17-byte blocks = 136
//   bytes, the last piece starting at 120 like q2_k's): a byte holds weights j and j + 16 of its block, as in iq4_xs
template <>
struct StGeom<KQ_IQ4_NL> {
  static constexpr int BPB = 144, PP = 9, LBPB = 144, NAP = 4, XSG = 8;
  static constexpr bool SIDE_D = false;
};
template <>
struct StGeom<KQ_Q4_0> {
  static constexpr int BPB = 144, PP = 9, LBPB = 144, NAP = 4, XSG = 8;
  static constexpr bool SIDE_D = false;
};
template <>
struct StGeom<KQ_MXFP4> {
  static constexpr int BPB = 136, PP = 9, LBPB = 144, NAP = 4, XSG = 8;
  static constexpr bool SIDE_D = false;
};
//   nvfp4: four 36-byte blocks of 64 weights (four e4m3 scales, then 8 bytes per 16 weights whose byte j holds
//   weights j and j + 8 of its 16), 144 bytes copied as they lie
template <>
struct StGeom<KQ_NVFP4> {
  static constexpr int BPB = 144, PP = 9, LBPB = 144, NAP = 4, XSG = 8;
  static constexpr bool SIDE_D = false;
};
// codecs decoded through the byte -> f16 pair table (one copy per LDS bank)
template <int C>
constexpr bool st_pair_table() {
  return C == KQ_IQ4_XS || C == KQ_IQ4_NL || C == KQ_Q4_0 || C == KQ_MXFP4 || C == KQ_NVFP4;
}
// block byte of the f16 d that travels on its own (SIDE_D)
template <int C>
constexpr uint32_t st_side_d_off() { return C == KQ_Q6_K ? 208u : 0u; }
// byte offset of piece p inside a block
template <int C>
__device__ __forceinline__ uint32_t st_piece_off(int p) {
  using G = StGeom<C>;
  if constexpr (C == KQ_Q2_K || C == KQ_Q3_K || C == KQ_MXFP4)
    return p == G::PP - 1 ? (uint32_t)(G::BPB - 16) : 16u * (uint32_t)p;
  if constexpr (C == KQ_IQ4_XS) return p == 0 ? 0u : 16u * (uint32_t)p - 8u;
  if constexpr (C == KQ_IQ2_XXS) return p == 0 ? 0u : 16u * (uint32_t)p - 14u;
  if constexpr (C == KQ_IQ3_S) return p == 6 ? 94u : 16u * (uint32_t)p + 2u;
  return 16u * (uint32_t)p;
}
// Order of the staged f16 activations inside a group: 0 = k0 k2 k1 k3 per four (the order the masked-in-place codes
// leave a 32-bit word in), 1 = k0 k1 k2 k3 (codebook entries), 2 = x[j], x[j + 16] interleaved over 32 (iq4_xs: a
// byte holds weights j and j + 16 of its sub-block), 3 = x[j], x[j + 8] interleaved over 16 (nvfp4).
template <int C>
constexpr int st_xord() {
  return C == KQ_NVFP4 ? 3 : st_pair_table<C>() ? 2 : C == KQ_IQ2_XXS || C == KQ_IQ3_S || C == KQ_Q8_0 ? 1 : 0;
}
// LDS bytes of the decode tables a workgroup builds for itself
//   iq4_xs:  [256][32] byte -> f16 pair (kvalues[low nibble], kvalues[high nibble]), one copy per LDS bank: lane l
//            reads copy l % 32, so the 64 data-dependent reads of an instruction never meet in a bank (with a single
//            copy the bank conflicts took about half of the kernel's time)
//   iq2_xxs: [256] grid entry as eight f16 | [128] sign index -> eight f16 sign masks
//   iq3_s:   [512] grid entry as four f16 | [256] sign byte -> eight f16 sign masks; the one-row eight-wave kernel
//            has the LDS for [16 sign nibbles][512] entries with the signs applied (64 KiB, in front of the plain
//            entries it is built from): one table read per four weights and no XOR.  With the two-table form the
//            kernel is bound by the LDS (88 % busy, 63 % of that bank conflicts of the data-dependent reads).
template <int C, int MB = 0, int NW = 0, int GM = 0>
constexpr bool st_iq3s_merged() { return C == KQ_IQ3_S && MB == 1 && NW == 8 && GM == 0; }
// iq2_xxs, one-row eight-wave kernel: 16 copies of both tables, entry e copy c at 256 e + 16 c, lane l reads copy
// l % 16, so the sixteen lanes of a 16-byte read never meet in a bank (with single copies the kernel is bound by the
// LDS: 90 % busy, 60 % of that bank conflicts).
template <int C, int MB = 0, int NW = 0, int GM = 0>
constexpr int st_iq2_copies() { return C == KQ_IQ2_XXS && MB == 1 && NW == 8 && GM == 0 ? 16 : 1; }
// (gathered launches, whose workgroups live for one to four units, keep the plain iq2_xxs / iq3_s tables)
template <int C, int MB = 0, int NW = 0, int GM = 0>
constexpr int st_tbl_bytes() {
  return st_pair_table<C>() ? 32768 : C == KQ_IQ2_XXS ? (4096 + 2048) * st_iq2_copies<C, MB, NW, GM>() :
         st_iq3s_merged<C, MB, NW, GM>() ? 65536 + 4096 : C == KQ_IQ3_S ? 4096 + 4096 : 0;
}
// Codecs of 32-weight blocks whose unit is eight blocks copied as they lie: K may end inside a unit (any multiple
// of 32).  The last unit of a row then holds K % 256 / 32 blocks, T bytes.  Nothing past the row's end is read:
// pieces that lie inside the T bytes travel as usual; the piece the row ends in (16 ps < T < 16 ps + 16) is fetched
// from T - 16, so that it ends with the row, and the wave then moves its bytes down to where the unit expects them;
// pieces that start past the end are fetched from the unit's start (their blocks get a zero scale and zero
// activations, whatever bytes they hold).
template <int C>
constexpr bool st_tail_codec() { return C == KQ_MXFP4 || C == KQ_Q4_0 || C == KQ_IQ4_NL || C == KQ_Q8_0; }
template <int C>
struct StUnit {
  using G = StGeom<C>;
  static constexpr int PIECES = ST_ROWS * G::PP;
  static constexpr int FULL = PIECES / 64;                // load instructions with all 64 lanes
  static constexpr bool HALF = (PIECES % 64) != 0;        // one more with 32 lanes
  static constexpr int UPI = FULL + (HALF ? 1 : 0) + (G::SIDE_D ? 1 : 0);  // load instructions per unit
  static constexpr int SLOT = ST_ROWS * G::LBPB + (G::SIDE_D ? 128 : 0);   // LDS bytes per unit
};

struct StArgs {
  const void* x;
  const uint8_t* w;
  void* y;
  int M, N, K, tiles;
  const uint8_t* grids;  // device copy of the IQ codebooks (codebook codecs)
  int rpt;  // weight rows per tile (<= 32): fewer than 32 evens the rows out over one round of workgroups
  float* partial;  // split-K: [ksplit][M][N] f32
  const uint16_t* bias16;  // dense calls without a K split: null, or [N] in the activation dtype, added in f32
  int ksplit, sb_per_split;
  // gathered calls (one activation row per entry, MoE decode): entry p = blockIdx.x / tiles_per_entry multiplies row
  // p / x_div of x by rows of expert rhs[p] (w, and w2 = the up stack of the fused gate / up form) into output row
  // out_row(om, p); entries whose expert id is >= E are skipped
  const uint8_t* w2;
  const uint32_t* rhs;
  const uint32_t* lhs;     // null, or the entry's activation row: x + lhs[p] * x_row_stride (x_div is then unused)
  int64_t x_row_stride;
  int tiles_per_entry, x_div, E, act;
  float limit, alpha;
  const float* bias;   // null, or f32 [E][N] added to the (gate) sums before the epilogue
  const float* bias2;  // the same for the up sums of the fused form
  int64_t w_expert_stride;
  KqOutMap om;
};

// ------------------------------------------------------------------ q4_k / q5_k unit
// Lane (row, kg) owns sub-blocks 4 kg .. 4 kg + 3.  LDS row: d, dmin, scales[12] | (q5_k: qh[32]) | qs[128].
// Pieces qs[64 kg + 16 pc ..), pc = 0..3: pair pc / 2 of the half, weights 16 (pc % 2) .. + 15 of the low-nibble
// sub-block 2 (pc / 2) and of the high-nibble sub-block 2 (pc / 2) + 1.  MFMA (pc, e, h): word e of the piece,
// nibble h; activations = A pair pc, block 2 e + h.
// R activation rows in RG = ceil(R / 4) groups of four; group g keeps its A registers at areg[g * AS + ...].
template <int C, int R, int AS>
__device__ __forceinline__ void q45k_unit(const uint8_t* __restrict__ bl, int kg, float xscale, const u32x2* areg,
                                          const float* __restrict__ xsum, int xsum_row_stride, float* acc) {
  constexpr int QS = C == KQ_Q4_K ? 16 : 48;
  constexpr int RG = (R + 3) / 4;
  const u32x4 hdr = *reinterpret_cast<const u32x4*>(bl);
  u32x4 q[4];
#pragma unroll
  for (int i = 0; i < 4; i++) q[i] = *reinterpret_cast<const u32x4*>(bl + QS + 64 * kg + 16 * i);
  uint32_t hw[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if constexpr (C == KQ_Q5_K) {
    // fifth bits: bit j of qh[l] belongs to sub-block j; shifted down by 4 kg they sit at bits 0..3 of every byte
    const u32x4 h0 = *reinterpret_cast<const u32x4*>(bl + 16), h1 = *reinterpret_cast<const u32x4*>(bl + 32);
    const int sh = 4 * kg;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      hw[e] = h0[e] >> sh;
      hw[4 + e] = h1[e] >> sh;
    }
  }
  float xs[R][4];
#pragma unroll
  for (int r = 0; r < R; r++) {
    const float4 t4 = *reinterpret_cast<const float4*>(xsum + r * xsum_row_stride + 4 * kg);
    xs[r][0] = t4.x;
    xs[r][1] = t4.y;
    xs[r][2] = t4.z;
    xs[r][3] = t4.w;
  }
  // scales of this lane's four sub-blocks
  float mul[4], sub[4];
  {
    const float d = kq::h2f((uint16_t)(hdr.x & 0xffff)) * xscale;
    const float dmin = kq::h2f((uint16_t)(hdr.x >> 16)) * xscale;
    const float d16 = d * 0.0625f;
    const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
    const uint32_t sc_lo = s0 & 0x3f3f3f3fu, mn_lo = s1 & 0x3f3f3f3fu;
    const uint32_t sc_hi = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
    const uint32_t scw = kg ? sc_hi : sc_lo, mnw = kg ? mn_hi : mn_lo;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const float sc = (float)((scw >> (8 * j)) & 0xff);
      const float mn = (float)((mnw >> (8 * j)) & 0xff);
      // even sub-blocks read low nibbles (1024 + q), odd ones high nibbles in place (1024 + 16 q)
      mul[j] = ((j & 1) ? d16 : d) * sc;
      sub[j] = fmaf(mul[j], 1024.0f, dmin * mn);
    }
  }
  const uint32_t magic = opaque_vgpr(0x64006400u);
  const uint32_t mask_lo = opaque_sgpr(0x000f000fu), mask_hi = opaque_sgpr(0x00f000f0u);
  const uint32_t bit_lo = opaque_sgpr(0x00100010u), bit_hi = opaque_sgpr(0x01000100u);
  SFor<2>::run([&](auto gg) {
    constexpr int gl = decltype(gg)::value;
    f32x4 p[RG][2];
#pragma unroll
    for (int g = 0; g < RG; g++) p[g][0] = p[g][1] = f32x4{0, 0, 0, 0};
    SFor<2>::run([&](auto pp) {
      constexpr int pc = 2 * gl + decltype(pp)::value;
      f16x4 av[RG];
#pragma unroll
      for (int g = 0; g < RG; g++) av[g] = __builtin_bit_cast(f16x4, areg[g * AS + pc]);
      SFor<4>::run([&](auto ee) {
        constexpr int e = decltype(ee)::value;
        const uint32_t w0 = q[pc][e], w8 = w0 >> 8;
        SFor<2>::run([&](auto hh) {
          constexpr int h = decltype(hh)::value;
          u32x2 bv;
          bv.x = and_or(w0, h ? mask_hi : mask_lo, magic);  // weights l, l + 2
          bv.y = and_or(w8, h ? mask_hi : mask_lo, magic);  // weights l + 1, l + 3
          if constexpr (C == KQ_Q5_K) {
            // bit jl = 2 gl + h of the four qh bytes of weights l .. l + 3 goes to bit 4 (1024 + q + 16 b) or
            // bit 8 (1024 + 16 q + 256 b) of the 16-bit code
            constexpr int jl = 2 * gl + h, tgt = h ? 8 : 4;
            const uint32_t hq = hw[4 * (pc & 1) + e];
            bv.x = and_or(hq << (tgt - jl), h ? bit_hi : bit_lo, opaque_vgpr(bv.x));
            bv.y = and_or(hq >> (8 + jl - tgt), h ? bit_hi : bit_lo, opaque_vgpr(bv.y));
          }
#pragma unroll
          for (int g = 0; g < RG; g++)
            p[g][h] = __builtin_amdgcn_mfma_f32_4x4x4f16(av[g], __builtin_bit_cast(f16x4, bv), p[g][h], 3, 2 * e + h, 0);
        });
      });
    });
    SFor<2>::run([&](auto hh) {
      constexpr int h = decltype(hh)::value;
      constexpr int jl = 2 * gl + h;
      SFor<R>::run([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        acc[r] = fmaf(mul[jl], p[r / 4][h][r % 4], acc[r]);
        acc[r] = fmaf(-sub[jl], xs[r][jl], acc[r]);
      });
    });
  });
}

// ------------------------------------------------------------------ q2_k / q3_k unit
// Lane (row, kg) owns half kg of the superblock: weights 128 kg + 32 j + l, field j = 0..3 (bits 2 j, 2 j + 1 of
// qs[32 kg + l]), l = 0..31; sub-block (16 weights, one scale) 8 kg + 2 j + l / 16.  Fields are masked in place:
// 1024 + 4^j q.  q3_k: the third bit of the weight (hmask[l] bit 4 kg + j) is moved next to its field, bit
// 2 j + 2, so the code reads 1024 + 4^j (q2 + 4 h), and the weight is q - 4.
// MFMA (j, wi): word wi of the half, l = 4 wi .. 4 wi + 3; activations = A pair j, block wi.
template <int C, int R, int AS>
__device__ __forceinline__ void q23k_unit(const uint8_t* __restrict__ bl, int kg, float xscale, const u32x2* areg,
                                          const float* __restrict__ xsum, int xsum_row_stride, float* acc) {
  constexpr int RG = (R + 3) / 4;
  constexpr int QS = C == KQ_Q2_K ? 16 : 32;
  u32x4 q[2];
#pragma unroll
  for (int i = 0; i < 2; i++) q[i] = *reinterpret_cast<const u32x4*>(bl + QS + 32 * kg + 16 * i);
  uint32_t w8[8];
#pragma unroll
  for (int i = 0; i < 8; i++) w8[i] = q[i >> 2][i & 3] >> 8;
  uint32_t hw[8] = {0, 0, 0, 0, 0, 0, 0, 0}, hw8[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  float mul[8], sub[8];
  if constexpr (C == KQ_Q2_K) {
    const uint2 scw = *reinterpret_cast<const uint2*>(bl + 8 * kg);
    const uint32_t dd = *reinterpret_cast<const uint32_t*>(bl + 92);
    const float d = kq::h2f((uint16_t)(dd & 0xffff)) * xscale, dmin = kq::h2f((uint16_t)(dd >> 16)) * xscale;
#pragma unroll
    for (int sl = 0; sl < 8; sl++) {
      const uint32_t b = ((sl < 4 ? scw.x : scw.y) >> (8 * (sl & 3))) & 0xff;
      const float sc = (float)(b & 0xf), mn = (float)(b >> 4);
      const float f = 1.0f / (float)(1 << (2 * (sl >> 1)));  // 1 / 4^j
      mul[sl] = d * sc * f;
      sub[sl] = fmaf(mul[sl], 1024.0f, dmin * mn);
    }
  } else {
    const u32x4 hm0 = *reinterpret_cast<const u32x4*>(bl), hm1 = *reinterpret_cast<const u32x4*>(bl + 16);
    const int sh = 4 * kg;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      hw[i] = hm0[i] >> sh;
      hw[4 + i] = hm1[i] >> sh;
    }
#pragma unroll
    for (int i = 0; i < 8; i++) hw8[i] = hw[i] >> 8;
    // block bytes 94 .. 109 sit at 96 .. 111: scales[12] from 98, d at 110
    const u32x4 t = *reinterpret_cast<const u32x4*>(bl + 96);
    const uint32_t aux0 = __builtin_amdgcn_alignbyte(t[1], t[0], 2), aux1 = __builtin_amdgcn_alignbyte(t[2], t[1], 2);
    const uint32_t tmp = __builtin_amdgcn_alignbyte(t[3], t[2], 2) >> sh;
    const float d = kq::h2f((uint16_t)(t[3] >> 16)) * xscale;
    const uint32_t lo = ((aux0 >> sh) & 0x0f0f0f0fu) | ((tmp & 0x03030303u) << 4);
    const uint32_t hi = ((aux1 >> sh) & 0x0f0f0f0fu) | (((tmp >> 2) & 0x03030303u) << 4);
#pragma unroll
    for (int sl = 0; sl < 8; sl++) {
      const float sc = (float)(int)(((sl < 4 ? lo : hi) >> (8 * (sl & 3))) & 0xff) - 32.0f;
      const float f = 1.0f / (float)(1 << (2 * (sl >> 1)));
      mul[sl] = d * sc * f;
      sub[sl] = d * sc * (1024.0f * f + 4.0f);
    }
  }
  float xs[R][8];
#pragma unroll
  for (int r = 0; r < R; r++) {
    const float4 t0 = *reinterpret_cast<const float4*>(xsum + r * xsum_row_stride + 8 * kg);
    const float4 t1 = *reinterpret_cast<const float4*>(xsum + r * xsum_row_stride + 8 * kg + 4);
    xs[r][0] = t0.x; xs[r][1] = t0.y; xs[r][2] = t0.z; xs[r][3] = t0.w;
    xs[r][4] = t1.x; xs[r][5] = t1.y; xs[r][6] = t1.z; xs[r][7] = t1.w;
  }
  const uint32_t magic = opaque_vgpr(0x64006400u);
  const uint32_t mask_f[4] = {opaque_sgpr(0x00030003u), opaque_sgpr(0x000c000cu), opaque_sgpr(0x00300030u),
                              opaque_sgpr(0x00c000c0u)};
  const uint32_t bit_f[4] = {opaque_sgpr(0x00040004u), opaque_sgpr(0x00100010u), opaque_sgpr(0x00400040u),
                             opaque_sgpr(0x01000100u)};
  (void)bit_f;
  SFor<4>::run([&](auto jj) {
    constexpr int j = decltype(jj)::value;
    f16x4 av[RG];
#pragma unroll
    for (int g = 0; g < RG; g++) av[g] = __builtin_bit_cast(f16x4, areg[g * AS + j]);
    SFor<2>::run([&](auto hh) {
      constexpr int hs = decltype(hh)::value;  // l / 16
      f32x4 p[RG];
#pragma unroll
      for (int g = 0; g < RG; g++) p[g] = f32x4{0, 0, 0, 0};
      SFor<4>::run([&](auto ee) {
        constexpr int wi = 4 * hs + decltype(ee)::value;
        u32x2 bv;
        bv.x = and_or(q[wi >> 2][wi & 3], mask_f[j], magic);  // weights l, l + 2
        bv.y = and_or(w8[wi], mask_f[j], magic);              // weights l + 1, l + 3
        if constexpr (C == KQ_Q3_K) {
          bv.x = and_or(hw[wi] << (j + 2), bit_f[j], opaque_vgpr(bv.x));
          bv.y = and_or(hw8[wi] << (j + 2), bit_f[j], opaque_vgpr(bv.y));
        }
#pragma unroll
        for (int g = 0; g < RG; g++)
          p[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(av[g], __builtin_bit_cast(f16x4, bv), p[g], 3, wi, 0);
      });
      constexpr int sl = 2 * j + hs;
      SFor<R>::run([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        acc[r] = fmaf(mul[sl], p[r / 4][r % 4], acc[r]);
        acc[r] = fmaf(-sub[sl], xs[r][sl], acc[r]);
      });
    });
  });
}

// ------------------------------------------------------------------ q8_0 unit
// Lane (row, kg) owns blocks 4 kg .. 4 kg + 3 of the row's eight: 136 bytes at 136 kg, read as 34 dwords.  A block
// at an even position has its quants 2 bytes past a dword boundary (realigned with v_alignbyte), an odd one on it.
// A quant byte b becomes the f16 1024 + (b ^ 0x80) = q + 1152 by a byte permute, and the exact packed subtraction of
// 1152 leaves q.  MFMA (ib, q): weights 4 q .. 4 q + 3 of block ib; activations = A pair ib, block q.
template <int R, int AS>
__device__ __forceinline__ void q80_unit(const uint8_t* __restrict__ bl, int kg, float xscale, const u32x2* areg,
                                         float* acc, int nvalid) {
  constexpr int RG = (R + 3) / 4;
  typedef _Float16 f16x2v __attribute__((ext_vector_type(2)));
  const uint8_t* p8 = bl + 136 * kg;
  uint32_t w[34];
#pragma unroll
  for (int i = 0; i < 17; i++) {
    const u32x2 v = *reinterpret_cast<const u32x2*>(p8 + 8 * i);
    w[2 * i] = v.x;
    w[2 * i + 1] = v.y;
  }
  const uint32_t flip = opaque_sgpr(0x80808080u), magic = opaque_vgpr(0x64646464u);
  const f16x2v off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
  SFor<4>::run([&](auto ii) {
    constexpr int ib = decltype(ii)::value;
    // byte offset of block ib inside the 136: 34 ib -> dword 8.5 ib
    constexpr int d0 = (34 * ib) / 4;            // dword holding d
    constexpr bool even = (ib & 1) == 0;         // d in the low half of dword d0, quants straddle dwords
    // blocks past the end of K (the last unit of a row whose K ends inside it): scale 0 on sums of zero activations
    const float dl = 4 * kg + ib < nvalid ? kq::h2f((uint16_t)(even ? (w[d0] & 0xffffu) : (w[d0] >> 16))) * xscale : 0.f;
    f32x4 p[RG];
#pragma unroll
    for (int g = 0; g < RG; g++) p[g] = f32x4{0, 0, 0, 0};
    SFor<8>::run([&](auto qq) {
      constexpr int q = decltype(qq)::value;
      uint32_t qd;
      if constexpr (even)
        qd = __builtin_amdgcn_alignbyte(w[d0 + q + 1], w[d0 + q], 2);
      else
        qd = w[d0 + 1 + q];
      qd ^= flip;
      u32x2 bv;
      bv.x = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2v, __builtin_amdgcn_perm(magic, qd, 0x04010400u)) + off);
      bv.y = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2v, __builtin_amdgcn_perm(magic, qd, 0x04030402u)) + off);
#pragma unroll
      for (int g = 0; g < RG; g++)
        p[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, areg[g * AS + ib]),
                                                  __builtin_bit_cast(f16x4, bv), p[g], 3, q, 0);
    });
    SFor<R>::run([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      acc[r] = fmaf(dl, p[r / 4][r % 4], acc[r]);
    });
  });
}

// ------------------------------------------------------------------ iq4_xs unit
// Lane (row, kg) owns sub-blocks 4 kg .. 4 kg + 3 (16 bytes of qs each; byte j = weights j and j + 16).  One table
// read turns a byte into the f16 pair of its two codebook values; two bytes make the B operand of one MFMA,
// whose activations are staged in the matching order x[j], x[j + 16], x[j + 1], x[j + 17].
// MFMA (ib, q): bytes 2 q, 2 q + 1 of sub-block ib; activations = A pair ib, block q.
template <int R, int AS>
__device__ __forceinline__ void iq4xs_unit(const uint8_t* __restrict__ bl, int kg, float xscale, const u32x2* areg,
                                           const uint8_t* __restrict__ tbl, float* acc) {
  constexpr int RG = (R + 3) / 4;
  const u32x2 hdr = *reinterpret_cast<const u32x2*>(bl);
  const float d = kq::h2f((uint16_t)(hdr.x & 0xffff)) * xscale;
  const uint32_t sh = (hdr.x >> 16) >> (8 * kg), sl = hdr.y >> (16 * kg);
  // The table reads of sub-block ib + 1 are issued before the MFMAs of sub-block ib: left to itself the compiler
  // waits for every pair of reads right before the MFMA that uses it, one LDS round trip per MFMA.
  u32x2 bv[4][8];
  auto lookup = [&](auto ii) {
    constexpr int ib = decltype(ii)::value;
    const u32x4 qv = *reinterpret_cast<const u32x4*>(bl + 16 + 64 * kg + 16 * ib);
    SFor<8>::run([&](auto qq) {
      constexpr int q = decltype(qq)::value;
      const uint32_t w = qv[q >> 1];
      const uint32_t i0 = (w >> (16 * (q & 1))) & 0xff, i1 = (w >> (16 * (q & 1) + 8)) & 0xff;
      bv[ib][q].x = *reinterpret_cast<const uint32_t*>(tbl + 128 * i0);
      bv[ib][q].y = *reinterpret_cast<const uint32_t*>(tbl + 128 * i1);
    });
    __builtin_amdgcn_sched_barrier(0);
  };
  lookup(std::integral_constant<int, 0>{});
  SFor<4>::run([&](auto ii) {
    constexpr int ib = decltype(ii)::value;
    if constexpr (ib < 3) lookup(std::integral_constant<int, ib + 1>{});
    f32x4 p[RG];
#pragma unroll
    for (int g = 0; g < RG; g++) p[g] = f32x4{0, 0, 0, 0};
    SFor<8>::run([&](auto qq) {
      constexpr int q = decltype(qq)::value;
#pragma unroll
      for (int g = 0; g < RG; g++)
        p[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, areg[g * AS + ib]),
                                                  __builtin_bit_cast(f16x4, bv[ib][q]), p[g], 3, q, 0);
    });
    const int ls = (int)(((sl >> (4 * ib)) & 15) | (((sh >> (2 * ib)) & 3) << 4));
    const float dl = d * (float)(ls - 32);
    SFor<R>::run([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      acc[r] = fmaf(dl, p[r / 4][r % 4], acc[r]);
    });
  });
}

// ------------------------------------------------------------------ iq4_nl / q4_0 / mxfp4 / nvfp4 unit
// Lane (row, kg) owns blocks 4 kg .. 4 kg + 3 of the row's eight (18 or 17 bytes each: scale, then 16 bytes whose
// byte j holds weights j and j + 16).  The blocks' bytes are read as dwords and the 16 quant bytes of a block are
// brought onto dword boundaries with v_alignbyte; everything else is the iq4_xs unit: table read per byte, MFMA
// (ib, q) on bytes 2 q, 2 q + 1 of block ib, block scale on the partial sum.  nvfp4: the lane's 72 bytes are two
// 36-byte blocks, all fields on dword boundaries; "block" ib is then a pair of 16-weight groups with a scale each.
// half of an unsigned e4m3 scale (0 and 0x7f decode to 0), the value kq::ue4m3_half returns, without branches
__device__ __forceinline__ float ue4m3_half_fast(uint32_t x) {
  const uint32_t ex = (x >> 3) & 15u, man = x & 7u;
  const float normal = __builtin_bit_cast(float, ((ex + 119u) << 23) | (man << 20));
  const float sub = (float)man * 0x1p-10f;
  const float v = ex ? normal : sub;
  return x == 0x7fu ? 0.0f : v;
}
template <int C, int R, int AS>
__device__ __forceinline__ void nib32_unit(const uint8_t* __restrict__ bl, int kg, float xscale, const u32x2* areg,
                                           const uint8_t* __restrict__ tbl, float* acc, int nvalid) {
  constexpr int RG = (R + 3) / 4;
  constexpr bool NV = C == KQ_NVFP4;            // 36-byte blocks of 64: scale bytes 0 .. 3, 8 quant bytes per 16 weights
  constexpr int BB = C == KQ_MXFP4 ? 17 : 18;   // block bytes
  constexpr int HB = C == KQ_MXFP4 ? 1 : 2;     // scale bytes in front of the quants
  constexpr int NDW = 4 * BB / 4;               // 17 or 18 dwords per lane
  uint32_t w[NDW + 1];
  if constexpr (C == KQ_MXFP4) {
    // LDS row: block bytes 0 .. 127 as they lie, bytes 120 .. 135 again at 128: this lane's bytes 68 kg .. 68 kg + 67
    // are contiguous for kg = 0; for kg = 1 bytes 128 .. 135 sit at 136
#pragma unroll
    for (int i = 0; i < 15; i++) w[i] = *reinterpret_cast<const uint32_t*>(bl + 68 * kg + 4 * i);
    w[15] = *reinterpret_cast<const uint32_t*>(bl + (kg ? 136 : 60));
    w[16] = *reinterpret_cast<const uint32_t*>(bl + (kg ? 140 : 64));
    w[17] = 0u;
  } else {
#pragma unroll
    for (int i = 0; i < 9; i++) {
      const u32x2 v = *reinterpret_cast<const u32x2*>(bl + 72 * kg + 8 * i);
      w[2 * i] = v.x;
      w[2 * i + 1] = v.y;
    }
    w[18] = 0u;
  }
  u32x2 bv[4][8];
  auto lookup = [&](auto ii) {
    constexpr int ib = decltype(ii)::value;
    // first quant byte of the block (nvfp4: of the 16 bytes of groups 2 (ib % 2), 2 (ib % 2) + 1 of block ib / 2)
    constexpr int o = NV ? 36 * (ib / 2) + 4 + 16 * (ib % 2) : BB * ib + HB, base = o / 4, sh = o % 4;
    uint32_t qv[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
      qv[i] = sh == 0 ? w[base + i] : __builtin_amdgcn_alignbyte(w[base + i + 1], w[base + i], sh);
    SFor<8>::run([&](auto qq) {
      constexpr int q = decltype(qq)::value;
      const uint32_t ww = qv[q >> 1];
      const uint32_t i0 = (ww >> (16 * (q & 1))) & 0xff, i1 = (ww >> (16 * (q & 1) + 8)) & 0xff;
      bv[ib][q].x = *reinterpret_cast<const uint32_t*>(tbl + 128 * i0);
      bv[ib][q].y = *reinterpret_cast<const uint32_t*>(tbl + 128 * i1);
    });
    __builtin_amdgcn_sched_barrier(0);
  };
  lookup(std::integral_constant<int, 0>{});
  SFor<4>::run([&](auto ii) {
    constexpr int ib = decltype(ii)::value;
    if constexpr (ib < 3) lookup(std::integral_constant<int, ib + 1>{});
    f32x4 p[RG], p2[RG];  // p2: the second 16 weights of the 32 (nvfp4: a scale of their own)
#pragma unroll
    for (int g = 0; g < RG; g++) p[g] = p2[g] = f32x4{0, 0, 0, 0};
    SFor<8>::run([&](auto qq) {
      constexpr int q = decltype(qq)::value;
#pragma unroll
      for (int g = 0; g < RG; g++) {
        if constexpr (NV && q >= 4)
          p2[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, areg[g * AS + ib]),
                                                     __builtin_bit_cast(f16x4, bv[ib][q]), p2[g], 3, q, 0);
        else
          p[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(f16x4, areg[g * AS + ib]),
                                                    __builtin_bit_cast(f16x4, bv[ib][q]), p[g], 3, q, 0);
      }
    });
    if constexpr (NV) {
      const uint32_t sw = w[9 * (ib / 2)] >> (16 * (ib % 2));
      const float d0 = ue4m3_half_fast(sw & 0xffu) * xscale, d1 = ue4m3_half_fast((sw >> 8) & 0xffu) * xscale;
      SFor<R>::run([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        acc[r] = fmaf(d0, p[r / 4][r % 4], acc[r]);
        acc[r] = fmaf(d1, p2[r / 4][r % 4], acc[r]);
      });
      return;
    }
    constexpr int so = BB * ib;  // scale byte(s) of the block
    float dl;
    if constexpr (C == KQ_MXFP4)
      dl = kq::e8m0_half((w[so / 4] >> (8 * (so % 4))) & 0xffu) * xscale;
    else
      dl = kq::h2f((uint16_t)((w[so / 4] >> (8 * (so % 4))) & 0xffffu)) * xscale;
    dl = 4 * kg + ib < nvalid ? dl : 0.f;  // blocks past the end of K: scale 0 on sums of zero activations
    SFor<R>::run([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      acc[r] = fmaf(dl, p[r / 4][r % 4], acc[r]);
    });
  });
}

// ------------------------------------------------------------------ iq2_xxs unit
// Lane (row, kg) owns the 8-byte groups 4 kg .. 4 kg + 3 (32 weights each): four grid index bytes, then a word of
// four 7-bit sign indices and the 4-bit scale.  Index -> eight f16 magnitudes, sign index -> eight f16 sign
// masks (16-byte table reads), XOR.  MFMAs (ib, l, half): A pair ib, block 2 l + half.
// COP copies of every table entry, 16 bytes apart (tbl already points at the lane's copy).
template <int R, int AS, int COP>
__device__ __forceinline__ void iq2xxs_unit(const uint8_t* __restrict__ bl, int kg, float xscale, const u32x2* areg,
                                            const uint8_t* __restrict__ tbl, float* acc) {
  constexpr int RG = (R + 3) / 4;
  const float d = kq::h2f(*reinterpret_cast<const uint16_t*>(bl)) * xscale * 0.25f;
  const u32x4 q0 = *reinterpret_cast<const u32x4*>(bl + 16 + 32 * kg), q1 = *reinterpret_cast<const u32x4*>(bl + 32 + 32 * kg);
  const uint8_t* stbl = tbl + 4096 * COP;
  // The table reads of group ib + 1 are issued before the MFMAs of group ib (see iq4xs_unit).
  u32x4 gv[4][4], sm[4][4];
  uint32_t a1s[4];
  auto lookup = [&](auto ii) {
    constexpr int ib = decltype(ii)::value;
    const uint32_t gi = ib < 2 ? q0[2 * ib] : q1[2 * (ib - 2)], a1 = ib < 2 ? q0[2 * ib + 1] : q1[2 * (ib - 2) + 1];
    a1s[ib] = a1;
    SFor<4>::run([&](auto ll) {
      constexpr int l = decltype(ll)::value;
      const uint32_t idx = (gi >> (8 * l)) & 0xff, si = (a1 >> (7 * l)) & 127;
      gv[ib][l] = *reinterpret_cast<const u32x4*>(tbl + 16 * COP * idx);
      sm[ib][l] = *reinterpret_cast<const u32x4*>(stbl + 16 * COP * si);
    });
    __builtin_amdgcn_sched_barrier(0);
  };
  lookup(std::integral_constant<int, 0>{});
  SFor<4>::run([&](auto ii) {
    constexpr int ib = decltype(ii)::value;
    if constexpr (ib < 3) lookup(std::integral_constant<int, ib + 1>{});
    f32x4 p[RG];
#pragma unroll
    for (int g = 0; g < RG; g++) p[g] = f32x4{0, 0, 0, 0};
    SFor<4>::run([&](auto ll) {
      constexpr int l = decltype(ll)::value;
      const u32x4 v = gv[ib][l] ^ sm[ib][l];
      const u32x2 lo = {v[0], v[1]}, hi = {v[2], v[3]};
#pragma unroll
      for (int g = 0; g < RG; g++) {
        const f16x4 av = __builtin_bit_cast(f16x4, areg[g * AS + ib]);
        p[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(av, __builtin_bit_cast(f16x4, lo), p[g], 3, 2 * l, 0);
        p[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(av, __builtin_bit_cast(f16x4, hi), p[g], 3, 2 * l + 1, 0);
      }
    });
    const float dl = d * (0.5f + (float)(a1s[ib] >> 28));
    SFor<R>::run([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      acc[r] = fmaf(dl, p[r / 4][r % 4], acc[r]);
    });
  });
}

// ------------------------------------------------------------------ iq3_s unit
// Lane (row, kg) owns the 32-weight blocks 4 kg .. 4 kg + 3: eight index bytes each (the ninth index bit is bit j
// of the block's qh byte), four sign bytes (one per eight weights) and a 4-bit scale.  Index -> four f16
// magnitudes (8-byte table read), sign byte -> eight f16 sign masks (16-byte read), XOR.  MFMAs (ib, l, half):
// index 2 l + half of the block; A pair ib, block 2 l + half.
// MERGED: tbl holds [16][512] entries with the signs of a nibble applied; index | nibble << 9.
template <int R, int AS, bool MERGED>
__device__ __forceinline__ void iq3s_unit(const uint8_t* __restrict__ bl, int kg, float dx, const u32x2* areg,
                                          const uint8_t* __restrict__ tbl, float* acc) {
  constexpr int RG = (R + 3) / 4;
  const u32x4 qa = *reinterpret_cast<const u32x4*>(bl + 32 * kg), qb = *reinterpret_cast<const u32x4*>(bl + 32 * kg + 16);
  const uint32_t qh = *reinterpret_cast<const uint32_t*>(bl + 64 + 4 * kg);
  const uint32_t scw = *reinterpret_cast<const uint32_t*>(bl + 108) >> (16 * kg);
  const uint8_t* sgp = bl + 72 + 16 * kg;
  const uint8_t* stbl = tbl + 4096;
  u32x2 gv[4][8];
  u32x4 sm[4][4];
  auto lookup = [&](auto ii) {
    constexpr int ib = decltype(ii)::value;
    const uint32_t w0 = ib < 2 ? qa[2 * ib] : qb[2 * (ib - 2)], w1 = ib < 2 ? qa[2 * ib + 1] : qb[2 * (ib - 2) + 1];
    const uint32_t hb = qh >> (8 * ib);
    // sign words 6 and 7 of the block sit four bytes further (behind the two bytes the last piece repeats)
    const uint32_t sw = *reinterpret_cast<const uint32_t*>(sgp + 4 * ib + (ib >= 2 ? 4 * kg : 0));
    if constexpr (MERGED) {
      // 13-bit table index of value j = index byte | high bit << 8 | sign nibble << 9, built two per dword with byte
      // permutes: the high bits spread to the low bit of each byte (even and odd values apart, by a 24-bit multiply
      // whose partial products meet only beside the kept bits), the sign nibbles shifted beside them, then
      // interleaved with the index bytes.
      const uint32_t he = __umul24(hb & 0x55u, 0x41041u) & 0x01010101u;
      const uint32_t ho = __umul24((hb >> 1) & 0x55u, 0x41041u) & 0x01010101u;
      const uint32_t ce = ((sw << 1) & 0x1e1e1e1eu) | he, co = ((sw >> 3) & 0x1e1e1e1eu) | ho;
      const uint32_t c03 = __builtin_amdgcn_perm(co, ce, 0x05010400u), c47 = __builtin_amdgcn_perm(co, ce, 0x07030602u);
      const uint32_t pr[4] = {__builtin_amdgcn_perm(c03, w0, 0x05010400u), __builtin_amdgcn_perm(c03, w0, 0x07030602u),
                              __builtin_amdgcn_perm(c47, w1, 0x05010400u), __builtin_amdgcn_perm(c47, w1, 0x07030602u)};
      SFor<8>::run([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        const uint32_t idx = (j & 1) ? pr[j / 2] >> 16 : pr[j / 2] & 0xffffu;
        gv[ib][j] = *reinterpret_cast<const u32x2*>(tbl + 8 * idx);
      });
    } else {
      SFor<8>::run([&](auto jj) {
        constexpr int j = decltype(jj)::value;
        const uint32_t w = j < 4 ? w0 : w1;
        const uint32_t idx = ((w >> (8 * (j & 3))) & 0xff) | (((hb >> j) & 1) << 8);
        gv[ib][j] = *reinterpret_cast<const u32x2*>(tbl + 8 * idx);
      });
    }
    if constexpr (!MERGED) {
      SFor<4>::run([&](auto ll) {
        constexpr int l = decltype(ll)::value;
        sm[ib][l] = *reinterpret_cast<const u32x4*>(stbl + 16 * ((sw >> (8 * l)) & 0xff));
      });
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  lookup(std::integral_constant<int, 0>{});
  SFor<4>::run([&](auto ii) {
    constexpr int ib = decltype(ii)::value;
    if constexpr (ib < 3) lookup(std::integral_constant<int, ib + 1>{});
    f32x4 p[RG];
#pragma unroll
    for (int g = 0; g < RG; g++) p[g] = f32x4{0, 0, 0, 0};
    SFor<4>::run([&](auto ll) {
      constexpr int l = decltype(ll)::value;
      u32x2 lo = gv[ib][2 * l], hi = gv[ib][2 * l + 1];
      if constexpr (!MERGED) {
        lo = u32x2{lo[0] ^ sm[ib][l][0], lo[1] ^ sm[ib][l][1]};
        hi = u32x2{hi[0] ^ sm[ib][l][2], hi[1] ^ sm[ib][l][3]};
      }
#pragma unroll
      for (int g = 0; g < RG; g++) {
        const f16x4 av = __builtin_bit_cast(f16x4, areg[g * AS + ib]);
        p[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(av, __builtin_bit_cast(f16x4, lo), p[g], 3, 2 * l, 0);
        p[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(av, __builtin_bit_cast(f16x4, hi), p[g], 3, 2 * l + 1, 0);
      }
    });
    const float dl = dx * (float)(1 + 2 * (int)((scw >> (4 * ib)) & 15));
    SFor<R>::run([&](auto rr) {
      constexpr int r = decltype(rr)::value;
      acc[r] = fmaf(dl, p[r / 4][r % 4], acc[r]);
    });
  });
}

// ------------------------------------------------------------------ q6_k unit
// Lane (row, hf) owns half hf of the superblock: weights 128 hf + 32 t + l, t = 0..3, l = 0..31.  LDS row:
// ql[128] | qh[64] | int8 scales[16]; d sits in the slot's side area (one dword per row).  Low nibble of the
// weight: ql[64 hf + 32 (t & 1) + l] (high nibble of the byte for t >= 2); high bits: bits 2 t, 2 t + 1 of
// qh[32 hf + l]; scale 8 hf + 2 t + l / 16.  Both fields are masked in place: 1024 + s ql with s = 1 (t < 2) or
// 16, 1024 + 4^t qh.  Per scale group of 16 weights two accumulators P, H and
//   sum x w = d sc (P / s + 16 H / 4^t - (1024 / s + 16 * 1024 / 4^t + 32) X).
// MFMA (t, e): weights l = 4 e .. 4 e + 3; activations = A pair 2 t + e / 4, block 2 (e % 4) [+ 1 unused].
template <int R, int AS>
__device__ __forceinline__ void q6k_unit(const uint8_t* __restrict__ bl, float dx, int hf, const u32x2* areg,
                                         const float* __restrict__ xsum, int xsum_row_stride, float* acc) {
  constexpr int RG = (R + 3) / 4;
  u32x4 ql[4], qh[2];
#pragma unroll
  for (int i = 0; i < 4; i++) ql[i] = *reinterpret_cast<const u32x4*>(bl + 64 * hf + 16 * i);
#pragma unroll
  for (int i = 0; i < 2; i++) qh[i] = *reinterpret_cast<const u32x4*>(bl + 128 + 32 * hf + 16 * i);
  const uint2 scw = *reinterpret_cast<const uint2*>(bl + 192 + 8 * hf);
  float xs[R][8];
#pragma unroll
  for (int r = 0; r < R; r++) {
    const float4 t0 = *reinterpret_cast<const float4*>(xsum + r * xsum_row_stride + 8 * hf);
    const float4 t1 = *reinterpret_cast<const float4*>(xsum + r * xsum_row_stride + 8 * hf + 4);
    xs[r][0] = t0.x; xs[r][1] = t0.y; xs[r][2] = t0.z; xs[r][3] = t0.w;
    xs[r][4] = t1.x; xs[r][5] = t1.y; xs[r][6] = t1.z; xs[r][7] = t1.w;
  }
  const uint32_t magic = opaque_vgpr(0x64006400u);
  const uint32_t mask_lo = opaque_sgpr(0x000f000fu), mask_hi = opaque_sgpr(0x00f000f0u);
  const uint32_t mask_h[4] = {opaque_sgpr(0x00030003u), opaque_sgpr(0x000c000cu), opaque_sgpr(0x00300030u),
                              opaque_sgpr(0x00c000c0u)};
  uint32_t ql8[16], qh8[8];
#pragma unroll
  for (int i = 0; i < 16; i++) ql8[i] = ql[i >> 2][i & 3] >> 8;
#pragma unroll
  for (int i = 0; i < 8; i++) qh8[i] = qh[i >> 2][i & 3] >> 8;
  SFor<4>::run([&](auto tt) {
    constexpr int t = decltype(tt)::value;
    SFor<2>::run([&](auto ss) {
      constexpr int s = decltype(ss)::value;  // scale group 2 t + s: weights l = 16 s .. 16 s + 15
      f32x4 pq[RG], ph[RG];
#pragma unroll
      for (int g = 0; g < RG; g++) pq[g] = ph[g] = f32x4{0, 0, 0, 0};
      SFor<4>::run([&](auto ee) {
        constexpr int e = 4 * s + decltype(ee)::value;  // l = 4 e .. 4 e + 3
        constexpr int wq = 8 * (t & 1) + e;             // ql word: bytes 32 (t & 1) + 4 e ..
        u32x2 bq, bh;
        bq.x = and_or(ql[wq >> 2][wq & 3], t >= 2 ? mask_hi : mask_lo, magic);
        bq.y = and_or(ql8[wq], t >= 2 ? mask_hi : mask_lo, magic);
        bh.x = and_or(qh[e >> 2][e & 3], mask_h[t], magic);
        bh.y = and_or(qh8[e], mask_h[t], magic);
#pragma unroll
        for (int g = 0; g < RG; g++) {
          const f16x4 av = __builtin_bit_cast(f16x4, areg[g * AS + 2 * t + e / 4]);
          pq[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(av, __builtin_bit_cast(f16x4, bq), pq[g], 3, 2 * (e & 3), 0);
          ph[g] = __builtin_amdgcn_mfma_f32_4x4x4f16(av, __builtin_bit_cast(f16x4, bh), ph[g], 3, 2 * (e & 3), 0);
        }
      });
      constexpr int g = 2 * t + s;
      const int sc = __builtin_amdgcn_sbfe((int)(g < 4 ? scw.x : scw.y), 8 * (g & 3), 8);
      const float dsc = dx * (float)sc;
      constexpr float fq = t >= 2 ? 0.0625f : 1.0f;       // 1 / s
      constexpr float fh = 16.0f / (float)(1 << (2 * t));  // 16 / 4^t
      constexpr float fx = 1024.0f * fq + 1024.0f * fh + 32.0f;
      SFor<R>::run([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        const float v = fmaf(fq, pq[r / 4][r % 4], fmaf(fh, ph[r / 4][r % 4], -fx * xs[r][g]));
        acc[r] = fmaf(dsc, v, acc[r]);
      });
    });
  });
}

// ------------------------------------------------------------------ the kernel
// MB = M rounded up to a power of two (1, 2, 4, 8); D = units a wave keeps in LDS (in flight or being read);
// WGS = workgroups per CU the register budget is set for.  Eight rows are two groups of four for the 4-row
// MFMA; their f16 fragments pass through the wave's LDS staging area two rows at a time.
template <int MB>
constexpr int st_xch() { return MB > 4 ? 2 : MB; }  // activation rows staged at a time

// XU = units (superblocks) a wave handles per tile at most: 4 or 8, i.e. K ranges of up to 16 or 32 superblocks
// per workgroup (the A registers of all of them stay resident).
// NW = waves per workgroup (4 or 8): wave w owns superblocks sb_begin + w + NW u of the workgroup's K range.
// GM = 0: dense.  GM = 1: gathered, one tile of one entry per workgroup.  GM = 2: gathered gate / up pair: a
// superblock is two units (the gate rows, then the same rows of the up matrix) with an accumulator each, and the
// tile's result is act(gate) * up.
template <int C, int DT, int MB, int D, int WGS, int XU, int NW, int GM = 0>
__global__ __launch_bounds__(64 * NW, WGS) void stream_gemv_kernel(StArgs a) {
  static_assert(GM == 0 || MB == 1, "gathered entries carry one activation row");
  constexpr int ST_XU = XU, ST_WAVES = NW;
  constexpr int UPS = GM == 2 ? 2 : 1;  // units per superblock
  using G = StGeom<C>;
  using U = StUnit<C>;
  constexpr int R = MB;
  constexpr int RG = (MB + 3) / 4, XCH = st_xch<MB>(), NCH = MB / XCH;
  constexpr int NAP = G::NAP, XSG = G::XSG;
  constexpr int AS = ST_XU * NAP;  // A register pairs per row group
  constexpr int XL = XU / 2;  // 16-byte activation loads per lane and row: XU units x 256 values

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, kg = lane >> 5;
  constexpr bool TAIL = st_tail_codec<C>();
  // units per row; a tail-capable codec's last one may hold fewer than eight blocks
  const int M = a.M, N = a.N, K = a.K, nsb = TAIL ? (K + 255) >> 8 : K >> 8, rpt = a.rpt;
  const uint32_t row_bytes = TAIL ? (uint32_t)(K >> 5) * (G::BPB / 8) : (uint32_t)nsb * G::BPB;
  const int tail_sb = TAIL && (K & 255) ? K >> 8 : -1;             // the unit K ends in
  const int tail_blocks = (K & 255) >> 5;                           // its blocks
  const uint32_t tail_bytes = (uint32_t)tail_blocks * (G::BPB / 8);  // and their bytes
  // gathered: this workgroup's entry and its tile inside the entry's matrix (the tile loop below runs once)
  const int g_entry = GM ? __builtin_amdgcn_readfirstlane((int)blockIdx.x / a.tiles_per_entry) : 0;
  const int g_tile = GM ? (int)blockIdx.x - g_entry * a.tiles_per_entry : 0;
  const uint8_t* wmat = a.w;
  const uint8_t* wmat2 = a.w;
  uint32_t g_expert = 0;
  if constexpr (GM != 0) {
    const uint32_t e = (uint32_t)__builtin_amdgcn_readfirstlane((int)a.rhs[g_entry]);
    if (e >= (uint32_t)a.E) return;  // the whole workgroup, ahead of every barrier
    g_expert = e;
    wmat = a.w + (int64_t)e * a.w_expert_stride;
    if constexpr (GM == 2) wmat2 = a.w2 + (int64_t)e * a.w_expert_stride;
  }
  const int tiles = GM ? g_tile + 1 : a.tiles;
  const int tile0 = GM ? g_tile : (int)blockIdx.x;
  const int G_x = GM ? 1 << 30 : (int)gridDim.x;

  // LDS: per wave [D slots][x fragments MB x 4 x 256 f16][x sums MB x 4 x 2 XSG f32]; then red [2][waves][R][64] f32
  constexpr int XS_BYTES = XCH * ST_XU * 512, XSUM_BYTES = MB * ST_XU * 2 * XSG * 4;
  constexpr int WAVE_BYTES = D * U::SLOT + XS_BYTES + XSUM_BYTES;
  uint8_t* wb = smem + wave * WAVE_BYTES;
  _Float16* xs = reinterpret_cast<_Float16*>(wb + D * U::SLOT);
  float* xsum = reinterpret_cast<float*>(wb + D * U::SLOT + XS_BYTES);
  float* red_all = reinterpret_cast<float*>(smem + ST_WAVES * WAVE_BYTES);
  uint8_t* tbl = smem + ST_WAVES * WAVE_BYTES + UPS * 2 * ST_WAVES * R * 64 * 4;  // decode tables (codebook codecs)
  (void)tbl;
  const uint32_t wb_lds = lds_addr(wb);

  // this workgroup's K range and this wave's units: superblocks sb_begin + wave + 4 u
  const int sb_begin = a.ksplit > 1 ? (int)blockIdx.z * a.sb_per_split : 0;
  int sb_end = a.ksplit > 1 ? sb_begin + a.sb_per_split : nsb;
  sb_end = sb_end < nsb ? sb_end : nsb;
  const int sbn = sb_end - sb_begin;
  const int nu = UPS * (sbn > wave ? (sbn - wave + ST_WAVES - 1) / ST_WAVES : 0);  // wave-uniform, 0..XU

  // ---- activation loads first: they are the oldest loads of the wave
  const uint16_t* x16 = static_cast<const uint16_t*>(a.x);
  if constexpr (GM != 0)
    x16 += a.lhs ? (size_t)__builtin_amdgcn_readfirstlane((int)a.lhs[g_entry]) * (size_t)a.x_row_stride
                 : (size_t)(g_entry / a.x_div) * K;
  // codebook codecs: threads 0 .. 127 fetch 16 bytes each of the 2 KiB grid the tables are built from
  u32x4 greg = {0, 0, 0, 0};
  // replicated iq2_xxs tables: the sixteen lanes of a quarter wave write the sixteen copies of one entry (a wave
  // store covers 1 KiB of consecutive LDS); wave w converts the grid entries 32 i + 4 w + lane / 16, i = 0 .. 7
  constexpr int IQ2_COP = st_iq2_copies<C, MB, NW, GM>();
  u32x2 gq[IQ2_COP > 1 ? 8 : 1];
  if constexpr (C == KQ_IQ2_XXS) {
    if constexpr (IQ2_COP == 1) {
      greg = gload16(a.grids + KQ_GRID_IQ2XXS + 16 * (tid & 127));
    } else {
      SFor<8>::run([&](auto ii) {
        constexpr int i = decltype(ii)::value;
        gq[i] = gload8(a.grids + KQ_GRID_IQ2XXS + 8 * (32 * i + 4 * wave + (lane >> 4)));
      });
    }
  }
  if constexpr (C == KQ_IQ3_S) greg = gload16(a.grids + KQ_GRID_IQ3S + 16 * (tid & 127));  // four entries
  u32x4 xreg[MB * XL];
  SFor<MB * XL>::run([&](auto t) {
    constexpr int T = decltype(t)::value;
    constexpr int m = T / XL, s = T % XL;
    const int gi = lane + 64 * s, uu = gi >> 5, grp = gi & 31;
    int sb = wave + ST_WAVES * uu;
    sb = sb < sbn ? sb : (wave < sbn ? wave : 0);  // spare units re-read a valid superblock
    const int mm = m < M ? m : M - 1;
    int k0 = (sb_begin + sb) * 256 + 8 * grp;
    if constexpr (TAIL) k0 = k0 < K ? k0 : 0;  // past the end of K: any valid address, zeroed once it has landed
    xreg[T] = gload16(x16 + (size_t)mm * K + k0);
  });
  __builtin_amdgcn_sched_barrier(0);  // nothing below is scheduled ahead of these loads

  // ---- weight stream.  Piece i = lane + 64 t of a unit -> (row i / PP, piece i % PP); rows past the end of the
  // tile or of the matrix re-read the last row inside both (their results are dropped).
  uint32_t goff[U::FULL + 1];
  const int row_lim = N - 1;
  auto piece_off = [&](int i, int row0) {
    int r = i / G::PP;
    const int p = i - r * G::PP;
    r = r < rpt ? r : rpt - 1;
    r = row0 + r;
    r = r < row_lim ? r : row_lim;
    return (uint32_t)(r - row0) * row_bytes + st_piece_off<C>(p);  // r >= row0: a tile always starts inside the matrix
  };
  // (offsets are relative to the tile's first row; a tile always starts inside the matrix)
  // Elements of the stream: (tile, unit) in tile-major order.  `it`, `iu`, `islot`: next element to issue.
  int it = tile0, iu = 0, islot = 0, inflight = 0;
  int goff_row0 = -1;
  auto issue_next = [&]() {
    if (it >= tiles) return;
    const int row0 = it * rpt;
    if (row0 + rpt > N && goff_row0 != row0) {  // ragged last tile: rebuild the piece map with clamped rows
      SFor<U::FULL + 1>::run([&](auto t) { constexpr int T = decltype(t)::value; goff[T] = piece_off(lane + 64 * T, row0); });
      goff_row0 = row0;
    }
    const uint8_t* base = ((GM == 2 && (iu & 1)) ? wmat2 : wmat) + (size_t)row0 * row_bytes +
                          (size_t)(sb_begin + wave + ST_WAVES * (iu / UPS)) * G::BPB;
    const uint32_t l0 = (uint32_t)__builtin_amdgcn_readfirstlane((int)(wb_lds + islot * U::SLOT));
    bool tail_unit = false;
    if constexpr (TAIL) tail_unit = sb_begin + wave + ST_WAVES * (iu / UPS) == tail_sb;
    if (tail_unit) {
      SFor<U::FULL + 1>::run([&](auto t) {
        constexpr int T = decltype(t)::value;
        if constexpr (T < U::FULL || U::HALF) {
          const int i = lane + 64 * T;
          const uint32_t po = st_piece_off<C>(i - (i / G::PP) * G::PP);
          // whole piece inside the row: as usual; the piece the row ends in: the row's last 16 bytes; past the end:
          // the unit's first 16 bytes
          const uint32_t off = po + 16 <= tail_bytes ? goff[T] : goff[T] - po + (po < tail_bytes ? tail_bytes - 16 : 0u);
          if (T < U::FULL || lane < 32) dma16(base, off, l0 + T * 1024);
        }
      });
    } else {
      SFor<U::FULL>::run([&](auto t) { constexpr int T = decltype(t)::value; dma16(base, goff[T], l0 + T * 1024); });
      if constexpr (U::HALF) {
        if (lane < 32) dma16(base, goff[U::FULL], l0 + U::FULL * 1024);
      }
    }
    if constexpr (G::SIDE_D) {
      int r = row0 + (lane < rpt ? lane : rpt - 1);
      r = r < row_lim ? r : row_lim;
      if (lane < 32) dma2(base + st_side_d_off<C>(), (uint32_t)(r - row0) * row_bytes, l0 + ST_ROWS * G::LBPB);
    }
    inflight++;
    islot = islot + 1 == D ? 0 : islot + 1;
    if (++iu == nu) {
      iu = 0;
      it += G_x;
    }
  };
  SFor<U::FULL + 1>::run([&](auto t) {
    constexpr int T = decltype(t)::value;
    const int i = lane + 64 * T, r = i / G::PP;
    goff[T] = (uint32_t)(r < rpt ? r : rpt - 1) * row_bytes + st_piece_off<C>(i - r * G::PP);
  });
  if (nu == 0) it = tiles;  // a wave without superblocks (short K range) only joins the barriers

  // every wave of the workgroup has queued its activation loads before any weight load is queued
  __builtin_amdgcn_s_barrier();
  issue_next();
  // wait for the activations alone: the first unit stays in flight
  if (inflight) vmwait<U::UPI>(); else vmwait<0>();
  SFor<MB * XL>::run([&](auto t) { tie_v(xreg[decltype(t)::value]); });
  if constexpr (TAIL) {
    if (tail_sb >= 0) {  // the activations a short last unit has no weights for
      SFor<MB * XL>::run([&](auto t) {
        constexpr int T = decltype(t)::value;
        constexpr int s = T % XL;
        const int gi = lane + 64 * s, uu = gi >> 5, grp = gi & 31;
        const int sb = wave + ST_WAVES * uu;
        if ((sb_begin + sb) * 256 + 8 * grp >= K && sb < sbn) xreg[T] = u32x4{0, 0, 0, 0};
      });
    }
  }
  tie_v(greg);
  if constexpr (IQ2_COP > 1) SFor<8>::run([&](auto ii) { tie_v2(gq[decltype(ii)::value]); });

  // ---- activations -> f16 fragments (+ sums) in the wave's LDS, then this lane's A registers
  float xscale = 1.0f, inv = 1.0f;
  if constexpr (DT == KQ_BF16) {
    // largest magnitude: bf16 magnitudes order like their bit patterns, two per packed integer maximum
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    u16x2 am2 = {0, 0};
    const uint32_t absmask = opaque_sgpr(0x7fff7fffu);
    SFor<MB * XL>::run([&](auto t) {
      const u32x4 v = xreg[decltype(t)::value];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const uint32_t mag = v[e] & absmask;
        am2 = __builtin_elementwise_max(am2, __builtin_bit_cast(u16x2, mag));
      }
    });
    float amax = __builtin_bit_cast(float, (uint32_t)(am2[0] > am2[1] ? am2[0] : am2[1]) << 16);
    amax = wave_max_nonneg(amax);
    if (((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff) == 0xff) {
      // an infinity or a NaN among the activations (their patterns order above every finite one): the largest
      // finite-or-infinite magnitude the floating-point maximum finds, which ignores NaNs
      amax = 0.f;
      SFor<MB * XL>::run([&](auto t) {
        const u32x4 v = xreg[decltype(t)::value];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] << 16)));
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] & 0xffff0000u)));
        }
      });
      amax = wave_max_nonneg(amax);
    }
    // bring the largest magnitude into [2^14, 2^15): exact power-of-two scaling
    const uint32_t eb = (__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff;
    if (eb != 0 && eb != 0xff) {
      int e = (int)eb - 127 - 14;
      if (e < -100) e = -100;
      xscale = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
      inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
    }
  }
  // A registers.  Lane (kg, fa, fi) keeps, for every row group, unit and register pair, the four activations of
  // row 4 g + fi that MFMA block fa needs.
  //   q4_k / q5_k: pair pc, block 2 e + h  -> k = 128 kg + 32 (2 (pc / 2) + h) + 16 (pc % 2) + 4 e
  //   q6_k:        pair 2 t + e / 4, block 2 (e % 4) -> k = 128 hf + 32 t + 4 e  (odd blocks unused)
  //   q2_k / q3_k: pair j, block wi -> k = 128 kg + 32 j + 4 wi
  //   codebook codecs: pair ib, block b -> staged positions 128 kg + 32 ib + 4 b .. + 3
  const int fa = (lane >> 2) & 7, fi = lane & 3;
  u32x2 areg[RG * AS];
  SFor<NCH>::run([&](auto cc) {
    constexpr int c = decltype(cc)::value;  // rows c XCH .. c XCH + XCH - 1 pass through the staging area
    if constexpr (c > 0) wave_lds_fence();  // the previous rows have been read
    SFor<XCH * XL>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      constexpr int ml = T / XL, m = c * XCH + ml, s = T % XL;
      const int gi = lane + 64 * s, uu = gi >> 5, grp = gi & 31;
      const u32x4 v = xreg[m * XL + s];
      _Float16 h[8];
      typedef _Float16 f16x2p __attribute__((ext_vector_type(2)));
      f16x2p hp[4];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        if constexpr (DT == KQ_BF16) {
          // a bf16 number times a power of two is an f16 number unless it falls below the f16 normals, where the
          // truncating pair conversion drops bits under 2^-38 of the largest magnitude
          hp[e] = __builtin_bit_cast(f16x2p, __builtin_amdgcn_cvt_pkrtz(__builtin_bit_cast(float, v[e] << 16) * inv,
                                                                        __builtin_bit_cast(float, v[e] & 0xffff0000u) * inv));
        } else {
          const uint32_t word = v[e];  // (a bit cast of the vector element itself reads element 0 every time)
          hp[e] = __builtin_bit_cast(f16x2p, word);
        }
        h[2 * e] = hp[e][0];
        h[2 * e + 1] = hp[e][1];
      }
      constexpr int XORD = st_xord<C>();
      if constexpr (XORD == 0) {  // k0 k2 k1 k3 inside every group of four
        const f16x8 v8 = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
        *reinterpret_cast<f16x8*>(xs + (ml * ST_XU + uu) * 256 + 8 * grp) = v8;
      } else if constexpr (XORD == 1) {
        const f16x8 v8 = {h[0], h[1], h[2], h[3], h[4], h[5], h[6], h[7]};
        *reinterpret_cast<f16x8*>(xs + (ml * ST_XU + uu) * 256 + 8 * grp) = v8;
      } else {
        // x[j], x[j + 16] interleaved over each 32: lanes a and a + 2 of a quad hold x[8 a ..] and x[16 + 8 a ..]
        // and write one half each of the 16 interleaved values (XORD 3: x[j], x[j + 8] over each 16, lanes a and
        // a + 1)
        typedef _Float16 f16x2v __attribute__((ext_vector_type(2)));
        uint32_t own[4], par[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          own[e] = __builtin_bit_cast(uint32_t, f16x2v{h[2 * e], h[2 * e + 1]});
          if constexpr (XORD == 2)
            par[e] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)own[e], 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
          else
            par[e] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)own[e], 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
        }
        const bool high = (grp & (XORD == 2 ? 2 : 1)) != 0;
        // low lane: own h0..h3 with the partner's h0..h3 behind each; high lane: the partner's h4..h7 ahead of own
        const uint32_t a0 = high ? par[2] : own[0], a1 = high ? par[3] : own[1];  // first of each pair
        const uint32_t b0 = high ? own[2] : par[0], b1 = high ? own[3] : par[1];  // second of each pair
        u32x4 o;
        o[0] = (a0 & 0xffffu) | (b0 << 16);
        o[1] = (a0 >> 16) | (b0 & 0xffff0000u);
        o[2] = (a1 & 0xffffu) | (b1 << 16);
        o[3] = (a1 >> 16) | (b1 & 0xffff0000u);
        if constexpr (XORD == 2)
          *reinterpret_cast<u32x4*>(xs + (ml * ST_XU + uu) * 256 + 32 * (grp >> 2) + 16 * (grp & 1) + (high ? 8 : 0)) = o;
        else
          *reinterpret_cast<u32x4*>(xs + (ml * ST_XU + uu) * 256 + 16 * (grp >> 1) + (high ? 8 : 0)) = o;
      }
      float sum = 0.f;
      {
        const f16x2p ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
        for (int e = 0; e < 4; e++) sum = __builtin_amdgcn_fdot2(hp[e], ones, sum, false);
      }
      sum += dpp_f<0xB1>(sum);  // lanes l ^ 1: 16 values
      if constexpr (XSG == 8) {
        if ((lane & 1) == 0) xsum[(m * ST_XU + uu) * 16 + (grp >> 1)] = sum;
      } else {
        sum += dpp_f<0x4E>(sum);  // lanes l ^ 2: 32 values
        if ((lane & 3) == 0) xsum[(m * ST_XU + uu) * 8 + (grp >> 2)] = sum;
      }
    });
    wave_lds_fence();
    constexpr int g = c * XCH / 4;  // the row group these rows belong to
    // staged row of this lane: MB <= 4 keeps all rows staged (spare lanes alias row fi % MB); MB = 8 stages
    // rows 2 c, 2 c + 1 = rows 2 (c % 2), 2 (c % 2) + 1 of group c / 2
    const bool mine = MB <= 4 || (fi >> 1) == (c & 1);
    const int lrow = MB <= 4 ? (fi & (MB - 1)) : (fi & 1);
    if (mine) {
      const uint8_t* xb = reinterpret_cast<const uint8_t*>(xs) + lrow * (ST_XU * 512) + 256 * kg;
      SFor<AS>::run([&](auto t) {
        constexpr int T = decltype(t)::value;
        constexpr int u = T / NAP, pr = T % NAP;
        int koff;  // in f16 elements inside the half
        if constexpr (C == KQ_Q6_K)
          koff = 32 * (pr >> 1) + 16 * (pr & 1) + 4 * (fa >> 1);
        else if constexpr (C == KQ_Q2_K || C == KQ_Q3_K || C == KQ_Q8_0 || st_tbl_bytes<C>() != 0)
          koff = 32 * pr + 4 * fa;
        else
          koff = 64 * (pr >> 1) + 32 * (fa & 1) + 16 * (pr & 1) + 4 * (fa >> 1);
        areg[g * AS + T] = *reinterpret_cast<const u32x2*>(xb + u * 512 + koff * 2);
      });
    }
  });

  // ---- decode tables of the codebook codecs (their grid bytes arrived with the activations)
  if constexpr (st_pair_table<C>()) {
    // entry b = dwords 32 b .. 32 b + 31 (one copy per LDS bank).  Eight lanes write the 128 bytes of an entry, so
    // a wave store covers 1 KiB of consecutive LDS (entry-per-lane stores, 128 bytes apart, all meet in two banks)
    typedef _Float16 f16x2v __attribute__((ext_vector_type(2)));
    constexpr int PER_WAVE = 256 / 8 / ST_WAVES;  // store instructions per wave: 8 entries each
#pragma unroll
    for (int i = 0; i < PER_WAVE; i++) {
      const int b = 8 * (PER_WAVE * wave + i) + (lane >> 3);
      auto val = [](int i) -> float {
        if constexpr (C == KQ_MXFP4 || C == KQ_NVFP4) return kq::kv_mxfp4(i);
        else if constexpr (C == KQ_Q4_0) return (float)(i - 8);
        else return kq::kv_iq4nl(i);
      };
      const f16x2v e = {(_Float16)val(b & 15), (_Float16)val(b >> 4)};
      const uint32_t ev = __builtin_bit_cast(uint32_t, e);
      *reinterpret_cast<u32x4*>(tbl + 128 * b + 16 * (lane & 7)) = u32x4{ev, ev, ev, ev};
    }
  }
  if constexpr (C == KQ_IQ2_XXS && st_iq2_copies<C, MB, NW, GM>() > 1) {
    constexpr int COP = st_iq2_copies<C, MB, NW, GM>();
    static_assert(COP == 1 || (COP == 16 && NW == 8), "eight waves write 16 copies");
    typedef _Float16 f16x2v __attribute__((ext_vector_type(2)));
    uint8_t* dst = tbl + 256 * (4 * wave + (lane >> 4)) + 16 * (lane & 15);
    SFor<8>::run([&](auto ii) {  // grid entries: eight bytes -> eight f16
      constexpr int i = decltype(ii)::value;
      u32x4 o;
#pragma unroll
      for (int k = 0; k < 8; k += 2) {
        const uint32_t gw = gq[i][k >> 2];
        const f16x2v e = {(_Float16)(float)((gw >> (8 * (k & 3))) & 0xff), (_Float16)(float)((gw >> (8 * ((k + 1) & 3))) & 0xff)};
        o[k >> 1] = __builtin_bit_cast(uint32_t, e);
      }
      *reinterpret_cast<u32x4*>(dst + 256 * 32 * i) = o;
    });
    SFor<4>::run([&](auto ii) {  // sign indices 32 i + 4 w + lane / 16 -> eight f16 sign masks
      constexpr int i = decltype(ii)::value;
      const uint32_t sb = kq::ksigns((uint32_t)(32 * i + 4 * wave + (lane >> 4)));
      u32x4 o;
#pragma unroll
      for (int w = 0; w < 4; w++) o[w] = (((sb >> (2 * w)) & 1) << 15) | (((sb >> (2 * w + 1)) & 1) << 31);
      *reinterpret_cast<u32x4*>(dst + 4096 * COP + 256 * 32 * i) = o;
    });
  } else if constexpr (C == KQ_IQ2_XXS) {
    if (tid < 128) {  // 16 grid bytes -> 16 f16 magnitudes
      u32x4 o[2];
#pragma unroll
      for (int k = 0; k < 16; k += 2) {
        typedef _Float16 f16x2v __attribute__((ext_vector_type(2)));
        const f16x2v e = {(_Float16)(float)((greg[k >> 2] >> (8 * (k & 3))) & 0xff),
                          (_Float16)(float)((greg[(k + 1) >> 2] >> (8 * ((k + 1) & 3))) & 0xff)};
        o[k >> 3][(k >> 1) & 3] = __builtin_bit_cast(uint32_t, e);
      }
      *reinterpret_cast<u32x4*>(tbl + 32 * tid) = o[0];
      *reinterpret_cast<u32x4*>(tbl + 32 * tid + 16) = o[1];
    }
    if (tid < 128) {  // sign table: 7-bit index -> eight f16 sign masks
      const uint32_t sb = kq::ksigns((uint32_t)tid);
      u32x4 o;
#pragma unroll
      for (int w = 0; w < 4; w++) o[w] = (((sb >> (2 * w)) & 1) << 15) | (((sb >> (2 * w + 1)) & 1) << 31);
      *reinterpret_cast<u32x4*>(tbl + 4096 + 16 * tid) = o;
    }
  }
  if constexpr (C == KQ_IQ3_S) {
    constexpr bool MERGED = st_iq3s_merged<C, MB, NW, GM>();
    uint8_t* plain = MERGED ? tbl + 65536 : tbl;
    if (tid < 128) {  // four grid entries of four bytes -> four times four f16 magnitudes
      typedef _Float16 f16x2v __attribute__((ext_vector_type(2)));
      u32x4 o[2];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const uint32_t gw = greg[e];
        const f16x2v e0 = {(_Float16)(float)(gw & 0xff), (_Float16)(float)((gw >> 8) & 0xff)};
        const f16x2v e1 = {(_Float16)(float)((gw >> 16) & 0xff), (_Float16)(float)(gw >> 24)};
        o[e >> 1][2 * (e & 1)] = __builtin_bit_cast(uint32_t, e0);
        o[e >> 1][2 * (e & 1) + 1] = __builtin_bit_cast(uint32_t, e1);
      }
      *reinterpret_cast<u32x4*>(plain + 32 * tid) = o[0];
      *reinterpret_cast<u32x4*>(plain + 32 * tid + 16) = o[1];
    }
    if constexpr (MERGED) {
      static_assert(!MERGED || 64 * NW == 512, "one thread per grid entry");
      wg_lds_barrier();
      const u32x2 e = *reinterpret_cast<const u32x2*>(plain + 8 * tid);
      SFor<16>::run([&](auto nn) {
        constexpr uint32_t nib = decltype(nn)::value;
        constexpr uint32_t m0 = ((nib & 1) << 15) | ((nib & 2) << 30), m1 = ((nib & 4) << 13) | ((nib & 8) << 28);
        *reinterpret_cast<u32x2*>(tbl + 8 * (tid | (nib << 9))) = u32x2{e[0] ^ m0, e[1] ^ m1};
      });
    } else if (tid < 256) {  // sign byte -> eight f16 sign masks
      u32x4 o;
#pragma unroll
      for (int w = 0; w < 4; w++) o[w] = ((((uint32_t)tid >> (2 * w)) & 1) << 15) | ((((uint32_t)tid >> (2 * w + 1)) & 1) << 31);
      *reinterpret_cast<u32x4*>(tbl + 4096 + 16 * tid) = o;
    }
  }
  if constexpr (st_tbl_bytes<C>() != 0) wg_lds_barrier();

  // The other D - 1 units are queued only now: a wave that queues loads faster than the memory system takes them
  // stalls in the issue, and the activation work above would have waited behind that stall.
  SFor<D - 1>::run([&](auto) { issue_next(); });
  float acc_a[R], acc_b[GM == 2 ? R : 1];
  int ct = tile0, cslot = 0;  // tile / slot being consumed
  int parity = 0;
  for (; ct < tiles; ct += G_x) {
#pragma unroll
    for (int r = 0; r < R; r++) acc_a[r] = 0.f;
    acc_b[0] = 0.f;
    const int row0 = ct * rpt;
    const int nrows = N - row0 < rpt ? N - row0 : rpt;
    const int crow = n < nrows ? n : nrows - 1;
    SFor<ST_XU>::run([&](auto uu) {
      constexpr int u = decltype(uu)::value;
      if (u < nu) {
        // loads issued after this unit's: inflight - 1 units
        const int younger = inflight - 1;
        if (younger >= 3) vmwait<3 * U::UPI>();
        else if (younger == 2) vmwait<2 * U::UPI>();
        else if (younger == 1) vmwait<1 * U::UPI>();
        else vmwait<0>();
        const uint8_t* slot = wb + cslot * U::SLOT;
        const uint8_t* bl = slot + crow * G::LBPB;
        constexpr int us = u / UPS;  // the wave's superblock this unit belongs to
        float* acc = (GM == 2 && (u & 1)) ? acc_b : acc_a;
        const int nvalid = sb_begin + wave + ST_WAVES * us == tail_sb ? tail_blocks : 8;
        (void)nvalid;
        if constexpr (TAIL) {
          if (nvalid != 8) {
            // the piece the row ends in arrived as the row's last 16 bytes: move them down by the 16 ps + 16 - T bytes
            // they sit too high (lane n < 32 does LDS row n of the slot, every row once)
            const uint32_t ps = tail_bytes >> 4, sh = 16 * ps + 16 - tail_bytes;  // sh = 1 .. 15
            if (lane < 32) {
              uint8_t* pr = wb + cslot * U::SLOT + lane * G::LBPB + 16 * ps;
              const u32x4 v = *reinterpret_cast<const u32x4*>(pr);
              uint32_t e0 = v[0], e1 = v[1], e2 = v[2], e3 = v[3];
              const uint32_t dq = sh >> 2;  // whole dwords (wave-uniform)
              if (dq == 1) { e0 = e1; e1 = e2; e2 = e3; e3 = 0; }
              else if (dq == 2) { e0 = e2; e1 = e3; e2 = 0; e3 = 0; }
              else if (dq == 3) { e0 = e3; e1 = 0; e2 = 0; e3 = 0; }
              const uint32_t db = sh & 3;   // then bytes
              u32x4 o;
              o[0] = __builtin_amdgcn_alignbyte(e1, e0, db);
              o[1] = __builtin_amdgcn_alignbyte(e2, e1, db);
              o[2] = __builtin_amdgcn_alignbyte(e3, e2, db);
              o[3] = __builtin_amdgcn_alignbyte(0u, e3, db);
              *reinterpret_cast<u32x4*>(pr) = o;
            }
            wave_lds_fence();
          }
        }
        if constexpr (C == KQ_Q6_K) {
          const float dx = kq::h2f((uint16_t)*reinterpret_cast<const uint32_t*>(slot + ST_ROWS * G::LBPB + 4 * crow)) * xscale;
          q6k_unit<R, AS>(bl, dx, kg, areg + us * NAP, xsum + us * 16, ST_XU * 16, acc);
        } else if constexpr (C == KQ_Q2_K || C == KQ_Q3_K) {
          q23k_unit<C, R, AS>(bl, kg, xscale, areg + us * NAP, xsum + us * 16, ST_XU * 16, acc);
        } else if constexpr (C == KQ_Q8_0) {
          q80_unit<R, AS>(bl, kg, xscale, areg + us * NAP, acc, nvalid);
        } else if constexpr (C == KQ_IQ4_XS) {
          iq4xs_unit<R, AS>(bl, kg, xscale, areg + us * NAP, tbl + 4 * (lane & 31), acc);
        } else if constexpr (C == KQ_IQ4_NL || C == KQ_Q4_0 || C == KQ_MXFP4 || C == KQ_NVFP4) {
          nib32_unit<C, R, AS>(bl, kg, xscale, areg + us * NAP, tbl + 4 * (lane & 31), acc, nvalid);
        } else if constexpr (C == KQ_IQ2_XXS) {
          constexpr int COP = st_iq2_copies<C, MB, NW, GM>();
          iq2xxs_unit<R, AS, COP>(bl, kg, xscale, areg + us * NAP, COP > 1 ? tbl + 16 * (lane & 15) : tbl, acc);
        } else if constexpr (C == KQ_IQ3_S) {
          const float dx = kq::h2f((uint16_t)*reinterpret_cast<const uint32_t*>(slot + ST_ROWS * G::LBPB + 4 * crow)) * xscale;
          iq3s_unit<R, AS, st_iq3s_merged<C, MB, NW, GM>()>(bl, kg, dx, areg + us * NAP, tbl, acc);
        } else {
          q45k_unit<C, R, AS>(bl, kg, xscale, areg + us * NAP, xsum + us * 8, ST_XU * 8, acc);
        }
        // the slot has been read: refill it with the next element of the stream
        lgkm_drain();
        inflight--;
        cslot = cslot + 1 == D ? 0 : cslot + 1;
        issue_next();
      }
    });

    // ---- cross-wave + cross-half reduction of the tile
    float* red = red_all + (parity * ST_WAVES + wave) * (UPS * R * 64);
#pragma unroll
    for (int r = 0; r < R; r++) red[r * 64 + lane] = acc_a[r];
    if constexpr (GM == 2) red[R * 64 + lane] = acc_b[0];
    wg_lds_barrier();
    if (tid < R * 32) {
      const int r = tid >> 5, nn = tid & 31;
      float v = 0.f, vu = 0.f;
#pragma unroll
      for (int wv = 0; wv < ST_WAVES; wv++) {
        const float* rw = red_all + (parity * ST_WAVES + wv) * (UPS * R * 64);
        v += rw[r * 64 + nn] + rw[r * 64 + nn + 32];
        if constexpr (GM == 2) vu += rw[R * 64 + nn] + rw[R * 64 + nn + 32];
      }
      if constexpr (GM != 0) {
        if (nn < nrows) {
          if (a.bias) v += a.bias[(size_t)g_expert * N + row0 + nn];
          if constexpr (GM == 2) {
            if (a.bias2) vu += a.bias2[(size_t)g_expert * N + row0 + nn];
            v = kq::glu_epilogue(a.act, v, vu, a.limit, a.alpha);
          }
          kq::store_result<DT>(a.y, a.om, (size_t)kq::out_row(a.om, g_entry) * N + row0 + nn, v);
        }
      } else if (r < M && nn < nrows) {
        if (a.ksplit > 1) {
          a.partial[(size_t)blockIdx.z * M * N + (size_t)r * N + row0 + nn] = v;
        } else {
          if (a.bias16) v += DT == KQ_F16 ? kq::h2f(a.bias16[row0 + nn]) : kq::bf162f(a.bias16[row0 + nn]);
          uint16_t* yo = static_cast<uint16_t*>(a.y) + (size_t)r * N + row0 + nn;
          *yo = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
        }
      }
    }
    parity ^= 1;
  }
}

// K the kernel takes: whole 256-weight units, or, for the codecs of 32-weight blocks copied as they lie, a last unit
// of one to seven whole blocks behind at least one whole unit.
bool st_tail_ok(int codec) { return codec == KQ_MXFP4 || codec == KQ_Q4_0 || codec == KQ_IQ4_NL || codec == KQ_Q8_0; }
bool st_k_ok(int K, int codec) { return K >= 256 && ((K & 255) == 0 || (st_tail_ok(codec) && (K & 31) == 0)); }
int st_k_units(int K) { return (K + 255) >> 8; }

template <int C, int MB, int D, int ST_XU, int ST_WAVES, int GM = 0>
constexpr size_t st_lds_bytes() {
  return (size_t)ST_WAVES * (D * StUnit<C>::SLOT + st_xch<MB>() * ST_XU * 512 + MB * ST_XU * 2 * StGeom<C>::XSG * 4) +
         (GM == 2 ? 2 : 1) * 2 * ST_WAVES * MB * 64 * 4 + st_tbl_bytes<C, MB, ST_WAVES, GM>();
}

template <int DT>
__global__ __launch_bounds__(256) void st_splitk_reduce_kernel(const float* __restrict__ partial, uint16_t* __restrict__ y,
                                                               int count, int ksplit) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  float v = 0.f;
  for (int sp = 0; sp < ksplit; sp++) v += partial[(size_t)sp * count + i];
  y[i] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
}

int st_num_cus() {
  // compute units of the current device, looked up once per device
  static std::atomic<int> cus[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// K split: a workgroup takes at most 16 superblocks (32 where the kernel with eight units per wave applies: codecs
// with four A register pairs per unit, up to four rows); with fewer row tiles than g_st_fill_pct per 100 CUs the
// range is cut further so that about two workgroups per CU exist.
struct StSplit {
  int ksplit, sb_per_split;
  int rpt;  // rows per tile the plan asks for (0: 32, levelled by the launcher)
};
constexpr int g_st_fill_pct = 150;  // row tiles x splits per 100 CUs below which K is split further
constexpr int g_st_min_rpt = 24;    // fewest rows a levelled tile may have (16 measured slower than 32)
constexpr bool g_st_nw8 = true;
#ifndef KQ_ST_SHORT_TILES
#define KQ_ST_SHORT_TILES 1
#endif
constexpr bool g_st_short_tiles = KQ_ST_SHORT_TILES != 0;
int st_max_sb(int codec, int M);
// superblocks a workgroup can take: 32 with the eight-wave kernel where its LDS fits (every codec for up to two
// rows, the codecs with small units for up to four)
template <int C>
constexpr int st_nw8_rows() {
  return st_lds_bytes<C, 4, 2, 4, 8>() <= 160 * 1024 ? 4 : st_lds_bytes<C, 2, 2, 4, 8>() <= 160 * 1024 ? 2 :
         st_lds_bytes<C, 1, 2, 4, 8>() <= 160 * 1024 ? 1 : 0;
}
int st_max_sb(int codec, int M) {
  if (!g_st_nw8) return 16;
  int rows = 0;
  switch (codec) {
    case KQ_Q2_K: rows = st_nw8_rows<KQ_Q2_K>(); break;
    case KQ_Q3_K: rows = st_nw8_rows<KQ_Q3_K>(); break;
    case KQ_Q4_K: rows = st_nw8_rows<KQ_Q4_K>(); break;
    case KQ_Q5_K: rows = st_nw8_rows<KQ_Q5_K>(); break;
    case KQ_Q6_K: rows = st_nw8_rows<KQ_Q6_K>(); break;
    case KQ_IQ4_XS: rows = st_nw8_rows<KQ_IQ4_XS>(); break;
    case KQ_IQ2_XXS: rows = st_nw8_rows<KQ_IQ2_XXS>(); break;
    case KQ_IQ3_S: rows = st_nw8_rows<KQ_IQ3_S>(); break;
    case KQ_Q8_0: rows = st_nw8_rows<KQ_Q8_0>(); break;
    case KQ_IQ4_NL: rows = st_nw8_rows<KQ_IQ4_NL>(); break;
    case KQ_Q4_0: rows = st_nw8_rows<KQ_Q4_0>(); break;
    case KQ_MXFP4: rows = st_nw8_rows<KQ_MXFP4>(); break;
    case KQ_NVFP4: rows = st_nw8_rows<KQ_NVFP4>(); break;
  }
  return M <= rows ? 32 : 16;
}
StSplit st_split_plan(int M, int N, int K, int codec, int cus) {
  const int nsb = K >> 8, tiles = (N + ST_ROWS - 1) / ST_ROWS, maxsb = st_max_sb(codec, M);
  int want = (nsb + maxsb - 1) / maxsb;
  // one or two rows: a single workgroup per CU over the whole K range beats a split with its reduction launch
  const int fill = M <= 2 && g_st_fill_pct == 150 ? 100 : g_st_fill_pct;
  if (tiles * want * 100 < cus * fill) {
    int more = (2 * cus + tiles - 1) / tiles;
    if (more > nsb / 4) more = nsb / 4;  // at least one superblock per wave
    if (more > want) want = more;
  }
  if (want < 1) want = 1;
  // one or two rows, fewer 32-row tiles than CUs and a K range one eight-wave workgroup can take: shorter tiles
  // (one per CU) instead of a K split, which would add the reduction launch (4096 x 4096: 7.0 -> 5.6 us)
  if (g_st_short_tiles && want > 1 && M <= 4 && maxsb >= 32 && nsb >= 8 && nsb <= 32 && tiles < cus) {
    int r = (N + cus - 1) / cus;
    if (r < 8) r = 8;
    if (r < ST_ROWS) return StSplit{1, nsb > 16 ? nsb : 17, r};  // sb_per_split > 16 selects the eight-wave kernel
  }
  int per = (nsb + want - 1) / want;
  if (per > maxsb) per = maxsb;
  StSplit p{(nsb + per - 1) / per, per, 0};
  return p;
}

template <int C, int DT, int MB, int D, int XU, int NW = 4>
int st_launch_one(StArgs a, int splits, hipStream_t s) {
  constexpr size_t lds = st_lds_bytes<C, MB, D, XU, NW>();
  static_assert(lds <= 160 * 1024, "workgroup does not fit the LDS of a CU");
  constexpr int WGS = lds <= 80 * 1024 && NW == 4 ? 2 : 1;
  auto kern = stream_gemv_kernel<C, DT, MB, D, WGS, XU, NW>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  int gx = WGS * st_num_cus() / splits;
  if (gx < 1) gx = 1;
  // rows per tile: when the 32-row tiles do not fill a whole number of rounds of the resident workgroups, the
  // busiest CU decides the time (448 tiles on 512 slots: two tiles on 192 CUs, one on 64).  Spreading the rows
  // over rounds x slots equal tiles of 24 ... 32 rows levels that; the rows a short tile leaves out cost idle lanes,
  // not bandwidth.
  if (a.rpt > 0) {  // the plan's short tiles
    a.tiles = (a.N + a.rpt - 1) / a.rpt;
  } else {
    const int tiles32 = (a.N + ST_ROWS - 1) / ST_ROWS;
    const int rounds = (tiles32 + gx - 1) / gx;
    const int rpt = (a.N + rounds * gx - 1) / (rounds * gx);
    a.rpt = rpt >= g_st_min_rpt && rpt < ST_ROWS ? rpt : ST_ROWS;
    a.tiles = (a.N + a.rpt - 1) / a.rpt;
  }
  if (gx > a.tiles) gx = a.tiles;
  hipLaunchKernelGGL(kern, dim3(gx, 1, splits), dim3(64 * NW), lds, s, a);
  KQ_HIP_CHECK(hipGetLastError());
  if (splits > 1) {
    const int count = a.M * a.N;
    hipLaunchKernelGGL((st_splitk_reduce_kernel<DT>), dim3((count + 255) / 256), dim3(256), 0, s, a.partial,
                       static_cast<uint16_t*>(a.y), count, splits);
    KQ_HIP_CHECK(hipGetLastError());
  }
  return KQ_OK;
}

template <int C, int DT>
int st_launch_m(const StArgs& a, int splits, hipStream_t s) {
  constexpr int D = 2;  // units in LDS per wave; 3 and 4 measured slower for every codec
  if (a.sb_per_split > 16) {
    // K ranges of 17 .. 32 superblocks: eight waves of four units (st_max_sb allows this for up to four rows).
    // Four waves of eight units, the alternative without more waves, took 9.0 instead of 7.1 us on q2_k 8192^2.
    if constexpr (st_nw8_rows<C>() >= 1)
      if (a.M == 1) return st_launch_one<C, DT, 1, D, 4, 8>(a, splits, s);
    if constexpr (st_nw8_rows<C>() >= 2)
      if (a.M == 2) return st_launch_one<C, DT, 2, D, 4, 8>(a, splits, s);
    if constexpr (st_nw8_rows<C>() >= 4) return st_launch_one<C, DT, 4, D, 4, 8>(a, splits, s);
  }
  if (a.M == 1) return st_launch_one<C, DT, 1, D, 4>(a, splits, s);
  if (a.M == 2) return st_launch_one<C, DT, 2, D, 4>(a, splits, s);
  if (a.M <= 4) return st_launch_one<C, DT, 4, D, 4>(a, splits, s);
  return st_launch_one<C, DT, 8, D, 4>(a, splits, s);
}

// Gathered calls: one workgroup per (entry, 32-row tile); NW waves share the entry's K range, XU = 4 units per
// wave, i.e. at most 4 NW superblocks (2 NW for the gate / up pair, whose superblocks are two units).
template <int C, int DT, int NW, int GM>
int st_launch_gather(StArgs a, int entries, hipStream_t s) {
  constexpr int D = 2, XU = 4;
  constexpr size_t lds = st_lds_bytes<C, 1, D, XU, NW, GM>();
  static_assert(lds <= 160 * 1024, "workgroup does not fit the LDS of a CU");
  constexpr int WGS = lds <= 80 * 1024 && NW == 4 ? 2 : 1;
  auto kern = stream_gemv_kernel<C, DT, 1, D, WGS, XU, NW, GM>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  a.rpt = ST_ROWS;
  a.tiles_per_entry = (a.N + ST_ROWS - 1) / ST_ROWS;
  a.tiles = a.tiles_per_entry;
  hipLaunchKernelGGL(kern, dim3((unsigned)(entries * a.tiles_per_entry)), dim3(64 * NW), lds, s, a);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

template <int C, int DT>
int st_launch_gather_nw(const StArgs& a, int entries, bool glu, hipStream_t s) {
  const int nsb = st_k_units(a.K);
  // gate / up pair: two units per superblock; beyond four superblocks eight waves keep a wave at two to four units
  // (a codec whose eight-wave workgroup does not fit the LDS stays on four waves as far as their units reach)
  if (glu) {
    if (nsb <= 4) return st_launch_gather<C, DT, 4, 2>(a, entries, s);
    if constexpr (st_lds_bytes<C, 1, 2, 4, 8, 2>() <= 160 * 1024) return st_launch_gather<C, DT, 8, 2>(a, entries, s);
    if (nsb <= 8) return st_launch_gather<C, DT, 4, 2>(a, entries, s);
    return KQ_ERR_UNSUPPORTED;
  }
  if (nsb <= 16) return st_launch_gather<C, DT, 4, 1>(a, entries, s);
  if constexpr (st_lds_bytes<C, 1, 2, 4, 8, 1>() <= 160 * 1024) return st_launch_gather<C, DT, 8, 1>(a, entries, s);
  return KQ_ERR_UNSUPPORTED;
}

bool st_codec_ok(int codec) {
  return codec == KQ_Q4_K || codec == KQ_Q5_K || codec == KQ_Q6_K || codec == KQ_Q2_K || codec == KQ_Q3_K ||
         codec == KQ_IQ4_XS || codec == KQ_IQ2_XXS || codec == KQ_IQ3_S || codec == KQ_Q8_0 || codec == KQ_IQ4_NL ||
         codec == KQ_Q4_0 || codec == KQ_MXFP4 || codec == KQ_NVFP4;
}

}  // namespace

// The dense and the gathered launchers can be compiled into separate objects (KQ_STREAM_PART = 1 dense, 2 gathered).
#if !defined(KQ_STREAM_PART) || KQ_STREAM_PART == 1
bool kq_stream_supported(int M, int N, int K, int codec, const void* x, const void* w) {
  if (!st_codec_ok(codec) || M < 1 || M > 8 || N < 1 || !st_k_ok(K, codec)) return false;
  if ((int64_t)N * st_k_units(K) * 272 >= (int64_t)1 << 40) return false;
  // q4_k / q5_k pieces are fetched 16-byte aligned; iq4_xs blocks are 8-byte multiples, q2_k blocks 4-byte ones, the
  // others 2-byte ones
  const uintptr_t wmask = codec == KQ_Q4_K || codec == KQ_Q5_K ? 15 : codec == KQ_IQ4_XS ? 7 : codec == KQ_Q2_K ? 3 : codec == KQ_MXFP4 ? 0 : 1;
  if (reinterpret_cast<uintptr_t>(w) & wmask) return false;
  return (reinterpret_cast<uintptr_t>(x) & 15) == 0;
}

size_t kq_stream_workspace_bytes(int M, int N, int K, int codec) {
  if (!st_codec_ok(codec) || M < 1 || M > 8 || !st_k_ok(K, codec)) return 0;
  const StSplit p = st_split_plan(M, N, 256 * st_k_units(K), codec, st_num_cus());
  return p.ksplit > 1 ? (size_t)p.ksplit * M * N * sizeof(float) : 0;
}

int kq_launch_qmm_stream(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                         size_t ws_bytes, hipStream_t s, const void* bias) {
  if (!kq_stream_supported(M, N, K, codec, x, w)) return KQ_ERR_UNSUPPORTED;
  const StSplit p = st_split_plan(M, N, 256 * st_k_units(K), codec, st_num_cus());
  if (bias && p.ksplit > 1) return KQ_ERR_UNSUPPORTED;  // the bias joins the sum in the unsplit epilogue only
  // three or more rows of a table-decoded 4-bit codec whose K range has to be cut (few row tiles): the code-level
  // kernel needs no reduction launch and is ahead (mxfp4 3072 -> 2880: 4 rows 7.8 us against 10.4 here, 8 rows 9.1
  // against 11.3; 2880 -> 5760: 4 rows 8.5 against 12.0; q4_0 4128 -> 11008: 15.9 against 17.4)
  if (p.ksplit > 1 && M >= 3 && !bias && (codec == KQ_MXFP4 || codec == KQ_Q4_0 || codec == KQ_IQ4_NL))
    return KQ_ERR_UNSUPPORTED;
  if (p.ksplit > 1 && (!ws || ws_bytes < (size_t)p.ksplit * M * N * sizeof(float) || (reinterpret_cast<uintptr_t>(ws) & 3)))
    return KQ_ERR_UNSUPPORTED;  // the caller falls through to the kernels that can run unsplit
  StArgs a{};
  a.x = x;
  a.w = w;
  a.y = y;
  a.M = M;
  a.N = N;
  a.K = K;
  a.tiles = (N + ST_ROWS - 1) / ST_ROWS;
  a.partial = static_cast<float*>(ws);
  a.bias16 = static_cast<const uint16_t*>(bias);
  a.ksplit = p.ksplit;
  a.sb_per_split = p.sb_per_split;
  a.rpt = p.rpt;
  if (codec == KQ_Q4_K)
    return dtype == KQ_F16 ? st_launch_m<KQ_Q4_K, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_Q4_K, KQ_BF16>(a, p.ksplit, s);
  if (codec == KQ_Q5_K)
    return dtype == KQ_F16 ? st_launch_m<KQ_Q5_K, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_Q5_K, KQ_BF16>(a, p.ksplit, s);
  if (codec == KQ_IQ4_XS || codec == KQ_IQ2_XXS || codec == KQ_IQ3_S) {
    a.grids = kq_device_grids();
    if (!a.grids) return KQ_ERR_HIP;
    if (codec == KQ_IQ3_S)
      return dtype == KQ_F16 ? st_launch_m<KQ_IQ3_S, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_IQ3_S, KQ_BF16>(a, p.ksplit, s);
    if (codec == KQ_IQ4_XS)
      return dtype == KQ_F16 ? st_launch_m<KQ_IQ4_XS, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_IQ4_XS, KQ_BF16>(a, p.ksplit, s);
    return dtype == KQ_F16 ? st_launch_m<KQ_IQ2_XXS, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_IQ2_XXS, KQ_BF16>(a, p.ksplit, s);
  }
  if (codec == KQ_Q8_0)
    return dtype == KQ_F16 ? st_launch_m<KQ_Q8_0, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_Q8_0, KQ_BF16>(a, p.ksplit, s);
  if (codec == KQ_IQ4_NL)
    return dtype == KQ_F16 ? st_launch_m<KQ_IQ4_NL, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_IQ4_NL, KQ_BF16>(a, p.ksplit, s);
  if (codec == KQ_Q4_0)
    return dtype == KQ_F16 ? st_launch_m<KQ_Q4_0, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_Q4_0, KQ_BF16>(a, p.ksplit, s);
  if (codec == KQ_MXFP4)
    return dtype == KQ_F16 ? st_launch_m<KQ_MXFP4, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_MXFP4, KQ_BF16>(a, p.ksplit, s);
  if (codec == KQ_NVFP4)
    return dtype == KQ_F16 ? st_launch_m<KQ_NVFP4, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_NVFP4, KQ_BF16>(a, p.ksplit, s);
  if (codec == KQ_Q2_K)
    return dtype == KQ_F16 ? st_launch_m<KQ_Q2_K, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_Q2_K, KQ_BF16>(a, p.ksplit, s);
  if (codec == KQ_Q3_K)
    return dtype == KQ_F16 ? st_launch_m<KQ_Q3_K, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_Q3_K, KQ_BF16>(a, p.ksplit, s);
  return dtype == KQ_F16 ? st_launch_m<KQ_Q6_K, KQ_F16>(a, p.ksplit, s) : st_launch_m<KQ_Q6_K, KQ_BF16>(a, p.ksplit, s);
}

#endif  // dense part

#if !defined(KQ_STREAM_PART) || KQ_STREAM_PART == 2
// Gathered matvec of MoE decode on the streamed kernel: entry p (0 .. entries - 1) multiplies row p / x_div of x
// [.., K] by the [N, K] matrix of expert rhs[p] (w; with w2 the fused gate / up form act(x . gate) * (x . up)) into
// output row out_row(om, p).  Every codec of the streamed kernel, K of at most 32 superblocks (16 for the fused form).
#ifndef KQ_GATHER_STREAM_MAX_ENTRIES
#define KQ_GATHER_STREAM_MAX_ENTRIES 256
#endif
int kq_gather_stream_max_entries() { return KQ_GATHER_STREAM_MAX_ENTRIES; }

// Whether the streamed gathered kernel takes a call of this shape and alignment (the launcher's own test, also asked
// by the router that chooses between the per-entry and the expert-grouped kernels before either runs).
bool kq_gather_stream_takes(const void* x, const void* w, const void* w2, int entries, int N, int K, bool strided_x,
                            int64_t x_row_stride, int64_t w_expert_stride, bool second_bias_without_glu, int codec) {
  if (!st_codec_ok(codec)) return false;
  if (entries < 1 || entries > KQ_GATHER_STREAM_MAX_ENTRIES || N < 1 || !st_k_ok(K, codec)) return false;
  const bool glu = w2 != nullptr;
  if (st_k_units(K) > (glu ? 16 : 32) || second_bias_without_glu) return false;
  // the fused gate / up form on stacks whose K ends inside a unit stays on the code-level kernels, which are ahead
  // there (32 experts of 2880 x 2880 in mxfp4: 4 pairs 16.4 us against 18.3 here, whose 360 eight-wave workgroups
  // take two rounds of one per CU; 8 pairs 24.6 on the block-scaled kernel against 26.7)
  if (glu && (K & 255)) return false;
  if ((int64_t)entries * ((N + ST_ROWS - 1) / ST_ROWS) > 65535 * 16) return false;
  const uintptr_t wmask = codec == KQ_Q4_K || codec == KQ_Q5_K ? 15 : codec == KQ_IQ4_XS ? 7 : codec == KQ_Q2_K ? 3 : codec == KQ_MXFP4 ? 0 : 1;
  if ((reinterpret_cast<uintptr_t>(w) & wmask) || (reinterpret_cast<uintptr_t>(w2) & wmask) ||
      ((uintptr_t)w_expert_stride & wmask) || (reinterpret_cast<uintptr_t>(x) & 15) || ((K * 2) & 15) ||
      (strided_x && ((x_row_stride * 2) & 15)))
    return false;
  return true;
}

int kq_launch_gather_stream(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* lhs, const uint32_t* rhs,
                            void* out, int entries, int N, int K, int x_div, int64_t x_row_stride,
                            int64_t w_expert_stride, int act, float limit, float alpha, const float* bias,
                            const float* bias2, int codec, int dtype, int E, KqOutMap om, hipStream_t s) {
  if (!rhs || !kq_gather_stream_takes(x, w, w2, entries, N, K, lhs != nullptr, x_row_stride, w_expert_stride,
                                      !w2 && bias2, codec))
    return KQ_ERR_UNSUPPORTED;
  const bool glu = w2 != nullptr;
  StArgs a{};
  a.x = x;
  a.w = w;
  a.w2 = w2;
  a.rhs = rhs;
  a.lhs = lhs;
  a.x_row_stride = x_row_stride;
  a.y = out;
  a.M = 1;
  a.N = N;
  a.K = K;
  a.ksplit = 1;
  a.sb_per_split = st_k_units(K);
  a.x_div = x_div < 1 ? 1 : x_div;
  a.E = E;
  a.act = act;
  a.limit = limit;
  a.alpha = alpha;
  a.bias = bias;
  a.bias2 = bias2;
  a.w_expert_stride = w_expert_stride;
  a.om = om;
  if (codec == KQ_IQ4_XS || codec == KQ_IQ2_XXS || codec == KQ_IQ3_S) {
    a.grids = kq_device_grids();
    if (!a.grids) return KQ_ERR_HIP;
  }
  switch (codec) {
#define KQ_CASE(c)                                                                    \
  case c:                                                                             \
    return dtype == KQ_F16 ? st_launch_gather_nw<c, KQ_F16>(a, entries, glu, s)       \
                           : st_launch_gather_nw<c, KQ_BF16>(a, entries, glu, s);
    KQ_CASE(KQ_Q2_K) KQ_CASE(KQ_Q3_K) KQ_CASE(KQ_Q4_K) KQ_CASE(KQ_Q5_K) KQ_CASE(KQ_Q6_K) KQ_CASE(KQ_IQ4_XS)
    KQ_CASE(KQ_IQ3_S) KQ_CASE(KQ_IQ2_XXS) KQ_CASE(KQ_Q8_0) KQ_CASE(KQ_IQ4_NL) KQ_CASE(KQ_Q4_0) KQ_CASE(KQ_MXFP4)
    KQ_CASE(KQ_NVFP4)
#undef KQ_CASE
  }
  return KQ_ERR_UNSUPPORTED;
}
#endif  // gathered part
