// Tuned skinny-M (decode) kernels: y[M,N] = x[M,K] . W^T for M <= 8, weights streamed once from
// HBM, all multiply-accumulates on the matrix cores.  Codecs: q2_k, q3_k, q4_k, q5_k, q6_k.  Dense calls
// go to the streamed kernel of kq_stream.hip first; the kernels here serve the gathered ops (one grid
// row per (activation matrix, expert) item) and the fused gate/up GLU op, where a tile holds rows
// [n0, n0 + h) of the gate matrix followed by the same rows of the up matrix and the epilogue combines
// them, and the dense calls the streamed kernel declines.
//
// Mapping.  One workgroup (4 waves) owns a tile of up to 32 weight rows; its waves split K by
// superblock.  Inside a wave the weights are the B operand of v_mfma_f32_32x32x16_f16: lane l
// serves weight row n = l % 32 and K-half kg = l / 32.  Activations are the A operand: the
// workgroup converts x to f16 once (scaled by a power of two so bf16 inputs cannot overflow),
// keeps it in LDS, and every wave reads fragments back with ds_read_b128.  M is padded to the 32
// rows of the MFMA by letting the spare rows alias real ones; only the accumulator registers of
// real rows are carried.
//
// q4_k.  Nibbles become exact f16 integers with one AND-OR each (0x6400 | q = 1024 + q; high
// nibbles stay in place and read as 1024 + 16 q), so the MFMAs over one 32-weight sub-block return
//     P = sum_k x_k (1024 + s q_k),  s in {1, 16}
// and the sub-block contributes  (d sc / s) P - (1024 d sc / s + dmin m) X,  X = sum_k x_k,
// applied in f32 on the accumulator registers.
//
// q6_k.  sc (q - 32) with sc the int8 scale of the weight's 16-group reaches 4096 and is not always
// an f16 number, so a weight is fed to the matrix cores as two exact f16 terms, sc ql (the low
// nibble, <= 1920) and 16 sc (qh - 2) (the two high bits, a multiple of 16 up to 4096): the nibble
// is masked in place as 1024 + 16 ql, the high bits as 1024 + 256 qh, and one v_pk_fma_f16 each
// removes the 1024 and applies sc.  Two MFMAs per 16 weights share the activation fragment; one
// accumulator collects the superblock and is folded in with a single multiply by d.
#include <type_traits>

#include "kq_decode.h"
#include "kq_epilogue.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// 16-byte global load from a 2-byte-aligned address (q6_k blocks are 210 bytes long): the
// hardware serves unaligned vector loads, the type only stops the compiler from assuming more
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));

constexpr int SK_WAVES = 4;
constexpr int SK_THREADS = SK_WAVES * 64;
constexpr int SK_MAXM = 8;
constexpr int SK_MAXROWS = 32;

// Compile-time loop: the body sees its index as a constant from the start, so register arrays
// indexed by it are split into scalars (a '#pragma unroll' loop is unrolled too late for that
// and leaves the array in scratch memory).
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

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences global memory,
// which on this target drains every outstanding global load (s_waitcnt vmcnt(0)) and would
// serialise the weight stream behind each barrier.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// (a & mask) | magic should be ONE v_and_or_b32.  VOP3 on gfx9 takes no literal operands, so
// with constant mask/magic the compiler emits v_and + v_or; callers therefore pass mask and magic
// through opaque registers (see kq_opaque_*).  No instruction is written in inline asm: the
// hazard recognizer does not see inside asm statements, and VALU writes racing an in-flight MFMA
// destination need its wait states.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) { return (a & mask) | magic; }
__device__ __forceinline__ uint32_t kq_opaque_vgpr(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}
__device__ __forceinline__ uint32_t kq_opaque_sgpr(uint32_t v) {
  asm volatile("" : "+s"(v));
  return v;
}

// Per-codec geometry of the weight stream.  A superblock travels as PP 16-byte pieces (q6_k: the
// first 208 bytes; its trailing 2-byte d goes through a side channel) and is parked in LDS LBPB
// bytes apart, so that every block starts 16-byte aligned there.
template <int C>
struct SkGeom;
// TAIL: the block's last 16 bytes [BPB - 16, BPB) travel as one extra piece and are parked at
// LDS offset 16 PP of the block (q2_k: d / dmin, q3_k: scales + d).  XSUM: granularity of the
// activation sums kept in LDS (0 = none).  KGOFF: consecutive weights a lane owns inside each
// 32-weight sub-block half -- 16 (lane kg takes weights 16 kg .. 16 kg + 15 of the sub-block) or 8
// (weights 8 kg .. 8 kg + 7 of each 16-weight scale group, so one MFMA covers one scale group).
template <>
struct SkGeom<KQ_Q4_K> {
  static constexpr int BPB = 144, LBPB = 144, PP = 9, XSUM = 32, KGOFF = 16;
  static constexpr bool SIDE_D = false, TAIL = false;
  typedef u32x4 piece_t;
};
template <>
struct SkGeom<KQ_Q5_K> {
  static constexpr int BPB = 176, LBPB = 176, PP = 11, XSUM = 32, KGOFF = 16;
  static constexpr bool SIDE_D = false, TAIL = false;
  typedef u32x4 piece_t;
};
template <>
struct SkGeom<KQ_Q6_K> {
  static constexpr int BPB = 210, LBPB = 208, PP = 13, XSUM = 0, KGOFF = 16;
  static constexpr bool SIDE_D = true, TAIL = false;
  typedef u32x4_a2 piece_t;
};
template <>
struct SkGeom<KQ_Q2_K> {  // LDS block: scales[16] | qs[64] | tail (wire bytes 68..83: d at +12, dmin at +14) | pad
  static constexpr int BPB = 84, LBPB = 112, PP = 5, XSUM = 16, KGOFF = 8;
  static constexpr bool SIDE_D = false, TAIL = true;
  typedef u32x4_a2 piece_t;
};
template <>
struct SkGeom<KQ_Q3_K> {  // LDS block: hmask[32] | qs[64] | tail (wire bytes 94..109: scales at +2, d at +14)
  static constexpr int BPB = 110, LBPB = 112, PP = 6, XSUM = 16, KGOFF = 8;
  static constexpr bool SIDE_D = false, TAIL = true;
  typedef u32x4_a2 piece_t;
};

// Accumulator rows of the "diagonal" kernel: a lane whose MFMA column is (row r, superblock q) wants
// D rows 8 q + 4 kg + j, i.e. registers 4 q + j of the 16 it holds.
// (J is a template parameter: with a function argument the element access is lowered as a dynamic
// index -- sixteen selects per pick -- before inlining can make it constant.)
template <bool DIAG, int J>
__device__ __forceinline__ float pick_row(const f32x16& p, int q) {
  if constexpr (!DIAG) {
    return p[J];
  } else {
    const float lo = (q & 1) ? p[4 + J] : p[J], hi = (q & 1) ? p[12 + J] : p[8 + J];
    return (q & 2) ? hi : lo;
  }
}

// ------------------------------------------------------------------ q4_k superblock
struct Q4kRaw {
  uint4 hdr;
  uint4 q[4];
};

// per-lane scales of one superblock: mul[j] multiplies P_j, sub[j] multiplies X_j
__device__ __forceinline__ void q4k_scales(const uint4& hdr, float xscale, float* mul, float* sub) {
  const float d = kq::h2f((uint16_t)(hdr.x & 0xffff)) * xscale;
  const float dmin = kq::h2f((uint16_t)(hdr.x >> 16)) * xscale;
  const float d16 = d * 0.0625f;
  const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
  const uint32_t sc_lo = s0 & 0x3f3f3f3fu, mn_lo = s1 & 0x3f3f3f3fu;
  const uint32_t sc_hi = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
  const uint32_t mn_hi = ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u);
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const uint32_t scw = j < 4 ? sc_lo : sc_hi, mnw = j < 4 ? mn_lo : mn_hi;
    const float sc = (float)((scw >> (8 * (j & 3))) & 0xff);
    const float mn = (float)((mnw >> (8 * (j & 3))) & 0xff);
    // even sub-blocks read low nibbles (1024 + q), odd ones high nibbles in place (1024 + 16 q)
    mul[j] = ((j & 1) ? d16 : d) * sc;
    sub[j] = fmaf(mul[j], 1024.0f, dmin * mn);
  }
}

__device__ __forceinline__ f16x8 q4k_frag(uint32_t wa, uint32_t wa8, uint32_t wb, uint32_t wb8, uint32_t mask,
                                          uint32_t magic) {
  uint4 v;
  v.x = and_or(wa, mask, magic);   // k0, k2
  v.y = and_or(wa8, mask, magic);  // k1, k3
  v.z = and_or(wb, mask, magic);   // k4, k6
  v.w = and_or(wb8, mask, magic);  // k5, k7
  return __builtin_bit_cast(f16x8, v);
}

// One superblock of one 32-row tile (q4_k / q5_k): 16 MFMAs + the f32 fix-up on R accumulator
// registers.  bl: this lane's row of the superblock in LDS; xs_lane: this lane's A-fragment base
// (f16 index) for the superblock; xsum: X_j for the superblock, [8][XS] floats.
// q5_k: the fifth bit of weight (sub-block j, i) is bit j of qh[i]; it is OR-ed into the code at
// bit 4 (low-nibble sub-blocks, 1024 + q) or bit 8 (high-nibble ones, 1024 + 16 q).
template <int C, int R, int XS, bool DIAG = false>
__device__ __forceinline__ void q45k_superblock(const uint8_t* __restrict__ bl, int kg, float xscale,
                                                const _Float16* __restrict__ xs_lane,
                                                const float* __restrict__ xsum, float* acc, int q = 0) {
  constexpr int QS = C == KQ_Q4_K ? 16 : 48;  // offset of the nibble array
  Q4kRaw raw;
  const uint4* p4 = reinterpret_cast<const uint4*>(bl);
  raw.hdr = p4[0];
#pragma unroll
  for (int g = 0; g < 4; g++) raw.q[g] = *reinterpret_cast<const uint4*>(bl + QS + 32 * g + 16 * kg);
  uint32_t hw[4] = {0, 0, 0, 0};
  if constexpr (C == KQ_Q5_K) {
    const uint4 hv = p4[1 + kg];  // qh[16 kg .. 16 kg + 15]
    hw[0] = hv.x;
    hw[1] = hv.y;
    hw[2] = hv.z;
    hw[3] = hv.w;
  }
  float mul[8], sub[8];
  q4k_scales(raw.hdr, xscale, mul, sub);
  const uint32_t magic = kq_opaque_vgpr(0x64006400u);
  const uint32_t mask_lo = kq_opaque_sgpr(0x000f000fu), mask_hi = kq_opaque_sgpr(0x00f000f0u);
  const uint32_t bit_lo = kq_opaque_sgpr(0x00100010u), bit_hi = kq_opaque_sgpr(0x01000100u);
#pragma unroll
  for (int g = 0; g < 4; g++) {
    const uint32_t qw[4] = {raw.q[g].x, raw.q[g].y, raw.q[g].z, raw.q[g].w};
    const uint32_t qw8[4] = {qw[0] >> 8, qw[1] >> 8, qw[2] >> 8, qw[3] >> 8};
#pragma unroll
    for (int h = 0; h < 2; h++) {  // h = 0: sub-block 2g (low nibbles), h = 1: 2g + 1 (high nibbles)
      const int j = 2 * g + h;
      f32x16 p = {0};
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const f16x8 a = *reinterpret_cast<const f16x8*>(xs_lane + 32 * j + 8 * s);
        f16x8 b = q4k_frag(qw[2 * s], qw8[2 * s], qw[2 * s + 1], qw8[2 * s + 1], h ? mask_hi : mask_lo, magic);
        if constexpr (C == KQ_Q5_K) {
          // even bytes of a qh word (bits j, 16 + j) go to bits 4 / 20 (h = 0) or 8 / 24 (h = 1) of the
          // fragment word, odd bytes (bits 8 + j, 24 + j) likewise
          const int tgt = h ? 8 : 4;
          const uint32_t bm = h ? bit_hi : bit_lo;
          uint4 v = __builtin_bit_cast(uint4, b);
          const uint32_t ha = hw[2 * s], hb = hw[2 * s + 1];
          const uint32_t ea = tgt >= j ? (ha << (tgt - j)) : (ha >> (j - tgt));
          const uint32_t eb = tgt >= j ? (hb << (tgt - j)) : (hb >> (j - tgt));
          const uint32_t oa = ha >> (8 + j - tgt), ob = hb >> (8 + j - tgt);
          v.x = and_or(ea, bm, kq_opaque_vgpr(v.x));
          v.y = and_or(oa, bm, kq_opaque_vgpr(v.y));
          v.z = and_or(eb, bm, kq_opaque_vgpr(v.z));
          v.w = and_or(ob, bm, kq_opaque_vgpr(v.w));
          b = __builtin_bit_cast(f16x8, v);
        }
        p = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, p, 0, 0, 0);
      }
      StaticFor<R>::run([&](auto rr) {
        constexpr int r = decltype(rr)::value;
        acc[r] = fmaf(mul[j], pick_row<DIAG, r>(p, q), acc[r]);
        acc[r] = fmaf(-sub[j], xsum[j * XS + r], acc[r]);
      });
    }
  }
}

// ------------------------------------------------------------------ q2_k / q3_k superblocks
// Weight 128 half + 32 si + l (l = 0..31) is the 2-bit field si of qs[32 half + l]; its scale group is
// 8 half + 2 si + l / 16.  Lane (row, kg) owns l = 16 s + 8 kg .. + 7 of MFMA s, so every MFMA covers
// exactly one scale group and is folded with that group's scale.  The field is masked in place and
// reads 1024 + 4^si q; the 4^si goes into the scale.
template <int R, int XS, bool DIAG = false>
__device__ __forceinline__ void q2k_superblock(const uint8_t* __restrict__ bl, int kg, float xscale,
                                               const _Float16* __restrict__ xs_lane,
                                               const float* __restrict__ xsum, float* acc, int q = 0) {
  const uint32_t magic = kq_opaque_vgpr(0x64006400u);
  const uint32_t mask[4] = {kq_opaque_sgpr(0x00030003u), kq_opaque_sgpr(0x000c000cu), kq_opaque_sgpr(0x00300030u),
                            kq_opaque_sgpr(0x00c000c0u)};
  const uint4 scv = *reinterpret_cast<const uint4*>(bl);
  const uint32_t scw[4] = {scv.x, scv.y, scv.z, scv.w};
  const uint32_t dm = *reinterpret_cast<const uint32_t*>(bl + 80 + 12);
  const float d = kq::h2f((uint16_t)(dm & 0xffff)) * xscale, dmin = kq::h2f((uint16_t)(dm >> 16)) * xscale;
#pragma unroll
  for (int half = 0; half < 2; half++) {
    const uint2 q0 = *reinterpret_cast<const uint2*>(bl + 16 + 32 * half + 8 * kg);
    const uint2 q1 = *reinterpret_cast<const uint2*>(bl + 32 + 32 * half + 8 * kg);
    const uint32_t qv[2][4] = {{q0.x, q0.x >> 8, q0.y, q0.y >> 8}, {q1.x, q1.x >> 8, q1.y, q1.y >> 8}};
#pragma unroll
    for (int si = 0; si < 4; si++) {
      const int j = 4 * half + si;
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const int g = 8 * half + 2 * si + s;
        const uint32_t scb = (scw[g >> 2] >> (8 * (g & 3))) & 0xff;
        uint4 v;
        v.x = and_or(qv[s][0], mask[si], magic);
        v.y = and_or(qv[s][1], mask[si], magic);
        v.z = and_or(qv[s][2], mask[si], magic);
        v.w = and_or(qv[s][3], mask[si], magic);
        const f16x8 a = *reinterpret_cast<const f16x8*>(xs_lane + 32 * j + 16 * s);
        const f32x16 p = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, __builtin_bit_cast(f16x8, v), f32x16{0}, 0, 0, 0);
        const float mulg = d * (float)(scb & 15) * (1.0f / (float)(1 << (2 * si)));
        const float subg = fmaf(mulg, 1024.0f, dmin * (float)(scb >> 4));
        StaticFor<R>::run([&](auto rr) {
          constexpr int r = decltype(rr)::value;
          acc[r] = fmaf(mulg, pick_row<DIAG, r>(p, q), acc[r]);
          acc[r] = fmaf(-subg, xsum[g * XS + r], acc[r]);
        });
      }
    }
  }
}

// q3_k: same 2-bit fields plus the high bit (bit 4 half + si of hmask[l], set = +4): the code is
// 1024 + 4^si (q + 4 h) with zero point 4, scale d (sc - 32), sc the 6-bit scale of the group.
template <int R, int XS, bool DIAG = false>
__device__ __forceinline__ void q3k_superblock(const uint8_t* __restrict__ bl, int kg, float xscale,
                                               const _Float16* __restrict__ xs_lane,
                                               const float* __restrict__ xsum, float* acc, int q = 0) {
  const uint32_t magic = kq_opaque_vgpr(0x64006400u);
  const uint32_t mask[4] = {kq_opaque_sgpr(0x00030003u), kq_opaque_sgpr(0x000c000cu), kq_opaque_sgpr(0x00300030u),
                            kq_opaque_sgpr(0x00c000c0u)};
  const uint32_t hmask[4] = {kq_opaque_sgpr(0x00040004u), kq_opaque_sgpr(0x00100010u), kq_opaque_sgpr(0x00400040u),
                             kq_opaque_sgpr(0x01000100u)};
  const uint4 tl = *reinterpret_cast<const uint4*>(bl + 96);  // wire bytes 94..109
  // 12 scale bytes start at tail byte 2
  const uint32_t s0 = __builtin_amdgcn_alignbyte(tl.y, tl.x, 2), s1 = __builtin_amdgcn_alignbyte(tl.z, tl.y, 2),
                 s2 = __builtin_amdgcn_alignbyte(tl.w, tl.z, 2);
  const float d = kq::h2f((uint16_t)(tl.w >> 16)) * xscale;
  const uint2 h0 = *reinterpret_cast<const uint2*>(bl + 8 * kg);
  const uint2 h1 = *reinterpret_cast<const uint2*>(bl + 16 + 8 * kg);
  const uint32_t hv[2][4] = {{h0.x, h0.x >> 8, h0.y, h0.y >> 8}, {h1.x, h1.x >> 8, h1.y, h1.y >> 8}};
#pragma unroll
  for (int half = 0; half < 2; half++) {
    const uint2 q0 = *reinterpret_cast<const uint2*>(bl + 32 + 32 * half + 8 * kg);
    const uint2 q1 = *reinterpret_cast<const uint2*>(bl + 48 + 32 * half + 8 * kg);
    const uint32_t qv[2][4] = {{q0.x, q0.x >> 8, q0.y, q0.y >> 8}, {q1.x, q1.x >> 8, q1.y, q1.y >> 8}};
#pragma unroll
    for (int si = 0; si < 4; si++) {
      const int j = 4 * half + si;
      const int sh = si + 2 - 4 * half;  // hmask bit 4 half + si -> code bit 2 si + 2
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const int g = 8 * half + 2 * si + s, k = g & 3, grp = g >> 2;
        uint32_t lo4 = ((grp & 1) ? s1 : s0) >> (8 * k);
        lo4 = (grp & 2) ? ((lo4 >> 4) & 15) : (lo4 & 15);
        const uint32_t sc = lo4 | (((s2 >> (8 * k + 2 * grp)) & 3) << 4);
        uint32_t fr[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const uint32_t hb = sh >= 0 ? (hv[s][e] << (sh >= 0 ? sh : 0)) : (hv[s][e] >> (sh < 0 ? -sh : 0));
          fr[e] = and_or(hb, hmask[si], kq_opaque_vgpr(and_or(qv[s][e], mask[si], magic)));
        }
        const uint4 v = make_uint4(fr[0], fr[1], fr[2], fr[3]);
        const f16x8 a = *reinterpret_cast<const f16x8*>(xs_lane + 32 * j + 16 * s);
        const f32x16 p = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, __builtin_bit_cast(f16x8, v), f32x16{0}, 0, 0, 0);
        const float mulg = d * (float)((int)sc - 32) * (1.0f / (float)(1 << (2 * si)));
        const float subg = mulg * (1024.0f + (float)(4 << (2 * si)));
        StaticFor<R>::run([&](auto rr) {
          constexpr int r = decltype(rr)::value;
          acc[r] = fmaf(mulg, pick_row<DIAG, r>(p, q), acc[r]);
          acc[r] = fmaf(-subg, xsum[g * XS + r], acc[r]);
        });
      }
    }
  }
}

// ------------------------------------------------------------------ q6_k superblock
// LDS block: ql[128] | qh[64] | int8 scales[16]; d arrives separately.  Weight 128 hf + 32 t + l
// (hf = half, t = 0..3, l = 0..31) has its low nibble in ql[64 hf + 32 (t & 1) + l] (high nibble of
// the byte when t >= 2), its high bits in bits 2t, 2t+1 of qh[32 hf + l] and scale 8 hf + 2 t +
// l / 16.  Lane (row, kg) takes l = 16 kg .. 16 kg + 15: one scale per lane and sub-block.
template <int R, bool DIAG = false>
__device__ __forceinline__ void q6k_superblock(const uint8_t* __restrict__ bl, int kg, float dx,
                                               const _Float16* __restrict__ xs_lane, float* acc, int q = 0) {
  const uint32_t magic = kq_opaque_vgpr(0x64006400u);
  const uint32_t mask_q = kq_opaque_sgpr(0x00f000f0u), mask_h = kq_opaque_sgpr(0x03000300u);
  const uint4 scv = *reinterpret_cast<const uint4*>(bl + 192);
  const uint32_t scw[4] = {scv.x, scv.y, scv.z, scv.w};
  f32x16 p = {0};
#pragma unroll
  for (int hf = 0; hf < 2; hf++) {
    const uint4 hv = *reinterpret_cast<const uint4*>(bl + 128 + 32 * hf + 16 * kg);
    const uint32_t hw[4] = {hv.x, hv.y, hv.z, hv.w};
#pragma unroll
    for (int qr = 0; qr < 2; qr++) {
      const uint4 qv = *reinterpret_cast<const uint4*>(bl + 64 * hf + 32 * qr + 16 * kg);
      const uint32_t qw[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int t = qr + 2 * h, j = 4 * hf + t;
        const int sc = __builtin_amdgcn_sbfe((int)scw[2 * hf + (t >> 1)], 8 * (2 * (t & 1) + kg), 8);
        const float scf = (float)sc;
        const _Float16 sch = (_Float16)(scf * 0.0625f), ofl = (_Float16)(-64.0f * scf), ofh = (_Float16)(-96.0f * scf);
        const f16x2 scp = {sch, sch}, oflp = {ofl, ofl}, ofhp = {ofh, ofh};
#pragma unroll
        for (int s = 0; s < 2; s++) {
          uint32_t fl[4], fh[4];
#pragma unroll
          for (int e = 0; e < 2; e++) {
            const uint32_t q = qw[2 * s + e], hq = hw[2 * s + e];
            const uint32_t qe = h ? q : (q << 4), qo = h ? (q >> 8) : (q >> 4);
            const uint32_t he = hq << (8 - 2 * t), ho = t ? (hq >> (2 * t)) : hq;
            fl[2 * e] = and_or(qe, mask_q, magic);  // bytes 0, 2 of the word: 1024 + 16 ql
            fl[2 * e + 1] = and_or(qo, mask_q, magic);  // bytes 1, 3
            fh[2 * e] = and_or(he, mask_h, magic);  // 1024 + 256 qh
            fh[2 * e + 1] = and_or(ho, mask_h, magic);
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
          const f16x8 a = *reinterpret_cast<const f16x8*>(xs_lane + 32 * j + 8 * s);
          p = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, blo, p, 0, 0, 0);
          p = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bhi, p, 0, 0, 0);
        }
      }
    }
  }
  StaticFor<R>::run([&](auto rr) {
    constexpr int r = decltype(rr)::value;
    acc[r] = fmaf(dx, pick_row<DIAG, r>(p, q), acc[r]);
  });
}

// ------------------------------------------------------------------ the kernel
struct SkArgs {
  const void* x;
  const uint8_t* w;
  const uint8_t* w2;    // up stack (GLU) or null
  void* y;
  const uint32_t* lhs;  // activation-matrix index per item, or null: item / x_div
  const uint32_t* rhs;  // expert index per item, or null: expert 0
  int M, N, K, rows_per_tile, kch, x_div, act;
  int64_t x_batch_stride;   // elements between activation matrices
  int64_t w_expert_stride;  // bytes between expert matrices
  float limit;
  // split-K (dense calls with few row tiles): grid z = K split; partial sums [ksplit][M][N] f32
  float* partial;
  int ksplit, sb_per_split;
  KqOutMap om;  // gathered calls: output row of an item, 16-bit or f32 (dense calls: identity)
  int E;        // gathered calls: items whose expert id is >= E are skipped (output rows left untouched)
};

// MB = M rounded up to a power of two (1, 2, 4, 8).  Rows of the 32-row A operand beyond MB alias
// row (r % MB); their accumulator rows are never read.  Grid: x = row tile, y = item.
//
// Weight traffic: a tile (rows_per_tile rows x KCH superblocks) is fetched with coalesced
// 16-byte loads -- consecutive lanes read consecutive 16-byte pieces of a row, so every wave
// load covers about 1 KiB of contiguous HBM -- and parked in LDS with the row stride an odd
// multiple of 16 bytes (keeps the row-per-lane ds_read_b128 of the MFMA operand fetch free of
// bank conflicts).  A row-per-lane pattern straight from global memory runs 6x slower: each
// wave load would touch 32 different cache lines for 32 bytes apiece.
// Sub-chunks (synchronous kernel) / units (decoupled kernel) in flight beyond the one being
// consumed.  One is best: with 2, 3 and 4 the 33 MB gate/up GEMV took 11.3, 12.4 and 12.9 us instead of
// 10.2 -- a single resident round of workgroups already keeps ~8 MB outstanding, which covers the
// bandwidth-latency product; anything more only queues in the memory system.
#ifndef SK_INF
#define SK_INF 1
#endif
template <int C, int DT, int MB, bool GLU>
__global__ __launch_bounds__(SK_THREADS, 2) void skinny_kernel(SkArgs a) {
  using G = SkGeom<C>;
  constexpr int R = MB < 4 ? MB : 4;  // accumulator registers carried per lane
  constexpr int SBC = 4;              // superblocks per sub-chunk: one per wave
  constexpr int NCH = 4;              // sub-chunks per chunk (kch <= 16)
  constexpr int PPR = SBC * G::PP;    // 16-byte pieces per row and sub-chunk
  constexpr int PPC = (SK_MAXROWS * PPR + SK_THREADS - 1) / SK_THREADS;  // pieces per thread and sub-chunk
  // activation staging slots per thread: slot t = (row t / XK, k-pass t % XK); a chunk holds at
  // most min(512, 2048 / MB) 8-element groups per row because kch <= 16 and kch * MB <= 64
  constexpr int XK = MB <= 4 ? 2 : 1;
  constexpr int XG = MB * XK;
  constexpr int INF = SK_INF;  // sub-chunks in flight

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int M = a.M, N = a.N, K = a.K, rows_per_tile = a.rows_per_tile, kch = a.kch;
  // layout: wt [rows_per_tile][wstride] | xs f16 [MB][kch*256] | xsum f32 [kch*8][MB] | red | scratch | dump | dq
  const int wstride = kch * G::LBPB + (((kch * (G::LBPB / 16)) & 1) ? 0 : 16), kchunk = kch * 256;
  uint8_t* wt = smem;
  _Float16* xs = reinterpret_cast<_Float16*>(smem + rows_per_tile * wstride);
  float* xsum = reinterpret_cast<float*>(smem + rows_per_tile * wstride + (size_t)MB * kchunk * 2);
  float* red = xsum + kch * 16 * MB;
  float* scratch = red + SK_WAVES * R * 64;
  uint8_t* dump = reinterpret_cast<uint8_t*>(scratch + 16) + 16 * threadIdx.x;  // per-thread 16-byte dump slot
  uint16_t* dq = reinterpret_cast<uint16_t*>(reinterpret_cast<uint8_t*>(scratch + 16) + 16 * SK_THREADS);  // [32][16]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_in = lane & 31, kg = lane >> 5;
  const int nsb = K >> 8;
  const size_t row_bytes = (size_t)nsb * G::BPB;
  // GLU tiles hold `half` gate rows then `half` up rows; plain tiles rows_per_tile rows
  const int half = GLU ? (rows_per_tile >> 1) : rows_per_tile;
  const int row0 = blockIdx.x * half;
  const int nrows = (N - row0 < half) ? (N - row0) : half;
  const int item = blockIdx.y;
  const size_t expert = a.rhs ? a.rhs[item] : 0;
  if (a.rhs && expert >= (size_t)a.E) return;  // uniform over the workgroup, ahead of every barrier
  const size_t xsel = a.lhs ? a.lhs[item] : (size_t)(item / a.x_div);
  const uint8_t* wtile = a.w + expert * (size_t)a.w_expert_stride + (size_t)row0 * row_bytes;
  const uint8_t* wtile2 = GLU ? a.w2 + expert * (size_t)a.w_expert_stride + (size_t)row0 * row_bytes : wtile;
  const uint16_t* x16 = static_cast<const uint16_t*>(a.x) + xsel * (size_t)a.x_batch_stride;
  // compute-phase row of this lane (spare lanes re-read tile row 0, their results are dropped)
  const bool lane_live = GLU ? (n_in < 2 * half && (n_in < half ? n_in : n_in - half) < nrows) : n_in < nrows;
  const int crow = lane_live ? n_in : 0;

  float acc[R];
#pragma unroll
  for (int r = 0; r < R; r++) acc[r] = 0.f;

  // piece map of the weight stream (see step 2): global / LDS byte offsets inside a sub-chunk
  uint32_t goff[PPC], loff[PPC];
  int ppc[PPC];
  bool piece_ok[PPC], piece_up[PPC];
  {
    int r = tid / PPR, pc = tid % PPR;
    StaticFor<PPC>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      const bool up = GLU && r >= half;
      const int srow = up ? r - half : r;
      piece_ok[T] = srow < nrows && r < rows_per_tile;
      piece_up[T] = up;
      ppc[T] = pc;
      const int sbl = pc / G::PP, p = pc % G::PP;
      goff[T] = (uint32_t)srow * (uint32_t)row_bytes + sbl * G::BPB + 16 * p;
      loff[T] = (uint32_t)r * (uint32_t)wstride + sbl * G::LBPB + 16 * p;
      r += SK_THREADS / PPR;
      pc += SK_THREADS % PPR;
      if (pc >= PPR) {
        pc -= PPR;
        r++;
      }
    });
  }
  // side channel for the 2-byte d of q6_k: thread -> (row tid / 4, superblock tid % 4) of a sub-chunk
  const int d_row = tid >> 2, d_sbl = tid & 3;
  const bool d_up = GLU && d_row >= half;
  const int d_srow = d_up ? d_row - half : d_row;
  const bool d_ok = G::SIDE_D && d_row < rows_per_tile && d_srow < nrows;
  const uint8_t* d_src = (d_up ? wtile2 : wtile) + (d_ok ? (size_t)d_srow * row_bytes : 0) + 208;
  // tail piece (last 16 bytes of a block), same thread -> (row, superblock) map
  const bool t_ok = G::TAIL && d_row < rows_per_tile && d_srow < nrows;
  const uint8_t* t_src = (d_up ? wtile2 : wtile) + (t_ok ? (size_t)d_srow * row_bytes : 0) + (G::BPB - 16);
  uint8_t* t_dst = wt + d_row * wstride + d_sbl * G::LBPB + 16 * G::PP;

  const int sb_begin = a.ksplit > 1 ? (int)blockIdx.z * a.sb_per_split : 0;
  const int sb_end = a.ksplit > 1 ? (sb_begin + a.sb_per_split < nsb ? sb_begin + a.sb_per_split : nsb) : nsb;
  for (int sb0 = sb_begin; sb0 < sb_end; sb0 += kch) {
    const int sbn = (sb_end - sb0 < kch) ? (sb_end - sb0) : kch;
    const int kc = sbn << 8, k0 = sb0 << 8;

    // ---- 1. activation loads first, so waiting for them does not wait for the weights
    const int gpr = kc >> 3;  // 8-element groups per activation row in this chunk
    u32x4 xreg[XG];
    // (loads are unconditional and branch-free -- out-of-range slots re-read valid data -- so the
    // compiler can count outstanding loads exactly and wait for the activations alone)
    StaticFor<XG>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      int m = T / XK;
      m = m < M ? m : M - 1;  // spare rows of the MB-row block mirror the last real row
      int kgi = tid + (T % XK) * SK_THREADS;
      kgi = kgi < gpr ? kgi : 0;
      xreg[T] = *reinterpret_cast<const u32x4*>(x16 + (size_t)m * K + k0 + 8 * kgi);
    });

    // ---- 2. weight stream.  Sub-chunk c covers superblocks [4c, 4c+4) = PPR 16-byte pieces per
    // row; piece i = tid + 256 t maps to (row i / PPR, piece i % PPR), so consecutive lanes read
    // consecutive 16-byte pieces of a row.  The map is the same for every sub-chunk (goff / loff);
    // pieces outside the tile or a ragged last sub-chunk re-read the tile's first bytes and
    // land in a dump slot.  INF sub-chunks are in flight at any time (register sets c % INF); the
    // next one is issued as soon as its register set has been parked in LDS.
    u32x4 wreg[INF * PPC], treg[INF];
    uint16_t dreg[INF];
    auto issue = [&](auto cc) {
      constexpr int c = decltype(cc)::value;
      const int sbc = sbn - SBC * c;  // superblocks left from this sub-chunk on (uniform)
      const size_t sboff = (size_t)(sb0 + SBC * c) * G::BPB;
      StaticFor<PPC>::run([&](auto t) {
        constexpr int T = decltype(t)::value;
        const bool ok = piece_ok[T] && ppc[T] < sbc * G::PP;
        const uint8_t* base = (GLU && piece_up[T]) ? wtile2 : wtile;
        wreg[(c % INF) * PPC + T] = *reinterpret_cast<const typename G::piece_t*>(ok ? base + sboff + goff[T] : wtile);
      });
      if constexpr (G::SIDE_D) {
        const bool ok = d_ok && d_sbl < sbc;
        dreg[c % INF] = *reinterpret_cast<const uint16_t*>(ok ? d_src + sboff + d_sbl * G::BPB : wtile);
      }
      if constexpr (G::TAIL) {
        const bool ok = t_ok && d_sbl < sbc;
        treg[c % INF] = *reinterpret_cast<const u32x4_a2*>(ok ? t_src + sboff + d_sbl * G::BPB : wtile);
      }
    };
    StaticFor<INF>::run([&](auto cc) { issue(cc); });

    // ---- 3. activations -> f16 in LDS (+ per-sub-block sums)
    if (sb0 > sb_begin) lds_barrier();
    float xscale = 1.0f, inv = 1.0f;  // true x = xscale * stored f16 x
    if constexpr (DT == KQ_BF16) {
      float amax = 0.f;
      StaticFor<XG>::run([&](auto t) {
        const u32x4 v = xreg[decltype(t)::value];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] << 16)));
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] & 0xffff0000u)));
        }
      });
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
      if (lane == 0) scratch[wave] = amax;
      lds_barrier();
      amax = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
      // bring the largest magnitude into [2^14, 2^15): exact power-of-two scaling
      const uint32_t eb = (__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff;
      if (eb != 0 && eb != 0xff) {
        int e = (int)eb - 127 - 14;
        if (e < -100) e = -100;
        xscale = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
        inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
      }
    }
    StaticFor<XG>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      constexpr int m = T / XK;
      const int kgi = tid + (T % XK) * SK_THREADS;
      if (kgi < gpr) {
        const int kk = kgi << 3;
        const u32x4 v = xreg[T];
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
        // MFMA fragment order inside an 8-group: k0 k2 k1 k3 k4 k6 k5 k7
        const f16x8 v8 = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
        *reinterpret_cast<f16x8*>(xs + (size_t)m * kchunk + kk) = v8;
        if constexpr (G::XSUM != 0) {
          float sum = 0.f;
#pragma unroll
          for (int e = 0; e < 8; e++) sum += (float)h[e];
          sum += __shfl_xor(sum, 1);  // 2 threads cover a 16-wide scale group, 4 a 32-wide sub-block
          if constexpr (G::XSUM == 32) {
            sum += __shfl_xor(sum, 2);
            if ((tid & 3) == 0) xsum[(kk >> 5) * MB + m] = sum;
          } else {
            if ((tid & 1) == 0) xsum[(kk >> 4) * MB + m] = sum;
          }
        }
      }
    });

    // ---- 4. sub-chunk by sub-chunk: park the arrived bytes in LDS, then one superblock per wave
    // while the later sub-chunks are still streaming in
    const _Float16* xs_lane = xs + (size_t)(n_in & (MB - 1)) * kchunk + G::KGOFF * kg;
    const float* xsum_lane = xsum + (MB == 8 ? 4 * kg : 0);
    const uint8_t* wt_lane = wt + crow * wstride;
    StaticFor<NCH>::run([&](auto cc) {
      constexpr int c = decltype(cc)::value;
      const int sbc = sbn - SBC * c;
      if (sbc > 0) {
        StaticFor<PPC>::run([&](auto t) {
          constexpr int T = decltype(t)::value;
          const bool ok = piece_ok[T] && ppc[T] < sbc * G::PP;
          *reinterpret_cast<u32x4*>(ok ? wt + SBC * c * G::LBPB + loff[T] : dump) = wreg[(c % INF) * PPC + T];
        });
        if constexpr (G::SIDE_D) {
          if (d_ok && d_sbl < sbc) dq[d_row * 16 + SBC * c + d_sbl] = dreg[c % INF];
        }
        if constexpr (G::TAIL) {
          *reinterpret_cast<u32x4*>((t_ok && d_sbl < sbc) ? t_dst + SBC * c * G::LBPB : dump) = treg[c % INF];
        }
      }
      if constexpr (c + INF < NCH) issue(std::integral_constant<int, c + INF>{});
      if (sbc > 0) {
        lds_barrier();
        const int sb = SBC * c + wave;
        if (sb < sbn) {
          if constexpr (C == KQ_Q4_K || C == KQ_Q5_K) {
            q45k_superblock<C, R, MB>(wt_lane + sb * G::LBPB, kg, xscale, xs_lane + 256 * sb, xsum_lane + 8 * MB * sb,
                                      acc);
          } else if constexpr (C == KQ_Q2_K) {
            q2k_superblock<R, MB>(wt_lane + sb * G::LBPB, kg, xscale, xs_lane + 256 * sb, xsum_lane + 16 * MB * sb, acc);
          } else if constexpr (C == KQ_Q3_K) {
            q3k_superblock<R, MB>(wt_lane + sb * G::LBPB, kg, xscale, xs_lane + 256 * sb, xsum_lane + 16 * MB * sb, acc);
          } else {
            const float dx = kq::h2f(dq[crow * 16 + sb]) * xscale;
            q6k_superblock<R>(wt_lane + sb * G::LBPB, kg, dx, xs_lane + 256 * sb, acc);
          }
        }
      }
    });
  }

  // ---- cross-wave reduction and store
#pragma unroll
  for (int r = 0; r < R; r++) red[(wave * R + r) * 64 + lane] = acc[r];
  lds_barrier();
  if constexpr (!GLU) {
    if (a.ksplit > 1) {
      // split-K: store this workgroup's partial sums; a second kernel adds the splits up in order
      const size_t plane = (size_t)M * N;
      for (int o = tid; o < R * 64; o += SK_THREADS) {
        const int r = o >> 6, l = o & 63;
        const int m = 4 * (l >> 5) + r, n = l & 31;
        if (m >= M || n >= nrows) continue;
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < SK_WAVES; wv++) v += red[(wv * R + r) * 64 + l];
        a.partial[blockIdx.z * plane + (size_t)m * N + row0 + n] = v;
      }
      return;
    }
  }
  for (int o = tid; o < R * 64; o += SK_THREADS) {
    const int r = o >> 6, l = o & 63;
    const int m = 4 * (l >> 5) + r, n = l & 31;
    if (m >= M || n >= nrows) continue;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < SK_WAVES; wv++) v += red[(wv * R + r) * 64 + l];
    if constexpr (GLU) {
      float u = 0.f;
#pragma unroll
      for (int wv = 0; wv < SK_WAVES; wv++) u += red[(wv * R + r) * 64 + l + half];
      v = kq::glu_epilogue(a.act, v, u, a.limit, 1.0f);
    }
    // gathered calls may remap the item's output row (M = 1 there) or ask for f32
    kq::store_result<DT>(a.y, a.om, ((size_t)kq::out_row(a.om, item) * M + m) * N + row0 + n, v);
  }
}

// ------------------------------------------------------------------ decoupled-wave variant (dense calls)
// Same tiles, same superblock routines, but every wave fetches, parks and consumes ITS OWN
// superblocks: the weight stream needs no workgroup barrier, so a wave that has its bytes never
// waits for the slowest of four.  A wave owns a run of adjacent superblocks of the chunk and moves
// it in units of USB superblocks x 32 rows.  USB = 2: consecutive lanes read the 2 PP consecutive
// pieces of a row (288 B for q4_k), then the next row -- reading the 33 MB gate/up matrix with
// nothing but this pattern takes 7.3 us, with 144-byte runs 8.2 us, with whole 576-byte runs 6.7 us (as
// fast as a linear sweep) but then nothing overlaps the decode.  USB = 1 serves short K ranges.
// Units are parked in a wave-private LDS buffer; LDS operations of one wave execute in order, so
// park -> fragment reads -> next park need no synchronisation.
#ifndef SK2_DEPTH
#define SK2_DEPTH 1
#endif
template <int C, int DT, int MB, int USB>
// (one activation row: held to 128 registers so that four workgroups fit a CU -- down 21.8 -> 19.6 us, lm_head
// 112 -> 107 us; q5_k would spill and keeps its 144)
__global__ __launch_bounds__(SK_THREADS, (MB == 1 && C != KQ_Q5_K) ? 4 : 2) void skinny2_kernel(SkArgs a) {
  using G = SkGeom<C>;
  constexpr int R = MB < 4 ? MB : 4;
  constexpr int NU = 4 / USB;                                  // units per wave and chunk (kch <= 16)
  constexpr int UPIECES = SK_MAXROWS * USB * G::PP;            // pieces of a unit
  constexpr int UP = (UPIECES + 63) / 64;                      // pieces per lane and unit
  constexpr int WROW = USB * G::LBPB + (USB == 2 ? 16 : 0);    // LDS row stride: an odd number of 16-byte pieces
  constexpr int WBUF = SK_MAXROWS * WROW + 128;                // wave buffer (+ 64 d values of q6_k)
  constexpr int XK = MB <= 4 ? 2 : 1;
  constexpr int XG = MB * XK;
  constexpr int DEPTH = SK2_DEPTH;                             // units in flight per wave

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int M = a.M, N = a.N, K = a.K, rows_per_tile = a.rows_per_tile, kch = a.kch;
  const int kchunk = kch * 256;
  // layout: xs f16 [MB][kch*256] | xsum f32 [kch*16][MB] | red | scratch | wave buffers
  _Float16* xs = reinterpret_cast<_Float16*>(smem);
  float* xsum = reinterpret_cast<float*>(smem + (size_t)MB * kchunk * 2);
  float* red = xsum + kch * 16 * MB;
  float* scratch = red + SK_WAVES * R * 64;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint8_t* wbuf = reinterpret_cast<uint8_t*>(scratch + 16) + wave * WBUF;
  uint16_t* dq = reinterpret_cast<uint16_t*>(wbuf + SK_MAXROWS * WROW);  // [row][USB]

  const int n_in = lane & 31, kg = lane >> 5;
  const int nsb = K >> 8;
  const size_t row_bytes = (size_t)nsb * G::BPB;
  const int row0 = blockIdx.x * rows_per_tile;
  const int nrows = (N - row0 < rows_per_tile) ? (N - row0) : rows_per_tile;
  const uint8_t* wtile = a.w + (size_t)row0 * row_bytes;
  const uint16_t* x16 = static_cast<const uint16_t*>(a.x);
  const int crow = n_in < nrows ? n_in : 0;

  float acc[R];
#pragma unroll
  for (int r = 0; r < R; r++) acc[r] = 0.f;

  // piece map of a unit: piece i = lane + 64 t -> (row, superblock of the unit, piece of the block)
  uint32_t goff[UP], loff[UP];
  StaticFor<UP>::run([&](auto t) {
    constexpr int T = decltype(t)::value;
    const int i = lane + 64 * T, r = i / (USB * G::PP), q = i % (USB * G::PP), sbl = q / G::PP, pc = q % G::PP;
    goff[T] = r < nrows ? (uint32_t)r * (uint32_t)row_bytes + sbl * G::BPB + 16 * pc : 0;  // spare slots re-read the tile start
    loff[T] = (uint32_t)r * WROW + sbl * G::LBPB + 16 * pc;
  });
  // side channel (tail piece / d): lane -> (row lane / USB, superblock lane % USB)
  const int s_row = lane / USB, s_sbl = lane % USB;
  const bool side_ok = s_row < nrows && lane < SK_MAXROWS * USB;
  const uint8_t* side_src = wtile + (side_ok ? (size_t)s_row * row_bytes + s_sbl * G::BPB : 0);

  const int sb_begin = a.ksplit > 1 ? (int)blockIdx.z * a.sb_per_split : 0;
  const int sb_end = a.ksplit > 1 ? (sb_begin + a.sb_per_split < nsb ? sb_begin + a.sb_per_split : nsb) : nsb;
  for (int sb0 = sb_begin; sb0 < sb_end; sb0 += kch) {
    const int sbn = (sb_end - sb0 < kch) ? (sb_end - sb0) : kch;
    const int kc = sbn << 8, k0 = sb0 << 8;
    // this wave's superblocks of the chunk: USB = 2 -> a run of 2 nu adjacent ones, USB = 1 -> wave, wave + 4, ...
    const int nu = USB == 2 ? (sbn + 7) >> 3 : NU;
    auto unit_first = [&](int u) { return USB == 2 ? (wave * nu + u) * 2 : 4 * u + wave; };

    // ---- activation loads first
    const int gpr = kc >> 3;
    u32x4 xreg[XG];
    StaticFor<XG>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      int m = T / XK;
      m = m < M ? m : M - 1;
      int kgi = tid + (T % XK) * SK_THREADS;
      kgi = kgi < gpr ? kgi : 0;
      xreg[T] = *reinterpret_cast<const u32x4*>(x16 + (size_t)m * K + k0 + 8 * kgi);
    });

    // ---- this wave's weight stream, DEPTH units in flight
    u32x4 wreg[DEPTH * UP], treg[DEPTH];
    uint16_t dreg[DEPTH];
    auto issue = [&](auto uu) {
      constexpr int u = decltype(uu)::value;
      const int sb = unit_first(u);
      const bool live = u < nu && sb < sbn;  // wave-uniform
      // (a unit whose second superblock lies past the chunk reads the following superblock or row:
      // the bytes exist unless this is the matrix end, see the launcher)
      const size_t sboff = (size_t)(sb0 + (live ? sb : 0)) * G::BPB;
      StaticFor<UP>::run([&](auto t) {
        constexpr int T = decltype(t)::value;
        wreg[(u % DEPTH) * UP + T] = *reinterpret_cast<const typename G::piece_t*>(wtile + sboff + goff[T]);
      });
      if constexpr (G::SIDE_D) dreg[u % DEPTH] = *reinterpret_cast<const uint16_t*>(side_src + sboff + 208);
      if constexpr (G::TAIL) treg[u % DEPTH] = *reinterpret_cast<const u32x4_a2*>(side_src + sboff + (G::BPB - 16));
    };
    StaticFor<DEPTH>::run([&](auto uu) { issue(uu); });

    // ---- activations -> f16 in LDS (+ sums)
    if (sb0 > sb_begin) lds_barrier();
    float xscale = 1.0f, inv = 1.0f;
    if constexpr (DT == KQ_BF16) {
      float amax = 0.f;
      StaticFor<XG>::run([&](auto t) {
        const u32x4 v = xreg[decltype(t)::value];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] << 16)));
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] & 0xffff0000u)));
        }
      });
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
      if (lane == 0) scratch[wave] = amax;
      lds_barrier();
      amax = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
      const uint32_t eb = (__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff;
      if (eb != 0 && eb != 0xff) {
        int e = (int)eb - 127 - 14;
        if (e < -100) e = -100;
        xscale = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
        inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
      }
    }
    StaticFor<XG>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      constexpr int m = T / XK;
      const int kgi = tid + (T % XK) * SK_THREADS;
      if (kgi < gpr) {
        const int kk = kgi << 3;
        const u32x4 v = xreg[T];
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
        const f16x8 v8 = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
        *reinterpret_cast<f16x8*>(xs + (size_t)m * kchunk + kk) = v8;
        if constexpr (G::XSUM != 0) {
          float sum = 0.f;
#pragma unroll
          for (int e = 0; e < 8; e++) sum += (float)h[e];
          sum += __shfl_xor(sum, 1);
          if constexpr (G::XSUM == 32) {
            sum += __shfl_xor(sum, 2);
            if ((tid & 3) == 0) xsum[(kk >> 5) * MB + m] = sum;
          } else {
            if ((tid & 1) == 0) xsum[(kk >> 4) * MB + m] = sum;
          }
        }
      }
    });
    lds_barrier();  // the chunk's activations are visible to every wave; from here on waves run free

    const _Float16* xs_lane = xs + (size_t)(n_in & (MB - 1)) * kchunk + G::KGOFF * kg;
    const float* xsum_lane = xsum + (MB == 8 ? 4 * kg : 0);
    const uint8_t* wt_lane = wbuf + crow * WROW;
    StaticFor<NU>::run([&](auto uu) {
      constexpr int u = decltype(uu)::value;
      const int sbf = unit_first(u);
      const bool live = u < nu && sbf < sbn;
      if (live) {
        StaticFor<UP>::run([&](auto t) {
          constexpr int T = decltype(t)::value;
          if (lane + 64 * T < UPIECES) *reinterpret_cast<u32x4*>(wbuf + loff[T]) = wreg[(u % DEPTH) * UP + T];
        });
        if constexpr (G::SIDE_D) {
          if (lane < SK_MAXROWS * USB) dq[lane] = dreg[u % DEPTH];
        }
        if constexpr (G::TAIL) {
          if (lane < SK_MAXROWS * USB)
            *reinterpret_cast<u32x4*>(wbuf + s_row * WROW + s_sbl * G::LBPB + 16 * G::PP) = treg[u % DEPTH];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      if constexpr (u + DEPTH < NU) issue(std::integral_constant<int, u + DEPTH>{});
      if (live) {
#pragma unroll
        for (int q = 0; q < USB; q++) {
          const int sb = sbf + q;
          if (sb < sbn) {
            const uint8_t* bl = wt_lane + q * G::LBPB;
            if constexpr (C == KQ_Q4_K || C == KQ_Q5_K) {
              q45k_superblock<C, R, MB>(bl, kg, xscale, xs_lane + 256 * sb, xsum_lane + 8 * MB * sb, acc);
            } else if constexpr (C == KQ_Q2_K) {
              q2k_superblock<R, MB>(bl, kg, xscale, xs_lane + 256 * sb, xsum_lane + 16 * MB * sb, acc);
            } else if constexpr (C == KQ_Q3_K) {
              q3k_superblock<R, MB>(bl, kg, xscale, xs_lane + 256 * sb, xsum_lane + 16 * MB * sb, acc);
            } else {
              const float dx = kq::h2f(dq[crow * USB + q]) * xscale;
              q6k_superblock<R>(bl, kg, dx, xs_lane + 256 * sb, acc);
            }
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
    });
  }

  // ---- cross-wave reduction and store
#pragma unroll
  for (int r = 0; r < R; r++) red[(wave * R + r) * 64 + lane] = acc[r];
  lds_barrier();
  const size_t plane = (size_t)M * N;
  for (int o = tid; o < R * 64; o += SK_THREADS) {
    const int r = o >> 6, l = o & 63;
    const int m = 4 * (l >> 5) + r, n = l & 31;
    if (m >= M || n >= nrows) continue;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < SK_WAVES; wv++) v += red[(wv * R + r) * 64 + l];
    if (a.ksplit > 1) {
      a.partial[blockIdx.z * plane + (size_t)m * N + row0 + n] = v;
    } else {
      uint16_t* yo = static_cast<uint16_t*>(a.y) + (size_t)m * N + row0 + n;
      *yo = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
    }
  }
}

// ------------------------------------------------------------------ diagonal variant (dense calls, K % 1024 == 0)
// The 32 columns of the MFMA are 8 weight rows x 4 ADJACENT superblocks instead of 32 rows x 1
// superblock: lane l serves row l % 8 and superblock (l % 32) / 8 of the wave's current group of
// four, and the 32 rows of the A operand are (superblock of the group, activation row), so the
// useful results sit on the block diagonal (D rows 8 q + m for the columns of superblock q; the rest
// of the MFMA is idle arithmetic on matrix cores that have nothing else to do).  What it buys:
//   * a wave's unit of weight traffic is 8 rows x 576 contiguous bytes (q4_k) instead of 32 rows x
//     144: reading the 33 MB gate/up matrix with nothing but that pattern takes 6.7 us, as fast as a
//     linear sweep, against 8.2 us for 144-byte runs (fewer cache lines touched per load instruction);
//   * a wave owns its 8 rows for all of K, so there is no cross-wave reduction; the four
//     superblock partials of a row are summed with two shuffles at the end.
#ifndef SK3_DEPTH
#define SK3_DEPTH 1
#endif
template <int C, int DT, int MB>
__global__ __launch_bounds__(SK_THREADS, 2) void skinny3_kernel(SkArgs a) {
  using G = SkGeom<C>;
  constexpr int R = MB < 4 ? MB : 4;
  constexpr int NU = 4;                                        // units (groups of 4 superblocks) per chunk
  constexpr int UPIECES = 8 * 4 * G::PP;                       // pieces of a unit: 8 rows x 4 superblocks
  constexpr int UP = (UPIECES + 63) / 64;
  constexpr int WROW = 4 * G::LBPB + 16;                       // LDS row stride: an odd number of 16-byte pieces
  constexpr int WBUF = 8 * WROW + 64;                          // wave buffer (+ 32 d values of q6_k)
  constexpr int XK = MB <= 4 ? 2 : 1;
  constexpr int XG = MB * XK;
  constexpr int D3 = SK3_DEPTH;                                // units in flight per wave
  constexpr int XSB = 256 + 32;  // f16 per superblock of activations in LDS: the four superblocks a wave reads
                                 // together start 64 bytes apart modulo the bank window

  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const int M = a.M, N = a.N, K = a.K, kch = a.kch;
  const int kchunk = kch * XSB + 8;  // row stride: rows start 16 bytes apart modulo the bank window
  // layout: xs f16 [MB][kchunk] | xsum f32 [kch*16][MB] | scratch | wave buffers
  _Float16* xs = reinterpret_cast<_Float16*>(smem);
  float* xsum = reinterpret_cast<float*>(smem + (size_t)MB * kchunk * 2);
  float* scratch = xsum + kch * 16 * MB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  uint8_t* wbuf = reinterpret_cast<uint8_t*>(scratch + 16) + wave * WBUF;
  uint16_t* dq = reinterpret_cast<uint16_t*>(wbuf + 8 * WROW);  // [q][row]

  const int n_in = lane & 31, kg = lane >> 5;
  const int r8 = n_in & 7, q4 = n_in >> 3;  // this lane's MFMA column: row r8 of the wave, superblock q4 of the group
  const int nsb = K >> 8;
  const size_t row_bytes = (size_t)nsb * G::BPB;
  const int row0 = blockIdx.x * 32 + 8 * wave;  // first row of this wave
  int nrows = N - row0;
  nrows = nrows < 0 ? 0 : (nrows > 8 ? 8 : nrows);
  const uint8_t* wtile = a.w + (size_t)(nrows > 0 ? row0 : 0) * row_bytes;
  const uint16_t* x16 = static_cast<const uint16_t*>(a.x);
  const int crow = r8 < nrows ? r8 : 0;

  float acc[R];
#pragma unroll
  for (int r = 0; r < R; r++) acc[r] = 0.f;

  // piece map of a unit: piece i = lane + 64 t -> (row, superblock of the group, piece of the block)
  uint32_t goff[UP], loff[UP];
  StaticFor<UP>::run([&](auto t) {
    constexpr int T = decltype(t)::value;
    const int i = lane + 64 * T, r = i / (4 * G::PP), qq = i % (4 * G::PP), sbl = qq / G::PP, pc = qq % G::PP;
    goff[T] = (r < nrows && i < UPIECES) ? (uint32_t)r * (uint32_t)row_bytes + sbl * G::BPB + 16 * pc : 0;
    loff[T] = (uint32_t)r * WROW + sbl * G::LBPB + 16 * pc;
  });
  // side channel (tail piece / d): lane < 32 -> its own MFMA column (row r8, superblock q4)
  const bool side_ok = lane < 32 && r8 < nrows;
  const uint8_t* side_src = wtile + (side_ok ? (size_t)r8 * row_bytes + q4 * G::BPB : 0);

  const int sb_begin = a.ksplit > 1 ? (int)blockIdx.z * a.sb_per_split : 0;
  const int sb_end = a.ksplit > 1 ? (sb_begin + a.sb_per_split < nsb ? sb_begin + a.sb_per_split : nsb) : nsb;
  for (int sb0 = sb_begin; sb0 < sb_end; sb0 += kch) {
    const int sbn = (sb_end - sb0 < kch) ? (sb_end - sb0) : kch;  // a multiple of 4
    const int kc = sbn << 8, k0 = sb0 << 8;

    // ---- activation loads first
    const int gpr = kc >> 3;
    u32x4 xreg[XG];
    StaticFor<XG>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      int m = T / XK;
      m = m < M ? m : M - 1;
      int kgi = tid + (T % XK) * SK_THREADS;
      kgi = kgi < gpr ? kgi : 0;
      xreg[T] = *reinterpret_cast<const u32x4*>(x16 + (size_t)m * K + k0 + 8 * kgi);
    });

    // ---- this wave's weight stream: unit u = superblocks [4 u, 4 u + 4) of its 8 rows, one unit in flight
    u32x4 wreg[D3 * UP], treg[D3];
    uint16_t dreg[D3];
    auto issue = [&](auto uu) {
      constexpr int u = decltype(uu)::value;
      const bool live = 4 * u < sbn;  // uniform
      const size_t sboff = (size_t)(sb0 + (live ? 4 * u : 0)) * G::BPB;
      StaticFor<UP>::run([&](auto t) {
        constexpr int T = decltype(t)::value;
        wreg[(u % D3) * UP + T] = *reinterpret_cast<const typename G::piece_t*>(wtile + sboff + goff[T]);
      });
      if constexpr (G::SIDE_D) dreg[u % D3] = *reinterpret_cast<const uint16_t*>(side_src + sboff + 208);
      if constexpr (G::TAIL) treg[u % D3] = *reinterpret_cast<const u32x4_a2*>(side_src + sboff + (G::BPB - 16));
    };
    StaticFor<D3>::run([&](auto uu) { issue(uu); });

    // ---- activations -> f16 in LDS (+ sums)
    if (sb0 > sb_begin) lds_barrier();
    float xscale = 1.0f, inv = 1.0f;
    if constexpr (DT == KQ_BF16) {
      float amax = 0.f;
      StaticFor<XG>::run([&](auto t) {
        const u32x4 v = xreg[decltype(t)::value];
#pragma unroll
        for (int e = 0; e < 4; e++) {
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] << 16)));
          amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, v[e] & 0xffff0000u)));
        }
      });
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
      if (lane == 0) scratch[wave] = amax;
      lds_barrier();
      amax = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
      const uint32_t eb = (__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff;
      if (eb != 0 && eb != 0xff) {
        int e = (int)eb - 127 - 14;
        if (e < -100) e = -100;
        xscale = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
        inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
      }
    }
    StaticFor<XG>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      constexpr int m = T / XK;
      const int kgi = tid + (T % XK) * SK_THREADS;
      if (kgi < gpr) {
        const int kk = kgi << 3;
        const u32x4 v = xreg[T];
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
        const f16x8 v8 = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
        *reinterpret_cast<f16x8*>(xs + (size_t)m * kchunk + (kk >> 8) * XSB + (kk & 255)) = v8;
        if constexpr (G::XSUM != 0) {
          float sum = 0.f;
#pragma unroll
          for (int e = 0; e < 8; e++) sum += (float)h[e];
          sum += __shfl_xor(sum, 1);
          if constexpr (G::XSUM == 32) {
            sum += __shfl_xor(sum, 2);
            if ((tid & 3) == 0) xsum[(kk >> 5) * MB + m] = sum;
          } else {
            if ((tid & 1) == 0) xsum[(kk >> 4) * MB + m] = sum;
          }
        }
      }
    });
    lds_barrier();  // the chunk's activations are visible to every wave; from here on waves run free

    // A operand: MFMA row l % 32 = (superblock q of the group, activation row): rows beyond MB alias real ones
    const _Float16* xs_lane = xs + (size_t)(r8 & (MB - 1)) * kchunk + XSB * q4 + G::KGOFF * kg;
    const float* xsum_lane = xsum + (size_t)(G::XSUM == 16 ? 16 : 8) * MB * q4 + (MB == 8 ? 4 * kg : 0);
    const uint8_t* bl = wbuf + crow * WROW + q4 * G::LBPB;
    StaticFor<NU>::run([&](auto uu) {
      constexpr int u = decltype(uu)::value;
      if (4 * u >= sbn) return;  // uniform
      StaticFor<UP>::run([&](auto t) {
        constexpr int T = decltype(t)::value;
        if (lane + 64 * T < UPIECES) *reinterpret_cast<u32x4*>(wbuf + loff[T]) = wreg[(u % D3) * UP + T];
      });
      if constexpr (G::SIDE_D) {
        if (lane < 32) dq[lane] = dreg[u % D3];
      }
      if constexpr (G::TAIL) {
        if (lane < 32) *reinterpret_cast<u32x4*>(wbuf + r8 * WROW + q4 * G::LBPB + 16 * G::PP) = treg[u % D3];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      if constexpr (u + D3 < NU) issue(std::integral_constant<int, u + D3>{});
      constexpr int sb = 4 * u;  // superblock of q4 = 0 within the chunk
      if constexpr (C == KQ_Q4_K || C == KQ_Q5_K) {
        q45k_superblock<C, R, MB, true>(bl, kg, xscale, xs_lane + XSB * sb, xsum_lane + 8 * MB * sb, acc, q4);
      } else if constexpr (C == KQ_Q2_K) {
        q2k_superblock<R, MB, true>(bl, kg, xscale, xs_lane + XSB * sb, xsum_lane + 16 * MB * sb, acc, q4);
      } else if constexpr (C == KQ_Q3_K) {
        q3k_superblock<R, MB, true>(bl, kg, xscale, xs_lane + XSB * sb, xsum_lane + 16 * MB * sb, acc, q4);
      } else {
        const float dx = kq::h2f(dq[n_in < 32 ? (crow + 8 * q4) : 0]) * xscale;
        q6k_superblock<R, true>(bl, kg, dx, xs_lane + XSB * sb, acc, q4);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    });
  }

  // ---- sum the four superblock partials of a row (lanes r8 + 8 q), store
  const size_t plane = (size_t)M * N;
#pragma unroll
  for (int r = 0; r < R; r++) {
    float v = acc[r];
    v += __shfl_xor(v, 8);
    v += __shfl_xor(v, 16);
    const int m = 4 * kg + r;
    if (q4 == 0 && m < M && r8 < nrows) {
      if (a.ksplit > 1) {
        a.partial[blockIdx.z * plane + (size_t)m * N + row0 + r8] = v;
      } else {
        uint16_t* yo = static_cast<uint16_t*>(a.y) + (size_t)m * N + row0 + r8;
        *yo = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
      }
    }
  }
}

template <int C>
size_t sk3_lds_bytes(int kch, int MB) {
  using G = SkGeom<C>;
  return (size_t)MB * (kch * 288 + 8) * 2 + (size_t)kch * 16 * MB * 4 + 64 + SK_WAVES * (8 * (4 * G::LBPB + 16) + 64);
}

template <int C>
size_t sk2_lds_bytes(int kch, int MB, int usb) {
  using G = SkGeom<C>;
  const int R = MB < 4 ? MB : 4;
  const size_t wrow = (size_t)usb * G::LBPB + (usb == 2 ? 16 : 0);
  return (size_t)MB * kch * 512 + (size_t)kch * 16 * MB * 4 + SK_WAVES * R * 64 * 4 + 64 +
         SK_WAVES * (SK_MAXROWS * wrow + 128);
}

template <int DT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, uint16_t* __restrict__ y,
                                                            int count, int ksplit) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  float v = 0.f;
  for (int sp = 0; sp < ksplit; sp++) v += partial[(size_t)sp * count + i];
  y[i] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
}

template <int C>
size_t sk_lds_bytes(int rows, int kch, int MB) {
  using G = SkGeom<C>;
  const int R = MB < 4 ? MB : 4;
  const size_t wstride = (size_t)kch * G::LBPB + (((kch * (G::LBPB / 16)) & 1) ? 0 : 16);
  return rows * wstride + (size_t)MB * kch * 512 + (size_t)kch * 16 * MB * 4 + SK_WAVES * R * 64 * 4 + 64 +
         16 * SK_THREADS + 32 * 16 * 2;
}

int g_sk_variant = 0;  // kq_set_skinny_variant: 0 default, 1 synchronous, 2 decoupled, 3 two-superblock units, 4 diagonal, 5 streamed

// Split-K plan of a dense call: with few row tiles the K range is cut so that about 768
// workgroups of full 32-row tiles exist; every split keeps at least one superblock per wave.
struct SkSplit {
  int ksplit, sb_per_split;
};
SkSplit sk_split_plan(int N, int K) {
  const int nsb = K >> 8, tiles = (N + SK_MAXROWS - 1) / SK_MAXROWS;
  SkSplit p{1, nsb};
  if (tiles >= 384 || nsb < 8) return p;
  int want = (768 + tiles - 1) / tiles;
  if (want > nsb / 4) want = nsb / 4;
  if (want < 2) return p;
  int per = (nsb + want - 1) / want;
  per = (per + 3) & ~3;  // whole sub-chunks
  p.ksplit = (nsb + per - 1) / per;
  p.sb_per_split = per;
  if (p.ksplit < 2) return SkSplit{1, nsb};
  return p;
}

template <int C, int DT, int MB, bool GLU>
int launch_skinny(SkArgs a, int items, void* ws, hipStream_t s) {
  // balanced row tiles: about two workgroups per CU over the whole launch, at most 32 rows each
  const int64_t total = (int64_t)a.N * items * (GLU ? 2 : 1);
  int rows = (int)((total + 511) / 512);
  rows = (rows + 7) & ~7;
  if (rows > SK_MAXROWS) rows = SK_MAXROWS;
  if (rows < 8) rows = 8;
  int splits = 1;
  a.ksplit = 1;
  // a dense call: one item, no index arrays, the result as 16-bit values at row 0 (a gathered call of one
  // item keeps the synchronous kernel, which honours the indices and the output map)
  const bool dense = items == 1 && !a.lhs && !a.rhs && !a.om.f32 && a.om.in == a.om.out && a.om.off == 0;
  if (!GLU && dense && ws) {
    const SkSplit p = sk_split_plan(a.N, a.K);
    if (p.ksplit > 1) {
      rows = SK_MAXROWS;
      splits = a.ksplit = p.ksplit;
      a.sb_per_split = p.sb_per_split;
      a.partial = static_cast<float*>(ws);
    }
  }
  const int half = GLU ? rows / 2 : rows;
  const int tiles = (a.N + half - 1) / half;
  int kch = splits > 1 ? a.sb_per_split : a.K >> 8;
  if (kch > 16) kch = 16;            // four sub-chunks of four superblocks
  if (kch * MB > 64) kch = 64 / MB;  // keep the f16 activations of a chunk within 32 KiB
  if constexpr (!GLU) {
    // dense call: decoupled-wave variant (measured 3 - 25 % faster than the synchronous kernel on every
    // decode shape of the sweep)
    if (dense && g_sk_variant != 1) {
      // Diagonal variant (a wave owns 8 rows x 4 adjacent superblocks, no cross-wave reduction): measured
      // 4 - 10 % faster at 5 - 8 activation rows and level or slightly slower below, so it is the default
      // only there; kq_set_skinny_variant(4) selects it wherever the shape allows.
      const bool diag_shape = ((a.K >> 8) & 3) == 0 && (kch & 3) == 0 && (splits == 1 || (a.sb_per_split & 3) == 0);
      if (diag_shape && (g_sk_variant == 4 || (g_sk_variant == 0 && MB == 8))) {
        // 32-row tiles always (8 rows per wave)
        const int tiles3 = (a.N + 31) / 32;
        const size_t lds3 = sk3_lds_bytes<C>(kch, MB);
        a.rows_per_tile = 32;
        a.kch = kch;
        KQ_SET_MAX_LDS_ONCE((skinny3_kernel<C, DT, MB>), 120 * 1024);
        hipLaunchKernelGGL((skinny3_kernel<C, DT, MB>), dim3(tiles3, 1, splits), dim3(SK_THREADS), lds3, s, a);
        KQ_HIP_CHECK(hipGetLastError());
        if (splits > 1) {
          const int count = a.M * a.N;
          hipLaunchKernelGGL((splitk_reduce_kernel<DT>), dim3((count + 255) / 256), dim3(256), 0, s, a.partial,
                             static_cast<uint16_t*>(a.y), count, splits);
          KQ_HIP_CHECK(hipGetLastError());
        }
        return KQ_OK;
      }
      // Units of two adjacent superblocks read HBM in a friendlier pattern but measured 15 - 60 % slower
      // end to end (two superblocks of decode per unit leave too little overlap), so they are only
      // selectable through kq_set_skinny_variant(3).  Such a unit may read one superblock past an
      // odd-length K range, i.e. into the next row: fine except at the very end of the matrix, so odd
      // superblock counts always keep single-superblock units.
      const bool two = g_sk_variant == 3 && kch >= 8 && ((a.K >> 8) & 1) == 0 &&
                       (splits == 1 || (a.sb_per_split & 1) == 0);
      const size_t lds2 = sk2_lds_bytes<C>(kch, MB, two ? 2 : 1);
      a.rows_per_tile = rows;
      a.kch = kch;
      KQ_SET_MAX_LDS_ONCE((skinny2_kernel<C, DT, MB, 1>), 120 * 1024);
      KQ_SET_MAX_LDS_ONCE((skinny2_kernel<C, DT, MB, 2>), 120 * 1024);
      if (two)
        hipLaunchKernelGGL((skinny2_kernel<C, DT, MB, 2>), dim3(tiles, 1, splits), dim3(SK_THREADS), lds2, s, a);
      else
        hipLaunchKernelGGL((skinny2_kernel<C, DT, MB, 1>), dim3(tiles, 1, splits), dim3(SK_THREADS), lds2, s, a);
      KQ_HIP_CHECK(hipGetLastError());
      if (splits > 1) {
        const int count = a.M * a.N;
        hipLaunchKernelGGL((splitk_reduce_kernel<DT>), dim3((count + 255) / 256), dim3(256), 0, s, a.partial,
                           static_cast<uint16_t*>(a.y), count, splits);
        KQ_HIP_CHECK(hipGetLastError());
      }
      return KQ_OK;
    }
  }
  while (kch > 1 && sk_lds_bytes<C>(rows, kch, MB) > 76 * 1024) kch >>= 1;  // two workgroups per CU must fit in 160 KiB
  const size_t lds = sk_lds_bytes<C>(rows, kch, MB);
  a.rows_per_tile = rows;
  a.kch = kch;
  auto kern = skinny_kernel<C, DT, MB, GLU>;
  KQ_SET_MAX_LDS_ONCE((kern), 120 * 1024);
  hipLaunchKernelGGL(kern, dim3(tiles, items, splits), dim3(SK_THREADS), lds, s, a);
  KQ_HIP_CHECK(hipGetLastError());
  if (splits > 1) {
    const int count = a.M * a.N;
    hipLaunchKernelGGL((splitk_reduce_kernel<DT>), dim3((count + 255) / 256), dim3(256), 0, s, a.partial,
                       static_cast<uint16_t*>(a.y), count, splits);
    KQ_HIP_CHECK(hipGetLastError());
  }
  return KQ_OK;
}

template <int C, int DT, bool GLU>
int launch_skinny_m(const SkArgs& a, int items, void* ws, hipStream_t s) {
  if (a.M == 1) return launch_skinny<C, DT, 1, GLU>(a, items, ws, s);
  if constexpr (GLU) {
    return KQ_ERR_UNSUPPORTED;
  } else {
    if (a.M == 2) return launch_skinny<C, DT, 2, false>(a, items, ws, s);
    if (a.M <= 4) return launch_skinny<C, DT, 4, false>(a, items, ws, s);
    return launch_skinny<C, DT, 8, false>(a, items, ws, s);
  }
}

template <bool GLU>
int launch_skinny_any(const SkArgs& a, int items, int codec, int dtype, void* ws, hipStream_t s) {
  if (codec == KQ_Q4_K)
    return dtype == KQ_F16 ? launch_skinny_m<KQ_Q4_K, KQ_F16, GLU>(a, items, ws, s)
                           : launch_skinny_m<KQ_Q4_K, KQ_BF16, GLU>(a, items, ws, s);
  if (codec == KQ_Q5_K)
    return dtype == KQ_F16 ? launch_skinny_m<KQ_Q5_K, KQ_F16, GLU>(a, items, ws, s)
                           : launch_skinny_m<KQ_Q5_K, KQ_BF16, GLU>(a, items, ws, s);
  if (codec == KQ_Q2_K)
    return dtype == KQ_F16 ? launch_skinny_m<KQ_Q2_K, KQ_F16, GLU>(a, items, ws, s)
                           : launch_skinny_m<KQ_Q2_K, KQ_BF16, GLU>(a, items, ws, s);
  if (codec == KQ_Q3_K)
    return dtype == KQ_F16 ? launch_skinny_m<KQ_Q3_K, KQ_F16, GLU>(a, items, ws, s)
                           : launch_skinny_m<KQ_Q3_K, KQ_BF16, GLU>(a, items, ws, s);
  return dtype == KQ_F16 ? launch_skinny_m<KQ_Q6_K, KQ_F16, GLU>(a, items, ws, s)
                         : launch_skinny_m<KQ_Q6_K, KQ_BF16, GLU>(a, items, ws, s);
}

bool sk_codec_ok(int codec) {
  return codec == KQ_Q2_K || codec == KQ_Q3_K || codec == KQ_Q4_K || codec == KQ_Q5_K || codec == KQ_Q6_K;
}
// q4_k / q5_k pieces are fetched with aligned 16-byte loads; the other blocks are 2-byte multiples
uintptr_t sk_wire_align_mask(int codec) { return (codec == KQ_Q4_K || codec == KQ_Q5_K) ? 15 : 1; }

bool sk_shape_ok(int M, int K, int codec, const void* x, const void* w, const void* w2) {
  if (!sk_codec_ok(codec) || M < 1 || M > SK_MAXM || (K & 255) || K == 0) return false;
  const uintptr_t wmask = sk_wire_align_mask(codec);
  if ((reinterpret_cast<uintptr_t>(w) & wmask) || (reinterpret_cast<uintptr_t>(w2) & wmask)) return false;
  return (reinterpret_cast<uintptr_t>(x) & 15) == 0;
}

}  // namespace

size_t kq_qmm_tuned_workspace_bytes(int M, int N, int K, int codec) {
  if (M < 1 || M > SK_MAXM || K == 0) return 0;
  const size_t st = kq_stream_workspace_bytes(M, N, K, codec);  // also covers codecs only the streamed kernel takes
  if (!sk_codec_ok(codec) || (K & 255)) return st;
  const SkSplit p = sk_split_plan(N, K);
  const size_t own = p.ksplit > 1 ? (size_t)p.ksplit * M * N * sizeof(float) : 0;
  return own > st ? own : st;
}

int kq_launch_qmm_tuned(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                        size_t ws_bytes, hipStream_t s) {
  // up to eight activation rows of the K-quants, iq4_xs, iq3_s, iq2_xxs: the streamed kernel (variant 5), unless a
  // test pins another
  if (g_sk_variant == 0 || g_sk_variant == 5) {
    const int rc = kq_launch_qmm_stream(x, w, y, M, N, K, codec, dtype, ws, ws_bytes, s);
    if (rc != KQ_ERR_UNSUPPORTED) return rc;
  }
  if (!sk_shape_ok(M, K, codec, x, w, nullptr)) return KQ_ERR_UNSUPPORTED;
  SkArgs a{};
  a.x = x;
  a.w = w;
  a.y = y;
  a.M = M;
  a.N = N;
  a.K = K;
  a.x_div = 1;
  const SkSplit own = sk_split_plan(N, K);
  if (ws_bytes < (own.ksplit > 1 ? (size_t)own.ksplit * M * N * sizeof(float) : 0) || (reinterpret_cast<uintptr_t>(ws) & 3)) ws = nullptr;
  return launch_skinny_any<false>(a, 1, codec, dtype, ws, s);
}

int kq_launch_gather_tuned(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* lhs,
                           const uint32_t* rhs, void* out, int B, int M, int N, int K, int x_div,
                           int64_t x_batch_stride, int64_t w_expert_stride, int glu, int act, float limit, int codec,
                           int dtype, int E, KqOutMap om, hipStream_t s) {
  // one activation row per entry (MoE decode: entries in order of x; gather_qmm: any row index): the streamed
  // kernel, which also takes the codebook codecs it has units for
  if (M == 1 && rhs && (lhs || x_batch_stride == K) && g_sk_variant == 0 && B >= 1 &&
      (!glu || act != KQ_ACT_SWIGLU_CLAMP)) {
    const int rcs = kq_launch_gather_stream(x, w, glu ? w2 : nullptr, lhs, rhs, out, B, N, K, x_div, x_batch_stride,
                                            w_expert_stride, act, limit, 1.0f, nullptr, nullptr, codec, dtype, E, om, s);
    if (rcs != KQ_ERR_UNSUPPORTED) return rcs;
  }
  if (!sk_shape_ok(M, K, codec, x, w, w2) || B < 1 || B > 65535) return KQ_ERR_UNSUPPORTED;
  if (glu && (M != 1 || act == KQ_ACT_SWIGLU_CLAMP)) return KQ_ERR_UNSUPPORTED;
  const int64_t wmask = (int64_t)sk_wire_align_mask(codec);
  if ((w_expert_stride & wmask) || ((x_batch_stride * 2) & 15)) return KQ_ERR_UNSUPPORTED;
  SkArgs a{};
  a.x = x;
  a.w = w;
  a.w2 = w2;
  a.y = out;
  a.lhs = lhs;
  a.rhs = rhs;
  a.M = M;
  a.N = N;
  a.K = K;
  a.x_div = x_div < 1 ? 1 : x_div;
  a.act = act;
  a.x_batch_stride = x_batch_stride;
  a.w_expert_stride = w_expert_stride;
  a.limit = limit;
  a.om = om;
  a.E = E;
  return glu ? launch_skinny_any<true>(a, B, codec, dtype, nullptr, s)
             : launch_skinny_any<false>(a, B, codec, dtype, nullptr, s);
}

extern "C" void kq_set_skinny_variant(int v) { g_sk_variant = v; }
