// Prefill GEMM for the codebook codecs (iq2_xxs, iq2_xs, iq2_s, iq3_xxs, iq3_s, iq1_s, iq1_m): y[M,N] = x[M,K] . W^T
// on the f16 matrix cores, 256-row (or 128-row) wave tiles, ONE exact f16 term per weight.
//
// A weight of these codecs is d (f16, one per superblock of 256) times a sub-block factor times a codebook value
// times a sign; everything but d is an integer multiple of 1/8 below 512 (what the reference-order decoder gives with
// d taken as 1), i.e. an f16 number.  Those go into the MFMA as they are; d goes into the unit of the running sums
// exactly as in kq_gemm3.hip: entering a superblock with scale d, S is multiplied by r / d and r becomes d (one
// multiply per accumulator and superblock; a superblock with d = 0 keeps the unit and feeds zeros).  The f16 values
// are made in packed f16 arithmetic from the block's fields (kq::iq_group / kq::iq1_group, the field readers of the
// shared decoder): codebook byte m as the f16 number 1024 + m by its bit pattern, one fused (1024 + m) s - 1024 s
// with the group's scale s, which is exact, signs as XOR masks from a 256-entry table in LDS.
//
// Workgroup = 8 waves = 256 (MT = 8) or 128 (MT = 4) activation rows x 256 weight rows, one per CU.  K steps of 64,
// two activation stages filled by the whole workgroup with direct-to-LDS loads (one barrier per step).  Every wave
// streams the wire bytes of its own 32 weight rows, whole superblocks, into two private stages with 4-byte
// direct-to-LDS loads (blocks are 50 ... 110 bytes long and 2-byte aligned; a block's last dword may reach two bytes
// past it, into the next block - except at the very end of the matrix, where the one lane that would read past the
// buffer loads two bytes earlier and shifts the dword once it has landed).  The codec's codebook lies in LDS.
// Block layouts as the reference decodes them: src/kquant_cpu_decode.cpp:467-735 (through kq_decode.h); the M > 8
// matmul this serves: src/kquant_cpu_decode.cpp:1209-1359.
#include "kq_decode.h"
#include "kq_dma.h"
#include "kq_mma.h"

namespace {

using namespace kqmma;
using namespace kqdma;

constexpr int I3_WAVES = 8, I3_BN = 256, I3_KS = 64;

template <int C>
struct I3Geom;
template <>
struct I3Geom<KQ_IQ2_XXS> {
  static constexpr int BPB = 66, TBL_OFF = KQ_GRID_IQ2XXS, TBL_BYTES = 2048;
};
template <>
struct I3Geom<KQ_IQ2_XS> {
  static constexpr int BPB = 74, TBL_OFF = KQ_GRID_IQ2XS, TBL_BYTES = 4096;
};
template <>
struct I3Geom<KQ_IQ2_S> {
  static constexpr int BPB = 82, TBL_OFF = KQ_GRID_IQ2S, TBL_BYTES = 8192;
};
template <>
struct I3Geom<KQ_IQ3_XXS> {
  static constexpr int BPB = 98, TBL_OFF = KQ_GRID_IQ3XXS, TBL_BYTES = 1024;
};
template <>
struct I3Geom<KQ_IQ3_S> {
  static constexpr int BPB = 110, TBL_OFF = KQ_GRID_IQ3S, TBL_BYTES = 2048;
};
template <>
struct I3Geom<KQ_IQ1_S> {
  static constexpr int BPB = 50, TBL_OFF = KQ_GRID_IQ1S, TBL_BYTES = 16384;
};
template <>
struct I3Geom<KQ_IQ1_M> {
  static constexpr int BPB = 56, TBL_OFF = KQ_GRID_IQ1S, TBL_BYTES = 16384;
};

template <int C>
constexpr int i3_dpr() { return (I3Geom<C>::BPB + 3) / 4; }  // dwords that hold a block
template <int C>
constexpr int i3_dpl() { return i3_dpr<C>() | 1; }           // dwords of a row in LDS: odd, so that the 32 rows' fields lie in 32 banks
template <int C>
constexpr int i3_stage() { return 32 * 4 * i3_dpl<C>(); }    // bytes of a wave's stage (32 rows)
template <int C, int MT>
constexpr int i3_lds_bytes() {
  return 2 * (32 * MT * I3_KS * 2) + I3_WAVES * 2 * i3_stage<C>() + I3Geom<C>::TBL_BYTES +
         (kq::is_sign_grid_codec(C) ? 4096 : 0);  // two activation stages, the wire stages, the codebook, the sign masks
}

// Activations of one row: xh = f16(x 2^-e) in their own order, rs = 2^e (bf16 rows scaled so that the largest
// magnitude lands in [2^14, 2^15); f16 rows pass through).
template <int DT>
__global__ __launch_bounds__(256) void i3_prepass_kernel(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
                                                         float* __restrict__ rs, int K) {
  __shared__ float red[4];
  const int m = blockIdx.x, tid = threadIdx.x, ngroups = K >> 3;
  const uint16_t* xi = x + (size_t)m * K;
  _Float16* xo = xh + (size_t)m * K;
  float inv = 1.f, scale = 1.f;
  if constexpr (DT == KQ_BF16) {
    float amax = 0.f;
    for (int g = tid; g < ngroups; g += 256) {
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
      int e = (int)eb - 127 - 14;
      if (e < -100) e = -100;
      scale = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
      inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
    }
  }
  if (tid == 0) rs[m] = scale;
  for (int g = tid; g < ngroups; g += 256) {
    const u32x4 v = *reinterpret_cast<const u32x4*>(xi + 8 * g);
    if constexpr (DT == KQ_BF16) {
      _Float16 h[8];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        h[2 * e] = (_Float16)(__builtin_bit_cast(float, v[e] << 16) * inv);
        h[2 * e + 1] = (_Float16)(__builtin_bit_cast(float, v[e] & 0xffff0000u) * inv);
      }
      *reinterpret_cast<f16x8*>(xo + 8 * g) = f16x8{h[0], h[1], h[2], h[3], h[4], h[5], h[6], h[7]};
    } else {
      *reinterpret_cast<u32x4*>(xo + 8 * g) = v;
    }
  }
}

template <int C, int DT, int MT>
__global__ __launch_bounds__(64 * I3_WAVES, 1) void iq_gemm3_kernel(const _Float16* __restrict__ xh,
                                                                   const float* __restrict__ rs,
                                                                   const uint8_t* __restrict__ w,
                                                                   const uint8_t* __restrict__ grids,
                                                                   uint16_t* __restrict__ y, int M, int N, int K,
                                                                   int mtiles, int nt0) {
  using G = I3Geom<C>;
  constexpr int BPB = G::BPB, DPR = i3_dpr<C>(), DPL = i3_dpl<C>(), STAGE = i3_stage<C>();
  constexpr int NEL = 32 * DPL, NI = (NEL + 63) / 64;  // dwords of a stage, load instructions for them
  constexpr int W_LAST = NEL - 64 * (NI - 1);
  constexpr bool OVER = (BPB & 3) != 0;                // a block's last dword reaches two bytes past it
  constexpr int TM = 32 * MT, A_STAGE = TM * I3_KS * 2, AQ = MT / 2;
  constexpr int W_OFF = 2 * A_STAGE, T_OFF = W_OFF + I3_WAVES * 2 * STAGE;
  constexpr int S_OFF = T_OFF + G::TBL_BYTES;  // the sign masks, 4 KiB
  constexpr int GPS = I3_KS / 16;   // MFMA groups per step: 4
  constexpr int SPS = 256 / I3_KS;  // steps per superblock: 4
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, kg = lane >> 5;
  const int mt = blockIdx.x % mtiles, nt = nt0 + blockIdx.x / mtiles;  // consecutive workgroups share the weight columns
  const int m0 = mt * TM, n0 = nt * I3_BN;
  const int nsb = K >> 8, nsteps = SPS * nsb;
  const uint32_t row_bytes = (uint32_t)nsb * BPB;
  const int nrows = N - n0 < I3_BN ? N - n0 : I3_BN;
  const uint32_t lds0 = lds_addr(smem);

  // ---- the codebook into LDS (every wave is past the first barrier before it is read)
  for (int bi = 64 * wave; bi < G::TBL_BYTES / 16; bi += 64 * I3_WAVES)  // 64 pieces of 16 bytes per instruction
    dma16(grids + G::TBL_OFF + (size_t)bi * 16, 16u * (uint32_t)lane, lds0 + T_OFF + (uint32_t)bi * 16);

  // ---- the sign masks of the codecs that keep 8 sign bits per group: entry e, dword i = bit 2 i of e on bit 15, bit
  // 2 i + 1 on bit 31
  if constexpr (kq::is_sign_grid_codec(C)) {
    uint32_t* st = reinterpret_cast<uint32_t*>(smem + S_OFF);
    for (int i = tid; i < 1024; i += 64 * I3_WAVES) {
      const uint32_t two = ((uint32_t)i >> 2) >> (2 * (i & 3));
      st[i] = ((two & 1u) << 15) | ((two & 2u) << 30);
    }
  }

  // ---- load maps
  // activations: load q covers rows 8 (wave + 8 q) + lane / 8, piece lane % 8 of the step; LDS piece p of row r holds
  // global piece p ^ swz(r).  Rows past M re-read the last one (never stored).
  auto swz = [](int row) { return (row >> 1) & 7; };
  uint32_t a_voff[AQ];
#pragma unroll
  for (int q = 0; q < AQ; q++) {
    const int r = 8 * (wave + 8 * q) + (lane >> 3);
    const int gr = m0 + r < M ? m0 + r : M - 1;
    a_voff[q] = (uint32_t)gr * (uint32_t)K * 2u + 16u * (uint32_t)((lane & 7) ^ swz(r));
  }
  const uint8_t* a_base = reinterpret_cast<const uint8_t*>(xh);
  // wire: dword i = 64 q + lane of a stage -> row i / DPL, dword i % DPL of its block (a row's padding dword, where
  // DPL > DPR, re-reads the block's first dword and is never looked at).  Rows past N read the tile's
  // first row (their columns are not stored) and never a block's last dword.  The last dword of the matrix's last
  // row is read two bytes early (fix = its LDS offset in a stage, shifted down once landed).
  uint32_t w_voff[NI];
  int fix = -1;
#pragma unroll
  for (int q = 0; q < NI; q++) {
    int i = 64 * q + lane;
    i = i < NEL ? i : NEL - 1;
    const int r = wave * 32 + i / DPL;
    int dw = i % DPL;
    dw = dw < DPR ? dw : 0;
    uint32_t off;
    if (r < nrows) {
      off = (uint32_t)r * row_bytes + 4u * (uint32_t)dw;
      if (OVER && dw == DPR - 1 && n0 + r == N - 1) {
        off -= 2u;
        if (64 * q + lane < NEL) fix = 4 * i;
      }
    } else {
      dw = OVER && dw == DPR - 1 ? dw - 1 : dw;
      off = 4u * (uint32_t)dw;
    }
    w_voff[q] = off;
  }
  const uint8_t* w_base = w + (size_t)n0 * row_bytes;

  auto issue_a = [&](int step) {
    const uint8_t* base = a_base + (size_t)step * (I3_KS * 2);
    const uint32_t l = lds0 + (step & 1) * A_STAGE + wave * 1024;
#pragma unroll
    for (int q = 0; q < AQ; q++) dma16(base, a_voff[q], l + q * (I3_WAVES * 1024));
  };
  const uint32_t w_lds = lds0 + W_OFF + wave * (2 * STAGE);
  uint8_t* w_smem = smem + W_OFF + wave * (2 * STAGE);
  auto issue_w = [&](int sb) {  // superblock sb of this wave's rows -> its stage sb % 2
    const uint8_t* base = w_base + (size_t)sb * BPB;
    const uint32_t l = w_lds + (sb & 1) * STAGE;
#pragma unroll
    for (int q = 0; q < NI - 1; q++) dma4(base, w_voff[q], l + q * 256);
    if (W_LAST == 64 || lane < W_LAST) dma4(base, w_voff[NI - 1], l + (NI - 1) * 256);
  };
  auto fix_tail = [&](int sb) {  // after stage sb % 2 has landed
    if constexpr (OVER) {
      if (fix >= 0) {
        uint32_t* p = reinterpret_cast<uint32_t*>(w_smem + (sb & 1) * STAGE + fix);
        *p = *p >> 16;
      }
    }
  };

  // A fragment of m-tile t, group g: lane half kg holds weights 16 g + 8 kg .. + 7 of the step
  uint32_t a_addr[GPS];
#pragma unroll
  for (int g = 0; g < GPS; g++) a_addr[g] = (uint32_t)l32 * 128u + 16u * (uint32_t)((2 * g + kg) ^ swz(l32));
  const uint8_t* tbl = smem + T_OFF - G::TBL_OFF;  // decode8 adds the codec's offset in the codebook blob

  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) acc[t] = f32x16{0};

  float r = 1.0f, ratio = 1.0f, live = 1.0f, live_n = 1.0f;
  // entering superblock sb (its stage has landed): the unit change it asks for; commit = false leaves r alone
  auto head = [&](int sb, bool commit) {
    const float d = kq::iq_block_d<C>(w_smem + (sb & 1) * STAGE + l32 * (4 * DPL));
    const float rn = d != 0.f ? d : r;  // a superblock with d = 0 keeps the unit and is fed as zeros
    ratio = r * __builtin_amdgcn_rcpf(rn);
    live_n = d != 0.f ? 1.0f : 0.0f;
    r = commit ? rn : r;
  };
  // B fragment of group g of step p of superblock sb: weights 64 p + 16 g + 8 kg .. + 7 of this lane's row
  auto decode = [&](int sb, int p, int g, float lv) -> f16x8 {
    const uint8_t* blk = w_smem + (sb & 1) * STAGE + l32 * (4 * DPL);
    if constexpr (kq::is_sign_grid_codec(C)) {
      // magnitude byte m as the f16 1024 + m (bits 0x6400 | m), then (1024 + m) * db - 1024 * db in one fused step:
      // db has at most 5 significant bits and m * db below 2048 units, so the result is m * db itself; the signs
      // are the table's masks on the f16 sign bits.  A dead superblock is fed with db = 0.
      uint32_t lo, hi, sg;
      float db;
      kq::iq_group<C, true, true>(blk, 8 * p + 2 * g + kg, tbl, lo, hi, sg, db);
      const _Float16 dh = (_Float16)(lv != 0.f ? db : 0.f);
      const f16x2 mul = {dh, dh}, sub = mul * f16x2{(_Float16)-1024.f, (_Float16)-1024.f};
      const u32x4 mask = *reinterpret_cast<const u32x4*>(smem + S_OFF + 16 * sg);
      const uint32_t pair[4] = {__builtin_amdgcn_perm(lo, 0x64646464u, 0x00050004u), __builtin_amdgcn_perm(lo, 0x64646464u, 0x00070006u),
                                __builtin_amdgcn_perm(hi, 0x64646464u, 0x00050004u), __builtin_amdgcn_perm(hi, 0x64646464u, 0x00070006u)};
      u32x4 out;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const f16x2 mag = __builtin_bit_cast(f16x2, pair[i]);
        const f16x2 val = __builtin_elementwise_fma(mag, mul, sub);
        out[i] = __builtin_bit_cast(uint32_t, val) ^ mask[i];
      }
      return __builtin_bit_cast(f16x8, out);
    } else {
      // ternary codecs: entry byte e in {-1, 0, 1} as the f16 1152 + e (bits 0x6400 | (e ^ 0x80)), then
      // (1152 + e) * dl - 1152 * dl = e * dl in one fused step (dl is an odd integer up to 15) and + dl * delta, a
      // multiple of 1/8 below 17: both exact.  A dead superblock is fed with dl = 0.
      uint32_t lo, hi;
      float dl, delta;
      kq::iq1_group<C, true, true>(blk, 8 * p + 2 * g + kg, tbl, lo, hi, dl, delta);
      lo ^= 0x80808080u;
      hi ^= 0x80808080u;
      const _Float16 dh = (_Float16)(lv != 0.f ? dl : 0.f), sh = (_Float16)(lv != 0.f ? dl * delta : 0.f);
      const f16x2 mul = {dh, dh}, sub = mul * f16x2{(_Float16)-1152.f, (_Float16)-1152.f}, shift = {sh, sh};
      const uint32_t pair[4] = {__builtin_amdgcn_perm(lo, 0x64646464u, 0x00050004u), __builtin_amdgcn_perm(lo, 0x64646464u, 0x00070006u),
                                __builtin_amdgcn_perm(hi, 0x64646464u, 0x00050004u), __builtin_amdgcn_perm(hi, 0x64646464u, 0x00070006u)};
      u32x4 out;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const f16x2 mag = __builtin_bit_cast(f16x2, pair[i]);
        const f16x2 val = __builtin_elementwise_fma(mag, mul, sub) + shift;
        out[i] = __builtin_bit_cast(uint32_t, val);
      }
      return __builtin_bit_cast(f16x8, out);
    }
  };

  // ---- prologue
  issue_a(0);
  issue_w(0);
  vmwait<0>();
  fix_tail(0);
  lds_barrier();  // the codebook is every wave's loads
  head(0, true);
  live = live_n;
  f16x8 bfr[2];
  bfr[0] = decode(0, 0, 0, live);

  // ---- main loop: step s = 4 sb + p.  The activation loads of step s + 1 are queued right after the barrier that
  // opens step s; this wave's superblock sb + 1 follows in part 0 (its stage held superblock sb - 1, last decoded in
  // part 3 of that superblock) and may stay in flight over the next barrier; it has landed by part 2.
  for (int sb = 0; sb < nsb; sb++) {
    const bool more = sb + 1 < nsb;
    StaticFor<SPS>::run([&](auto pc) {
      constexpr int p = decltype(pc)::value;
      const int step = SPS * sb + p;
      const uint8_t* a_stage = smem + (p & 1) * A_STAGE;
      if (p == 1 && more) vmwait<NI>(); else vmwait<0>();
      if constexpr (p == 2) {
        if (more) fix_tail(sb + 1);
      }
      lds_barrier();
      if (step + 1 < nsteps) issue_a(step + 1);
      if (p == 0 && more) issue_w(sb + 1);
      f16x8 afr[MT];
#pragma unroll
      for (int t = 0; t < MT; t++) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[0] + t * 4096);
      StaticFor<GPS>::run([&](auto gc) {
        constexpr int g = decltype(gc)::value;
        if constexpr (g + 1 < GPS) {
          bfr[(g + 1) & 1] = decode(sb, p, g + 1, live);
        } else if constexpr (p + 1 < SPS) {
          bfr[0] = decode(sb, p + 1, 0, live);
        } else {
          head(more ? sb + 1 : sb, more);  // past the end: a dry run on this superblock's bytes
          bfr[0] = decode(more ? sb + 1 : sb, 0, 0, live_n);
        }
#pragma unroll
        for (int t = 0; t < MT; t++) {
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[t], bfr[g & 1], acc[t], 0, 0, 0);
          if constexpr (g + 1 < GPS) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[g + 1] + t * 4096);
        }
      });
      if constexpr (p == SPS - 1) {
        live = live_n;
        if (more) {  // the running sums change unit
#pragma unroll
          for (int t = 0; t < MT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[t][i] *= ratio;
        }
      }
    });
  }

  // ---- epilogue: back to plain units, undo the per-row activation scale, round once, store
  const int n = n0 + wave * 32 + l32;
#pragma unroll
  for (int t = 0; t < MT; t++) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int m = m0 + t * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);
      if (m < M && n < N) {
        const float v = acc[t][i] * r * rs[m];
        y[(size_t)m * N + n] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
      }
    }
  }
}

template <int C, int DT, int MT>
int launch_i3(const _Float16* xh, const float* rs, const uint8_t* w, const uint8_t* grids, void* y, int M, int N, int K,
              int nt0, int ntiles, hipStream_t s) {
  if (ntiles <= 0) return KQ_OK;
  const int mtiles = (M + 32 * MT - 1) / (32 * MT);
  constexpr int lds = i3_lds_bytes<C, MT>();
  static_assert(lds <= 160 * 1024, "tile does not fit the LDS of a CU");
  auto kern = iq_gemm3_kernel<C, DT, MT>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  hipLaunchKernelGGL(kern, dim3(mtiles * ntiles), dim3(64 * I3_WAVES), lds, s, xh, rs, w, grids, static_cast<uint16_t*>(y), M,
                     N, K, mtiles, nt0);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

int i3_num_cus() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
  return n;
}

static int g_i3_force = 0;  // kq_set_gemm_tile_rows: 1024 / 1025 force one tile height for every column tile, 64 switches the kernel off

template <int C, int DT>
int launch_i3_call(const void* x, const uint8_t* w, void* y, int M, int N, int K, void* ws, int force, hipStream_t s) {
  const uint8_t* grids = kq_device_grids();
  if (!grids) return KQ_ERR_HIP;
  _Float16* xh = static_cast<_Float16*>(ws);
  float* rs = reinterpret_cast<float*>(xh + (size_t)M * K);
  hipLaunchKernelGGL((i3_prepass_kernel<DT>), dim3(M), dim3(256), 0, s, static_cast<const uint16_t*>(x), xh, rs, K);
  KQ_HIP_CHECK(hipGetLastError());
  auto tiles = [&](int nt0, int ntiles, int rows) {
    return rows == 128 ? launch_i3<C, DT, 4>(xh, rs, w, grids, y, M, N, K, nt0, ntiles, s)
                       : launch_i3<C, DT, 8>(xh, rs, w, grids, y, M, N, K, nt0, ntiles, s);
  };
  // tile heights by whole rounds of one workgroup per CU, as for the other tall-tile kernels
  const int nt256 = (N + 255) / 256, mt256 = (M + 255) / 256, mt128 = (M + 127) / 128;
  if (force) return tiles(0, nt256, force);
  const int64_t cus = i3_num_cus();
  auto rounds = [&](int64_t wgs) { return (wgs + cus - 1) / cus; };
  const int64_t c128 = rounds((int64_t)mt128 * nt256) * 119;
  const int64_t full = (int64_t)mt256 * nt256 / cus;
  const int tall = full > 0 ? (int)(full * cus / mt256) : 0;
  const int rest = nt256 - tall;
  const int64_t rest256 = rounds((int64_t)mt256 * rest) * 200, rest128 = rounds((int64_t)mt128 * rest) * 119;
  const int64_t c256 = full * 200 + (rest128 < rest256 ? rest128 : rest256);
  if (c128 < c256) return tiles(0, nt256, 128);
  const int rc = tiles(0, tall, 256);
  if (rc != KQ_OK) return rc;
  return tiles(tall, rest, rest128 < rest256 ? 128 : 256);
}

bool i3_codec(int codec) {
  return codec == KQ_IQ2_XXS || codec == KQ_IQ2_XS || codec == KQ_IQ2_S || codec == KQ_IQ3_XXS || codec == KQ_IQ3_S ||
         codec == KQ_IQ1_S || codec == KQ_IQ1_M;
}

}  // namespace

// Taken for calls of 128 rows or more whose half-height tiles fill three quarters of the CUs; smaller calls stay on
// the any-codec kernel.
bool kq_gemm3i_supported(int M, int N, int K, int codec) {
  if (!i3_codec(codec)) return false;
  if (M < 128 || N <= 0 || K < 256 || (K & 255)) return false;
  if ((int64_t)256 * (K >> 8) * 110 >= ((int64_t)1 << 32) || (int64_t)M * K * 2 >= ((int64_t)1 << 32)) return false;
  if (g_i3_force > 0) return true;  // a forced tile height takes every shape (tests reach the kernel on small matrices)
  return 4 * (int64_t)((M + 127) / 128) * ((N + 255) / 256) >= 3 * (int64_t)i3_num_cus();
}

size_t kq_gemm3i_workspace_bytes(int M, int K) { return (size_t)M * K * 2 + (size_t)M * 4 + 256; }

void kq_gemm3i_force_tile(int rows) { g_i3_force = rows == 1024 ? 256 : rows == 1025 ? 128 : rows == 64 ? -1 : 0; }

int kq_launch_gemm3i(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                     hipStream_t s) {
  if (g_i3_force < 0 || !kq_gemm3i_supported(M, N, K, codec)) return KQ_ERR_UNSUPPORTED;
  if ((reinterpret_cast<uintptr_t>(w) & 1) || (reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(ws) & 15))
    return KQ_ERR_UNSUPPORTED;
  const int force = g_i3_force;
#define KQ_I3_CASE(CODEC)                                                                                   \
  if (codec == CODEC)                                                                                        \
    return dtype == KQ_F16 ? launch_i3_call<CODEC, KQ_F16>(x, w, y, M, N, K, ws, force, s)                   \
                           : launch_i3_call<CODEC, KQ_BF16>(x, w, y, M, N, K, ws, force, s);
  KQ_I3_CASE(KQ_IQ2_XXS)
  KQ_I3_CASE(KQ_IQ2_XS)
  KQ_I3_CASE(KQ_IQ2_S)
  KQ_I3_CASE(KQ_IQ3_XXS)
  KQ_I3_CASE(KQ_IQ3_S)
  KQ_I3_CASE(KQ_IQ1_S)
  KQ_I3_CASE(KQ_IQ1_M)
#undef KQ_I3_CASE
  return KQ_ERR_UNSUPPORTED;
}
