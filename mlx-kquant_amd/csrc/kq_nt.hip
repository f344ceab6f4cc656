// transpose = false on the matrix cores: y[m, n] = sum_k x[m, k] * W[k, n], W stored as K wire rows of N weights
// (the orientation of the reference's qmm_n, src/kquant_matmul.cpp:455-527, and of its gathered form
// src/kquant_gather.cpp:470-746 with transpose = false: MLA's absorbed projections and the LoRA vjp).
//
// The reduction runs over wire ROWS, so a decoded 8-weight group (8 consecutive n of one row k) is not an MFMA
// operand by itself: an operand wants 8 consecutive k of one column.  The kernel gets there without any
// transpose: lane (c = lane % 16, h = lane / 16) decodes the SAME 8-column group c of 8 consecutive rows
// k0 + 8h ... k0 + 8h + 7; value t of those eight groups, taken over the rows, is the B operand of MFMA number t
// (v_mfma_f32_16x16x32_bf16: 32 rows of K a step), whose 16 columns are then the strided set {8c + t}.  Eight
// accumulator tiles (t = 0 ... 7) cover 128 consecutive output columns, and the eight results of a lane for one
// output row are 8 consecutive columns: one 16-byte store.
//
// Numerics: every decoded weight (f32, reference order, kq_decode.h) is split into two bf16 terms (16 mantissa
// bits), f16 activations into two exact bf16 terms, bf16 activations are used as they are; the MFMA forms exact
// products and sums in f32.
//
// Workgroup = 4 waves on one (entry, 16 or 32 activation rows, 128 columns) tile; the waves take the 32-row steps
// of K in turn and their accumulators meet in LDS.  A wave copies the 32 row pieces of its step (the wire bytes of
// the tile's columns, contiguous per row; for the 256-weight codecs the whole superblock, which two column tiles
// share) into its own LDS area with dword loads issued one step ahead, and the decoders read the bytes from there:
// decoding straight from global memory costs about 130 byte-wide loads a step.  Calls of 96 rows and more run
// gemm_nt_wide_kernel below, which decodes a step once for 128 activation rows.
#include <type_traits>

#include "kq_decode.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32_a1 __attribute__((aligned(1)));  // the hardware serves unaligned dword loads

constexpr int NT_WAVES = 4, NT_THREADS = 64 * NT_WAVES;
constexpr int NT_KSTEP = 32, NT_COLS = 128;
// Codecs whose 32-row form does not fit 256 registers (it spills up to 248 bytes per lane) take 64-row tiles on one
// wave per SIMD beyond 32 rows (q6_k 4096 x 4096, 512 rows: 292 -> 146 us); for the others the 64-row form measured
// level or slower (q8_0 93 -> 111 us).
constexpr bool nt_wide(int codec) { return codec == KQ_Q6_K; }
// Calls of this many activation rows take the kernel that decodes a step once for 128 rows
#ifndef KQ_NT_SHARED_ROWS
#define KQ_NT_SHARED_ROWS 96
#endif
constexpr int NT_SHARED_ROWS = KQ_NT_SHARED_ROWS;

struct NtArgs {
  const void* x;
  const uint8_t* w;
  void* y;
  const uint32_t* lhs;
  const uint32_t* rhs;
  int M, N, K, E;
  int64_t x_batch_stride, w_expert_stride;
  int x_vec;  // activation rows can be read 16 bytes at a time (K % 8 == 0, aligned base and stride)
  // dense calls with few tiles: grid z cuts the K steps into ksplit ranges whose f32 partial sums go to `part`
  // ([ksplit, M, N]) and are added by nt_reduce_kernel
  int ksplit, steps_per_split;
  float* part;
};

__device__ __forceinline__ uint32_t pack_hi(float a, float b) {
  // upper halves of two f32 = their bf16 truncations, a in the low half
  return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, b), __builtin_bit_cast(uint32_t, a), 0x07060302u);
}
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_rne(float a, float b) {
  // two f32 rounded to nearest-even bf16 (v_cvt_pk_bf16_f32), a in the low half
  const bf16x2 v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float trunc_bf16(float a) {
  return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, a) & 0xffff0000u);
}

template <int C>
struct NtGeom {
  static constexpr int WPB = kq_geom(C).wpb, BPB = kq_geom(C).bpb, GPB = WPB / 8;
  static constexpr bool SUPER = WPB > NT_COLS;          // two column tiles share the row piece of a superblock
  static constexpr int PCOLS = SUPER ? WPB : NT_COLS;    // columns a row piece covers
  static constexpr int PIECE = PCOLS / WPB * BPB;        // ... and its wire bytes
  static constexpr int PDW = 2 * ((PIECE + 7) / 8), STRIDE = 4 * PDW;  // rows 8-byte aligned in LDS
  static constexpr int NDW = (NT_KSTEP * PDW + 63) / 64;  // dwords a lane copies per step
  static constexpr int STAGE_BYTES = NT_WAVES * NT_KSTEP * STRIDE;
};

// MR = 16-row groups of activations per workgroup (1: up to 16 rows, 2: 32, 4: 64 rows on one wave per SIMD, for
// calls of many rows: every decoded weight then feeds four MFMAs)
template <int C, int DT, int MR>
__global__ __launch_bounds__(NT_THREADS, MR == 4 ? 1 : 2) void gemm_nt_mfma_kernel(NtArgs a, const uint8_t* __restrict__ grids) {
  using G = NtGeom<C>;
  constexpr int BPB = G::BPB, GPB = G::GPB, PDW = G::PDW, STRIDE = G::STRIDE, NDW = G::NDW;
  constexpr int RED_BYTES = 2 * 32 * MR * 64 * 4;  // two waves' accumulators; shares the space of the staging areas
  __shared__ __attribute__((aligned(16))) uint8_t lds[G::STAGE_BYTES > RED_BYTES ? G::STAGE_BYTES : RED_BYTES];
  float* red = reinterpret_cast<float*>(lds);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, h = lane >> 4;
  const int item = a.ksplit > 1 ? 0 : blockIdx.z, split = a.ksplit > 1 ? blockIdx.z : 0;
  const uint32_t e = a.rhs ? a.rhs[item] : 0u;
  if (e >= (uint32_t)a.E) return;  // the whole workgroup leaves: the entry's output rows stay untouched
  const int tile = blockIdx.x;
  const int ngroups = a.N / 8;
  const int gi = tile * 16 + c;  // this lane's 8-column group
  const bool col_ok = gi < ngroups;
  const size_t row_bytes = (size_t)(a.N / G::WPB) * BPB;
  const int pi = G::SUPER ? tile >> 1 : tile;  // row piece the tile reads
  // group inside the piece; lanes past the last column decode the last group and store nothing
  const int gp = (col_ok ? gi : ngroups - 1) - pi * (G::PCOLS / 8);
  const uint8_t* wt = a.w + (size_t)e * (size_t)a.w_expert_stride + (size_t)pi * G::PIECE;
  const int cols_here = a.N - G::PCOLS * pi < G::PCOLS ? a.N - G::PCOLS * pi : G::PCOLS;
  const int piece_here = cols_here / G::WPB * BPB;  // the last piece of a 32-weight codec may be shorter
  uint8_t* stage = lds + wave * NT_KSTEP * STRIDE;
  const uint8_t* blk = stage + (gp / GPB) * BPB;
  const int g = gp % GPB, klast = a.K - 1;
  const int m0 = blockIdx.y * 16 * MR;
  const uint16_t* xr[MR];
#pragma unroll
  for (int q = 0; q < MR; q++) {
    const int mrow = m0 + 16 * q + c < a.M ? m0 + 16 * q + c : a.M - 1;  // rows past M repeat the last, never stored
    xr[q] = static_cast<const uint16_t*>(a.x) + (a.lhs ? (size_t)a.lhs[item] * (size_t)a.x_batch_stride : 0) +
            (size_t)mrow * a.K;
  }

  f32x4 acc[MR][8];
#pragma unroll
  for (int q = 0; q < MR; q++)
#pragma unroll
    for (int t = 0; t < 8; t++) acc[q][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  uint32_t wreg[NDW], xreg[MR][4];
  // Rows past K repeat the last row (their activations are zero).  No branch stands between the loads, so they are
  // all in flight together: a lane past the end of the step or of a short piece reads a clamped address, and the
  // last bytes of a piece come out of the dword that ends with the piece, shifted (never a byte past a row's end).
  auto fetch = [&](int st) {
#pragma unroll
    for (int j = 0; j < NDW; j++) {
      const int idx = lane + 64 * j < NT_KSTEP * PDW ? lane + 64 * j : NT_KSTEP * PDW - 1;
      const int row = idx / PDW, boff = 4 * (idx - row * PDW);
      const int eoff = boff < piece_here - 4 ? boff : piece_here - 4;
      const int k = NT_KSTEP * st + row < a.K ? NT_KSTEP * st + row : klast;
      const uint32_t v = *reinterpret_cast<const u32_a1*>(wt + (size_t)k * row_bytes + eoff);
      wreg[j] = v >> (8 * ((boff - eoff) & 3));
    }
    const int k0 = NT_KSTEP * st + 8 * h;
#pragma unroll
    for (int q = 0; q < MR; q++) {
#pragma unroll
      for (int j = 0; j < 4; j++) xreg[q][j] = 0u;
      if (a.x_vec) {  // K is a multiple of 8 here: a group of 8 lies inside the row or past it
        const uint4 v = *reinterpret_cast<const uint4*>(xr[q] + (k0 < a.K ? k0 : 0));
        const bool in = k0 < a.K;
        xreg[q][0] = in ? v.x : 0u, xreg[q][1] = in ? v.y : 0u, xreg[q][2] = in ? v.z : 0u, xreg[q][3] = in ? v.w : 0u;
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++)
          if (k0 + i < a.K) xreg[q][i >> 1] |= (uint32_t)xr[q][k0 + i] << (16 * (i & 1));
      }
    }
  };

  const int steps_all = (a.K + NT_KSTEP - 1) / NT_KSTEP;
  const int st_begin = split * a.steps_per_split;
  const int nsteps = st_begin + a.steps_per_split < steps_all ? st_begin + a.steps_per_split : steps_all;
  if (st_begin + wave < nsteps) fetch(st_begin + wave);
  for (int st = st_begin + wave; st < nsteps; st += NT_WAVES) {
#pragma unroll
    for (int j = 0; j < NDW; j++) {
      const int idx = lane + 64 * j;
      if (idx < NT_KSTEP * PDW) *reinterpret_cast<uint32_t*>(stage + 4 * idx) = wreg[j];
    }
    bf16x8 ah[MR], al[MR];
#pragma unroll
    for (int q = 0; q < MR; q++) {
      if constexpr (DT == KQ_BF16) {
        ah[q] = __builtin_bit_cast(bf16x8, make_uint4(xreg[q][0], xreg[q][1], xreg[q][2], xreg[q][3]));
      } else {
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float f0 = kq::h2f((uint16_t)(xreg[q][j] & 0xffffu)), f1 = kq::h2f((uint16_t)(xreg[q][j] >> 16));
          hi[j] = pack_hi(f0, f1);
          lo[j] = pack_hi(f0 - trunc_bf16(f0), f1 - trunc_bf16(f1));  // exact: 11 significant bits in all
        }
        ah[q] = __builtin_bit_cast(bf16x8, make_uint4(hi[0], hi[1], hi[2], hi[3]));
        al[q] = __builtin_bit_cast(bf16x8, make_uint4(lo[0], lo[1], lo[2], lo[3]));
      }
    }
    if (st + NT_WAVES < nsteps) fetch(st + NT_WAVES);
    // weights: rows 8h ... 8h + 7 of the step, column group of this lane, split into bf16 hi / lo and regrouped by
    // column
    uint32_t bh[8][4], bl[8][4];
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      float w0[8], w1[8];
      kq::decode8<C>(blk + (8 * h + i) * STRIDE, g, grids, w0);
      kq::decode8<C>(blk + (8 * h + i + 1) * STRIDE, g, grids, w1);
#pragma unroll
      for (int t = 0; t < 8; t++) {
        bh[t][i >> 1] = pack_hi(w0[t], w1[t]);
        bl[t][i >> 1] = pack_rne(w0[t] - trunc_bf16(w0[t]), w1[t] - trunc_bf16(w1[t]));
      }
    }
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const bf16x8 wh = __builtin_bit_cast(bf16x8, make_uint4(bh[t][0], bh[t][1], bh[t][2], bh[t][3]));
      const bf16x8 wl = __builtin_bit_cast(bf16x8, make_uint4(bl[t][0], bl[t][1], bl[t][2], bl[t][3]));
#pragma unroll
      for (int q = 0; q < MR; q++) {
        acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[q], wh, acc[q][t], 0, 0, 0);
        acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[q], wl, acc[q][t], 0, 0, 0);
        if constexpr (DT == KQ_F16) acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[q], wh, acc[q][t], 0, 0, 0);
      }
    }
  }

  if (nsteps - st_begin > 1) {  // uniform over the workgroup: waves 2, 3 -> waves 0, 1, then wave 1 -> wave 0
    constexpr int NACC = 32 * MR;
    __syncthreads();  // every wave is done with its staging area
    float* mine = red + (size_t)(wave & 1) * NACC * 64 + lane;
    auto put = [&](float* dst) {
#pragma unroll
      for (int q = 0; q < MR; q++)
#pragma unroll
        for (int t = 0; t < 8; t++)
#pragma unroll
          for (int r = 0; r < 4; r++) dst[((q * 8 + t) * 4 + r) * 64] = acc[q][t][r];
    };
    auto add = [&](const float* src) {
#pragma unroll
      for (int q = 0; q < MR; q++)
#pragma unroll
        for (int t = 0; t < 8; t++)
#pragma unroll
          for (int r = 0; r < 4; r++) acc[q][t][r] += src[((q * 8 + t) * 4 + r) * 64];
    };
    if (wave >= 2) put(mine);
    __syncthreads();
    if (wave < 2) add(mine);
    __syncthreads();
    if (wave == 1) put(red + lane);
    __syncthreads();
    if (wave == 0) add(red + lane);
  }
  if (wave != 0 || !col_ok) return;
  if (a.ksplit > 1) {
    float* pb = a.part + (size_t)split * a.M * a.N + 8 * (size_t)gi;
#pragma unroll
    for (int q = 0; q < MR; q++) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int m = m0 + 16 * q + 4 * h + r;
        if (m < a.M) {
          float4* o = reinterpret_cast<float4*>(pb + (size_t)m * a.N);
          o[0] = make_float4(acc[q][0][r], acc[q][1][r], acc[q][2][r], acc[q][3][r]);
          o[1] = make_float4(acc[q][4][r], acc[q][5][r], acc[q][6][r], acc[q][7][r]);
        }
      }
    }
    return;
  }
  uint16_t* yb = static_cast<uint16_t*>(a.y) + (size_t)item * a.M * a.N + 8 * (size_t)gi;
#pragma unroll
  for (int q = 0; q < MR; q++) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int m = m0 + 16 * q + 4 * h + r;
      if (m < a.M) {
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float v0 = acc[q][2 * j][r], v1 = acc[q][2 * j + 1][r];
          const uint16_t lo = DT == KQ_F16 ? kq::f2f16(v0) : kq::f2bf16(v0);
          const uint16_t hi = DT == KQ_F16 ? kq::f2f16(v1) : kq::f2bf16(v1);
          o[j] = (uint32_t)lo | ((uint32_t)hi << 16);
        }
        *reinterpret_cast<uint4*>(yb + (size_t)m * a.N) = make_uint4(o[0], o[1], o[2], o[3]);
      }
    }
  }
}

// Many activation rows: 128 (MRW = 2) or 256 (MRW = 4) rows x 128 columns per workgroup.  Every wave owns a quarter
// of the rows and the four walk the
// K steps together, so the 4096 weights of a step are decoded ONCE per workgroup instead of once per 32 rows: wave w
// decodes rows 8w ... 8w + 7 of the step's 32 (lane (c, part): rows 8w + 2 part, + 1 of column group c), writes them
// as packed bf16 pairs where the MFMA operands of all four waves lie (LDS, [k group h][t][c] x 16 bytes, hi and lo
// planes), and after one barrier every wave reads its 16 operands back.  Staging and operand buffers are double:
// one barrier per step.
template <int C, int DT, int MRW>
__global__ __launch_bounds__(NT_THREADS, 2) void gemm_nt_wide_kernel(NtArgs a, const uint8_t* __restrict__ grids) {
  using G = NtGeom<C>;
  constexpr int BPB = G::BPB, GPB = G::GPB, PDW = G::PDW, STRIDE = G::STRIDE;
  constexpr int STG = NT_KSTEP * STRIDE;               // one staging buffer: the step's 32 row pieces
  constexpr int NDWW = (NT_KSTEP * PDW + NT_THREADS - 1) / NT_THREADS;  // dwords a thread copies per step
  constexpr int PLANE = 4 * 8 * 16 * 16;               // one operand plane: [h][t][c] x 16 bytes
  constexpr int OPB = 2 * PLANE;                       // hi + lo
  __shared__ __attribute__((aligned(16))) uint8_t lds[2 * STG + 2 * OPB];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, h = lane >> 4;  // h: k group as operand reader, row pair as decoder
  const int item = a.ksplit > 1 ? 0 : blockIdx.z, split = a.ksplit > 1 ? blockIdx.z : 0;
  const uint32_t e = a.rhs ? a.rhs[item] : 0u;
  if (e >= (uint32_t)a.E) return;  // the whole workgroup leaves: the entry's output rows stay untouched
  const int tile = blockIdx.x;
  const int ngroups = a.N / 8;
  const int gi = tile * 16 + c;
  const bool col_ok = gi < ngroups;
  const size_t row_bytes = (size_t)(a.N / G::WPB) * BPB;
  const int pi = G::SUPER ? tile >> 1 : tile;
  const int gp = (col_ok ? gi : ngroups - 1) - pi * (G::PCOLS / 8);
  const uint8_t* wt = a.w + (size_t)e * (size_t)a.w_expert_stride + (size_t)pi * G::PIECE;
  const int cols_here = a.N - G::PCOLS * pi < G::PCOLS ? a.N - G::PCOLS * pi : G::PCOLS;
  const int piece_here = cols_here / G::WPB * BPB;
  const int blk_off = (gp / GPB) * BPB + (8 * wave + 2 * h) * STRIDE;  // this lane's first row inside a staging buffer
  const int g = gp % GPB, klast = a.K - 1;
  const int m0 = blockIdx.y * (64 * MRW) + 16 * MRW * wave;
  const uint16_t* xr[MRW];
#pragma unroll
  for (int q = 0; q < MRW; q++) {
    const int mrow = m0 + 16 * q + c < a.M ? m0 + 16 * q + c : a.M - 1;
    xr[q] = static_cast<const uint16_t*>(a.x) + (a.lhs ? (size_t)a.lhs[item] * (size_t)a.x_batch_stride : 0) +
            (size_t)mrow * a.K;
  }
  f32x4 acc[MRW][8];
#pragma unroll
  for (int q = 0; q < MRW; q++)
#pragma unroll
    for (int t = 0; t < 8; t++) acc[q][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  uint32_t wreg[NDWW], xreg[MRW][4];
  auto fetch = [&](int st) {  // as in gemm_nt_mfma_kernel, the step's pieces spread over the whole workgroup
#pragma unroll
    for (int j = 0; j < NDWW; j++) {
      const int idx = tid + NT_THREADS * j < NT_KSTEP * PDW ? tid + NT_THREADS * j : NT_KSTEP * PDW - 1;
      const int row = idx / PDW, boff = 4 * (idx - row * PDW);
      const int eoff = boff < piece_here - 4 ? boff : piece_here - 4;
      const int k = NT_KSTEP * st + row < a.K ? NT_KSTEP * st + row : klast;
      const uint32_t v = *reinterpret_cast<const u32_a1*>(wt + (size_t)k * row_bytes + eoff);
      wreg[j] = v >> (8 * ((boff - eoff) & 3));
    }
    const int k0 = NT_KSTEP * st + 8 * h;
#pragma unroll
    for (int q = 0; q < MRW; q++) {
#pragma unroll
      for (int j = 0; j < 4; j++) xreg[q][j] = 0u;
      if (a.x_vec) {
        const uint4 v = *reinterpret_cast<const uint4*>(xr[q] + (k0 < a.K ? k0 : 0));
        const bool in = k0 < a.K;
        xreg[q][0] = in ? v.x : 0u, xreg[q][1] = in ? v.y : 0u, xreg[q][2] = in ? v.z : 0u, xreg[q][3] = in ? v.w : 0u;
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++)
          if (k0 + i < a.K) xreg[q][i >> 1] |= (uint32_t)xr[q][k0 + i] << (16 * (i & 1));
      }
    }
  };
  auto park = [&](uint8_t* stage) {
#pragma unroll
    for (int j = 0; j < NDWW; j++) {
      const int idx = tid + NT_THREADS * j;
      if (idx < NT_KSTEP * PDW) *reinterpret_cast<uint32_t*>(stage + 4 * idx) = wreg[j];
    }
  };

  const int steps_all = (a.K + NT_KSTEP - 1) / NT_KSTEP;
  const int st_begin = split * a.steps_per_split;
  const int nsteps = st_begin + a.steps_per_split < steps_all ? st_begin + a.steps_per_split : steps_all;
  if (st_begin < nsteps) {
    fetch(st_begin);
    park(lds);
  }
  for (int st = st_begin; st < nsteps; st++) {
    const int b = (st - st_begin) & 1;
    const uint8_t* stage = lds + b * STG;
    uint8_t* opnd = lds + 2 * STG + b * OPB;
    bf16x8 ah[MRW], al[MRW];
#pragma unroll
    for (int q = 0; q < MRW; q++) {
      if constexpr (DT == KQ_BF16) {
        ah[q] = __builtin_bit_cast(bf16x8, make_uint4(xreg[q][0], xreg[q][1], xreg[q][2], xreg[q][3]));
      } else {
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float f0 = kq::h2f((uint16_t)(xreg[q][j] & 0xffffu)), f1 = kq::h2f((uint16_t)(xreg[q][j] >> 16));
          hi[j] = pack_hi(f0, f1);
          lo[j] = pack_hi(f0 - trunc_bf16(f0), f1 - trunc_bf16(f1));
        }
        ah[q] = __builtin_bit_cast(bf16x8, make_uint4(hi[0], hi[1], hi[2], hi[3]));
        al[q] = __builtin_bit_cast(bf16x8, make_uint4(lo[0], lo[1], lo[2], lo[3]));
      }
    }
    if (st == st_begin) __syncthreads();  // the first staging buffer is complete (later ones: the barrier below)
    if (st + 1 < nsteps) fetch(st + 1);
    {  // decode this lane's two rows and put them where the operands lie
      float w0[8], w1[8];
      kq::decode8<C>(stage + blk_off, g, grids, w0);
      kq::decode8<C>(stage + blk_off + STRIDE, g, grids, w1);
      uint8_t* dst = opnd + ((wave * 8) * 16 + c) * 16 + 4 * h;
#pragma unroll
      for (int t = 0; t < 8; t++) {
        *reinterpret_cast<uint32_t*>(dst + t * 256) = pack_hi(w0[t], w1[t]);
        *reinterpret_cast<uint32_t*>(dst + t * 256 + PLANE) =
            pack_rne(w0[t] - trunc_bf16(w0[t]), w1[t] - trunc_bf16(w1[t]));
      }
    }
    if (st + 1 < nsteps) park(lds + (b ^ 1) * STG);
    __syncthreads();  // operands of this step are complete; the other staging buffer is written
    const uint8_t* src = opnd + ((h * 8) * 16 + c) * 16;
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const bf16x8 wh = *reinterpret_cast<const bf16x8*>(src + t * 256);
      const bf16x8 wl = *reinterpret_cast<const bf16x8*>(src + t * 256 + PLANE);
#pragma unroll
      for (int q = 0; q < MRW; q++) {
        acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[q], wh, acc[q][t], 0, 0, 0);
        acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[q], wl, acc[q][t], 0, 0, 0);
        if constexpr (DT == KQ_F16) acc[q][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[q], wh, acc[q][t], 0, 0, 0);
      }
    }
  }

  if (!col_ok) return;
  if (a.ksplit > 1) {
    float* pb = a.part + (size_t)split * a.M * a.N + 8 * (size_t)gi;
#pragma unroll
    for (int q = 0; q < MRW; q++) {
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int m = m0 + 16 * q + 4 * h + r;
        if (m < a.M) {
          float4* o = reinterpret_cast<float4*>(pb + (size_t)m * a.N);
          o[0] = make_float4(acc[q][0][r], acc[q][1][r], acc[q][2][r], acc[q][3][r]);
          o[1] = make_float4(acc[q][4][r], acc[q][5][r], acc[q][6][r], acc[q][7][r]);
        }
      }
    }
    return;
  }
  uint16_t* yb = static_cast<uint16_t*>(a.y) + (size_t)item * a.M * a.N + 8 * (size_t)gi;
#pragma unroll
  for (int q = 0; q < MRW; q++) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int m = m0 + 16 * q + 4 * h + r;
      if (m < a.M) {
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float v0 = acc[q][2 * j][r], v1 = acc[q][2 * j + 1][r];
          const uint16_t lo = DT == KQ_F16 ? kq::f2f16(v0) : kq::f2bf16(v0);
          const uint16_t hi = DT == KQ_F16 ? kq::f2f16(v1) : kq::f2bf16(v1);
          o[j] = (uint32_t)lo | ((uint32_t)hi << 16);
        }
        *reinterpret_cast<uint4*>(yb + (size_t)m * a.N) = make_uint4(o[0], o[1], o[2], o[3]);
      }
    }
  }
}

// y[i] = sum over the K ranges of part[s][i], 8 outputs per thread, ranges added in order
template <int DT>
__global__ __launch_bounds__(256) void nt_reduce_kernel(const float* __restrict__ part, void* __restrict__ y,
                                                        size_t groups, int ksplit) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= groups) return;
  float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < ksplit; s++) {
    const float4* p = reinterpret_cast<const float4*>(part + ((size_t)s * groups + i) * 8);
    const float4 lo = p[0], hi = p[1];
    v[0] += lo.x, v[1] += lo.y, v[2] += lo.z, v[3] += lo.w, v[4] += hi.x, v[5] += hi.y, v[6] += hi.z, v[7] += hi.w;
  }
  uint32_t o[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const uint16_t lo = DT == KQ_F16 ? kq::f2f16(v[2 * j]) : kq::f2bf16(v[2 * j]);
    const uint16_t hi = DT == KQ_F16 ? kq::f2f16(v[2 * j + 1]) : kq::f2bf16(v[2 * j + 1]);
    o[j] = (uint32_t)lo | ((uint32_t)hi << 16);
  }
  reinterpret_cast<uint4*>(y)[i] = make_uint4(o[0], o[1], o[2], o[3]);
}

// K ranges of a dense call: enough workgroups for two per CU, at least eight steps each
int nt_ksplit(int M, int N, int K) {
  const int rows = M <= 16 ? 16 : M < NT_SHARED_ROWS ? 32 : 128;  // activation rows per workgroup
  const int64_t tiles = (int64_t)((N + NT_COLS - 1) / NT_COLS) * ((M + rows - 1) / rows);
  const int steps = (K + NT_KSTEP - 1) / NT_KSTEP;
  if (tiles >= 256 || steps < 16) return 1;
  int s = (int)((512 + tiles - 1) / tiles);
  if (s > steps / 8) s = steps / 8;
  if (s > 32) s = 32;
  return s < 2 ? 1 : s;
}

template <int C>
struct NtRun {
  template <int DT, int MR>
  static void go(const NtArgs& a, int B, const uint8_t* grids, hipStream_t s) {
    dim3 grid((a.N + NT_COLS - 1) / NT_COLS, (a.M + 16 * MR - 1) / (16 * MR), a.ksplit > 1 ? a.ksplit : B);
    hipLaunchKernelGGL((gemm_nt_mfma_kernel<C, DT, MR>), grid, dim3(NT_THREADS), 0, s, a, grids);
    if (a.ksplit > 1) {
      const size_t groups = (size_t)a.M * a.N / 8;
      hipLaunchKernelGGL((nt_reduce_kernel<DT>), dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s, a.part, a.y,
                         groups, a.ksplit);
    }
  }
  template <int DT>
  static void go_shared(const NtArgs& a, int B, const uint8_t* grids, hipStream_t s) {
    // (256-row tiles, MRW = 4, measured slower: 316 against 223 us at 2048 rows of 4096 x 4096 q4_k; their 212 - 250
    // registers leave two workgroups per CU where the 128-row form runs three)
    dim3 grid((a.N + NT_COLS - 1) / NT_COLS, (a.M + 127) / 128, a.ksplit > 1 ? a.ksplit : B);
    hipLaunchKernelGGL((gemm_nt_wide_kernel<C, DT, 2>), grid, dim3(NT_THREADS), 0, s, a, grids);
    if (a.ksplit > 1) {
      const size_t groups = (size_t)a.M * a.N / 8;
      hipLaunchKernelGGL((nt_reduce_kernel<DT>), dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s, a.part, a.y,
                         groups, a.ksplit);
    }
  }
  static int run(const NtArgs& a, int B, int dt, const uint8_t* grids, hipStream_t s) {
    if (a.M >= NT_SHARED_ROWS) {
      dt == KQ_F16 ? go_shared<KQ_F16>(a, B, grids, s) : go_shared<KQ_BF16>(a, B, grids, s);
    } else if (a.M <= 16) {
      dt == KQ_F16 ? go<KQ_F16, 1>(a, B, grids, s) : go<KQ_BF16, 1>(a, B, grids, s);
    } else if (nt_wide(C) && a.M > 32) {
      if constexpr (nt_wide(C)) dt == KQ_F16 ? go<KQ_F16, 4>(a, B, grids, s) : go<KQ_BF16, 4>(a, B, grids, s);
    } else {
      dt == KQ_F16 ? go<KQ_F16, 2>(a, B, grids, s) : go<KQ_BF16, 2>(a, B, grids, s);
    }
    KQ_HIP_CHECK(hipGetLastError());
    return KQ_OK;
  }
};

template <template <int> class F, typename... A>
int nt_dispatch(int codec, const A&... a) {
  switch (codec) {
#define KQ_CASE(c) \
  case c:          \
    return F<c>::run(a...);
    KQ_CASE(KQ_Q2_K) KQ_CASE(KQ_Q3_K) KQ_CASE(KQ_Q4_K) KQ_CASE(KQ_Q5_K) KQ_CASE(KQ_Q6_K) KQ_CASE(KQ_Q4_0)
    KQ_CASE(KQ_Q4_1) KQ_CASE(KQ_Q5_0) KQ_CASE(KQ_Q5_1) KQ_CASE(KQ_Q8_0) KQ_CASE(KQ_IQ4_NL) KQ_CASE(KQ_IQ4_XS)
    KQ_CASE(KQ_IQ3_S) KQ_CASE(KQ_IQ3_XXS) KQ_CASE(KQ_IQ2_XXS) KQ_CASE(KQ_IQ2_XS) KQ_CASE(KQ_IQ2_S)
    KQ_CASE(KQ_IQ1_S) KQ_CASE(KQ_IQ1_M) KQ_CASE(KQ_MXFP4) KQ_CASE(KQ_NVFP4)
#undef KQ_CASE
  }
  return KQ_ERR_UNSUPPORTED;
}

}  // namespace

// f32 partial sums of a dense call whose K range is cut (0: the call runs uncut)
size_t kq_nt_workspace_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int s = nt_ksplit(M, N, K);
  return s > 1 ? (size_t)s * M * N * 4 : 0;
}

// Dense (lhs = rhs = null, B = 1, E = 1) or gathered.  KQ_ERR_UNSUPPORTED (nothing launched) when the output is
// not 16-byte aligned or the grid does not fit: the caller then runs the plain vector kernel.  A dense call cuts
// its K range when `ws` holds kq_nt_workspace_bytes and is 16-byte aligned; without it the call runs uncut.
int kq_launch_nt_mfma(const void* x, const uint8_t* w, const uint32_t* lhs, const uint32_t* rhs, void* out, int B,
                      int M, int E, int N, int K, int64_t x_batch_stride, int64_t w_expert_stride, int codec, int dtype,
                      void* ws, size_t ws_bytes, hipStream_t s) {
  if (B <= 0 || M <= 0 || N <= 0 || K <= 0 || (N & 7)) return KQ_ERR_UNSUPPORTED;
  if (B > 65535 || (M + 15) / 16 > 65535) return KQ_ERR_UNSUPPORTED;
  if (reinterpret_cast<uintptr_t>(out) & 15) return KQ_ERR_UNSUPPORTED;
  const uint8_t* grids = kq_device_grids();
  if (!grids) return KQ_ERR_HIP;
  NtArgs a{x, w, out, lhs, rhs, M, N, K, E, x_batch_stride, w_expert_stride, 0, 1, (K + NT_KSTEP - 1) / NT_KSTEP, nullptr};
  a.x_vec = !(K & 7) && !(reinterpret_cast<uintptr_t>(x) & 15) && !(x_batch_stride & 7);
  if (!rhs && B == 1 && ws && !(reinterpret_cast<uintptr_t>(ws) & 15)) {
    const int sp = nt_ksplit(M, N, K);
    if (sp > 1 && ws_bytes >= (size_t)sp * M * N * 4) {
      const int steps = (K + NT_KSTEP - 1) / NT_KSTEP;
      a.steps_per_split = (steps + sp - 1) / sp;
      a.ksplit = (steps + a.steps_per_split - 1) / a.steps_per_split;
      a.part = static_cast<float*>(ws);
    }
  }
  return nt_dispatch<NtRun>(codec, a, B, dtype, grids, s);
}
