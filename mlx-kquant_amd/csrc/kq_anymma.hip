// Matrix-core GEMM for EVERY codec: prefill (y[M,N] = x[M,K] . W^T, M > 8) and the batched MoE ops
// (pairs sorted by expert, 32-pair segments), for the codecs and options the tuned K-quant kernels
// do not cover (legacy, IQ, fp4, biases, swiglu_clamp).
//
// Numerics.  A wave decodes its 32 weight columns with the reference-order decoders of
// kq_decode.h (f32, bit-identical to dequantize) and splits every f32 weight into two bf16
// terms, the truncation and the remainder rounded to nearest (16 significand bits, an error below
// 2^-17 of the weight; bf16 has the f32 exponent range, so no codec scale can overflow or
// underflow; KQ_ANY_TERMS = 3 builds the exact three-term form).  Activations are bf16 as given, or
// f16 split exactly into two bf16 terms.  v_mfma_f32_32x32x16_bf16 then forms exact products and
// accumulates in f32.
//
// Tiling.  Workgroup = 4 waves, tile = (32 MT activation rows) x 128 weight rows, K advances one
// 256-weight step (a superblock, or 8 / 4 of the 32 / 64-weight blocks; the last step of a K that is
// not a multiple of 256 is zero-filled).  Wire bytes of the step (128 rows) and the activation tile
// are fetched with coalesced 16-byte loads one step ahead and parked in LDS; lane (column l % 32,
// K-half l / 32) decodes exactly the 8-weight groups its MFMA B operands need, so nothing decoded
// is ever shared or stored.
#include "kq_decode.h"
#include "kq_epilogue.h"

// kq_moe.hip
int kq_launch_moe_sort(const uint32_t* idx, int P, int E, void* order, void* segs, void* nseg, hipStream_t s);

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_a1 __attribute__((aligned(1)));  // the hardware serves unaligned vector loads

constexpr int AM_THREADS = 256;
constexpr int AM_BN = 128;          // weight rows per workgroup
constexpr int AM_STEP = 256;        // weights of K per step
constexpr int A_STRIDE = 512 + 16;  // bytes per activation row of one step in LDS (one bf16 plane)

struct Segment {
  int expert, start, count, pad;
};

__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int C>
struct StepGeom {
  static constexpr int WPB = kq_geom(C).wpb, BPB = kq_geom(C).bpb, GPB = WPB / 8;
  static constexpr int BLOCKS = AM_STEP / WPB;             // blocks per step and row
  static constexpr int BYTES = BLOCKS * BPB;               // wire bytes per step and row
  static constexpr int PIECES = (BYTES + 15) / 16;         // 16-byte pieces (the last may read past the step)
  static constexpr int LROW = (PIECES | 1) * 16;           // LDS row stride: an odd number of pieces
  static constexpr int WPT = (AM_BN * PIECES + AM_THREADS - 1) / AM_THREADS;
};

// f32 -> three bf16 terms by truncation, packed: out1/2/3[i] hold weights 2i (low half), 2i + 1 (high half)
__device__ __forceinline__ void split3(const float* w, uint32_t* o1, uint32_t* o2, uint32_t* o3) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    uint32_t t1[2], t2[2], t3[2];
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const float v = w[2 * i + e];
      const uint32_t u1 = __builtin_bit_cast(uint32_t, v) & 0xffff0000u;
      const float r1 = v - __builtin_bit_cast(float, u1);
      const uint32_t u2 = __builtin_bit_cast(uint32_t, r1) & 0xffff0000u;
      const float r2 = r1 - __builtin_bit_cast(float, u2);
      t1[e] = u1;
      t2[e] = u2;
      t3[e] = __builtin_bit_cast(uint32_t, r2) & 0xffff0000u;
    }
    o1[i] = (t1[0] >> 16) | t1[1];
    o2[i] = (t2[0] >> 16) | t2[1];
    o3[i] = (t3[0] >> 16) | t3[1];
  }
}

// f32 -> bf16 by truncation + the remainder rounded to nearest (v_cvt_pk_bf16_f32): 16 significand bits, an error
// below 2^-17 of the weight.  Two terms instead of three take a third off the MFMAs and 2.5 vector instructions per
// weight off the split; the kernel is bound by both.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void split2(const float* w, uint32_t* o1, uint32_t* o2) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const float v0 = w[2 * i], v1 = w[2 * i + 1];
    const uint32_t b0 = __builtin_bit_cast(uint32_t, v0), b1 = __builtin_bit_cast(uint32_t, v1);
    o1[i] = __builtin_amdgcn_perm(b1, b0, 0x07060302u);
    const float r0 = v0 - __builtin_bit_cast(float, b0 & 0xffff0000u);
    const float r1 = v1 - __builtin_bit_cast(float, b1 & 0xffff0000u);
    const bf16x2_t lo = {(__bf16)r0, (__bf16)r1};
    o2[i] = __builtin_bit_cast(uint32_t, lo);
  }
}

#ifndef KQ_ANY_TERMS
#define KQ_ANY_TERMS 2
#endif

struct AnyArgs {
  const void* x;        // dense: [M][K]; grouped: [rows][K], pair p reads row p / x_div
  const uint8_t* w;
  const uint8_t* w2;    // up stack (GLU) or null
  void* y;              // dense [M][N]; grouped [P][N]
  const float* bias;    // f32 [E][N] or null (grouped)
  const float* bias2;
  const int* order;     // grouped: pair ids sorted by expert
  const Segment* segs;
  const int* nseg;
  const uint8_t* grids;
  int M, N, K, x_div, act, mtiles;
  int64_t w_expert_stride;
  float limit, alpha;
  KqOutMap om;          // grouped: where pair results go
  float* partial;       // dense split-K: f32 partial sums [ksplit][M][N] (null: round and store y)
  int steps_per_split;  // dense: K steps per blockIdx.y
};

// MODE 0 = dense, 1 = grouped, 2 = grouped GLU (slab = 64 gate + 64 up rows; waves 0/2 gate, 1/3 up)
template <int C, int DT, int MT, int MODE>
__global__ __launch_bounds__(AM_THREADS, 1) void any_mma_kernel(AnyArgs a) {
  using G = StepGeom<C>;
  constexpr int NA = DT == KQ_F16 ? 2 : 1;         // bf16 planes of the activation tile
  constexpr int TM = 32 * MT;
  constexpr int APT = TM * 32 / AM_THREADS;        // 16-byte activation pieces per thread per step
  constexpr int NCOLS = MODE == 2 ? AM_BN / 2 : AM_BN;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* a_lds = smem;                                   // [NA][TM][A_STRIDE]
  uint8_t* b_lds = a_lds + NA * TM * A_STRIDE;             // [128][LROW]
  int* pair_lds = reinterpret_cast<int*>(b_lds + AM_BN * G::LROW);  // [32] output row per slot, -1 = none

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, kg = lane >> 5;
  const int N = a.N, K = a.K;
  const int nsteps = (K + AM_STEP - 1) / AM_STEP;
  const size_t row_bytes = (size_t)(K / G::WPB) * G::BPB;

  Segment seg{0, 0, 0, 0};
  int m0 = 0, n0;
  if constexpr (MODE == 0) {
    const int mt = blockIdx.x % a.mtiles, nt = blockIdx.x / a.mtiles;  // consecutive workgroups share the weight rows
    m0 = mt * TM;
    n0 = nt * NCOLS;
  } else {
    if ((int)blockIdx.y >= *a.nseg) return;  // uniform: the grid is sized for the worst case
    seg = a.segs[blockIdx.y];
    n0 = blockIdx.x * NCOLS;
  }
  const int ncols = N - n0 < NCOLS ? N - n0 : NCOLS;
  const uint8_t* wbase = a.w + (size_t)seg.expert * (size_t)a.w_expert_stride;
  const uint8_t* wbase2 = MODE == 2 ? a.w2 + (size_t)seg.expert * (size_t)a.w_expert_stride : wbase;
  const uint8_t* w_end = wbase + (size_t)N * row_bytes;  // one past the expert's matrix

  // slab row rr (= wave * 32 + l32 in the compute phase) -> (matrix, column)
  auto slab_col = [&](int rr, bool& up) {
    if constexpr (MODE == 2) {
      const int wv = rr >> 5;
      up = wv & 1;
      return (wv >> 1) * 32 + (rr & 31);
    } else {
      up = false;
      return rr;
    }
  };

  if constexpr (MODE != 0) {
    if (tid < 32) pair_lds[tid] = tid < seg.count ? a.order[seg.start + tid] : -1;
  }

  // ---- piece maps
  const int a_slot = tid >> 5, a_pc = tid & 31;  // activation piece i = tid + 256 t -> (row i / 32, piece i % 32)
  const uint16_t* a_src[APT];
#pragma unroll
  for (int t = 0; t < APT; t++) {
    const int slot = a_slot + 8 * t;
    size_t row;
    if constexpr (MODE == 0) {
      row = (size_t)(m0 + slot < a.M ? m0 + slot : a.M - 1);
    } else {
      row = (size_t)(a.order[seg.start + (slot < seg.count ? slot : 0)] / a.x_div);
    }
    a_src[t] = static_cast<const uint16_t*>(a.x) + row * K + 8 * a_pc;
  }
  const uint8_t* w_src[G::WPT];
  uint32_t w_loff[G::WPT];
  bool w_up[G::WPT];
#pragma unroll
  for (int t = 0; t < G::WPT; t++) {
    const int i = tid + AM_THREADS * t;
    const int r = i / G::PIECES, pc = i % G::PIECES;
    bool up;
    const int col = slab_col(r < AM_BN ? r : 0, up);
    const bool ok = r < AM_BN && col < ncols;  // rows past N re-read the slab's first row
    w_up[t] = up;
    w_src[t] = (up ? wbase2 : wbase) + (size_t)(n0 + (ok ? col : 0)) * row_bytes + 16 * pc;
    w_loff[t] = r < AM_BN ? (uint32_t)r * G::LROW + 16 * pc : 0xffffffffu;
  }
  const uint8_t* w_end2 = wbase2 + (size_t)N * row_bytes;

  // dense tiles past M are zero-filled without a load (a skinny call has 32 - M such rows)
  bool a_live[APT];
#pragma unroll
  for (int t = 0; t < APT; t++) a_live[t] = MODE != 0 || m0 + a_slot + 8 * t < a.M;

  u32x4 areg[APT], wreg[G::WPT];
  auto issue = [&](int st) {
    const int kvalid = K - AM_STEP * st;  // weights of this step that exist (>= 256 except in the last step)
#pragma unroll
    for (int t = 0; t < APT; t++) {
      u32x4 v = {0, 0, 0, 0};
      if (8 * a_pc < kvalid && a_live[t]) v = *reinterpret_cast<const u32x4*>(a_src[t] + (size_t)AM_STEP * st);
      areg[t] = v;
    }
    const int bvalid = kvalid >= AM_STEP ? G::BYTES : (kvalid / G::WPB) * G::BPB;  // wire bytes of this step per row
#pragma unroll
    for (int t = 0; t < G::WPT; t++) {
      const int pc = (tid + AM_THREADS * t) % G::PIECES;
      const uint8_t* p = w_src[t] + (size_t)st * G::BYTES;
      u32x4 v = {0, 0, 0, 0};
      if (16 * pc < bvalid) {
        const uint8_t* end = w_up[t] ? w_end2 : w_end;
        if (p + 16 <= end) {
          v = *reinterpret_cast<const u32x4_a1*>(p);
        } else {  // the last bytes of the matrix: never read past its end
          for (int b = 0; b < 16; b++)
            if (p + b < end) v[b >> 2] |= (uint32_t)p[b] << (8 * (b & 3));
        }
      }
      wreg[t] = v;
    }
  };
  auto park = [&]() {
#pragma unroll
    for (int t = 0; t < APT; t++) {
      uint8_t* dst = a_lds + (a_slot + 8 * t) * A_STRIDE + 16 * a_pc;
      if constexpr (DT == KQ_BF16) {
        *reinterpret_cast<u32x4*>(dst) = areg[t];
      } else {
        // f16 -> bf16 hi (truncated) + bf16 lo (exact remainder: at most 3 significant bits)
        u32x4 hi, lo;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          uint32_t hh[2], ll[2];
#pragma unroll
          for (int q = 0; q < 2; q++) {
            const uint16_t hbits = (uint16_t)(q ? (areg[t][e] >> 16) : (areg[t][e] & 0xffff));
            const float v = kq::h2f(hbits);
            const uint32_t u = __builtin_bit_cast(uint32_t, v) & 0xffff0000u;
            const float r = v - __builtin_bit_cast(float, u);
            hh[q] = u;
            ll[q] = __builtin_bit_cast(uint32_t, r) & 0xffff0000u;
          }
          hi[e] = (hh[0] >> 16) | hh[1];
          lo[e] = (ll[0] >> 16) | ll[1];
        }
        *reinterpret_cast<u32x4*>(dst) = hi;
        *reinterpret_cast<u32x4*>(dst + TM * A_STRIDE) = lo;
      }
    }
#pragma unroll
    for (int t = 0; t < G::WPT; t++)
      if (w_loff[t] != 0xffffffffu) *reinterpret_cast<u32x4*>(b_lds + w_loff[t]) = wreg[t];
  };

  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) acc[t] = f32x16{0};
  const uint8_t* b_lane = b_lds + (wave * 32 + l32) * G::LROW;
  const uint8_t* a_lane = a_lds + l32 * A_STRIDE + 16 * kg;

  // dense split-K: blockIdx.y owns K steps [st0, st1)
  int st0 = 0, st1 = nsteps;
  if constexpr (MODE == 0) {
    st0 = (int)blockIdx.y * a.steps_per_split;
    st1 = st0 + a.steps_per_split < nsteps ? st0 + a.steps_per_split : nsteps;
  }
  issue(st0);
  for (int st = st0; st < st1; st++) {
    if (st > st0) lds_barrier();  // everyone is done reading the previous step
    park();
    if (st + 1 < st1) issue(st + 1);
    lds_barrier();
    const int kvalid = K - AM_STEP * st;
#pragma unroll 2
    for (int i = 0; i < 16; i++) {  // 16 K-slices of 16: this lane decodes weights [16 i + 8 kg, + 8) of its column
      const int gk = 2 * i + kg;
      float w8[8];
      if (8 * gk < kvalid) {
        kq::decode8<C>(b_lane + (gk / G::GPB) * G::BPB, gk % G::GPB, a.grids, w8);
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++) w8[e] = 0.f;
      }
      uint32_t b1[4], b2[4], b3[4] = {0u, 0u, 0u, 0u};
      if constexpr (KQ_ANY_TERMS == 3)
        split3(w8, b1, b2, b3);
      else
        split2(w8, b1, b2);
      const bf16x8 f1 = __builtin_bit_cast(bf16x8, make_uint4(b1[0], b1[1], b1[2], b1[3]));
      const bf16x8 f2 = __builtin_bit_cast(bf16x8, make_uint4(b2[0], b2[1], b2[2], b2[3]));
      const bf16x8 f3 = __builtin_bit_cast(bf16x8, make_uint4(b3[0], b3[1], b3[2], b3[3]));
#pragma unroll
      for (int t = 0; t < MT; t++) {
#pragma unroll
        for (int pl = 0; pl < NA; pl++) {
          const bf16x8 av = *reinterpret_cast<const bf16x8*>(a_lane + (pl * TM + t * 32) * A_STRIDE + 32 * i);
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, f1, acc[t], 0, 0, 0);
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, f2, acc[t], 0, 0, 0);
          if constexpr (KQ_ANY_TERMS == 3) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, f3, acc[t], 0, 0, 0);
        }
      }
    }
  }

  // ---- epilogue
  uint16_t* y = static_cast<uint16_t*>(a.y);
  auto store = [&](size_t off, float v) { y[off] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v); };
  if constexpr (MODE == 0) {
    const int n = n0 + wave * 32 + l32;
    float* part = a.partial ? a.partial + (size_t)blockIdx.y * a.M * N : nullptr;
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int m = m0 + t * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);
        if (m < a.M && n < N) {
          if (part)
            part[(size_t)m * N + n] = acc[t][i];
          else
            store((size_t)m * N + n, acc[t][i]);
        }
      }
  } else if constexpr (MODE == 1) {
    const int col = wave * 32 + l32;
    const float bv = (a.bias && col < ncols) ? a.bias[(size_t)seg.expert * N + n0 + col] : 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int pr = pair_lds[8 * (i >> 2) + 4 * kg + (i & 3)];
      if (pr >= 0 && col < ncols)
        kq::store_result<DT>(a.y, a.om, (size_t)kq::out_row(a.om, pr) * N + n0 + col, acc[0][i] + bv);
    }
  } else {
    lds_barrier();  // the step buffers are free: reuse them for the up accumulators
    float* ex = reinterpret_cast<float*>(smem);  // [2 column blocks][16][64]
    const int nb = wave >> 1;
    if (wave & 1) {
#pragma unroll
      for (int i = 0; i < 16; i++) ex[(nb * 16 + i) * 64 + lane] = acc[0][i];
    }
    lds_barrier();
    if (!(wave & 1)) {
      const int col = nb * 32 + l32;
      const bool live = col < ncols;
      const float gb = (a.bias && live) ? a.bias[(size_t)seg.expert * N + n0 + col] : 0.f;
      const float ub = (a.bias2 && live) ? a.bias2[(size_t)seg.expert * N + n0 + col] : 0.f;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int pr = pair_lds[8 * (i >> 2) + 4 * kg + (i & 3)];
        if (pr >= 0 && live) {
          const float v = kq::glu_epilogue_fast(a.act, acc[0][i] + gb, ex[(nb * 16 + i) * 64 + lane] + ub, a.limit, a.alpha);
          kq::store_result<DT>(a.y, a.om, (size_t)kq::out_row(a.om, pr) * N + n0 + col, v);
        }
      }
    }
  }
}

// y[i] = round(sum over splits of partial[split][i])
template <int DT>
__global__ __launch_bounds__(256) void any_splitk_reduce_kernel(const float* __restrict__ partial, uint16_t* __restrict__ y,
                                                                int count, int splits) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  float v = 0.f;
  for (int sp = 0; sp < splits; sp++) v += partial[(size_t)sp * count + i];
  y[i] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
}

// 32-row activation groups per workgroup of a dense call: 128-row tiles for bf16 activations, 64-row tiles for
// f16 (two bf16 planes in LDS), smaller ones for fewer rows
int any_dense_mt(int M, int dt) { return M <= 32 ? 1 : (M <= 64 || dt == KQ_F16) ? 2 : 4; }

template <int C, int DT, int MT, int MODE>
int launch_any(const AnyArgs& a, dim3 grid, hipStream_t s) {
  using G = StepGeom<C>;
  constexpr int NA = DT == KQ_F16 ? 2 : 1;
  size_t lds = (size_t)NA * 32 * MT * A_STRIDE + (size_t)AM_BN * G::LROW + 128;
  if (MODE == 2 && lds < 8192 + 128) lds = 8192 + 128;
  auto kern = any_mma_kernel<C, DT, MT, MODE>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  hipLaunchKernelGGL(kern, grid, dim3(AM_THREADS), lds, s, a);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

constexpr int SEG_M = 32;

template <int C>
struct AnyRun {
  static int run(const AnyArgs& a, int mode, int dt, int P, int E, hipStream_t s) {
    if (mode == 0) {
      // one to four 32-row activation groups per workgroup; K split over blockIdx.y when the caller brought a
      // workspace (a.partial) and the plan asked for it
      AnyArgs b = a;
      const int mt = any_dense_mt(a.M, dt);
      b.mtiles = (a.M + 32 * mt - 1) / (32 * mt);
      const int nsteps = (a.K + AM_STEP - 1) / AM_STEP;
      const int splits = (nsteps + a.steps_per_split - 1) / a.steps_per_split;
      const dim3 grid(b.mtiles * ((a.N + AM_BN - 1) / AM_BN), splits);
      int rc;
      if (mt == 1)
        rc = dt == KQ_F16 ? launch_any<C, KQ_F16, 1, 0>(b, grid, s) : launch_any<C, KQ_BF16, 1, 0>(b, grid, s);
      else if (mt == 2)
        rc = dt == KQ_F16 ? launch_any<C, KQ_F16, 2, 0>(b, grid, s) : launch_any<C, KQ_BF16, 2, 0>(b, grid, s);
      else
        rc = launch_any<C, KQ_BF16, 4, 0>(b, grid, s);
      if (rc || !a.partial) return rc;
      const int count = a.M * a.N;
      if (dt == KQ_F16)
        hipLaunchKernelGGL(any_splitk_reduce_kernel<KQ_F16>, dim3((count + 255) / 256), dim3(256), 0, s, a.partial,
                           static_cast<uint16_t*>(a.y), count, splits);
      else
        hipLaunchKernelGGL(any_splitk_reduce_kernel<KQ_BF16>, dim3((count + 255) / 256), dim3(256), 0, s, a.partial,
                           static_cast<uint16_t*>(a.y), count, splits);
      KQ_HIP_CHECK(hipGetLastError());
      return KQ_OK;
    }
    int maxseg = E + P / SEG_M;
    if (maxseg > P) maxseg = P;
    const int ncols = mode == 2 ? AM_BN / 2 : AM_BN;
    const dim3 grid((a.N + ncols - 1) / ncols, maxseg);
    if (mode == 1)
      return dt == KQ_F16 ? launch_any<C, KQ_F16, 1, 1>(a, grid, s) : launch_any<C, KQ_BF16, 1, 1>(a, grid, s);
    return dt == KQ_F16 ? launch_any<C, KQ_F16, 1, 2>(a, grid, s) : launch_any<C, KQ_BF16, 1, 2>(a, grid, s);
  }
};

int dispatch_any(int codec, const AnyArgs& a, int mode, int dt, int P, int E, hipStream_t s) {
  switch (codec) {
#define KQ_CASE(c) \
  case c:          \
    return AnyRun<c>::run(a, mode, dt, P, E, s);
    KQ_CASE(KQ_Q2_K) KQ_CASE(KQ_Q3_K) KQ_CASE(KQ_Q4_K) KQ_CASE(KQ_Q5_K) KQ_CASE(KQ_Q6_K) KQ_CASE(KQ_Q4_0)
    KQ_CASE(KQ_Q4_1) KQ_CASE(KQ_Q5_0) KQ_CASE(KQ_Q5_1) KQ_CASE(KQ_Q8_0) KQ_CASE(KQ_IQ4_NL) KQ_CASE(KQ_IQ4_XS)
    KQ_CASE(KQ_IQ3_S) KQ_CASE(KQ_IQ3_XXS) KQ_CASE(KQ_IQ2_XXS) KQ_CASE(KQ_IQ2_XS) KQ_CASE(KQ_IQ2_S)
    KQ_CASE(KQ_IQ1_S) KQ_CASE(KQ_IQ1_M) KQ_CASE(KQ_MXFP4) KQ_CASE(KQ_NVFP4)
#undef KQ_CASE
  }
  return KQ_ERR_UNSUPPORTED;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

bool kq_anymma_supported(int M, int N, int K, int codec) {
  return codec >= 0 && codec < KQ_NUM_CODECS && M > 0 && N > 0 && K > 0 && (K & 7) == 0 &&
         K % kq_geom(codec).wpb == 0;
}

// K steps per workgroup of a dense call: K is split until about 512 workgroups exist (calls of more than 32 rows
// with 256 tiles or more run unsplit), with the partial sums held to 64 MiB.
static int any_steps_per_split(int M, int N, int K, int dt) {
  const int mt = any_dense_mt(M, dt);
  const int64_t tiles = (int64_t)((N + AM_BN - 1) / AM_BN) * ((M + 32 * mt - 1) / (32 * mt));
  const int nsteps = (K + AM_STEP - 1) / AM_STEP;
  int64_t want = (M > 32 && tiles >= 256) ? 1 : (512 + tiles - 1) / tiles;
  const int64_t cap = ((int64_t)64 << 20) / ((int64_t)M * N * 4);
  if (want > cap) want = cap;
  if (want > nsteps) want = nsteps;
  if (want < 1) want = 1;
  return (int)((nsteps + want - 1) / want);
}

// f32 partial sums of the split-K call (0: no split)
size_t kq_anymma_dense_workspace_bytes(int M, int N, int K, int dtype) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int nsteps = (K + AM_STEP - 1) / AM_STEP, per = any_steps_per_split(M, N, K, dtype);
  const int splits = (nsteps + per - 1) / per;
  return splits > 1 ? (size_t)splits * M * N * 4 : 0;
}

// Dense matmul, any codec; K is split across workgroups when the call has few tiles and `ws` holds
// kq_anymma_dense_workspace_bytes.
int kq_launch_anymma_dense(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype,
                           void* ws, size_t ws_bytes, hipStream_t s) {
  if (!kq_anymma_supported(M, N, K, codec) || (reinterpret_cast<uintptr_t>(x) & 15)) return KQ_ERR_UNSUPPORTED;
  AnyArgs a{};
  a.x = x;
  a.w = w;
  a.y = y;
  a.grids = kq_device_grids();
  if (!a.grids) return KQ_ERR_HIP;
  a.M = M;
  a.N = N;
  a.K = K;
  a.x_div = 1;
  a.steps_per_split = (K + AM_STEP - 1) / AM_STEP;
  const size_t need = kq_anymma_dense_workspace_bytes(M, N, K, dtype);
  if (need && ws && ws_bytes >= need && !(reinterpret_cast<uintptr_t>(ws) & 15)) {
    a.partial = static_cast<float*>(ws);
    a.steps_per_split = any_steps_per_split(M, N, K, dtype);
  }
  return dispatch_any(codec, a, 0, dtype, 0, 1, s);
}

// Workspace of the batched MoE path: sorted pair list, segment table, segment count.
size_t kq_anymma_moe_workspace_bytes(int P, int E) {
  return align256((size_t)P * 4) + align256(((size_t)E + P / SEG_M + 1) * sizeof(Segment)) + 256;
}

bool kq_anymma_moe_supported(int P, int E, int N, int K, int codec) {
  return kq_anymma_supported(1, N, K, codec) && P > 16 && E <= 4096 && (int64_t)E + P / SEG_M < 65535;
}

// x: [rows][K]; pair p reads row p / x_div and expert idx[p]; out [P][N].
int kq_launch_anymma_moe(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* idx, const float* bias,
                         const float* bias2, void* out, int P, int E, int N, int K, int x_div, int64_t w_expert_stride,
                         int glu, int act, float limit, float alpha, int codec, int dtype, void* ws, KqOutMap om,
                         hipStream_t s) {
  if (!kq_anymma_moe_supported(P, E, N, K, codec) || (reinterpret_cast<uintptr_t>(x) & 15) ||
      (reinterpret_cast<uintptr_t>(ws) & 255))
    return KQ_ERR_UNSUPPORTED;
  uint8_t* p = static_cast<uint8_t*>(ws);
  int* order = reinterpret_cast<int*>(p);
  Segment* segs = reinterpret_cast<Segment*>(p + align256((size_t)P * 4));
  int* nseg = reinterpret_cast<int*>(p + align256((size_t)P * 4) + align256(((size_t)E + P / SEG_M + 1) * sizeof(Segment)));
  int rc = kq_launch_moe_sort(idx, P, E, order, segs, nseg, s);
  if (rc) return rc;
  AnyArgs a{};
  a.x = x;
  a.w = w;
  a.w2 = w2;
  a.y = out;
  a.bias = bias;
  a.bias2 = bias2;
  a.order = order;
  a.segs = segs;
  a.nseg = nseg;
  a.grids = kq_device_grids();
  if (!a.grids) return KQ_ERR_HIP;
  a.M = P;
  a.N = N;
  a.K = K;
  a.x_div = x_div < 1 ? 1 : x_div;
  a.act = act;
  a.w_expert_stride = w_expert_stride;
  a.limit = limit;
  a.alpha = alpha;
  a.om = om;
  return dispatch_any(codec, a, glu ? 2 : 1, dtype, P, E, s);
}
