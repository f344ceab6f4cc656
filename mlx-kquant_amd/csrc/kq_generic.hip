// Bit-exact dequantize kernel and the generic (any codec, any shape) matmul kernels built on
// the reference-order decoders of kq_decode.h.  Compile with -ffp-contract=off.
//
// dequantize: a workgroup stages a run of consecutive wire blocks into LDS with coalesced
// dword loads, then every thread decodes 8-weight groups from LDS and issues one 16-byte
// (f16/bf16) or two 16-byte (f32) stores.  HBM-bound on the output write.
#include <type_traits>

#include "kq_decode.h"
#include "kq_epilogue.h"

namespace {

constexpr int DQ_THREADS = 256;
// Weights per workgroup: 4096 (16 / 64 / 128 blocks), or 16384 for superblock codecs on tensors large enough
// to give every CU a few such workgroups (measured 4 - 9 % faster there, slower on small tensors and on the
// 32-weight codecs, whose staged bytes then cost occupancy).
constexpr int DQ_WEIGHTS = 4096, DQ_WEIGHTS_BIG = 16384;

template <int C, int DT, int WEIGHTS>
__global__ __launch_bounds__(DQ_THREADS) void dequantize_kernel(const uint8_t* __restrict__ w,
                                                                void* __restrict__ out, uint64_t num_blocks,
                                                                const uint8_t* __restrict__ grids) {
  constexpr int WPB = kq_geom(C).wpb, BPB = kq_geom(C).bpb;
  constexpr int NBLK = WEIGHTS / WPB;  // multiple of 16 -> chunk bytes are a multiple of 16
  constexpr int GPB = WPB / 8;            // 8-weight groups per block
  __shared__ __attribute__((aligned(16))) uint8_t lds[NBLK * BPB];

  const uint64_t blk0 = (uint64_t)blockIdx.x * NBLK;
  const int nblk = (int)((num_blocks - blk0 < (uint64_t)NBLK) ? (num_blocks - blk0) : NBLK);
  const int nbytes = nblk * BPB;
  const uint8_t* src = w + blk0 * BPB;
  if ((((uintptr_t)src) & 3) == 0) {
    const int nw = nbytes >> 2;
    for (int i = threadIdx.x; i < nw; i += DQ_THREADS)
      reinterpret_cast<uint32_t*>(lds)[i] = reinterpret_cast<const uint32_t*>(src)[i];
    for (int i = (nw << 2) + threadIdx.x; i < nbytes; i += DQ_THREADS) lds[i] = src[i];
  } else {
    for (int i = threadIdx.x; i < nbytes; i += DQ_THREADS) lds[i] = src[i];
  }
  __syncthreads();

  const int ngroups = nblk * GPB;
  for (int gi = threadIdx.x; gi < ngroups; gi += DQ_THREADS) {
    const int b = gi / GPB, g = gi % GPB;
    float v[8];
    kq::decode8<C>(lds + b * BPB, g, grids, v);
    const uint64_t o = (blk0 + b) * WPB + 8 * g;
    if constexpr (DT == KQ_F32) {
      float4* p = reinterpret_cast<float4*>(static_cast<float*>(out) + o);
      p[0] = make_float4(v[0], v[1], v[2], v[3]);
      p[1] = make_float4(v[4], v[5], v[6], v[7]);
    } else {
      uint32_t r[4];
      for (int t = 0; t < 4; t++) {
        uint16_t lo = DT == KQ_F16 ? kq::f2f16(v[2 * t]) : kq::f2bf16(v[2 * t]);
        uint16_t hi = DT == KQ_F16 ? kq::f2f16(v[2 * t + 1]) : kq::f2bf16(v[2 * t + 1]);
        r[t] = (uint32_t)lo | ((uint32_t)hi << 16);
      }
      *reinterpret_cast<uint4*>(static_cast<uint16_t*>(out) + o) = make_uint4(r[0], r[1], r[2], r[3]);
    }
  }
}

// ---------------------------------------------------------------- generic matmul (VALU)
// y[m, n] = sum_k x[m, k] * W[n, k]: one wave per output row n, lanes stride over the row's
// 8-weight groups, f32 FMA, butterfly reduce.  Correct for every codec and K; the tuned MFMA
// kernels take over for the shapes that matter.
constexpr int GV_THREADS = 256;

template <int DT>
__device__ __forceinline__ void load_x8(const void* x, size_t off, float* v) {
  const uint16_t* p = static_cast<const uint16_t*>(x) + off;
  for (int t = 0; t < 8; t++) v[t] = DT == KQ_F16 ? kq::h2f(p[t]) : kq::bf162f(p[t]);
}
template <int DT>
__device__ __forceinline__ void store_y(void* y, size_t off, float v) {
  static_cast<uint16_t*>(y)[off] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
}

template <int C, int DT, int MT>
__global__ __launch_bounds__(GV_THREADS) void gemv_generic_kernel(const void* __restrict__ x,
                                                                  const uint8_t* __restrict__ w,
                                                                  void* __restrict__ y, int M, int N, int K,
                                                                  const uint8_t* __restrict__ grids) {
  constexpr int WPB = kq_geom(C).wpb, BPB = kq_geom(C).bpb, GPB = WPB / 8;
  const int lane = threadIdx.x & 63;
  const int wave = (blockIdx.x * GV_THREADS + threadIdx.x) >> 6;
  const int nwaves = (gridDim.x * GV_THREADS) >> 6;
  const int m0 = blockIdx.y * MT;
  const size_t row_bytes = (size_t)(K / WPB) * BPB;
  const int ngroups = K / 8;
  for (int n = wave; n < N; n += nwaves) {
    const uint8_t* wr = w + (size_t)n * row_bytes;
    float acc[MT];
    for (int m = 0; m < MT; m++) acc[m] = 0.f;
    for (int gi = lane; gi < ngroups; gi += 64) {
      float wv[8];
      kq::decode8<C>(wr + (size_t)(gi / GPB) * BPB, gi % GPB, grids, wv);
      for (int m = 0; m < MT; m++) {
        if (m0 + m < M) {
          float xv[8];
          load_x8<DT>(x, (size_t)(m0 + m) * K + 8 * (size_t)gi, xv);
          for (int t = 0; t < 8; t++) acc[m] = fmaf(xv[t], wv[t], acc[m]);
        }
      }
    }
    for (int m = 0; m < MT; m++) {
      float v = acc[m];
      for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
      if (lane == 0 && m0 + m < M) store_y<DT>(y, (size_t)(m0 + m) * N + n, v);
    }
  }
}

// y[m, n] = sum_k x[m, k] * W[k, n] (transpose = false: W decodes to [K, N]).  One thread per
// (m, 8 consecutive n); walks all K wire rows.  Grid z = gathered item: item b reads activation
// matrix lhs[b] and expert rhs[b] (both null for the plain op).
template <int C, int DT>
__global__ __launch_bounds__(GV_THREADS) void gemm_nt_generic_kernel(const void* __restrict__ x,
                                                                     const uint8_t* __restrict__ w,
                                                                     void* __restrict__ y, int M, int N, int K,
                                                                     const uint8_t* __restrict__ grids,
                                                                     const uint32_t* __restrict__ lhs,
                                                                     const uint32_t* __restrict__ rhs,
                                                                     int64_t x_batch_stride, int64_t w_expert_stride,
                                                                     int E) {
  constexpr int WPB = kq_geom(C).wpb, BPB = kq_geom(C).bpb, GPB = WPB / 8;
  const int gi = blockIdx.x * GV_THREADS + threadIdx.x;  // 8-column group
  const int item = blockIdx.z;
  if (gi >= N / 8) return;
  const uint32_t e = rhs ? rhs[item] : 0u;
  if (e >= (uint32_t)E) return;  // an expert id outside the stack: the entry's output is left untouched
  const size_t row_bytes = (size_t)(N / WPB) * BPB;
  const uint8_t* wb = w + (size_t)e * (size_t)w_expert_stride + (size_t)(gi / GPB) * BPB;
  for (int m = blockIdx.y; m < M; m += gridDim.y) {  // the grid's y extent is capped at 65535
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const uint16_t* xr =
        static_cast<const uint16_t*>(x) + (lhs ? (size_t)lhs[item] * (size_t)x_batch_stride : 0) + (size_t)m * K;
    for (int k = 0; k < K; k++) {
      float wv[8];
      kq::decode8<C>(wb + (size_t)k * row_bytes, gi % GPB, grids, wv);
      float xv = DT == KQ_F16 ? kq::h2f(xr[k]) : kq::bf162f(xr[k]);
      for (int t = 0; t < 8; t++) acc[t] = fmaf(xv, wv[t], acc[t]);
    }
    for (int t = 0; t < 8; t++) store_y<DT>(y, ((size_t)item * M + m) * N + 8 * (size_t)gi + t, acc[t]);
  }
}

// One wave per (item p, output row n).  Item p reads activation matrix x[lhs[p]] (or p / x_div
// when lhs is null) and expert rhs[p]; with GLU it also reads the `up` stack and applies the
// fused epilogue (metal/mlx/backend/metal/kernels/kq_moe_glu_kq.h:34-60 of the reference).
struct GatherArgs {
  const void* x;
  const uint8_t* w;
  const uint8_t* w2;  // up stack (GLU) or null
  const uint32_t* lhs;
  const uint32_t* rhs;
  const float* bias;
  const float* bias2;
  void* out;
  int B, M, N, K, x_div;
  int64_t x_batch_stride, w_expert_stride;
  int act;
  float limit, alpha;
  KqOutMap om;
  int E;  // entries whose expert id is >= E are skipped (their output rows stay untouched)
};

template <int C, int DT, int MT, bool GLU>
__global__ __launch_bounds__(GV_THREADS) void gather_generic_kernel(GatherArgs a, const uint8_t* __restrict__ grids) {
  constexpr int WPB = kq_geom(C).wpb, BPB = kq_geom(C).bpb, GPB = WPB / 8;
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * GV_THREADS + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * GV_THREADS) >> 6;
  const int m0 = blockIdx.y * MT;
  const size_t row_bytes = (size_t)(a.K / WPB) * BPB;
  const int ngroups = a.K / 8;
  for (int64_t item = wave; item < (int64_t)a.B * a.N; item += nwaves) {
    const int p = (int)(item / a.N), n = (int)(item % a.N);
    const uint32_t e = a.rhs[p];
    if (e >= (uint32_t)a.E) continue;  // wave-uniform
    const int64_t xi = a.lhs ? (int64_t)a.lhs[p] : (int64_t)(p / a.x_div);
    const size_t xoff = (size_t)(xi * a.x_batch_stride);
    const uint8_t* wr = a.w + (int64_t)e * a.w_expert_stride + (size_t)n * row_bytes;
    const uint8_t* wr2 = GLU ? a.w2 + (int64_t)e * a.w_expert_stride + (size_t)n * row_bytes : nullptr;
    float acc[MT], acc2[MT];
    for (int m = 0; m < MT; m++) acc[m] = acc2[m] = 0.f;
    for (int gi = lane; gi < ngroups; gi += 64) {
      float wv[8], wv2[8];
      kq::decode8<C>(wr + (size_t)(gi / GPB) * BPB, gi % GPB, grids, wv);
      if constexpr (GLU) kq::decode8<C>(wr2 + (size_t)(gi / GPB) * BPB, gi % GPB, grids, wv2);
      for (int m = 0; m < MT; m++) {
        if (m0 + m < a.M) {
          float xv[8];
          load_x8<DT>(a.x, xoff + (size_t)(m0 + m) * a.K + 8 * (size_t)gi, xv);
          for (int t = 0; t < 8; t++) {
            acc[m] = fmaf(xv[t], wv[t], acc[m]);
            if constexpr (GLU) acc2[m] = fmaf(xv[t], wv2[t], acc2[m]);
          }
        }
      }
    }
    for (int m = 0; m < MT; m++) {
      float v = acc[m], v2 = acc2[m];
      for (int off = 32; off > 0; off >>= 1) {
        v += __shfl_xor(v, off);
        if constexpr (GLU) v2 += __shfl_xor(v2, off);
      }
      if (lane == 0 && m0 + m < a.M) {
        if (a.bias) v += a.bias[(size_t)e * a.N + n];
        if constexpr (GLU) {
          if (a.bias2) v2 += a.bias2[(size_t)e * a.N + n];
          v = kq::glu_epilogue(a.act, v, v2, a.limit, a.alpha);
        }
        kq::store_result<DT>(a.out, a.om, ((size_t)kq::out_row(a.om, p) * a.M + (m0 + m)) * a.N + n, v);
      }
    }
  }
}

// Score-weighted slot sum in one launch (decode-sized calls):
// out[t][n] = T(sum_s scores[t][s] (x[t][s] . W[idx[t][s]][n] + bias[idx[t][s]][n])), f32 throughout.
// With a shared expert the last slot reads row n of the one-matrix stack shexp_w in codec C2 (the expert codec,
// q6_k or q8_0).  Slots whose expert id is >= E add nothing.
struct MixArgs {
  const void* x;           // [T][S][K]
  const uint8_t* w;        // [E][N][row bytes]
  const uint8_t* shexp_w;  // [N][row bytes of shexp_codec] or null
  const uint32_t* idx;     // [T][S - 1] with a shared expert, else [T][S]
  const float* scores;     // [T][S]
  const float* bias;       // [E][N] or null
  void* out;               // [T][N]
  int T, S, E, N, K, shexp_codec;
  int64_t w_expert_stride;
};

// this lane's share of x . w over one weight row (no reduction across the wave)
template <int C, int DT>
__device__ __forceinline__ float mix_row_dot(const uint8_t* wr, const void* x, size_t xoff, int ngroups, int lane,
                                             const uint8_t* grids) {
  constexpr int WPB = kq_geom(C).wpb, BPB = kq_geom(C).bpb, GPB = WPB / 8;
  float acc = 0.f;
  for (int gi = lane; gi < ngroups; gi += 64) {
    float wv[8], xv[8];
    kq::decode8<C>(wr + (size_t)(gi / GPB) * BPB, gi % GPB, grids, wv);
    load_x8<DT>(x, xoff + 8 * (size_t)gi, xv);
    for (int t = 0; t < 8; t++) acc = fmaf(xv[t], wv[t], acc);
  }
  return acc;
}

// One workgroup (four waves) per (token t, output row n): wave w takes the slots w, w + 4, ...; a lane sums
// score * (its share of the dot product) over the wave's slots, the wave reduces once, and the four wave sums are
// added in wave order.
template <int C, int DT>
__global__ __launch_bounds__(GV_THREADS) void gather_mix_generic_kernel(MixArgs a, const uint8_t* __restrict__ grids) {
  __shared__ float part[GV_THREADS / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const size_t row_bytes = (size_t)(a.K / kq_geom(C).wpb) * kq_geom(C).bpb;
  const int ngroups = a.K / 8;
  const int routed = a.shexp_w ? a.S - 1 : a.S;
  for (int64_t item = blockIdx.x; item < (int64_t)a.T * a.N; item += gridDim.x) {
    const int t = (int)(item / a.N), n = (int)(item % a.N);
    float tot = 0.f, btot = 0.f;
    for (int sl = wave; sl < a.S; sl += GV_THREADS / 64) {  // wave-uniform control flow
      const size_t xoff = ((size_t)t * a.S + sl) * a.K;
      const float score = a.scores[(size_t)t * a.S + sl];
      float v;
      if (sl < routed) {
        const uint32_t e = a.idx[(size_t)t * routed + sl];
        if (e >= (uint32_t)a.E) continue;
        v = mix_row_dot<C, DT>(a.w + (int64_t)e * a.w_expert_stride + (size_t)n * row_bytes, a.x, xoff, ngroups, lane, grids);
        if (a.bias) btot = fmaf(score, a.bias[(size_t)e * a.N + n], btot);
      } else if (a.shexp_codec == KQ_Q6_K) {
        v = mix_row_dot<KQ_Q6_K, DT>(a.shexp_w + (size_t)n * (a.K / 256) * 210, a.x, xoff, ngroups, lane, grids);
      } else if (a.shexp_codec == KQ_Q8_0) {
        v = mix_row_dot<KQ_Q8_0, DT>(a.shexp_w + (size_t)n * (a.K / 32) * 34, a.x, xoff, ngroups, lane, grids);
      } else {
        v = mix_row_dot<C, DT>(a.shexp_w + (size_t)n * row_bytes, a.x, xoff, ngroups, lane, grids);
      }
      tot = fmaf(score, v, tot);
    }
    for (int off = 32; off > 0; off >>= 1) tot += __shfl_xor(tot, off);
    if (lane == 0) part[wave] = tot + btot;
    __syncthreads();
    if (threadIdx.x == 0) {
      float r = part[0];
      for (int w = 1; w < GV_THREADS / 64; w++) r += part[w];
      uint16_t* o = static_cast<uint16_t*>(a.out) + (size_t)t * a.N + n;
      *o = DT == KQ_F16 ? kq::f2f16(r) : kq::f2bf16(r);
    }
    __syncthreads();
  }
}

template <int C>
struct MixRun {
  static int run(MixArgs a, int dt, const uint8_t* grids, hipStream_t s) {
    const int64_t items = (int64_t)a.T * a.N;
    if (items == 0) return KQ_OK;
    int64_t nwg = items;
    if (nwg > 65536) nwg = 65536;
    if (dt == KQ_F16)
      hipLaunchKernelGGL((gather_mix_generic_kernel<C, KQ_F16>), dim3((unsigned)nwg), dim3(GV_THREADS), 0, s, a, grids);
    else
      hipLaunchKernelGGL((gather_mix_generic_kernel<C, KQ_BF16>), dim3((unsigned)nwg), dim3(GV_THREADS), 0, s, a, grids);
    KQ_HIP_CHECK(hipGetLastError());
    return KQ_OK;
  }
};

template <template <int> class F, typename... A>
int dispatch_codec(int codec, A... a) {
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
  return kq_set_error(KQ_ERR_INVALID, "unknown codec id %d", codec);
}

template <int C>
struct DequantRun {
  template <int WEIGHTS>
  static int launch(const uint8_t* w, void* out, uint64_t num_blocks, int dt, const uint8_t* grids, hipStream_t s) {
    constexpr int NBLK = WEIGHTS / kq_geom(C).wpb;
    const uint64_t nwg = (num_blocks + NBLK - 1) / NBLK;
    if (nwg == 0) return KQ_OK;
    if (nwg > 0x7fffffffull) return kq_set_error(KQ_ERR_INVALID, "dequantize: tensor too large for one launch");
    dim3 grid((unsigned)nwg), block(DQ_THREADS);
    if (dt == KQ_F32)
      hipLaunchKernelGGL((dequantize_kernel<C, KQ_F32, WEIGHTS>), grid, block, 0, s, w, out, num_blocks, grids);
    else if (dt == KQ_F16)
      hipLaunchKernelGGL((dequantize_kernel<C, KQ_F16, WEIGHTS>), grid, block, 0, s, w, out, num_blocks, grids);
    else
      hipLaunchKernelGGL((dequantize_kernel<C, KQ_BF16, WEIGHTS>), grid, block, 0, s, w, out, num_blocks, grids);
    KQ_HIP_CHECK(hipGetLastError());
    return KQ_OK;
  }
  static int run(const uint8_t* w, void* out, uint64_t num_blocks, int dt, const uint8_t* grids, hipStream_t s) {
    if constexpr (kq_geom(C).wpb == 256) {
      if (num_blocks * 256ull >= (uint64_t)DQ_WEIGHTS_BIG * 256 * 16)
        return launch<DQ_WEIGHTS_BIG>(w, out, num_blocks, dt, grids, s);
    }
    return launch<DQ_WEIGHTS>(w, out, num_blocks, dt, grids, s);
  }
};

template <int C>
struct GemvRun {
  static int run(const void* x, const uint8_t* w, void* y, int M, int N, int K, int dt, const uint8_t* grids,
                 hipStream_t s) {
    int nwg = (N + 3) / 4;
    if (nwg > 8192) nwg = 8192;
    auto go = [&](auto mt) {
      constexpr int MT = decltype(mt)::value;
      dim3 grid(nwg, (M + MT - 1) / MT), block(GV_THREADS);
      if (dt == KQ_F16)
        hipLaunchKernelGGL((gemv_generic_kernel<C, KQ_F16, MT>), grid, block, 0, s, x, w, y, M, N, K, grids);
      else
        hipLaunchKernelGGL((gemv_generic_kernel<C, KQ_BF16, MT>), grid, block, 0, s, x, w, y, M, N, K, grids);
    };
    if (M == 1)
      go(std::integral_constant<int, 1>{});
    else if (M == 2)
      go(std::integral_constant<int, 2>{});
    else if (M <= 4)
      go(std::integral_constant<int, 4>{});
    else
      go(std::integral_constant<int, 8>{});
    KQ_HIP_CHECK(hipGetLastError());
    return KQ_OK;
  }
};

template <int C>
struct GemmNtRun {
  static int run(const void* x, const uint8_t* w, void* y, int M, int N, int K, int dt, const uint8_t* grids,
                 const uint32_t* lhs, const uint32_t* rhs, int B, int64_t xs, int64_t ws, int E, hipStream_t s) {
    dim3 grid((N / 8 + GV_THREADS - 1) / GV_THREADS, M < 65535 ? M : 65535, B), block(GV_THREADS);
    if (dt == KQ_F16)
      hipLaunchKernelGGL((gemm_nt_generic_kernel<C, KQ_F16>), grid, block, 0, s, x, w, y, M, N, K, grids, lhs, rhs, xs,
                         ws, E);
    else
      hipLaunchKernelGGL((gemm_nt_generic_kernel<C, KQ_BF16>), grid, block, 0, s, x, w, y, M, N, K, grids, lhs, rhs, xs,
                         ws, E);
    KQ_HIP_CHECK(hipGetLastError());
    return KQ_OK;
  }
};


template <int C>
struct GatherRun {
  static int run(GatherArgs a, int dt, bool glu, const uint8_t* grids, hipStream_t s) {
    int64_t items = (int64_t)a.B * a.N;
    if (items == 0 || a.M == 0) return KQ_OK;
    int64_t nwg = (items + 3) / 4;
    if (nwg > 16384) nwg = 16384;
    auto go = [&](auto mt, auto g) {
      constexpr int MT = decltype(mt)::value;
      constexpr bool G = decltype(g)::value;
      dim3 grid((unsigned)nwg, (a.M + MT - 1) / MT), block(GV_THREADS);
      if (dt == KQ_F16)
        hipLaunchKernelGGL((gather_generic_kernel<C, KQ_F16, MT, G>), grid, block, 0, s, a, grids);
      else
        hipLaunchKernelGGL((gather_generic_kernel<C, KQ_BF16, MT, G>), grid, block, 0, s, a, grids);
    };
    if (glu) {
      if (a.M == 1) go(std::integral_constant<int, 1>{}, std::true_type{});
      else go(std::integral_constant<int, 4>{}, std::true_type{});
    } else {
      if (a.M == 1) go(std::integral_constant<int, 1>{}, std::false_type{});
      else go(std::integral_constant<int, 8>{}, std::false_type{});
    }
    KQ_HIP_CHECK(hipGetLastError());
    return KQ_OK;
  }
};

}  // namespace

int kq_launch_dequantize(const uint8_t* w, void* out, uint64_t num_blocks, int codec, int out_dtype,
                         hipStream_t s) {
  const uint8_t* grids = kq_device_grids();
  if (!grids) return KQ_ERR_HIP;
  return dispatch_codec<DequantRun>(codec, w, out, num_blocks, out_dtype, grids, s);
}

int kq_launch_gemv_generic(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype,
                           hipStream_t s) {
  const uint8_t* grids = kq_device_grids();
  if (!grids) return KQ_ERR_HIP;
  return dispatch_codec<GemvRun>(codec, x, w, y, M, N, K, dtype, grids, s);
}

int kq_launch_gemm_nt_generic(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec,
                              int dtype, hipStream_t s) {
  const uint8_t* grids = kq_device_grids();
  if (!grids) return KQ_ERR_HIP;
  return dispatch_codec<GemmNtRun>(codec, x, w, y, M, N, K, dtype, grids, (const uint32_t*)nullptr,
                                   (const uint32_t*)nullptr, 1, (int64_t)0, (int64_t)0, 1, s);
}

int kq_launch_gather_nt_generic(const void* x, const uint8_t* w, const uint32_t* lhs, const uint32_t* rhs, void* out,
                                int B, int M, int E, int N, int K, int64_t x_batch_stride, int64_t w_expert_stride,
                                int codec, int dtype, hipStream_t s) {
  const uint8_t* grids = kq_device_grids();
  if (!grids) return KQ_ERR_HIP;
  if (B > 65535) return kq_set_error(KQ_ERR_INVALID, "gather_qmm: the batch must be below 65536 entries");
  return dispatch_codec<GemmNtRun>(codec, x, w, out, M, N, K, dtype, grids, lhs, rhs, B, x_batch_stride,
                                   w_expert_stride, E, s);
}

int kq_launch_gather_generic(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* lhs,
                             const uint32_t* rhs, const float* bias, const float* bias2, void* out, int B, int M,
                             int N, int K, int x_div, int64_t x_batch_stride, int64_t w_expert_stride, int glu,
                             int act, float limit, float alpha, int codec, int dtype, int E, KqOutMap om,
                             hipStream_t s) {
  const uint8_t* grids = kq_device_grids();
  if (!grids) return KQ_ERR_HIP;
  GatherArgs a{x, w, w2, lhs, rhs, bias, bias2, out, B, M, N, K, x_div, x_batch_stride, w_expert_stride,
               act, limit, alpha, om, E};
  return dispatch_codec<GatherRun>(codec, a, dtype, glu != 0, grids, s);
}

// x [T][S][K], idx [T][S] (or [T][S - 1] with a shared expert, whose one-matrix stack shexp_w supplies the last
// slot), scores [T][S], out [T][N].  shexp_codec: the expert codec, q6_k or q8_0.
int kq_launch_gather_mix_generic(const void* x, const uint8_t* w, const uint8_t* shexp_w, const uint32_t* idx,
                                 const float* scores, const float* bias, void* out, int T, int S, int E, int N, int K,
                                 int64_t w_expert_stride, int codec, int shexp_codec, int dtype, hipStream_t s) {
  const uint8_t* grids = kq_device_grids();
  if (!grids) return KQ_ERR_HIP;
  if (shexp_w && shexp_codec != codec && shexp_codec != KQ_Q6_K && shexp_codec != KQ_Q8_0) return KQ_ERR_UNSUPPORTED;
  MixArgs a{x, w, shexp_w, idx, scores, bias, out, T, S, E, N, K, shexp_w ? shexp_codec : codec, w_expert_stride};
  return dispatch_codec<MixRun>(codec, a, dtype, grids, s);
}
