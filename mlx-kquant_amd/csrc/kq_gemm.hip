// Prefill GEMM for q4_k / q5_k: y[M,N] = x[M,K] . W^T with M large, on the f16 matrix cores, exact
// in the weights.
//
// Numerics.  A weight is d*sc_j*q - dmin*m_j.  The B operand of the MFMA is the exact integer
// sc_j*q (<= 63*15 or 63*31 < 2048, so exact in f16), built from the wire nibbles with one
// v_and_or_b32 (0x6400 | q = 1024 + q) and one v_pk_fma_f16 per pair; one f32 accumulator set
// collects a whole 256-weight superblock and is folded into the running sum with a single
// multiply by d per superblock.  The -dmin*m_j term is a rank-8 update per superblock,
// sum_j m_j X_j[m] with X_j the sub-block sums of x: it runs as one extra MFMA whose A operand
// holds X_j split into two f16 halves (hi + lo, 22 bits) and whose B operand holds the 6-bit
// m_j.  Activations are converted to f16 once by a prepass (scaled per row by a power of two so
// bf16 inputs neither overflow nor lose bits) that also emits the X_j halves.  Products are exact
// and accumulate in f32, so the result differs from the f32 reference only by summation order.
//
// Tiling.  Workgroup = 4 waves, tile 128 (M) x 128 (N), one 256-wide superblock of K per step; each
// wave owns all 128 rows x 32 columns (4 accumulator tiles of v_mfma_f32_32x32x16_f16), so every
// weight is decoded by exactly one wave of the workgroup.  Wire bytes and activations are fetched
// with coalesced 16-byte loads into registers one step ahead and parked in LDS (activation rows
// padded by 16 bytes, wire rows 144 bytes apart: both strides are odd multiples of 16 bytes, which
// keeps the row-per-lane ds_read_b128 fragment fetch free of bank conflicts).
#include <type_traits>

#include "kq_decode.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}
__device__ __forceinline__ uint32_t opaque_vgpr(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}
__device__ __forceinline__ uint32_t opaque_sgpr(uint32_t v) {
  asm volatile("" : "+s"(v));
  return v;
}

// ------------------------------------------------------------------ activation prepass
// One workgroup per row m (rows >= M are written as zeros).  Outputs:
//   xh   f16 [Mpad][K]            x * 2^-e[m], k permuted inside 8-groups to k0 k2 k1 k3 k4 k6 k5 k7
//   xhl  f16 [Mpad][K/256][16]    per superblock: hi_j (8) then lo_j (8) with X_j = 32 (hi_j + lo_j)
//   rs   f32 [Mpad]               2^e[m]
constexpr int PP_THREADS = 256;

template <int DT>
__global__ __launch_bounds__(PP_THREADS) void gemm_prepass_kernel(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
                                                                  _Float16* __restrict__ xhl, float* __restrict__ rs,
                                                                  int M, int K) {
  __shared__ float red[PP_THREADS / 64];
  const int m = blockIdx.x, tid = threadIdx.x;
  const int ngroups = K >> 3;
  _Float16* xo = xh + (size_t)m * K;
  _Float16* ho = xhl + (size_t)m * (K >> 8) * 16;
  if (m >= M) {
    for (int g = tid; g < ngroups; g += PP_THREADS) *reinterpret_cast<u32x4*>(xo + 8 * g) = u32x4{0, 0, 0, 0};
    for (int i = tid; i < (K >> 8) * 16; i += PP_THREADS) ho[i] = (_Float16)0.f;
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
    const f16x8 o = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
    *reinterpret_cast<f16x8*>(xo + 8 * g) = o;
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) s += (float)h[e];
    s += __shfl_xor(s, 1);
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

// ------------------------------------------------------------------ main kernel
constexpr int GM_THREADS = 256;
constexpr int BM = 128, BN = 128;
constexpr int A_STRIDE = 512 + 16;  // bytes per activation row of one K step in LDS
constexpr int A_BYTES = BM * A_STRIDE;
constexpr int APT = BM * 32 / GM_THREADS;  // 16-byte activation pieces per thread per step (16)

template <int C>
struct WireGeom {
  static constexpr int BPB = C == KQ_Q4_K ? 144 : 176;
  static constexpr int PPR = BPB / 16;                                  // 16-byte pieces per row and step
  static constexpr int WPT = (BN * PPR + GM_THREADS - 1) / GM_THREADS;  // pieces per thread per step
  static constexpr int QS = C == KQ_Q4_K ? 16 : 48;                     // offset of the nibble array
};

template <int C, int DT>
__global__ __launch_bounds__(GM_THREADS, 1) void kquant_gemm_kernel(const _Float16* __restrict__ xh,
                                                                    const _Float16* __restrict__ xhl,
                                                                    const float* __restrict__ rs,
                                                                    const uint8_t* __restrict__ w,
                                                                    uint16_t* __restrict__ y, int M, int N, int K,
                                                                    int mtiles) {
  using G = WireGeom<C>;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* a_lds = smem;                          // [BM][A_STRIDE]
  uint8_t* b_lds = smem + A_BYTES;                // [BN][BPB]
  uint8_t* h_lds = b_lds + BN * G::BPB;           // [BM][32] X halves of the step

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, kg = lane >> 5;
  // consecutive workgroups share the weight columns (m fastest)
  const int mt = blockIdx.x % mtiles, nt = blockIdx.x / mtiles;
  const int m0 = mt * BM, n0 = nt * BN;
  const int nsb = K >> 8;
  const size_t row_bytes = (size_t)nsb * G::BPB;
  const int nrows = N - n0 < BN ? N - n0 : BN;

  // piece maps: activations piece i = tid + 256 t -> (row i / 32, piece i % 32); wire piece -> (row i / PPR, i % PPR)
  const int a_row = tid >> 5, a_pc = tid & 31;  // + 8 rows per t
  uint32_t w_goff[G::WPT], w_loff[G::WPT];
  {
    int r = tid / G::PPR, pc = tid % G::PPR;
    StaticFor<G::WPT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      const bool ok = r < nrows;  // rows past N and the pieces past the tile re-read the tile start
      w_goff[T] = ok ? (uint32_t)r * (uint32_t)row_bytes + 16 * pc : 0;
      w_loff[T] = r < BN ? (uint32_t)r * G::BPB + 16 * pc : 0xffffffffu;
      r += GM_THREADS / G::PPR;
      pc += GM_THREADS % G::PPR;
      if (pc >= G::PPR) {
        pc -= G::PPR;
        r++;
      }
    });
  }
  const uint8_t* wtile = w + (size_t)n0 * row_bytes;
  const _Float16* xtile = xh + (size_t)m0 * K;
  const _Float16* htile = xhl + (size_t)m0 * nsb * 16;

  u32x4 areg[APT], wreg[G::WPT], hreg;
  auto issue = [&](int sb) {
    StaticFor<APT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      areg[T] = *reinterpret_cast<const u32x4*>(xtile + (size_t)(a_row + 8 * T) * K + 256 * sb + 8 * a_pc);
    });
    StaticFor<G::WPT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      wreg[T] = *reinterpret_cast<const u32x4*>(wtile + (size_t)sb * G::BPB + w_goff[T]);
    });
    // X halves: 128 rows x 32 bytes = 256 pieces of 16 bytes
    hreg = *reinterpret_cast<const u32x4*>(htile + ((size_t)(tid >> 1) * nsb + sb) * 16 + 8 * (tid & 1));
  };
  auto park = [&]() {
    StaticFor<APT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      *reinterpret_cast<u32x4*>(a_lds + (a_row + 8 * T) * A_STRIDE + 16 * a_pc) = areg[T];
    });
    StaticFor<G::WPT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      if (w_loff[T] != 0xffffffffu) *reinterpret_cast<u32x4*>(b_lds + w_loff[T]) = wreg[T];
    });
    *reinterpret_cast<u32x4*>(h_lds + 16 * tid) = hreg;
  };

  f32x16 acc[4];
#pragma unroll
  for (int t = 0; t < 4; t++) acc[t] = f32x16{0};

  const uint32_t magic = opaque_vgpr(0x64006400u);
  const uint32_t mask_lo = opaque_sgpr(0x000f000fu), mask_hi = opaque_sgpr(0x00f000f0u);
  const uint8_t* b_lane = b_lds + (wave * 32 + l32) * G::BPB;
  const uint8_t* a_lane = a_lds + l32 * A_STRIDE + 32 * kg;

  issue(0);
  for (int sb = 0; sb < nsb; sb++) {
    if (sb > 0) lds_barrier();  // everyone is done reading the previous step
    park();
    if (sb + 1 < nsb) issue(sb + 1);
    lds_barrier();

    // ---- per-column scales of this superblock
    const uint4 hdr = *reinterpret_cast<const uint4*>(b_lane);
    const float d = kq::h2f((uint16_t)(hdr.x & 0xffff));
    const float dmin32 = kq::h2f((uint16_t)(hdr.x >> 16)) * 32.0f;
    const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
    const uint32_t scw[2] = {s0 & 0x3f3f3f3fu, (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u)};
    const uint32_t mnw[2] = {s1 & 0x3f3f3f3fu, ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u)};

    f32x16 part[4];
    // ---- main products: 8 sub-blocks x 2 K-steps of 16
#pragma unroll
    for (int g = 0; g < 4; g++) {
      const uint4 qv = *reinterpret_cast<const uint4*>(b_lane + G::QS + 32 * g + 16 * kg);
      const uint32_t qw[4] = {qv.x, qv.y, qv.z, qv.w};
      const uint32_t qw8[4] = {qw[0] >> 8, qw[1] >> 8, qw[2] >> 8, qw[3] >> 8};
      uint32_t hb[4] = {0, 0, 0, 0};  // q5_k: fifth bits of this lane's 16 weights, positioned per pair
      if constexpr (C == KQ_Q5_K) {
        const uint4 hv = *reinterpret_cast<const uint4*>(b_lane + 16 + 16 * kg);
        hb[0] = hv.x;
        hb[1] = hv.y;
        hb[2] = hv.z;
        hb[3] = hv.w;
      }
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int j = 2 * g + h;
        const float scf = (float)((scw[j >> 2] >> (8 * (j & 3))) & 0xff);
        // low nibbles read 1024 + q, high nibbles (in place) 1024 + 16 q: fold the 16 into the scale
        const _Float16 sch = (_Float16)(h ? scf * 0.0625f : scf);
        const _Float16 off = (_Float16)(-(h ? 64.0f : 1024.0f) * scf);
        const f16x2 scp = {sch, sch}, offp = {off, off};
#pragma unroll
        for (int s = 0; s < 2; s++) {
          const uint32_t mask = h ? mask_hi : mask_lo;
          uint32_t fr[4] = {(qw[2 * s] & mask) | magic, (qw8[2 * s] & mask) | magic, (qw[2 * s + 1] & mask) | magic,
                            (qw8[2 * s + 1] & mask) | magic};
          f16x2 bq[4];
#pragma unroll
          for (int e = 0; e < 4; e++)  // one rounding: (1024 + q) * sc - 1024 * sc = sc * q exactly
            bq[e] = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, fr[e]), scp, offp);
          if constexpr (C == KQ_Q5_K) {
            // fifth bit of weight (j, i) is bit j of qh[i]; this lane's bytes are qh[16 kg + 8 s + 0..7]
            const _Float16 s16 = (_Float16)(16.0f * scf);
            const uint32_t hwa = hb[2 * s] >> j, hwb = hb[2 * s + 1] >> j;
            const _Float16 z = (_Float16)0.f;
            const f16x2 add[4] = {{(hwa & 1) ? s16 : z, (hwa & 0x10000) ? s16 : z},
                                  {(hwa & 0x100) ? s16 : z, (hwa & 0x1000000) ? s16 : z},
                                  {(hwb & 1) ? s16 : z, (hwb & 0x10000) ? s16 : z},
                                  {(hwb & 0x100) ? s16 : z, (hwb & 0x1000000) ? s16 : z}};
#pragma unroll
            for (int e = 0; e < 4; e++) bq[e] += add[e];
          }
          const f16x8 b = {bq[0][0], bq[0][1], bq[1][0], bq[1][1], bq[2][0], bq[2][1], bq[3][0], bq[3][1]};
#pragma unroll
          for (int t = 0; t < 4; t++) {
            const f16x8 a = *reinterpret_cast<const f16x8*>(a_lane + t * 32 * A_STRIDE + 64 * j + 16 * s);
            if (j == 0 && s == 0)
              part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, f32x16{0}, 0, 0, 0);
            else
              part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, part[t], 0, 0, 0);
          }
        }
      }
    }
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[t][i] = fmaf(d, part[t][i], acc[t][i]);

    // ---- mins: sum_j m_j X_j = 32 sum_j m_j (hi_j + lo_j); K slots 0..7 = hi, 8..15 = lo
    _Float16 mj[8];
#pragma unroll
    for (int j = 0; j < 8; j++) mj[j] = (_Float16)(float)((mnw[j >> 2] >> (8 * (j & 3))) & 0xff);
    const f16x8 bm = {mj[0], mj[1], mj[2], mj[3], mj[4], mj[5], mj[6], mj[7]};
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const f16x8 a = *reinterpret_cast<const f16x8*>(h_lds + (t * 32 + l32) * 32 + 16 * kg);
      part[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, bm, f32x16{0}, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[t][i] = fmaf(-dmin32, part[t][i], acc[t][i]);
  }

  // ---- epilogue: undo the per-row activation scale, round once, store
  const int n = n0 + wave * 32 + l32;
#pragma unroll
  for (int t = 0; t < 4; t++) {
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

template <int C, int DT>
int launch_gemm(const void* x, const uint8_t* w, void* y, int M, int N, int K, void* ws, hipStream_t s) {
  using G = WireGeom<C>;
  const int mtiles = (M + BM - 1) / BM, ntiles = (N + BN - 1) / BN;
  const int mpad = mtiles * BM, nsb = K >> 8;
  _Float16* xh = static_cast<_Float16*>(ws);
  _Float16* xhl = xh + (size_t)mpad * K;
  float* rs = reinterpret_cast<float*>(xhl + (size_t)mpad * nsb * 16);
  hipLaunchKernelGGL((gemm_prepass_kernel<DT>), dim3(mpad), dim3(PP_THREADS), 0, s, static_cast<const uint16_t*>(x), xh,
                     xhl, rs, M, K);
  KQ_HIP_CHECK(hipGetLastError());
  const size_t lds = A_BYTES + BN * G::BPB + BM * 32;
  auto kern = kquant_gemm_kernel<C, DT>;
  static bool attr_set = false;
  if (!attr_set) {
    KQ_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(mtiles * ntiles), dim3(GM_THREADS), lds, s, xh, xhl, rs, w, static_cast<uint16_t*>(y), M,
                     N, K, mtiles);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

}  // namespace

size_t kq_gemm_workspace_bytes(int M, int K) {
  const size_t mpad = (size_t)((M + BM - 1) / BM) * BM;
  return mpad * K * 2 + mpad * (K >> 8) * 32 + mpad * 4 + 256;
}

bool kq_gemm_supported(int M, int N, int K, int codec) {
  return (codec == KQ_Q4_K || codec == KQ_Q5_K) && M > 8 && K > 0 && (K & 255) == 0 && N > 0;
}

int kq_launch_gemm(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                   hipStream_t s) {
  if (!kq_gemm_supported(M, N, K, codec)) return KQ_ERR_UNSUPPORTED;
  if ((reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(ws) & 15))
    return KQ_ERR_UNSUPPORTED;
  if (codec == KQ_Q4_K)
    return dtype == KQ_F16 ? launch_gemm<KQ_Q4_K, KQ_F16>(x, w, y, M, N, K, ws, s)
                           : launch_gemm<KQ_Q4_K, KQ_BF16>(x, w, y, M, N, K, ws, s);
  return dtype == KQ_F16 ? launch_gemm<KQ_Q5_K, KQ_F16>(x, w, y, M, N, K, ws, s)
                         : launch_gemm<KQ_Q5_K, KQ_BF16>(x, w, y, M, N, K, ws, s);
}
