// Tuned skinny-M (decode) kernels: y[M,N] = x[M,K] . W^T for M <= 8, weights streamed once from
// HBM, all multiply-accumulates on the matrix cores.
//
// Mapping (q4_k).  One workgroup (4 waves) owns a tile of up to 32 weight rows; its waves split
// K by superblock.  Inside a wave the weights are the B operand of v_mfma_f32_32x32x16_f16:
// lane l serves weight row n = l % 32 and K-half kg = l / 32, and loads, per 144-byte superblock,
// the 16-byte header (d, dmin, 6-bit scales/mins) plus four 16-byte chunks of the nibble array:
// every HBM byte is fetched by aligned 128-bit loads straight into registers.  Nibbles become
// exact f16 integers with one AND-OR each (0x6400 | q = 1024 + q; high nibbles stay in place and
// read as 1024 + 16 q), so the MFMAs over one 32-weight sub-block return
//     P = sum_k x_k (1024 + s q_k),  s in {1, 16}
// and the sub-block contributes  (d sc / s) P - (1024 d sc / s + dmin m) X,  X = sum_k x_k,
// applied in f32 on the accumulator registers.  Activations are the A operand: the workgroup
// converts x to f16 once (scaled by a power of two so bf16 inputs cannot overflow), keeps it and
// the per-sub-block sums X in LDS, and every wave reads fragments back with ds_read_b128.  M is
// padded to the 32 rows of the MFMA by letting the spare rows alias real ones; only the
// accumulator registers of real rows are carried.
#include <type_traits>

#include "kq_decode.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int SK_WAVES = 4;
constexpr int SK_THREADS = SK_WAVES * 64;
constexpr int SK_MAXM = 8;

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

struct Q4kRaw {
  uint4 hdr;
  uint4 q[4];
};

__device__ __forceinline__ void q4k_load(const uint8_t* __restrict__ blk, int kg, Q4kRaw& r) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const u32x4* p = reinterpret_cast<const u32x4*>(blk);
  auto ld = [](const u32x4* q) {
    const u32x4 v = __builtin_nontemporal_load(q);  // streamed once: keep it out of the caches' way
    return make_uint4(v.x, v.y, v.z, v.w);
  };
  r.hdr = ld(p);
#pragma unroll
  for (int g = 0; g < 4; g++) r.q[g] = ld(p + 1 + 2 * g + kg);
}

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

__device__ __forceinline__ f16x8 q4k_frag(uint32_t wa, uint32_t wa8, uint32_t wb, uint32_t wb8, uint32_t mask,
                                          uint32_t magic) {
  uint4 v;
  v.x = and_or(wa, mask, magic);   // k0, k2
  v.y = and_or(wa8, mask, magic);  // k1, k3
  v.z = and_or(wb, mask, magic);   // k4, k6
  v.w = and_or(wb8, mask, magic);  // k5, k7
  return __builtin_bit_cast(f16x8, v);
}

// One superblock of one 32-row tile: 16 MFMAs + the f32 fix-up on R accumulator registers.
// xs_lane: this lane's A-fragment base (f16 index) for the superblock; xsum: X_j for the
// superblock, [8][XS] floats with XS = row stride.
template <int R, int XS>
__device__ __forceinline__ void q4k_superblock(const Q4kRaw& raw, float xscale, const _Float16* __restrict__ xs_lane,
                                               const float* __restrict__ xsum, float* acc) {
  float mul[8], sub[8];
  q4k_scales(raw.hdr, xscale, mul, sub);
  const uint32_t magic = kq_opaque_vgpr(0x64006400u);
  const uint32_t mask_lo = kq_opaque_sgpr(0x000f000fu), mask_hi = kq_opaque_sgpr(0x00f000f0u);
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
        const f16x8 b = q4k_frag(qw[2 * s], qw8[2 * s], qw[2 * s + 1], qw8[2 * s + 1],
                                 h ? mask_hi : mask_lo, magic);
        p = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, p, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < R; r++) {
        acc[r] = fmaf(mul[j], p[r], acc[r]);
        acc[r] = fmaf(-sub[j], xsum[j * XS + r], acc[r]);
      }
    }
  }
}

// MB = M rounded up to a power of two (1, 2, 4, 8).  Rows of the 32-row A operand beyond MB alias
// row (r % MB); their accumulator rows are never read.
//
// Weight traffic: a tile (rows_per_tile rows x KCH superblocks) is fetched with fully coalesced
// 16-byte loads -- consecutive lanes read consecutive 16-byte pieces of a row, so every wave
// load covers 1 KiB of contiguous HBM -- and parked in LDS with a 16-byte pad per row (row
// stride = 16 mod 256 bytes keeps the row-per-lane ds_read_b128 of the MFMA operand fetch free
// of bank conflicts).  A row-per-lane pattern straight from global memory runs 6x slower: each
// wave load would touch 32 different cache lines for 32 bytes apiece.
template <int DT, int MB>
__global__ __launch_bounds__(SK_THREADS, 2) void q4k_skinny_kernel(const void* __restrict__ x,
                                                                   const uint8_t* __restrict__ w,
                                                                   void* __restrict__ y, int M, int N, int K,
                                                                   int rows_per_tile, int kch) {
  constexpr int R = MB < 4 ? MB : 4;  // accumulator registers carried per lane
  constexpr int MAXP = 18;            // 16-byte pieces per thread per chunk (32 rows x 16 superblocks)
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // layout: wt [rows_per_tile][kch*144 + 16] | xs f16 [MB][kch*256] | xsum f32 [kch*8][MB] | red | scratch
  const int chunk_bytes = kch * 144, wstride = chunk_bytes + 16, kchunk = kch * 256;
  uint8_t* wt = smem;
  _Float16* xs = reinterpret_cast<_Float16*>(smem + rows_per_tile * wstride);
  float* xsum = reinterpret_cast<float*>(smem + rows_per_tile * wstride + (size_t)MB * kchunk * 2);
  float* red = xsum + kch * 8 * MB;
  float* scratch = red + SK_WAVES * R * 64;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n_in = lane & 31, kg = lane >> 5;
  const int nsb = K >> 8;
  const size_t row_bytes = (size_t)nsb * 144;
  const int row0 = blockIdx.x * rows_per_tile;
  const int nrows = (N - row0 < rows_per_tile) ? (N - row0) : rows_per_tile;
  const uint8_t* wtile = w + (size_t)row0 * row_bytes;
  const uint16_t* x16 = static_cast<const uint16_t*>(x);
  // compute-phase row of this lane (clamped: spare lanes re-read row 0, their results are dropped)
  const int crow = n_in < nrows ? n_in : 0;

  float acc[R];
#pragma unroll
  for (int r = 0; r < R; r++) acc[r] = 0.f;

  for (int sb0 = 0; sb0 < nsb; sb0 += kch) {
    const int sbn = (nsb - sb0 < kch) ? (nsb - sb0) : kch;
    const int kc = sbn << 8, k0 = sb0 << 8;
    const int cpr = sbn * 9;  // 16-byte pieces per row in this chunk
    // ---- issue the weight loads: piece i = tid + 256 t -> (row i / cpr, 16-byte piece i % cpr),
    // tracked incrementally; out-of-range pieces re-read piece 0 and are not stored
    u32x4 wreg[MAXP];
    const int step_r = SK_THREADS / cpr, step_c = SK_THREADS % cpr;
    const int r_first = tid / cpr, c_first = tid % cpr;
    {
      int r = r_first, c = c_first;
      const uint8_t* src = wtile + (size_t)sb0 * 144;
      StaticFor<MAXP>::run([&](auto t) {
        const bool ok = r < nrows;
        const size_t off = ok ? (size_t)r * row_bytes + 16 * c : 0;
        wreg[decltype(t)::value] = *reinterpret_cast<const u32x4*>(src + off);
        r += step_r;
        c += step_c;
        if (c >= cpr) {
          c -= cpr;
          r++;
        }
      });
    }

    // ---- stage activations: thread handles 8 consecutive k of one row per step
    if (sb0 > 0) __syncthreads();
    const int ngroups = (kc >> 3) * MB;  // 8-element groups in the chunk
    float amax = 0.f;
    if constexpr (DT == KQ_BF16) {
      for (int gi = tid; gi < ngroups; gi += SK_THREADS) {
        const int m = gi / (kc >> 3), kk = (gi % (kc >> 3)) << 3;
        if (m < M) {
          const uint4 v = *reinterpret_cast<const uint4*>(x16 + (size_t)m * K + k0 + kk);
          const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int t = 0; t < 4; t++) {
            amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, u[t] << 16)));
            amax = fmaxf(amax, fabsf(__builtin_bit_cast(float, u[t] & 0xffff0000u)));
          }
        }
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
      if (lane == 0) scratch[wave] = amax;
      __syncthreads();
      amax = fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
    }
    float xscale = 1.0f, inv = 1.0f;  // true x = xscale * stored f16 x
    if constexpr (DT == KQ_BF16) {
      // bring the largest magnitude into [2^14, 2^15): exact power-of-two scaling
      const uint32_t eb = (__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff;
      if (eb != 0 && eb != 0xff) {
        int e = (int)eb - 127 - 14;
        if (e < -100) e = -100;
        xscale = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
        inv = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
      }
    }
    for (int gi = tid; gi < ngroups; gi += SK_THREADS) {
      const int m = gi / (kc >> 3), kk = (gi % (kc >> 3)) << 3;
      float f[8];
      if (m < M) {
        const uint4 v = *reinterpret_cast<const uint4*>(x16 + (size_t)m * K + k0 + kk);
        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int t = 0; t < 4; t++) {
          if constexpr (DT == KQ_BF16) {
            f[2 * t] = __builtin_bit_cast(float, u[t] << 16) * inv;
            f[2 * t + 1] = __builtin_bit_cast(float, u[t] & 0xffff0000u) * inv;
          } else {
            f[2 * t] = kq::h2f((uint16_t)(u[t] & 0xffff));
            f[2 * t + 1] = kq::h2f((uint16_t)(u[t] >> 16));
          }
        }
      } else {
#pragma unroll
        for (int t = 0; t < 8; t++) f[t] = 0.f;
      }
      _Float16 h[8];
#pragma unroll
      for (int t = 0; t < 8; t++) h[t] = (_Float16)f[t];
      // MFMA fragment order inside an 8-group: k0 k2 k1 k3 k4 k6 k5 k7
      const f16x8 v8 = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
      *reinterpret_cast<f16x8*>(xs + (size_t)m * kchunk + kk) = v8;
      float s = 0.f;
#pragma unroll
      for (int t = 0; t < 8; t++) s += (float)h[t];
      s += __shfl_xor(s, 1);  // 4 threads cover one 32-wide sub-block
      s += __shfl_xor(s, 2);
      if ((tid & 3) == 0) xsum[(kk >> 5) * MB + m] = s;
    }

    // ---- park the weights in LDS
    {
      int r = r_first, c = c_first;
      StaticFor<MAXP>::run([&](auto t) {
        if (r < nrows) *reinterpret_cast<u32x4*>(wt + r * wstride + 16 * c) = wreg[decltype(t)::value];
        r += step_r;
        c += step_c;
        if (c >= cpr) {
          c -= cpr;
          r++;
        }
      });
    }
    __syncthreads();

    // ---- this wave's superblocks of the chunk
    const _Float16* xs_lane = xs + (size_t)(n_in & (MB - 1)) * kchunk + 16 * kg;
    const float* xsum_lane = xsum + (MB == 8 ? 4 * kg : 0);
    const uint8_t* wt_lane = wt + crow * wstride;
    for (int s = wave; s < sbn; s += SK_WAVES) {
      Q4kRaw raw;
      const uint4* p = reinterpret_cast<const uint4*>(wt_lane + s * 144);
      raw.hdr = p[0];
#pragma unroll
      for (int g = 0; g < 4; g++) raw.q[g] = p[1 + 2 * g + kg];
      q4k_superblock<R, MB>(raw, xscale, xs_lane + 256 * s, xsum_lane + 8 * MB * s, acc);
    }
  }

  // ---- cross-wave reduction and store
#pragma unroll
  for (int r = 0; r < R; r++) red[(wave * R + r) * 64 + lane] = acc[r];
  __syncthreads();
  for (int o = tid; o < R * 64; o += SK_THREADS) {
    const int r = o >> 6, l = o & 63;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < SK_WAVES; wv++) v += red[(wv * R + r) * 64 + l];
    const int m = 4 * (l >> 5) + r, n = l & 31;
    if (m < M && n < nrows) {
      uint16_t* yo = static_cast<uint16_t*>(y) + (size_t)m * N + row0 + n;
      *yo = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
    }
  }
}

template <int DT, int MB>
int launch_q4k_skinny(const void* x, const uint8_t* w, void* y, int M, int N, int K, hipStream_t s) {
  constexpr int R = MB < 4 ? MB : 4;
  // balanced row tiles: about two workgroups per CU, at most 32 rows each
  int rows = (N + 511) / 512;
  rows = (rows + 3) & ~3;
  if (rows > 32) rows = 32;
  if (rows < 8) rows = 8;
  const int tiles = (N + rows - 1) / rows;
  int kch = K >> 8;
  if (kch > 16) kch = 16;            // 18 pieces per thread at most (32 rows x 16 superblocks)
  if (kch * MB > 32) kch = 32 / MB;  // keep the f16 activations of a chunk within 16 KiB
  auto lds_bytes = [&](int kc) {
    return (size_t)rows * (kc * 144 + 16) + (size_t)MB * kc * 512 + (size_t)kc * 8 * MB * 4 + SK_WAVES * R * 64 * 4 + 64;
  };
  while (kch > 1 && lds_bytes(kch) > 76 * 1024) kch >>= 1;  // two workgroups per CU must fit in 160 KiB
  const size_t lds = lds_bytes(kch);
  auto kern = q4k_skinny_kernel<DT, MB>;
  static bool attr_set = false;  // per instantiation
  if (!attr_set) {
    KQ_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     120 * 1024));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(SK_THREADS), lds, s, x, w, y, M, N, K, rows, kch);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

template <int DT>
int launch_q4k_skinny_m(const void* x, const uint8_t* w, void* y, int M, int N, int K, hipStream_t s) {
  if (M == 1) return launch_q4k_skinny<DT, 1>(x, w, y, M, N, K, s);
  if (M == 2) return launch_q4k_skinny<DT, 2>(x, w, y, M, N, K, s);
  if (M <= 4) return launch_q4k_skinny<DT, 4>(x, w, y, M, N, K, s);
  return launch_q4k_skinny<DT, 8>(x, w, y, M, N, K, s);
}

}  // namespace

int kq_launch_qmm_tuned(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype,
                        hipStream_t s) {
  if (codec != KQ_Q4_K || M < 1 || M > SK_MAXM || (K & 255) || K == 0) return KQ_ERR_UNSUPPORTED;
  if ((reinterpret_cast<uintptr_t>(w) & 15) || (reinterpret_cast<uintptr_t>(x) & 15)) return KQ_ERR_UNSUPPORTED;
  if (dtype == KQ_F16) return launch_q4k_skinny_m<KQ_F16>(x, w, y, M, N, K, s);
  return launch_q4k_skinny_m<KQ_BF16>(x, w, y, M, N, K, s);
}
