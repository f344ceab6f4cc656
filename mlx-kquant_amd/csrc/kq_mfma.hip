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

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences global memory,
// which on this target drains every outstanding global load (s_waitcnt vmcnt(0)) and would
// serialise the weight stream behind each barrier.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

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

  constexpr int SBC = 4;  // superblocks per sub-chunk: one per wave
  constexpr int NCH = 4;  // sub-chunks per chunk (kch <= 16), all in flight at once
  constexpr int PPC = 5;  // 16-byte pieces per thread per sub-chunk: ceil(32 rows * 36 / 256)
  // activation staging slots per thread: slot t = (row t / XK, k-pass t % XK); a chunk holds at
  // most min(512, 1024 / MB) 8-element groups per row because kch * MB <= 32
  constexpr int XK = MB <= 2 ? 2 : 1;
  constexpr int XG = MB * XK;

  // piece map of the weight stream (see step 2): global / LDS byte offsets inside a sub-chunk
  uint32_t goff[PPC], loff[PPC];
  int ppc[PPC];
  bool piece_ok[PPC];
  {
    int r = tid / 36, pc = tid % 36;
    StaticFor<PPC>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      piece_ok[T] = r < nrows;
      ppc[T] = pc;
      goff[T] = (uint32_t)r * (uint32_t)row_bytes + 16 * pc;
      loff[T] = (uint32_t)r * (uint32_t)wstride + 16 * pc;
      r += SK_THREADS / 36;
      pc += SK_THREADS % 36;
      if (pc >= 36) {
        pc -= 36;
        r++;
      }
    });
  }
  uint8_t* dump = reinterpret_cast<uint8_t*>(scratch + 16) + 16 * tid;  // per-thread 16-byte dump slot

  for (int sb0 = 0; sb0 < nsb; sb0 += kch) {
    const int sbn = (nsb - sb0 < kch) ? (nsb - sb0) : kch;
    const int kc = sbn << 8, k0 = sb0 << 8;

    // ---- 1. activation loads first, so waiting for them does not wait for the weights
    const int gpr = kc >> 3;         // 8-element groups per activation row in this chunk
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

    // ---- 2. weight stream.  Sub-chunk c covers superblocks [4c, 4c+4) = 36 16-byte pieces per
    // row; piece i = tid + 256 t maps to (row i / 36, piece i % 36), so consecutive lanes read
    // consecutive 16-byte pieces of a row.  The map is the same for every sub-chunk (goff / loff
    // below); pieces outside the tile or a ragged last sub-chunk re-read the tile's first bytes and
    // land in a dump slot.  Two sub-chunks are in flight at any time (register sets c % 2); the
    // next one is issued as soon as its register set has been parked in LDS.
    u32x4 wreg[2 * PPC];
    auto issue = [&](auto cc) {
      constexpr int c = decltype(cc)::value;
      const int sbc = sbn - SBC * c;  // superblocks left from this sub-chunk on (uniform)
      const uint8_t* src = wtile + (size_t)(sb0 + SBC * c) * 144;
      StaticFor<PPC>::run([&](auto t) {
        constexpr int T = decltype(t)::value;
        const bool ok = piece_ok[T] && ppc[T] < sbc * 9;
        wreg[(c & 1) * PPC + T] = *reinterpret_cast<const u32x4*>(ok ? src + goff[T] : wtile);
      });
    };
    issue(std::integral_constant<int, 0>{});
    issue(std::integral_constant<int, 1>{});

    // ---- 3. activations -> f16 in LDS (+ per-sub-block sums)
    if (sb0 > 0) lds_barrier();
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
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) sum += (float)h[e];
        sum += __shfl_xor(sum, 1);  // 4 threads cover one 32-wide sub-block
        sum += __shfl_xor(sum, 2);
        if ((tid & 3) == 0) xsum[(kk >> 5) * MB + m] = sum;
      }
    });

    // ---- 4. sub-chunk by sub-chunk: park the arrived bytes in LDS, then one superblock per wave
    // while the later sub-chunks are still streaming in
    const _Float16* xs_lane = xs + (size_t)(n_in & (MB - 1)) * kchunk + 16 * kg;
    const float* xsum_lane = xsum + (MB == 8 ? 4 * kg : 0);
    const uint8_t* wt_lane = wt + crow * wstride;
    StaticFor<NCH>::run([&](auto cc) {
      constexpr int c = decltype(cc)::value;
      const int sbc = sbn - SBC * c;
      if (sbc > 0) {
        StaticFor<PPC>::run([&](auto t) {
          constexpr int T = decltype(t)::value;
          const bool ok = piece_ok[T] && ppc[T] < sbc * 9;
          *reinterpret_cast<u32x4*>(ok ? wt + SBC * c * 144 + loff[T] : dump) = wreg[(c & 1) * PPC + T];
        });
      }
      if constexpr (c + 2 < NCH) issue(std::integral_constant<int, c + 2>{});
      if (sbc > 0) {
        lds_barrier();
        const int sb = SBC * c + wave;
        if (sb < sbn) {
          Q4kRaw raw;
          const uint4* p = reinterpret_cast<const uint4*>(wt_lane + sb * 144);
          raw.hdr = p[0];
#pragma unroll
          for (int g = 0; g < 4; g++) raw.q[g] = p[1 + 2 * g + kg];
          q4k_superblock<R, MB>(raw, xscale, xs_lane + 256 * sb, xsum_lane + 8 * MB * sb, acc);
        }
      }
    });
  }

  // ---- cross-wave reduction and store
#pragma unroll
  for (int r = 0; r < R; r++) red[(wave * R + r) * 64 + lane] = acc[r];
  lds_barrier();
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
    return (size_t)rows * (kc * 144 + 16) + (size_t)MB * kc * 512 + (size_t)kc * 8 * MB * 4 + SK_WAVES * R * 64 * 4 + 64 + 16 * SK_THREADS;
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
