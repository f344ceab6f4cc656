// Prefill GEMM for the fp4 codecs (mxfp4, nvfp4): y[M,N] = x[M,K] . W^T on the f16 matrix cores, 256-row (or
// 128-row) wave tiles, ONE exact f16 term per weight.
//
// An fp4 code is one of +-{0, 0.5, 1, 1.5, 2, 3, 4, 6} (two significant bits).  v_cvt_scalef32_pk_f16_fp4 turns a
// byte (two codes) into an f16 pair times a power of two (the exponent of its f32 scale operand; the mantissa is
// ignored): low nibble -> element 0, high nibble -> element 1, subnormal results included.
//   nvfp4: weight = code x (unsigned e4m3 scale), scale in [2^-9, 480] with four significant bits: the product
//          has six and lies in [2^-10, 2880], an f16 number.  B = cvt(byte, 1.0) x scale (one packed multiply).
//   mxfp4: weight = code x 2^(E - 127) for any byte E.  B = cvt(byte, 2^(E - uoff - 127)) with a per-column offset
//          uoff chosen so that the exponent stays inside the window in which every code is an f16 number
//          (2^-23 ... 2^13); the running sums are then in units of 2^uoff.  The offset moves only when a block
//          leaves the window (then the sums of that column are rescaled by an exact power of two), which ordinary
//          weights never do.  What cannot be held exactly: two blocks of one K step whose exponents differ by more
//          than 27, and blocks so far below sums already large (2^-100 of them) that f32 accumulation drops them too.
// A byte holds weights j and j + 8 (nvfp4, inside a 16-weight scale group) or j and j + 16 (mxfp4, inside the block):
// the activation prepass stores x in that pair order, so a lane's four quant bytes (one dword) become its B operand
// of one MFMA with four conversions and no shuffling.
//
// Workgroup, activation stages and the wave-private ring of four wire slots as in kq_gemm3b.hip; a K step (64
// weights: one nvfp4 block of 36 bytes, two mxfp4 blocks of 17) travels as three 16-byte pieces per row, the last
// one ending on the step's last byte (rows are 2-byte aligned whenever K is a multiple of 64).
// Block layouts and scale decoding as in the reference: src/kquant_cpu_decode.cpp:403-418 (mxfp4), :420-438 (nvfp4),
// src/kquant_fp_tables.h:21-41 (e8m0 / unsigned e4m3 scales); the M > 8 matmul this serves:
// src/kquant_cpu_decode.cpp:1209-1359, tile policy of the reference's own matrix path: src/kquant_matmul.cpp:77-134.
#include "kq_dma.h"
#include "kq_mma.h"

namespace {

using namespace kqmma;
using namespace kqdma;

constexpr int F3_WAVES = 8, F3_BN = 256, F3_KS = 64, F3_SLOTS = 4;
constexpr int F3_SLOT = 32 * 48;  // three pieces per row
constexpr int F3_W_INSTR = 2;     // 96 pieces: one full load instruction and a half one

template <int C>
struct F3Geom {
  static constexpr int STEP_BYTES = C == KQ_MXFP4 ? 34 : 36;
  static constexpr int P2 = C == KQ_MXFP4 ? 18 : 20;  // start of the third piece (the first two are bytes 0 .. 31)
};

template <int MT>
constexpr int f3_lds_bytes() {
  return 2 * (32 * MT * F3_KS * 2) + F3_WAVES * F3_SLOTS * F3_SLOT;
}

// Activations of one row: xh = f16(x 2^-e), rs = 2^e (bf16 rows scaled so that the largest magnitude lands in
// [2^14, 2^15); f16 rows pass through).  Piece p = 4 (G / 2) + 2 kg + G % 2 of a K step (8 values) holds, for MFMA
// group G and lane half kg, x[a], x[a + D], x[a + 1], x[a + 1 + D], ... with a = 16 G + 4 kg, D = 8 (nvfp4) or
// a = 32 (G / 2) + 8 (G % 2) + 4 kg, D = 16 (mxfp4).
template <int C, int DT>
__global__ __launch_bounds__(256) void f3_prepass_kernel(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
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
  for (int op = tid; op < ngroups; op += 256) {
    const int step = op >> 3, pi = op & 7;
    const int G = 2 * (pi >> 2) + (pi & 1), kg = (pi >> 1) & 1;
    const int a = 64 * step + (C == KQ_NVFP4 ? 16 * G + 4 * kg : 32 * (G >> 1) + 8 * (G & 1) + 4 * kg);
    constexpr int D = C == KQ_NVFP4 ? 8 : 16;
    const uint2 lo = *reinterpret_cast<const uint2*>(xi + a), hi = *reinterpret_cast<const uint2*>(xi + a + D);
    const uint32_t src[4] = {lo.x, lo.y, hi.x, hi.y};
    _Float16 h[8];  // a .. a + 3, then a + D .. a + D + 3
#pragma unroll
    for (int e = 0; e < 4; e++) {
      if constexpr (DT == KQ_BF16) {
        h[2 * e] = (_Float16)(__builtin_bit_cast(float, src[e] << 16) * inv);
        h[2 * e + 1] = (_Float16)(__builtin_bit_cast(float, src[e] & 0xffff0000u) * inv);
      } else {
        h[2 * e] = __builtin_bit_cast(_Float16, (uint16_t)(src[e] & 0xffff));
        h[2 * e + 1] = __builtin_bit_cast(_Float16, (uint16_t)(src[e] >> 16));
      }
    }
    *reinterpret_cast<f16x8*>(xo + 8 * op) = f16x8{h[0], h[4], h[1], h[5], h[2], h[6], h[3], h[7]};
  }
}

template <int C, int DT, int MT>
__global__ __launch_bounds__(64 * F3_WAVES, 1) void fp4_gemm3_kernel(const _Float16* __restrict__ xh,
                                                                    const float* __restrict__ rs,
                                                                    const uint8_t* __restrict__ w,
                                                                    uint16_t* __restrict__ y, int M, int N, int K,
                                                                    int mtiles, int nt0) {
  using G_ = F3Geom<C>;
  constexpr bool MX = C == KQ_MXFP4;
  constexpr int TM = 32 * MT, A_STAGE = TM * F3_KS * 2, AQ = MT / 2;
  constexpr int W_OFF = 2 * A_STAGE;
  constexpr int GPS = F3_KS / 16;  // MFMA groups per step: 4
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, kg = lane >> 5;
  const int mt = blockIdx.x % mtiles, nt = nt0 + blockIdx.x / mtiles;  // consecutive workgroups share the weight columns
  const int m0 = mt * TM, n0 = nt * F3_BN;
  const int nsteps = K / F3_KS;
  const uint32_t row_bytes = (uint32_t)nsteps * G_::STEP_BYTES;
  const int nrows = N - n0 < F3_BN ? N - n0 : F3_BN;
  const uint32_t lds0 = lds_addr(smem);

  // ---- load maps (activations as in kq_gemm3b.hip)
  auto swz = [](int row) { return (row >> 1) & 7; };
  uint32_t a_voff[AQ];
#pragma unroll
  for (int q = 0; q < AQ; q++) {
    const int r = 8 * (wave + 8 * q) + (lane >> 3);
    const int gr = m0 + r < M ? m0 + r : M - 1;
    a_voff[q] = (uint32_t)gr * (uint32_t)K * 2u + 16u * (uint32_t)((lane & 7) ^ swz(r));
  }
  const uint8_t* a_base = reinterpret_cast<const uint8_t*>(xh);
  // wire: piece i = 64 q + lane (i < 96) -> row i / 3, piece i % 3 of the row's step: bytes 0 .. 15, 16 .. 31 and the
  // step's last 16.  Rows past N re-read the last row (their columns are not stored).
  uint32_t v_q[2];
#pragma unroll
  for (int q = 0; q < 2; q++) {
    int i = 64 * q + lane;
    i = i < 96 ? i : 95;
    int r = wave * 32 + i / 3;
    const int p = i % 3;
    r = r < nrows ? r : nrows - 1;
    v_q[q] = (uint32_t)r * row_bytes + (uint32_t)(p == 0 ? 0 : p == 1 ? 16 : G_::P2);
  }
  const uint8_t* w_base = w + (size_t)n0 * row_bytes;

  auto issue_a = [&](int step) {
    const uint8_t* base = a_base + (size_t)step * (F3_KS * 2);
    const uint32_t l = lds0 + (step & 1) * A_STAGE + wave * 1024;
#pragma unroll
    for (int q = 0; q < AQ; q++) dma16(base, a_voff[q], l + q * (F3_WAVES * 1024));
  };
  const uint32_t w_lds = lds0 + W_OFF + wave * (F3_SLOTS * F3_SLOT);
  auto issue_w = [&](int step) {  // K step `step` of this wave's rows -> slot step % 4
    const uint8_t* base = w_base + (size_t)step * G_::STEP_BYTES;
    const uint32_t l = w_lds + (step & (F3_SLOTS - 1)) * F3_SLOT;
    dma16(base, v_q[0], l);
    if (lane < 32) dma16(base, v_q[1], l + 1024);
  };

  uint32_t a_addr[GPS];
#pragma unroll
  for (int g = 0; g < GPS; g++)
    a_addr[g] = (uint32_t)l32 * 128u + 16u * (uint32_t)((4 * (g >> 1) + 2 * kg + (g & 1)) ^ swz(l32));
  const uint8_t* slot0 = smem + W_OFF + wave * (F3_SLOTS * F3_SLOT);

  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) acc[t] = f32x16{0};

  // ---- this lane's weight row: registers of the step in hand
  struct Regs {
    uint32_t q[4];  // the lane's four quant bytes of each MFMA group
    uint32_t s[2];  // mxfp4: f32 bits of the two blocks' conversion scales; nvfp4: s[0] = the four scale bytes
  };
  // mxfp4: the running sums of this column are in units of 2^uoff; B = code x 2^(E - uoff - 127) with the exponent
  // field E - uoff kept inside [104, 140]
  int uoff = 0, uoff_n = 0, pending = 0;
  auto load_regs = [&](int slot, bool first) -> Regs {
    const uint8_t* rb = slot0 + slot * F3_SLOT + l32 * 48;
    Regs rg;
    if constexpr (MX) {
      // LDS row: step bytes 0 .. 31 as they lie (E0, 16 quant bytes, E1, ...), step bytes 18 .. 33 (the second
      // block's quant bytes) at 32
#pragma unroll
      for (int g = 0; g < 2; g++) {
        const uint32_t lo = *reinterpret_cast<const uint32_t*>(rb + 8 * g + 4 * kg);
        const uint32_t hi = *reinterpret_cast<const uint32_t*>(rb + 8 * g + 4 * kg + 4);
        rg.q[g] = __builtin_amdgcn_alignbyte(hi, lo, 1);  // step bytes 1 + 8 g + 4 kg .. + 3
        rg.q[2 + g] = *reinterpret_cast<const uint32_t*>(rb + 32 + 8 * g + 4 * kg);
      }
      const int e0 = (int)(*reinterpret_cast<const uint32_t*>(rb) & 0xffu);
      const int e1 = (int)((*reinterpret_cast<const uint32_t*>(rb + 16) >> 8) & 0xffu);
      const int hi = e0 > e1 ? e0 : e1, lo = e0 < e1 ? e0 : e1;
      // the offset moves when a block leaves the window; the larger exponent then lands at field 131
      const bool move = first || hi - uoff_n > 140 || lo - uoff_n < 104;
      int target = move ? hi - 131 : uoff_n;
      // A move to a smaller unit multiplies the sums by 2^(uoff_n - target).  Where they are large already that
      // would overflow, and the blocks that asked for it are far below one ulp of the sums anyway: the column keeps
      // its unit and those blocks go in as what is left of them in the window (f32 accumulation of the decoded
      // weights loses them the same way).  Rare: the sums are read only when some column wants to move down.
      if (!first && __builtin_amdgcn_ballot_w64(target < uoff_n) != 0) {
        float amax = 0.f;
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
          for (int i = 0; i < 16; i++) amax = fmaxf(amax, fabsf(acc[t][i]));
        const int ex = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xffu);  // biased exponent of the largest sum
        if (target < uoff_n && ex + (uoff_n - target) > 127 + 90) target = uoff_n;
      }
      pending = uoff_n - target;  // the sums change unit by 2^pending when this step is entered
      uoff_n = target;
      const int f0 = e0 - target, f1 = e1 - target;  // a block below the window becomes zeros (field <= 0: 2^-127)
      rg.s[0] = (uint32_t)(f0 > 0 ? f0 : 0) << 23;
      rg.s[1] = (uint32_t)(f1 > 0 ? f1 : 0) << 23;
    } else {
      // LDS row: block bytes 0 .. 31 as they lie (four scale bytes, then quant bytes), block bytes 20 .. 35 at 32
      rg.s[0] = *reinterpret_cast<const uint32_t*>(rb);
      rg.s[1] = 0;
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int off = 4 + 8 * g + 4 * kg;
        rg.q[g] = *reinterpret_cast<const uint32_t*>(rb + (off < 32 ? off : off + 12));
      }
    }
    return rg;
  };

  // B fragment of MFMA group g of the step
  auto decode = [&](auto gc, const Regs& rg) -> f16x8 {
    constexpr int g = decltype(gc)::value;
    f16x2 p[4];
    if constexpr (MX) {
      const float sc = __builtin_bit_cast(float, rg.s[g >> 1]);
      p[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(rg.q[g], sc, 0);
      p[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(rg.q[g], sc, 1);
      p[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(rg.q[g], sc, 2);
      p[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(rg.q[g], sc, 3);
    } else {
      // scale byte x -> the e4m3 value (the codes here are 0.5 ... 6, half the integers the scale's half goes
      // with): the f16 with bits (x & 0x7f) << 7 is that value / 256, subnormal scales included; x = 0x7f decodes to 0
      const uint32_t x = (rg.s[0] >> (8 * g)) & 0xffu;
      const uint32_t hb = x == 0x7fu ? 0u : (x & 0x7fu) << 7;
      const f16x2 sp = __builtin_bit_cast(f16x2, hb | (hb << 16)) * f16x2{(_Float16)256.0f, (_Float16)256.0f};
      p[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(rg.q[g], 1.0f, 0) * sp;
      p[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(rg.q[g], 1.0f, 1) * sp;
      p[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(rg.q[g], 1.0f, 2) * sp;
      p[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(rg.q[g], 1.0f, 3) * sp;
    }
    return f16x8{p[0][0], p[0][1], p[1][0], p[1][1], p[2][0], p[2][1], p[3][0], p[3][1]};
  };

  // ---- prologue: first loads, registers of step 0, its first fragment
  issue_a(0);
  issue_w(0);
  if (nsteps > 1) issue_w(1);
  if (nsteps > 2) issue_w(2);
  vmwait<0>();
  Regs cur = load_regs(0, true);
  uoff = uoff_n;
  Regs nxt = cur;
  f16x8 bfr[2];
  bfr[0] = decode(std::integral_constant<int, 0>{}, cur);

  // ---- main loop: as in kq_gemm3b.hip (step s + 3 queued in step s, registers of step s + 1 read in step s)
  for (int step = 0; step < nsteps; step++) {
    const uint8_t* a_stage = smem + (step & 1) * A_STAGE;
    if (step > 0 && step + 2 < nsteps) vmwait<F3_W_INSTR>(); else vmwait<0>();
    lds_barrier();
    if (step + 1 < nsteps) issue_a(step + 1);
    if (step + 3 < nsteps) issue_w(step + 3);
    f16x8 afr[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[0] + t * 4096);
    pending = 0;
    StaticFor<GPS>::run([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      if constexpr (g == GPS - 2) {
        if (step + 1 < nsteps) nxt = load_regs((step + 1) & (F3_SLOTS - 1), false);
      }
      if constexpr (g + 1 < GPS)
        bfr[(g + 1) & 1] = decode(std::integral_constant<int, g + 1>{}, cur);
      else
        bfr[0] = decode(std::integral_constant<int, 0>{}, nxt);
#pragma unroll
      for (int t = 0; t < MT; t++) {
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[t], bfr[g & 1], acc[t], 0, 0, 0);
        if constexpr (g + 1 < GPS) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[g + 1] + t * 4096);
      }
    });
    cur = nxt;
    if constexpr (MX) {
      // the next step's blocks left the exponent window of some column: its sums change unit (exact)
      if (__builtin_amdgcn_ballot_w64(pending != 0) != 0) {
#pragma unroll
        for (int t = 0; t < MT; t++)
#pragma unroll
          for (int i = 0; i < 16; i++) acc[t][i] = __builtin_ldexpf(acc[t][i], pending);
      }
      uoff = uoff_n;
    }
  }

  // ---- epilogue: back to plain units, undo the per-row activation scale, round once, store
  const int n = n0 + wave * 32 + l32;
#pragma unroll
  for (int t = 0; t < MT; t++) {
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int m = m0 + t * 32 + 8 * (i >> 2) + 4 * kg + (i & 3);
      if (m < M && n < N) {
        float v = acc[t][i] * rs[m];
        if constexpr (MX) v = __builtin_ldexpf(v, uoff);
        y[(size_t)m * N + n] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
      }
    }
  }
}

template <int C, int DT, int MT>
int launch_f3(const _Float16* xh, const float* rs, const uint8_t* w, void* y, int M, int N, int K, int nt0, int ntiles,
              hipStream_t s) {
  if (ntiles <= 0) return KQ_OK;
  const int mtiles = (M + 32 * MT - 1) / (32 * MT);
  constexpr int lds = f3_lds_bytes<MT>();
  static_assert(lds <= 160 * 1024, "tile does not fit the LDS of a CU");
  auto kern = fp4_gemm3_kernel<C, DT, MT>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  hipLaunchKernelGGL(kern, dim3(mtiles * ntiles), dim3(64 * F3_WAVES), lds, s, xh, rs, w, static_cast<uint16_t*>(y), M, N, K,
                     mtiles, nt0);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

template <int C, int DT>
int launch_f3_tiles(const _Float16* xh, const float* rs, const uint8_t* w, void* y, int M, int N, int K, int nt0,
                    int ntiles, int tile_rows, hipStream_t s) {
  return tile_rows == 128 ? launch_f3<C, DT, 4>(xh, rs, w, y, M, N, K, nt0, ntiles, s)
                          : launch_f3<C, DT, 8>(xh, rs, w, y, M, N, K, nt0, ntiles, s);
}

int f3_num_cus() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
  return n;
}

static int g_f3_force = 0;  // kq_set_gemm_tile_rows: 1024 / 1025 force one tile height for every column tile, 64 switches the kernel off

template <int C, int DT>
int launch_f3_call(const void* x, const uint8_t* w, void* y, int M, int N, int K, void* ws, int force, hipStream_t s) {
  _Float16* xh = static_cast<_Float16*>(ws);
  float* rs = reinterpret_cast<float*>(xh + (size_t)M * K);
  hipLaunchKernelGGL((f3_prepass_kernel<C, DT>), dim3(M), dim3(256), 0, s, static_cast<const uint16_t*>(x), xh, rs, K);
  KQ_HIP_CHECK(hipGetLastError());
  // tile heights by whole rounds of one workgroup per CU, as for the other tall-tile kernels
  const int nt256 = (N + 255) / 256, mt256 = (M + 255) / 256, mt128 = (M + 127) / 128;
  if (force) return launch_f3_tiles<C, DT>(xh, rs, w, y, M, N, K, 0, nt256, force, s);
  const int64_t cus = f3_num_cus();
  auto rounds = [&](int64_t wgs) { return (wgs + cus - 1) / cus; };
  const int64_t c128 = rounds((int64_t)mt128 * nt256) * 119;
  const int64_t full = (int64_t)mt256 * nt256 / cus;
  const int tall = full > 0 ? (int)(full * cus / mt256) : 0;
  const int rest = nt256 - tall;
  const int64_t rest256 = rounds((int64_t)mt256 * rest) * 200, rest128 = rounds((int64_t)mt128 * rest) * 119;
  const int64_t c256 = full * 200 + (rest128 < rest256 ? rest128 : rest256);
  if (c128 < c256) return launch_f3_tiles<C, DT>(xh, rs, w, y, M, N, K, 0, nt256, 128, s);
  const int rc = launch_f3_tiles<C, DT>(xh, rs, w, y, M, N, K, 0, tall, 256, s);
  if (rc != KQ_OK) return rc;
  return launch_f3_tiles<C, DT>(xh, rs, w, y, M, N, K, tall, rest, rest128 < rest256 ? 128 : 256, s);
}

}  // namespace

// Taken for calls of 128 rows or more whose half-height tiles fill three quarters of the CUs; smaller calls stay on
// the any-codec kernel.
bool kq_gemm3f_supported(int M, int N, int K, int codec) {
  if (codec != KQ_MXFP4 && codec != KQ_NVFP4) return false;
  if (M < 128 || N <= 0 || K < 64 || (K & 63)) return false;
  const int64_t row_bytes = (int64_t)(K >> 6) * (codec == KQ_MXFP4 ? 34 : 36);
  if (256 * row_bytes >= ((int64_t)1 << 32) || (int64_t)M * K * 2 >= ((int64_t)1 << 32)) return false;
  if (g_f3_force > 0) return true;  // a forced tile height takes every shape (tests reach the kernel on small matrices)
  return 4 * (int64_t)((M + 127) / 128) * ((N + 255) / 256) >= 3 * (int64_t)f3_num_cus();
}

size_t kq_gemm3f_workspace_bytes(int M, int K) { return (size_t)M * K * 2 + (size_t)M * 4 + 256; }

void kq_gemm3f_force_tile(int rows) { g_f3_force = rows == 1024 ? 256 : rows == 1025 ? 128 : rows == 64 ? -1 : 0; }

int kq_launch_gemm3f(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                     hipStream_t s) {
  if (g_f3_force < 0 || !kq_gemm3f_supported(M, N, K, codec)) return KQ_ERR_UNSUPPORTED;
  if ((reinterpret_cast<uintptr_t>(w) & 1) || (reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(ws) & 15))
    return KQ_ERR_UNSUPPORTED;
  const int force = g_f3_force;
  if (codec == KQ_MXFP4)
    return dtype == KQ_F16 ? launch_f3_call<KQ_MXFP4, KQ_F16>(x, w, y, M, N, K, ws, force, s)
                           : launch_f3_call<KQ_MXFP4, KQ_BF16>(x, w, y, M, N, K, ws, force, s);
  return dtype == KQ_F16 ? launch_f3_call<KQ_NVFP4, KQ_F16>(x, w, y, M, N, K, ws, force, s)
                         : launch_f3_call<KQ_NVFP4, KQ_BF16>(x, w, y, M, N, K, ws, force, s);
}
