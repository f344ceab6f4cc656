// Prefill GEMM for the 32-weight-block codecs whose weight is (f16 scale) x (small integer) [+ f16 minimum]: q8_0,
// q4_0, iq4_nl, q5_0, q4_1, q5_1.
// y[M,N] = x[M,K] . W^T on the f16 matrix cores, 256-row (or 128-row) wave tiles, exact in the weights.
//
// A block's scale d is not an integer, so the exact-integer operands of the K-quant kernels do not apply, and a
// scale fold per block would cost eight vector instructions per MFMA.  Instead every weight w = d q goes in as two
// f16 terms whose sum is w exactly: hi = round_f16(d q) (one packed multiply) and lo = d q - hi (one packed fused
// multiply-add: the product is formed exactly, and what is left after hi has at most eight significant bits, on the
// grid of d or coarser, so it is an f16 number, subnormal ones included).  Two MFMAs share the activation fragment;
// products of f16 numbers are exact in the f32 accumulator, so results differ from f32 arithmetic on the decoded
// weights by summation order only.  (|d q| beyond the f16 range, 65504, is not representable this way; no quantizer
// emits such scales.)  No per-block fold, no unit chain: 20 vector instructions decode eight weights for sixteen MFMAs.
// q4_1 / q5_1 add the block minimum m, an f16 number, as a third term on a third MFMA (the reference rounds d q + m
// to f32 once; the three-term sum is exact, the difference at most 2^-24 of the weight).
//
// Workgroup = 8 waves = 256 (MT = 8) or 128 (MT = 4) activation rows x 256 weight rows, one per CU, two waves per
// SIMD.  K advances in steps of 64 (two blocks): two activation stages filled by the whole workgroup with
// direct-to-LDS loads (one barrier per step); every wave streams the bytes of its own 32 weight rows, step by step,
// into a ring of four private slots (quant bytes as 16-byte pieces that start behind the 2-byte scale, scales as
// 2-byte loads) and needs no barrier for them: step s + 3 is queued in step s, registers of step s + 1 are read in
// step s.  Activations come from a prepass of their own (f16 scaled per row by a power of two, k permuted inside
// 8-groups to match the byte order of the decode).
// Block layouts as the reference decodes them: src/kquant_cpu_decode.cpp:49-63 (q8_0), :65-82 (q4_0), :84-102 (q4_1),
// :104-128 (q5_0), :130-153 (q5_1), :382-397 (iq4_nl); the M > 8 matmul this serves: src/kquant_cpu_decode.cpp:1209-1359,
// tile policy of the reference's own matrix path: src/kquant_matmul.cpp:77-134, 313-451.
#include "kq_dma.h"
#include "kq_mma.h"

namespace {

using namespace kqmma;
using namespace kqdma;

constexpr int B3_WAVES = 8, B3_BN = 256, B3_KS = 64, B3_SLOTS = 4;

template <int C>
struct B32;
template <>
struct B32<KQ_Q8_0> {
  static constexpr int BPB = 34, QB = 32;  // block bytes, quant bytes behind the scale
};
template <>
struct B32<KQ_Q4_0> {
  static constexpr int BPB = 18, QB = 16;
};
template <>
struct B32<KQ_IQ4_NL> {
  static constexpr int BPB = 18, QB = 16;  // as q4_0, the nibble indexing a table of sixteen int8 values
};
template <>
struct B32<KQ_Q4_1> {
  static constexpr int BPB = 20, QB = 16;  // d, m, 16 quant bytes
};
template <>
struct B32<KQ_Q5_0> {
  static constexpr int BPB = 22, QB = 16;  // d, 32 fifth bits, 16 quant bytes
};
template <>
struct B32<KQ_Q5_1> {
  static constexpr int BPB = 24, QB = 16;  // d, m, 32 fifth bits, 16 quant bytes
};

template <int C>
struct B3Geom : B32<C> {
  static constexpr int QP = 2 * B32<C>::QB / 16;   // 16-byte quant pieces per row and step
  static constexpr int Q_INSTR = 32 * QP / 64;     // load instructions for them
  static constexpr int SLOT_Q = 32 * 16 * QP;      // quant bytes of a slot (row-major, 16 QP bytes per row)
  // what stands in front of the quant bytes: a 2-byte scale (one 2-byte load per row and block, parked as a
  // zero-extended dword), or more (minimum, fifth bits): then the block's first 16 bytes travel as a piece
  static constexpr int HEAD = B32<C>::BPB - B32<C>::QB;
  static constexpr bool HEAD16 = HEAD > 2;
  static constexpr int SLOT = SLOT_Q + (HEAD16 ? 1024 : 256);
  static constexpr int W_INSTR = Q_INSTR + 1;
  static constexpr int STEP_BYTES = 2 * B32<C>::BPB;
  static constexpr bool MIN = C == KQ_Q4_1 || C == KQ_Q5_1;   // weight = d q + m
  static constexpr bool FIVE = C == KQ_Q5_0 || C == KQ_Q5_1;  // a fifth bit per weight
};

template <int C, int MT>
constexpr int b3_lds_bytes() {
  return 2 * (32 * MT * B3_KS * 2) + B3_WAVES * B3_SLOTS * B3Geom<C>::SLOT;
}

// Activations of one row: xh = f16(x 2^-e) with k permuted inside 8-groups to k0 k2 k1 k3 k4 k6 k5 k7, rs = 2^e
// (bf16 rows are scaled so that the largest magnitude lands in [2^14, 2^15); f16 rows pass through).
template <int DT>
__global__ __launch_bounds__(256) void b3_prepass_kernel(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
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
    *reinterpret_cast<f16x8*>(xo + 8 * g) = f16x8{h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
  }
}

template <int C, int DT, int MT>
__global__ __launch_bounds__(64 * B3_WAVES, 1) void block32_gemm3_kernel(const _Float16* __restrict__ xh,
                                                                        const float* __restrict__ rs,
                                                                        const uint8_t* __restrict__ w,
                                                                        uint16_t* __restrict__ y, int M, int N, int K,
                                                                        int mtiles, int nt0) {
  using G = B3Geom<C>;
  constexpr int TM = 32 * MT, A_STAGE = TM * B3_KS * 2, AQ = MT / 2;
  constexpr int W_OFF = 2 * A_STAGE;
  constexpr int GPS = B3_KS / 16;  // MFMA groups per step: 4 (block g / 2 of the step, K-half g % 2)
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, kg = lane >> 5;
  const int mt = blockIdx.x % mtiles, nt = nt0 + blockIdx.x / mtiles;  // consecutive workgroups share the weight columns
  const int m0 = mt * TM, n0 = nt * B3_BN;
  const int nsteps = K / B3_KS;
  const uint32_t row_bytes = (uint32_t)(K >> 5) * G::BPB;
  const int nrows = N - n0 < B3_BN ? N - n0 : B3_BN;
  const uint32_t lds0 = lds_addr(smem);

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
  // wire: quant piece i = 64 q + lane -> row i / QP, piece i % QP of the row's two blocks (block p / (QB / 16), its
  // 16-byte part p % (QB / 16)); scales: lane -> row lane / 2, block lane % 2.  Rows past N re-read the last row.
  auto wrow = [&](int r) -> uint32_t {
    r += wave * 32;
    return (uint32_t)(r < nrows ? r : nrows - 1) * row_bytes;
  };
  uint32_t v_q[G::Q_INSTR];
#pragma unroll
  for (int q = 0; q < G::Q_INSTR; q++) {
    const int i = 64 * q + lane, p = i % G::QP;
    v_q[q] = wrow(i / G::QP) + (uint32_t)(G::BPB * (p / (G::QB / 16)) + G::HEAD + 16 * (p % (G::QB / 16)));
  }
  const uint32_t v_d = wrow(lane >> 1) + (uint32_t)(G::BPB * (lane & 1));
  const uint8_t* w_base = w + (size_t)n0 * row_bytes;

  auto issue_a = [&](int step) {
    const uint8_t* base = a_base + (size_t)step * (B3_KS * 2);
    const uint32_t l = lds0 + (step & 1) * A_STAGE + wave * 1024;
#pragma unroll
    for (int q = 0; q < AQ; q++) dma16(base, a_voff[q], l + q * (B3_WAVES * 1024));
  };
  const uint32_t w_lds = lds0 + W_OFF + wave * (B3_SLOTS * G::SLOT);
  auto issue_w = [&](int step) {  // the two blocks of K step `step` of this wave's rows -> slot step % 4
    const uint8_t* base = w_base + (size_t)step * G::STEP_BYTES;
    const uint32_t l = w_lds + (step & (B3_SLOTS - 1)) * G::SLOT;
#pragma unroll
    for (int q = 0; q < G::Q_INSTR; q++) dma16(base, v_q[q], l + q * 1024);
    if constexpr (G::HEAD16)
      dma16(base, v_d, l + G::SLOT_Q);  // lane -> (row lane / 2, block lane % 2): 16 bytes each
    else
      dma2(base, v_d, l + G::SLOT_Q);
  };

  // A fragment of m-tile t, group g: lane half kg holds the weights 16 kg + 8 (g % 2) .. + 7 of block g / 2, i.e.
  // activation piece 4 (g / 2) + 2 kg + g % 2 of the step
  uint32_t a_addr[GPS];
#pragma unroll
  for (int g = 0; g < GPS; g++)
    a_addr[g] = (uint32_t)l32 * 128u + 16u * (uint32_t)((4 * (g >> 1) + 2 * kg + (g & 1)) ^ swz(l32));
  const uint8_t* slot0 = smem + W_OFF + wave * (B3_SLOTS * G::SLOT);

  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) acc[t] = f32x16{0};

  const uint32_t magic = opaque_vgpr(0x64006400u);
  const uint32_t mask_b = opaque_sgpr(C == KQ_Q4_0 || C == KQ_Q4_1 ? 0x000f000fu : G::FIVE ? 0x001f001fu : 0x00ff00ffu);
  // iq4_nl: the sixteen table values + 128 as bytes (entries 0 - 3, 4 - 7, 8 - 11, 12 - 15), looked up four at a time
  // with byte permutes: low three bits select inside each half, the fourth bit selects the half
  const uint32_t kv0 = opaque_sgpr(0x3f2d1801u), kv1 = opaque_sgpr(0x766a5d4fu), kv2 = opaque_sgpr(0xa6998d81u),
                 kv3 = opaque_sgpr(0xf1d9c5b5u);
  (void)kv0; (void)kv1; (void)kv2; (void)kv3;

  // ---- this lane's weight row: registers of the step in hand
  struct Regs {
    uint4 q[2];      // q8_0: bytes 16 kg .. + 15 of the block; the nibble codecs: its 16 bytes (this lane takes nibble kg)
    uint32_t d[2];   // f16 scale of the block, in both halves of the dword
    uint32_t m[2];   // q4_1 / q5_1: f16 minimum of the block, in both halves
    uint32_t qh[2];  // q5_0 / q5_1: the fifth bits of this lane's sixteen weights (bits 0 .. 15)
  };
  auto load_regs = [&](int slot) -> Regs {
    const uint8_t* sl = slot0 + slot * G::SLOT;
    Regs rg;
#pragma unroll
    for (int b = 0; b < 2; b++) {
      if constexpr (C == KQ_Q8_0)
        rg.q[b] = *reinterpret_cast<const uint4*>(sl + l32 * 64 + 32 * b + 16 * kg);
      else
        rg.q[b] = *reinterpret_cast<const uint4*>(sl + l32 * 32 + 16 * b);
    }
    if constexpr (G::HEAD16) {
#pragma unroll
      for (int b = 0; b < 2; b++) {
        const uint2 hd = *reinterpret_cast<const uint2*>(sl + G::SLOT_Q + l32 * 32 + 16 * b);  // block bytes 0 .. 7
        rg.d[b] = (hd.x & 0xffffu) | (hd.x << 16);
        rg.m[b] = G::MIN ? (hd.x >> 16) | (hd.x & 0xffff0000u) : 0u;
        // fifth bits: weight j of the block has bit j of the 32-bit field behind d (and m); this lane's are 16 kg ..
        const uint32_t field = G::MIN ? hd.y : (hd.x >> 16) | (hd.y << 16);
        rg.qh[b] = G::FIVE ? field >> (16 * kg) : 0u;
      }
    } else {
      const uint2 dd = *reinterpret_cast<const uint2*>(sl + G::SLOT_Q + l32 * 8);
      rg.d[0] = dd.x | (dd.x << 16);
      rg.d[1] = dd.y | (dd.y << 16);
      rg.m[0] = rg.m[1] = rg.qh[0] = rg.qh[1] = 0u;
    }
    return rg;
  };

  // the two exact terms of the weights 16 kg + 8 s .. + 7 of block b, (b, s) = (g / 2, g % 2)
  auto decode = [&](auto gc, const Regs& rg, f16x8& hi, f16x8& lo) {
    constexpr int g = decltype(gc)::value, b = g >> 1, s = g & 1;
    const uint32_t qw[4] = {rg.q[b].x, rg.q[b].y, rg.q[b].z, rg.q[b].w};
    const f16x2 dp = __builtin_bit_cast(f16x2, rg.d[b]);
    // q8_0: byte ^ 0x80 = q + 128, 0x6400 | that = 1024 + 128 + q (iq4_nl: the table holds value + 128);
    // q4_0: 0x6400 | nibble = 1024 + 8 + (n - 8); q5_0: 1024 + 16 + (q - 16); q4_1 / q5_1: 1024 + q
    constexpr float OFF = C == KQ_Q4_0 ? -1032.0f : C == KQ_Q5_0 ? -1040.0f : G::MIN ? -1024.0f : -1152.0f;
    const f16x2 off = {(_Float16)OFF, (_Float16)OFF};
    f16x2 h2[4], l2[4];
#pragma unroll
    for (int e = 0; e < 2; e++) {
      uint32_t x = qw[2 * s + e];
      if constexpr (C == KQ_Q8_0) {
        x ^= 0x80808080u;
      } else if constexpr (C == KQ_Q4_0 || C == KQ_Q4_1) {
        x >>= 4 * kg;
      } else if constexpr (G::FIVE) {
        // the four fifth bits of these four weights, one into bit 4 of each byte
        const uint32_t four = (rg.qh[b] >> (8 * s + 4 * e)) & 0xfu;
        const uint32_t spread = (four * 0x00204081u) & 0x01010101u;
        x = ((x >> (4 * kg)) & 0x0f0f0f0fu) | (spread << 4);
      } else {
        const uint32_t nib = (x >> (4 * kg)) & 0x0f0f0f0fu, low3 = nib & 0x07070707u;
        const uint32_t half0 = __builtin_amdgcn_perm(kv1, kv0, low3), half1 = __builtin_amdgcn_perm(kv3, kv2, low3);
        x = __builtin_amdgcn_perm(half1, half0, ((nib >> 1) & 0x04040404u) | 0x03020100u);
      }
      const uint32_t fe = (x & mask_b) | magic, fo = ((x >> 8) & mask_b) | magic;  // bytes 0, 2 / bytes 1, 3
      const f16x2 qe = __builtin_bit_cast(f16x2, fe) + off, qo = __builtin_bit_cast(f16x2, fo) + off;
      h2[2 * e] = qe * dp;
      h2[2 * e + 1] = qo * dp;
      l2[2 * e] = __builtin_elementwise_fma(qe, dp, -h2[2 * e]);
      l2[2 * e + 1] = __builtin_elementwise_fma(qo, dp, -h2[2 * e + 1]);
    }
    hi = f16x8{h2[0][0], h2[0][1], h2[1][0], h2[1][1], h2[2][0], h2[2][1], h2[3][0], h2[3][1]};
    lo = f16x8{l2[0][0], l2[0][1], l2[1][0], l2[1][1], l2[2][0], l2[2][1], l2[3][0], l2[3][1]};
  };

  // ---- prologue: first loads, registers of step 0, its first fragments
  issue_a(0);
  issue_w(0);
  if (nsteps > 1) issue_w(1);
  if (nsteps > 2) issue_w(2);
  vmwait<0>();
  Regs cur = load_regs(0);
  Regs nxt = cur;
  f16x8 bhi[2], blo[2];
  decode(std::integral_constant<int, 0>{}, cur, bhi[0], blo[0]);

  // ---- main loop.  The activation loads of step s + 1 are queued right after the barrier that opens step s; this
  // wave's wire bytes of step s + 3 follow (their slot held step s - 1, read into registers in step s - 2) and may
  // stay in flight over the next barrier; the bytes of step s + 1, queued in step s - 2, are older than this step's
  // activation loads and have landed with them.
  for (int step = 0; step < nsteps; step++) {
    const uint8_t* a_stage = smem + (step & 1) * A_STAGE;
    if (step > 0 && step + 2 < nsteps) vmwait<G::W_INSTR>(); else vmwait<0>();
    lds_barrier();
    if (step + 1 < nsteps) issue_a(step + 1);
    if (step + 3 < nsteps) issue_w(step + 3);
    f16x8 afr[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[0] + t * 4096);
    StaticFor<GPS>::run([&](auto gc) {
      constexpr int g = decltype(gc)::value;
      if constexpr (g == GPS - 2) nxt = load_regs((step + 1) & (B3_SLOTS - 1));  // past the end: a harmless re-read
      if constexpr (g + 1 < GPS)
        decode(std::integral_constant<int, g + 1>{}, cur, bhi[(g + 1) & 1], blo[(g + 1) & 1]);
      else
        decode(std::integral_constant<int, 0>{}, nxt, bhi[0], blo[0]);
#pragma unroll
      for (int t = 0; t < MT; t++) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[t], bhi[g & 1], acc[t], 0, 0, 0);
      if constexpr (G::MIN) {  // third term: the block minimum against the same activations
        const f16x2 mp = __builtin_bit_cast(f16x2, cur.m[g >> 1]);
        const f16x8 bm = {mp[0], mp[1], mp[0], mp[1], mp[0], mp[1], mp[0], mp[1]};
#pragma unroll
        for (int t = 0; t < MT; t++) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[t], bm, acc[t], 0, 0, 0);
      }
#pragma unroll
      for (int t = 0; t < MT; t++) {
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[t], blo[g & 1], acc[t], 0, 0, 0);
        if constexpr (g + 1 < GPS) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[g + 1] + t * 4096);
      }
    });
    cur = nxt;
  }

  // ---- epilogue: undo the per-row activation scale, round once, store
  const int n = n0 + wave * 32 + l32;
#pragma unroll
  for (int t = 0; t < MT; t++) {
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

template <int C, int DT, int MT>
int launch_b3(const _Float16* xh, const float* rs, const uint8_t* w, void* y, int M, int N, int K, int nt0, int ntiles,
              hipStream_t s) {
  const int mtiles = (M + 32 * MT - 1) / (32 * MT);
  constexpr int lds = b3_lds_bytes<C, MT>();
  static_assert(lds <= 160 * 1024, "tile does not fit the LDS of a CU");
  auto kern = block32_gemm3_kernel<C, DT, MT>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  hipLaunchKernelGGL(kern, dim3(mtiles * ntiles), dim3(64 * B3_WAVES), lds, s, xh, rs, w, static_cast<uint16_t*>(y), M, N, K,
                     mtiles, nt0);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

template <int C, int DT>
int launch_b3_tiles(const _Float16* xh, const float* rs, const uint8_t* w, void* y, int M, int N, int K, int nt0,
                    int ntiles, int tile_rows, hipStream_t s) {
  if (ntiles <= 0) return KQ_OK;
  return tile_rows == 128 ? launch_b3<C, DT, 4>(xh, rs, w, y, M, N, K, nt0, ntiles, s)
                          : launch_b3<C, DT, 8>(xh, rs, w, y, M, N, K, nt0, ntiles, s);
}

int b3_num_cus() {
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
  return n;
}

static int g_b3_force = 0;  // kq_set_gemm_tile_rows: 1024 / 1025 force one tile height for every column tile, 64 switches the kernel off

template <int C, int DT>
int launch_b3_call(const void* x, const uint8_t* w, void* y, int M, int N, int K, void* ws, int force, hipStream_t s) {
  _Float16* xh = static_cast<_Float16*>(ws);
  float* rs = reinterpret_cast<float*>(xh + (size_t)M * K);
  hipLaunchKernelGGL((b3_prepass_kernel<DT>), dim3(M), dim3(256), 0, s, static_cast<const uint16_t*>(x), xh, rs, K);
  KQ_HIP_CHECK(hipGetLastError());
  // One workgroup per CU, so a call costs whole rounds: a round of 256-row tiles counts 200, a round of 128-row
  // tiles 119 (measured on the q6_k kernel of the same structure).  Every column tile on one height, or the column
  // tiles that fill whole rounds at 256 rows and the rest at whichever height is cheaper.
  const int nt256 = (N + 255) / 256, mt256 = (M + 255) / 256, mt128 = (M + 127) / 128;
  if (force) return launch_b3_tiles<C, DT>(xh, rs, w, y, M, N, K, 0, nt256, force, s);
  const int64_t cus = b3_num_cus();
  auto rounds = [&](int64_t wgs) { return (wgs + cus - 1) / cus; };
  const int64_t c128 = rounds((int64_t)mt128 * nt256) * 119;
  const int64_t full = (int64_t)mt256 * nt256 / cus;
  const int tall = full > 0 ? (int)(full * cus / mt256) : 0;
  const int rest = nt256 - tall;
  const int64_t rest256 = rounds((int64_t)mt256 * rest) * 200, rest128 = rounds((int64_t)mt128 * rest) * 119;
  const int64_t c256 = full * 200 + (rest128 < rest256 ? rest128 : rest256);
  if (c128 < c256) return launch_b3_tiles<C, DT>(xh, rs, w, y, M, N, K, 0, nt256, 128, s);
  const int rc = launch_b3_tiles<C, DT>(xh, rs, w, y, M, N, K, 0, tall, 256, s);
  if (rc != KQ_OK) return rc;
  return launch_b3_tiles<C, DT>(xh, rs, w, y, M, N, K, tall, rest, rest128 < rest256 ? 128 : 256, s);
}

}  // namespace

// Taken for calls of 128 rows or more whose half-height tiles fill three quarters of the CUs; smaller calls stay on
// the any-codec kernel (small workgroups, K cut over the grid).
bool kq_gemm3b_supported(int M, int N, int K, int codec) {
  if (codec != KQ_Q8_0 && codec != KQ_Q4_0 && codec != KQ_IQ4_NL && codec != KQ_Q4_1 && codec != KQ_Q5_0 && codec != KQ_Q5_1)
    return false;
  if (M < 128 || N <= 0 || K < 64 || (K & 63)) return false;
  const int64_t row_bytes = (int64_t)(K >> 5) * 34;  // the largest block of the six
  if (256 * row_bytes >= ((int64_t)1 << 32) || (int64_t)M * K * 2 >= ((int64_t)1 << 32)) return false;
  if (g_b3_force > 0) return true;  // a forced tile height takes every shape (tests reach the kernel on small matrices)
  return 4 * (int64_t)((M + 127) / 128) * ((N + 255) / 256) >= 3 * (int64_t)b3_num_cus();
}

size_t kq_gemm3b_workspace_bytes(int M, int K) { return (size_t)M * K * 2 + (size_t)M * 4 + 256; }

void kq_gemm3b_force_tile(int rows) { g_b3_force = rows == 1024 ? 256 : rows == 1025 ? 128 : rows == 64 ? -1 : 0; }

int kq_launch_gemm3b(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                     hipStream_t s) {
  if (g_b3_force < 0 || !kq_gemm3b_supported(M, N, K, codec)) return KQ_ERR_UNSUPPORTED;
  if ((reinterpret_cast<uintptr_t>(w) & 1) || (reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(ws) & 15))
    return KQ_ERR_UNSUPPORTED;
  const int force = g_b3_force;
  if (codec == KQ_Q8_0)
    return dtype == KQ_F16 ? launch_b3_call<KQ_Q8_0, KQ_F16>(x, w, y, M, N, K, ws, force, s)
                           : launch_b3_call<KQ_Q8_0, KQ_BF16>(x, w, y, M, N, K, ws, force, s);
  if (codec == KQ_IQ4_NL)
    return dtype == KQ_F16 ? launch_b3_call<KQ_IQ4_NL, KQ_F16>(x, w, y, M, N, K, ws, force, s)
                           : launch_b3_call<KQ_IQ4_NL, KQ_BF16>(x, w, y, M, N, K, ws, force, s);
  if (codec == KQ_Q4_1)
    return dtype == KQ_F16 ? launch_b3_call<KQ_Q4_1, KQ_F16>(x, w, y, M, N, K, ws, force, s)
                           : launch_b3_call<KQ_Q4_1, KQ_BF16>(x, w, y, M, N, K, ws, force, s);
  if (codec == KQ_Q5_0)
    return dtype == KQ_F16 ? launch_b3_call<KQ_Q5_0, KQ_F16>(x, w, y, M, N, K, ws, force, s)
                           : launch_b3_call<KQ_Q5_0, KQ_BF16>(x, w, y, M, N, K, ws, force, s);
  if (codec == KQ_Q5_1)
    return dtype == KQ_F16 ? launch_b3_call<KQ_Q5_1, KQ_F16>(x, w, y, M, N, K, ws, force, s)
                           : launch_b3_call<KQ_Q5_1, KQ_BF16>(x, w, y, M, N, K, ws, force, s);
  return dtype == KQ_F16 ? launch_b3_call<KQ_Q4_0, KQ_F16>(x, w, y, M, N, K, ws, force, s)
                         : launch_b3_call<KQ_Q4_0, KQ_BF16>(x, w, y, M, N, K, ws, force, s);
}
