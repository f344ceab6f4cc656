// Prefill GEMM, 256-row wave tiles (q4_k / q5_k): y[M,N] = x[M,K] . W^T on the f16 matrix cores.
//
// The 128 x 256 kernel of kq_gemm2.hip decodes a weight fragment for every four MFMAs and keeps two accumulator
// sets (the running sums and the exact-integer sums of the superblock in hand, folded with d at its end), which is
// what stops its wave tile at 128 rows: 2 x 64 accumulator registers at two waves per SIMD.  Here a wave owns
// 256 activation rows x 32 weight rows on ONE accumulator set:
//   * the running sum S of a column is kept in units of that column's current scale r: entering a superblock with
//     scale d, S is multiplied by r / d (one multiply per accumulator and superblock, the cost of the old fold) and
//     r becomes d; the exact integers sc_j q then accumulate straight into S.  The result is S r at the end.  The
//     multiplications round like any f32 accumulation (2^-24 per superblock);
//   * the block minimum term is one extra MFMA per m-tile and superblock on exact integers (m_j against the hi / lo
//     sums of x) whose result joins S in the same pass that changes the unit: S <- S (r / d) + (-32 dmin / d) P;
//   * a decoded fragment feeds eight MFMAs: about 3.5 vector instructions per MFMA instead of 5.3.
// Workgroup = 8 waves = 256 activation rows x 256 weight rows, one per CU, two waves per SIMD.  K advances in steps
// of 64: two activation stages of 32 KiB filled by the whole workgroup (one barrier per step).  Every wave streams
// the wire bytes of its own 32 weight rows (two stages of one superblock) and needs no barrier for them, so the
// decode of the next fragment, of the next step and of the next superblock's header run ahead of the barriers.
// Activations come from the prepass of kq_gemm.hip (f16, k permuted inside 8-groups; hi / lo sub-block sums).
#include "kq_dma.h"
#include "kq_mma.h"

namespace {

using namespace kqmma;
using namespace kqdma;

constexpr int G3_TM = 256, G3_MT = 8, G3_WAVES = 8, G3_BN = 256, G3_KS = 64;
constexpr int G3_A_STAGE = G3_TM * G3_KS * 2;  // 32 KiB
constexpr int G3_H_BYTES = G3_TM * 32;         // hi / lo sums of x of one superblock: 8 KiB

template <int C>
constexpr int g3_lds_bytes() {
  return 2 * G3_A_STAGE + G3_WAVES * 2 * 32 * Wire<C>::LBPB + G3_H_BYTES;
}

template <int C, int DT>
__global__ __launch_bounds__(64 * G3_WAVES, 1) void kquant_gemm3_kernel(const _Float16* __restrict__ xh,
                                                                       const _Float16* __restrict__ xhl,
                                                                       const float* __restrict__ rs,
                                                                       const uint8_t* __restrict__ w,
                                                                       uint16_t* __restrict__ y, int M, int mrows, int N,
                                                                       int K, int mtiles, int nt0) {
  using G = Wire<C>;
  constexpr int MT = G3_MT, PP = G::PP, LBPB = G::LBPB;
  constexpr int W_STAGE = 32 * LBPB;
  constexpr int W_PIECES = 32 * PP;
  constexpr int W_INSTR = (W_PIECES + 63) / 64;      // 5 (q4_k), 6 (q5_k)
  constexpr int W_LAST = W_PIECES - 64 * (W_INSTR - 1);  // live lanes of the last one
  constexpr int A_OFF = 0, W_OFF = 2 * G3_A_STAGE, H_OFF = W_OFF + G3_WAVES * 2 * W_STAGE;
  constexpr int GPS = G3_KS / 16;  // MFMA groups per step: 4
  constexpr int SPS = 256 / G3_KS;  // steps per superblock: 4
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, kg = lane >> 5;
  const int mt = blockIdx.x % mtiles, nt = nt0 + blockIdx.x / mtiles;  // consecutive workgroups share the weight columns
  const int m0 = mt * G3_TM, n0 = nt * G3_BN;
  const int nsb = K >> 8;
  const uint32_t row_bytes = (uint32_t)nsb * G::BPB;
  const int nrows = N - n0 < G3_BN ? N - n0 : G3_BN;
  const uint32_t lds0 = lds_addr(smem);

  // ---- load maps
  // activations: load q of this wave covers rows 8 (wave + 8 q) + lane / 8, piece lane % 8 of the step; LDS piece p
  // of row r holds global piece p ^ swz(r).  Rows past the prepared ones re-read the last one (never stored).
  auto swz = [](int row) { return (row >> 1) & 7; };
  uint32_t a_voff[4];
#pragma unroll
  for (int q = 0; q < 4; q++) {
    const int r = 8 * (wave + 8 * q) + (lane >> 3);
    const int gr = m0 + r < mrows ? m0 + r : mrows - 1;
    a_voff[q] = (uint32_t)gr * (uint32_t)K * 2u + 16u * (uint32_t)((lane & 7) ^ swz(r));
  }
  const uint8_t* a_base = reinterpret_cast<const uint8_t*>(xh);
  // wire: load q covers pieces 64 q + lane of this wave's 32 rows x PP; piece i -> (row i / PP, i % PP)
  uint32_t w_voff[W_INSTR];
#pragma unroll
  for (int q = 0; q < W_INSTR; q++) {
    int i = 64 * q + lane;
    i = i < W_PIECES ? i : W_PIECES - 1;
    int r = wave * 32 + i / PP;
    const int p = i % PP;
    r = r < nrows ? r : nrows - 1;  // rows past N re-read the last row (their columns are not stored)
    w_voff[q] = (uint32_t)r * row_bytes + 16u * (uint32_t)p;
  }
  const uint8_t* w_base = w + (size_t)n0 * row_bytes;
  // hi / lo sums of x: 256 rows x 32 bytes = 8 loads, one per wave
  const int h_i = 64 * wave + lane;
  const int h_r = m0 + (h_i >> 1) < mrows ? m0 + (h_i >> 1) : mrows - 1;
  const uint32_t h_voff = (uint32_t)h_r * (uint32_t)nsb * 32u + 16u * (uint32_t)(h_i & 1);
  const uint8_t* h_base = reinterpret_cast<const uint8_t*>(xhl);

  auto issue_a = [&](int step) {  // K step `step` -> A stage step % 2
    const uint8_t* base = a_base + (size_t)step * (G3_KS * 2);
    const uint32_t l = lds0 + A_OFF + (step & 1) * G3_A_STAGE + wave * 1024;
#pragma unroll
    for (int q = 0; q < 4; q++) dma16(base, a_voff[q], l + q * (G3_WAVES * 1024));
  };
  const uint32_t w_lds = lds0 + W_OFF + wave * (2 * W_STAGE);
  auto issue_w = [&](int sb) {  // superblock sb of this wave's rows -> its W stage sb % 2
    const uint8_t* base = w_base + (size_t)sb * G::BPB;
    const uint32_t l = w_lds + (sb & 1) * W_STAGE;
#pragma unroll
    for (int q = 0; q < W_INSTR - 1; q++) dma16(base, w_voff[q], l + q * 1024);
    if (lane < W_LAST) dma16(base, w_voff[W_INSTR - 1], l + (W_INSTR - 1) * 1024);
  };
  auto issue_h = [&](int sb) { dma16(h_base + (size_t)sb * 32, h_voff, lds0 + H_OFF + wave * 1024); };

  // ---- fragment addresses
  // A fragment of m-tile t, MFMA group g of the step = (sub-block g / 2, K-half s = g % 2): lane half kg holds the
  // weights 16 kg + 8 s .. + 7 of the sub-block, i.e. activation piece 4 (g / 2) + 2 kg + s of the step
  uint32_t a_addr[GPS];
#pragma unroll
  for (int g = 0; g < GPS; g++)
    a_addr[g] = (uint32_t)l32 * 128u + 16u * (uint32_t)((4 * (g >> 1) + 2 * kg + (g & 1)) ^ swz(l32));
  const uint8_t* b_lane0 = smem + W_OFF + wave * (2 * W_STAGE) + l32 * LBPB;
  const uint8_t* h_lane = smem + H_OFF + l32 * 32 + 16 * kg;

  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) acc[t] = f32x16{0};

  const uint32_t magic = opaque_vgpr(0x64006400u);
  const uint32_t mask_lo = opaque_sgpr(0x000f000fu), mask_hi = opaque_sgpr(0x00f000f0u);
  const uint32_t mask5_lo = opaque_sgpr(0x00100010u), mask5_hi = opaque_sgpr(0x01000100u);
  (void)mask5_lo;
  (void)mask5_hi;

  // ---- per-superblock state of this lane's weight row
  struct Head {
    uint32_t scw[2];  // the eight 6-bit sub-block scales
    float klo, khi;   // what a low / high-nibble code (1024 + q, 1024 + 16 q) is multiplied by besides its scale
    float ratio;      // r_old / r_new: the running sums change unit when the superblock is entered
    float cm;         // -32 dmin / r_new: what the exact sum of m_j (hi_j + lo_j) is multiplied by
    f16x8 bm;         // the eight 6-bit sub-block minima m_j as f16 integers
  };
  float r = 1.0f;  // unit of the running sums
  auto decode_head = [&](const uint8_t* bl, bool commit) -> Head {  // commit = false: a dry run that leaves r alone
    Head h;
    const uint4 hdr = *reinterpret_cast<const uint4*>(bl);
    const float d = kq::h2f((uint16_t)(hdr.x & 0xffff)), dmin = kq::h2f((uint16_t)(hdr.x >> 16));
    const uint32_t s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
    h.scw[0] = s0 & 0x3f3f3f3fu;
    h.scw[1] = (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u);
    const uint32_t mnw[2] = {s1 & 0x3f3f3f3fu, ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u)};
    // a superblock with d = 0 keeps the unit (its integers are fed as zeros); f32 holds any dmin / d
    const float rn = d != 0.f ? d : r;
    const float inv = __builtin_amdgcn_rcpf(rn);  // 1 ulp: the sums pick up a factor 1 + 2^-23 per superblock at most
    h.ratio = r * inv;
    h.cm = -32.0f * dmin * inv;
    h.klo = d != 0.f ? 1.0f : 0.f;
    h.khi = h.klo * 0.0625f;
    // 1024 + m as f16 bits, minus 1024: the exact integers m_j, two per instruction
    const uint32_t k1024 = 0x64006400u;
    f16x2 mp[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const uint32_t wsel = mnw[e >> 1] >> (16 * (e & 1));  // bytes 2 e, 2 e + 1 of the eight
      const uint32_t pair = (wsel & 0xffu) | ((wsel & 0xff00u) << 8) | k1024;
      mp[e] = __builtin_bit_cast(f16x2, pair) - f16x2{(_Float16)1024.0f, (_Float16)1024.0f};
    }
    h.bm = f16x8{mp[0][0], mp[0][1], mp[1][0], mp[1][1], mp[2][0], mp[2][1], mp[3][0], mp[3][1]};
    r = commit ? rn : r;
    return h;
  };

  // B fragment of MFMA group `it` (0 .. 15) of a superblock: sub-block j = it / 2, K-half s = it % 2, from the 16
  // quant bytes qv (and q5_k: fifth-bit bytes hv) of this lane's half of the step's 32-byte chunk
  auto decode = [&](auto itc, const uint4& qv, const uint4& hv, const Head& hd) -> f16x8 {
    constexpr int it = decltype(itc)::value;
    constexpr int j = it >> 1, s = it & 1, h = j & 1;
    const uint32_t qw[4] = {qv.x, qv.y, qv.z, qv.w};
    const float scf = (float)((hd.scw[j >> 2] >> (8 * (j & 3))) & 0xff);
    // low nibbles read 1024 + q, high nibbles (in place) 1024 + 16 q: the 16 is in khi
    const _Float16 sch = (_Float16)(scf * (h ? hd.khi : hd.klo));
    const _Float16 off = sch * (_Float16)(-1024.0f);
    const f16x2 scp = {sch, sch}, offp = {off, off};
    const uint32_t mask = h ? mask_hi : mask_lo;
    uint32_t fr[4] = {(qw[2 * s] & mask) | magic, ((qw[2 * s] >> 8) & mask) | magic, (qw[2 * s + 1] & mask) | magic,
                      ((qw[2 * s + 1] >> 8) & mask) | magic};
    if constexpr (C == KQ_Q5_K) {
      // fifth bit of weight (j, i) is bit j of qh[i]; this lane's bytes are qh[16 kg + 8 s + 0..7]: bit 4 next
      // to a low nibble (1024 + q + 16 b), bit 8 next to a high nibble held in place (1024 + 16 (q + 16 b))
      constexpr int P = h ? 8 : 4;
      const uint32_t mbit = h ? mask5_hi : mask5_lo;
      const uint32_t hb[4] = {hv.x, hv.y, hv.z, hv.w};
      auto place = [&](uint32_t word, int from) -> uint32_t {
        return from >= P ? word >> (from - P) : word << (P - from);
      };
      fr[0] |= place(hb[2 * s], j) & mbit;
      fr[1] |= place(hb[2 * s], j + 8) & mbit;
      fr[2] |= place(hb[2 * s + 1], j) & mbit;
      fr[3] |= place(hb[2 * s + 1], j + 8) & mbit;
    }
    f16x2 bq[4];
#pragma unroll
    for (int e = 0; e < 4; e++)  // one rounding: (1024 + q) * sc - 1024 * sc = sc * q exactly
      bq[e] = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, fr[e]), scp, offp);
    return f16x8{bq[0][0], bq[0][1], bq[1][0], bq[1][1], bq[2][0], bq[2][1], bq[3][0], bq[3][1]};
  };
  auto load_q = [&](const uint8_t* bl, int p) -> uint4 {  // quant bytes of step p of the superblock at bl
    return *reinterpret_cast<const uint4*>(bl + G::QS + 32 * p + 16 * kg);
  };
  auto load_h5 = [&](const uint8_t* bl) -> uint4 {
    if constexpr (C == KQ_Q5_K) return *reinterpret_cast<const uint4*>(bl + 16 + 16 * kg);
    return uint4{0, 0, 0, 0};
  };

  // Entering a superblock: the running sums change unit and take the block minimum term, the exact
  // sum_j m_j (hi_j + lo_j) of one extra MFMA per m-tile times -32 dmin / r (two partial-sum tiles in rotation: the
  // MFMA of m-tile t + 1 runs while m-tile t is folded).  Runs at the end of the previous superblock's last step:
  // the sums of x it reads were queued three steps earlier and the loop-carried sums come out of plain FMAs.
  auto enter = [&](const Head& h) {
    f32x16 pm[2];
    f16x8 hfr[2];
    hfr[0] = *reinterpret_cast<const f16x8*>(h_lane);
    pm[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(hfr[0], h.bm, f32x16{0}, 0, 0, 0);
    StaticFor<MT>::run([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      if constexpr (t + 1 < MT) {
        hfr[(t + 1) & 1] = *reinterpret_cast<const f16x8*>(h_lane + (t + 1) * 1024);
        pm[(t + 1) & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(hfr[(t + 1) & 1], h.bm, f32x16{0}, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 16; i++) acc[t][i] = fmaf(pm[t & 1][i], h.cm, acc[t][i] * h.ratio);  // in place: multiply, then fmac
    });
  };

  // ---- prologue: first loads, the first superblock's header and first fragment
  issue_a(0);
  issue_w(0);
  issue_h(0);
  if (nsb > 1) issue_w(1);
  if (nsb > 1) vmwait<W_INSTR>(); else vmwait<0>();  // own wire bytes of superblock 0 (and everything older) have landed
  Head hd = decode_head(b_lane0, true);
  lds_barrier();  // the sums of x of superblock 0 are every wave's loads
  enter(hd);
  uint4 qv = load_q(b_lane0, 0), hv = load_h5(b_lane0);
  f16x8 bfr[2];
  bfr[0] = decode(std::integral_constant<int, 0>{}, qv, hv, hd);
  Head hn = hd;

  // ---- main loop: step s = 4 sb + p.  The activation loads of step s + 1 are queued right after the barrier that
  // opens step s (their stage was last read in step s - 1).  The sums of x of superblock sb + 1 follow in part 0
  // (every wave has then passed their only reader, the entry into superblock sb); this wave's wire bytes of
  // superblock sb + 2 follow in part 3, into the stage of superblock sb, whose last bytes went to registers at the
  // end of part 2.
  for (int sb = 0; sb < nsb; sb++) {
    const uint8_t* b_lane = b_lane0 + (sb & 1) * W_STAGE;
    const uint8_t* b_next = b_lane0 + ((sb + 1) & 1) * W_STAGE;
    const bool more = sb + 1 < nsb;
    StaticFor<SPS>::run([&](auto pc) {
      constexpr int p = decltype(pc)::value;
      const int step = SPS * sb + p;
      const uint8_t* a_stage = smem + A_OFF + (p & 1) * G3_A_STAGE;
      // own loads of this step's activations have landed; wire bytes queued after them may stay in flight
      if (p == 0 && more) vmwait<W_INSTR>(); else vmwait<0>();
      lds_barrier();
      if (p + 1 < SPS || more) issue_a(step + 1);
      if (p == 0 && more) issue_h(sb + 1);  // every wave is past the end of the previous part 3, their only reader
      if (p == SPS - 1 && sb + 2 < nsb) issue_w(sb + 2);
      f16x8 afr[MT];
#pragma unroll
      for (int t = 0; t < MT; t++) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[0] + t * 4096);
      // the next step's quant bytes (own wire stage: no barrier needed)
      const uint8_t* bl_n = p + 1 < SPS ? b_lane : (more ? b_next : b_lane);  // past the end: a harmless re-read
      const uint4 qv_n = load_q(bl_n, (p + 1) % SPS), hv_n = load_h5(bl_n);
      // the next superblock's header, decoded among this step's MFMAs (past the end: a dry run on this one's bytes)
      if constexpr (p == SPS - 1) hn = decode_head(bl_n, more);
      StaticFor<GPS>::run([&](auto gc) {
        constexpr int g = decltype(gc)::value;
        constexpr int it = GPS * p + g;
        // B fragment of the next group: of this step, or the first of the next step
        if constexpr (g + 1 < GPS)
          bfr[(g + 1) & 1] = decode(std::integral_constant<int, it + 1>{}, qv, hv, hd);
        else if constexpr (p + 1 < SPS)
          bfr[(g + 1) & 1] = decode(std::integral_constant<int, it + 1>{}, qv_n, hv_n, hd);
        else
          bfr[(g + 1) & 1] = decode(std::integral_constant<int, 0>{}, qv_n, hv_n, hn);
#pragma unroll
        for (int t = 0; t < MT; t++) {
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[t], bfr[g & 1], acc[t], 0, 0, 0);
          if constexpr (g + 1 < GPS) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[g + 1] + t * 4096);
        }
      });
      qv = qv_n;
      hv = hv_n;
      if constexpr (p == SPS - 1) {
        hd = hn;
        if (more) enter(hd);
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

template <int C, int DT>
int launch_gemm3(const _Float16* xh, const _Float16* xhl, const float* rs, const uint8_t* w, void* y, int M, int mrows,
                 int N, int K, int nt0, int ntiles, hipStream_t s) {
  const int mtiles = (M + G3_TM - 1) / G3_TM;
  constexpr int lds = g3_lds_bytes<C>();
  static_assert(lds <= 160 * 1024, "tile does not fit the LDS of a CU");
  auto kern = kquant_gemm3_kernel<C, DT>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  hipLaunchKernelGGL(kern, dim3(mtiles * ntiles), dim3(64 * G3_WAVES), lds, s, xh, xhl, rs, w, static_cast<uint16_t*>(y), M,
                     mrows, N, K, mtiles, nt0);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}


// ------------------------------------------------------------------ q6_k
// (block layout as the reference decodes it: src/kquant_cpu_decode.cpp:237-280)
// Same tile, same activation pipeline.  A q6_k weight sc (q - 32) reaches 4096 and goes in as two exact terms,
// sc ql and 16 sc (qh - 2), so a decoded fragment feeds sixteen MFMAs.  There is no minimum term: entering a
// superblock only changes the unit of the running sums.  Two superblock stages of 32 rows do not fit beside the
// activation stages, so the wire bytes travel by half superblocks (128 weights: 64 bytes of ql, 32 of qh, the
// scale piece, d) into two slots per wave: half h is consumed in K steps 2 h and 2 h + 1 from registers filled in
// step 2 h - 1, so its slot takes half h + 2 in step 2 h.
constexpr int Q6_SLOT_QH = 2048, Q6_SLOT_SC = 3072, Q6_SLOT_D = 3584, Q6_SLOT = 3712;
constexpr int Q6_W_INSTR = 5;  // load instructions per half: ql 2, qh 1, scales 1, d 1
template <int MT>
constexpr int g3_q6_lds_bytes() { return 2 * (32 * MT * G3_KS * 2) + G3_WAVES * 2 * Q6_SLOT; }

// MT = 8: 256 x 256 tiles; MT = 4: 128 x 256 tiles (a decoded fragment feeds eight MFMAs) for the column tiles
// that do not fill a round of one workgroup per CU.
template <int DT, int MT>
__global__ __launch_bounds__(64 * G3_WAVES, 1) void kquant_gemm3_q6k_kernel(const _Float16* __restrict__ xh,
                                                                           const float* __restrict__ rs,
                                                                           const uint8_t* __restrict__ w,
                                                                           uint16_t* __restrict__ y, int M, int mrows,
                                                                           int N, int K, int mtiles, int nt0) {
  constexpr int BPB = 210, TM = 32 * MT, A_STAGE = TM * G3_KS * 2, AQ = MT / 2;
  constexpr int A_OFF = 0, W_OFF = 2 * A_STAGE;
  constexpr int GPS = G3_KS / 16;   // MFMA groups per step: 4
  constexpr int SPS = 256 / G3_KS;  // steps per superblock: 4
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, kg = lane >> 5;
  const int mt = blockIdx.x % mtiles, nt = nt0 + blockIdx.x / mtiles;
  const int m0 = mt * TM, n0 = nt * G3_BN;
  const int nsb = K >> 8;
  const uint32_t row_bytes = (uint32_t)nsb * BPB;
  const int nrows = N - n0 < G3_BN ? N - n0 : G3_BN;
  const uint32_t lds0 = lds_addr(smem);

  // ---- load maps (activations as in the kernel above)
  auto swz = [](int row) { return (row >> 1) & 7; };
  uint32_t a_voff[AQ];
#pragma unroll
  for (int q = 0; q < AQ; q++) {
    const int r = 8 * (wave + 8 * q) + (lane >> 3);
    const int gr = m0 + r < mrows ? m0 + r : mrows - 1;
    a_voff[q] = (uint32_t)gr * (uint32_t)K * 2u + 16u * (uint32_t)((lane & 7) ^ swz(r));
  }
  const uint8_t* a_base = reinterpret_cast<const uint8_t*>(xh);
  // wire: a slot holds, for the wave's 32 rows, 64 bytes of ql (row-major, two load instructions), 32 bytes of qh
  // (one), the 16 scale bytes (half an instruction) and d (half a 2-byte instruction, zero-extended dwords).  Rows
  // past N re-read the last row (their columns are not stored).
  auto wrow = [&](int r) -> uint32_t {
    r += wave * 32;
    return (uint32_t)(r < nrows ? r : nrows - 1) * row_bytes;
  };
  uint32_t v_ql[2];
#pragma unroll
  for (int q = 0; q < 2; q++) v_ql[q] = wrow((64 * q + lane) >> 2) + 16u * (uint32_t)(lane & 3);
  const uint32_t v_qh = wrow(lane >> 1) + 128u + 16u * (uint32_t)(lane & 1);
  const uint32_t v_sc = wrow(l32) + 192u;
  const uint8_t* w_base = w + (size_t)n0 * row_bytes;

  auto issue_a = [&](int step) {
    const uint8_t* base = a_base + (size_t)step * (G3_KS * 2);
    const uint32_t l = lds0 + A_OFF + (step & 1) * A_STAGE + wave * 1024;
#pragma unroll
    for (int q = 0; q < AQ; q++) dma16(base, a_voff[q], l + q * (G3_WAVES * 1024));
  };
  const uint32_t w_lds = lds0 + W_OFF + wave * (2 * Q6_SLOT);
  auto issue_w = [&](int half) {  // half superblock `half` of this wave's rows -> slot half % 2
    const uint8_t* base = w_base + (size_t)(half >> 1) * BPB;
    const uint32_t hf = half & 1, l = w_lds + hf * Q6_SLOT;
    dma16(base + 64 * hf, v_ql[0], l);
    dma16(base + 64 * hf, v_ql[1], l + 1024);
    dma16(base + 32 * hf, v_qh, l + Q6_SLOT_QH);
    if (lane < 32) {
      dma16(base, v_sc, l + Q6_SLOT_SC);
      dma2(base, v_sc + 16u, l + Q6_SLOT_D);
    }
  };

  uint32_t a_addr[GPS];
#pragma unroll
  for (int g = 0; g < GPS; g++)
    a_addr[g] = (uint32_t)l32 * 128u + 16u * (uint32_t)((4 * (g >> 1) + 2 * kg + (g & 1)) ^ swz(l32));
  const uint8_t* slot0 = smem + W_OFF + wave * (2 * Q6_SLOT);

  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) acc[t] = f32x16{0};

  const uint32_t magic = opaque_vgpr(0x64006400u);
  const uint32_t mask_q = opaque_sgpr(0x00f000f0u), mask_h = opaque_sgpr(0x03000300u);

  // ---- this lane's weight row: registers of the half in hand
  struct Half {
    uint4 ql[2];      // ql[64 hf + 32 qr + 16 kg ..+15], qr = 0, 1
    uint4 qh;         // qh[32 hf + 16 kg ..+15]
    uint32_t scw[2];  // the half's eight int8 scales (zeros when d = 0: the half is fed as zeros)
  };
  float r = 1.0f, ratio = 1.0f;  // unit of the running sums; r_old / r_new of the superblock being entered
  // `first`: the half opens a superblock (its d changes the unit); commit = false leaves r alone (a dry run past K)
  auto load_half = [&](int hf, bool first, bool commit) -> Half {
    const uint8_t* sl = slot0 + hf * Q6_SLOT;
    Half hv;
    hv.ql[0] = *reinterpret_cast<const uint4*>(sl + l32 * 64 + 16 * kg);
    hv.ql[1] = *reinterpret_cast<const uint4*>(sl + l32 * 64 + 32 + 16 * kg);
    hv.qh = *reinterpret_cast<const uint4*>(sl + Q6_SLOT_QH + l32 * 32 + 16 * kg);
    const uint2 sc = *reinterpret_cast<const uint2*>(sl + Q6_SLOT_SC + l32 * 16 + 8 * hf);
    const float d = kq::h2f((uint16_t)(*reinterpret_cast<const uint32_t*>(sl + Q6_SLOT_D + l32 * 4) & 0xffff));
    hv.scw[0] = d != 0.f ? sc.x : 0u;
    hv.scw[1] = d != 0.f ? sc.y : 0u;
    if (first) {
      const float rn = d != 0.f ? d : r;  // a superblock with d = 0 keeps the unit
      ratio = r * __builtin_amdgcn_rcpf(rn);
      r = commit ? rn : r;
    }
    return hv;
  };

  // B fragments of MFMA group g of step p of a superblock: sub-block 32 t4 .. + 31 of the half with t4 = g / 2 +
  // 2 (p % 2) (low nibbles of the ql bytes in the half's first step, high nibbles in its second), K-half s = g % 2
  auto decode = [&](auto pc, auto gc, const Half& hv, f16x8& blo, f16x8& bhi) {
    constexpr int p = decltype(pc)::value, g = decltype(gc)::value;
    constexpr int h = p & 1, qr = g >> 1, s = g & 1, t4 = qr + 2 * h;
    const uint32_t qw[4] = {hv.ql[qr].x, hv.ql[qr].y, hv.ql[qr].z, hv.ql[qr].w};
    const uint32_t hw[4] = {hv.qh.x, hv.qh.y, hv.qh.z, hv.qh.w};
    const int sc = __builtin_amdgcn_sbfe((int)hv.scw[t4 >> 1], 8 * (2 * (t4 & 1) + kg), 8);
    const float scf = (float)sc;
    const _Float16 sch = (_Float16)(scf * 0.0625f), ofl = (_Float16)(-64.0f * scf), ofh = (_Float16)(-96.0f * scf);
    const f16x2 scp = {sch, sch}, oflp = {ofl, ofl}, ofhp = {ofh, ofh};
    uint32_t fl[4], fh[4];
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const uint32_t q = qw[2 * s + e], hq = hw[2 * s + e];
      const uint32_t qe = h ? q : (q << 4), qo = h ? (q >> 8) : (q >> 4);
      const uint32_t he = hq << (8 - 2 * t4), ho = t4 ? (hq >> (2 * t4)) : hq;
      fl[2 * e] = (qe & mask_q) | magic;      // bytes 0, 2 of the word: 1024 + 16 ql
      fl[2 * e + 1] = (qo & mask_q) | magic;  // bytes 1, 3
      fh[2 * e] = (he & mask_h) | magic;      // 1024 + 256 qh
      fh[2 * e + 1] = (ho & mask_h) | magic;
    }
    f16x2 bl2[4], bh2[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      // (1024 + 16 ql) sc / 16 - 64 sc = sc ql;  (1024 + 256 qh) sc / 16 - 96 sc = 16 sc (qh - 2)
      bl2[e] = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, fl[e]), scp, oflp);
      bh2[e] = __builtin_elementwise_fma(__builtin_bit_cast(f16x2, fh[e]), scp, ofhp);
    }
    blo = f16x8{bl2[0][0], bl2[0][1], bl2[1][0], bl2[1][1], bl2[2][0], bl2[2][1], bl2[3][0], bl2[3][1]};
    bhi = f16x8{bh2[0][0], bh2[0][1], bh2[1][0], bh2[1][1], bh2[2][0], bh2[2][1], bh2[3][0], bh2[3][1]};
  };

  // ---- prologue: first loads, registers of half 0, its first fragment
  const int nhalves = 2 * nsb, nsteps = SPS * nsb;
  issue_a(0);
  issue_w(0);
  issue_w(1);
  vmwait<Q6_W_INSTR>();  // own wire bytes of half 0 (and everything older) have landed
  Half cur = load_half(0, true, true);
  Half nxt = cur;
  f16x8 blo[2], bhi[2];
  decode(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, cur, blo[0], bhi[0]);

  // ---- main loop: step s = 4 sb + p.  The activation loads of step s + 1 are queued right after the barrier that
  // opens step s; half h + 2 follows in the first step of half h and may stay in flight over the next barrier.
  for (int sb = 0; sb < nsb; sb++) {
    const bool more = sb + 1 < nsb;
    StaticFor<SPS>::run([&](auto pc) {
      constexpr int p = decltype(pc)::value;
      constexpr int hf = p >> 1;
      const int step = SPS * sb + p, half = 2 * sb + hf;
      const uint8_t* a_stage = smem + A_OFF + (p & 1) * A_STAGE;
      // own loads of this step's activations have landed; a half queued after them may stay in flight
      if ((p & 1) && half + 2 < nhalves) vmwait<Q6_W_INSTR>(); else vmwait<0>();
      lds_barrier();
      if (step + 1 < nsteps) issue_a(step + 1);
      if (!(p & 1) && half + 2 < nhalves) issue_w(half + 2);
      f16x8 afr[MT];
#pragma unroll
      for (int t = 0; t < MT; t++) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[0] + t * 4096);
      StaticFor<GPS>::run([&](auto gc) {
        constexpr int g = decltype(gc)::value;
        // registers of the next half, from its slot (own loads, landed before the barrier that opened this step;
        // past the end: a harmless re-read)
        if constexpr ((p & 1) && g == GPS - 2) nxt = load_half(hf ^ 1, p == SPS - 1, more);
        // B fragments of the next group: of this step, of the half's second step, or of the next half
        if constexpr (g + 1 < GPS)
          decode(pc, std::integral_constant<int, g + 1>{}, cur, blo[(g + 1) & 1], bhi[(g + 1) & 1]);
        else if constexpr (!(p & 1))
          decode(std::integral_constant<int, p + 1>{}, std::integral_constant<int, 0>{}, cur, blo[0], bhi[0]);
        else
          decode(std::integral_constant<int, (p + 1) % SPS>{}, std::integral_constant<int, 0>{}, nxt, blo[0], bhi[0]);
#pragma unroll
        for (int t = 0; t < MT; t++) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[t], blo[g & 1], acc[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < MT; t++) {
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afr[t], bhi[g & 1], acc[t], 0, 0, 0);
          if constexpr (g + 1 < GPS) afr[t] = *reinterpret_cast<const f16x8*>(a_stage + a_addr[g + 1] + t * 4096);
        }
      });
      if constexpr (p & 1) cur = nxt;
      if constexpr (p == SPS - 1) {
        if (more) {  // the running sums change unit
#pragma unroll
          for (int t = 0; t < MT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[t][i] *= ratio;
        }
      }
    });
  }

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

template <int DT, int MT>
int launch_gemm3_q6k(const _Float16* xh, const float* rs, const uint8_t* w, void* y, int M, int mrows, int N, int K,
                     int nt0, int ntiles, hipStream_t s) {
  const int mtiles = (M + 32 * MT - 1) / (32 * MT);
  constexpr int lds = g3_q6_lds_bytes<MT>();
  static_assert(lds <= 160 * 1024, "tile does not fit the LDS of a CU");
  auto kern = kquant_gemm3_q6k_kernel<DT, MT>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  hipLaunchKernelGGL(kern, dim3(mtiles * ntiles), dim3(64 * G3_WAVES), lds, s, xh, rs, w, static_cast<uint16_t*>(y), M,
                     mrows, N, K, mtiles, nt0);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

}  // namespace

bool kq_gemm3_supported(int M, int mrows, int N, int K, int codec) {
  return (codec == KQ_Q4_K || codec == KQ_Q5_K || codec == KQ_Q6_K) && M >= 64 && mrows >= M && K >= 256 && (K & 255) == 0 &&
         N > 0 && (int64_t)256 * (K >> 8) * 210 < ((int64_t)1 << 32) && (int64_t)mrows * K * 2 < ((int64_t)1 << 32);
}

// Column tiles nt0 .. nt0 + ntiles - 1 (256 weight rows each) of y = x . W^T; xh / xhl / rs: outputs of the
// activation prepass with mrows >= M prepared rows (q6_k has no minimum term and reads no xhl; tile_rows = 128
// selects its 128-row form, any other value the 256-row tiles).
int kq_launch_gemm3(const void* xh, const void* xhl, const float* rs, const uint8_t* w, void* y, int M, int mrows, int N,
                    int K, int codec, int dtype, int nt0, int ntiles, hipStream_t s, int tile_rows) {
  if (!kq_gemm3_supported(M, mrows, N, K, codec)) return KQ_ERR_UNSUPPORTED;
  if (ntiles <= 0) return KQ_OK;
  const _Float16* a = static_cast<const _Float16*>(xh);
  const _Float16* h = static_cast<const _Float16*>(xhl);
  if (codec == KQ_Q6_K) {
    if (tile_rows == 128)
      return dtype == KQ_F16 ? launch_gemm3_q6k<KQ_F16, 4>(a, rs, w, y, M, mrows, N, K, nt0, ntiles, s)
                             : launch_gemm3_q6k<KQ_BF16, 4>(a, rs, w, y, M, mrows, N, K, nt0, ntiles, s);
    return dtype == KQ_F16 ? launch_gemm3_q6k<KQ_F16, 8>(a, rs, w, y, M, mrows, N, K, nt0, ntiles, s)
                           : launch_gemm3_q6k<KQ_BF16, 8>(a, rs, w, y, M, mrows, N, K, nt0, ntiles, s);
  }
  if (codec == KQ_Q4_K)
    return dtype == KQ_F16 ? launch_gemm3<KQ_Q4_K, KQ_F16>(a, h, rs, w, y, M, mrows, N, K, nt0, ntiles, s)
                           : launch_gemm3<KQ_Q4_K, KQ_BF16>(a, h, rs, w, y, M, mrows, N, K, nt0, ntiles, s);
  return dtype == KQ_F16 ? launch_gemm3<KQ_Q5_K, KQ_F16>(a, h, rs, w, y, M, mrows, N, K, nt0, ntiles, s)
                         : launch_gemm3<KQ_Q5_K, KQ_BF16>(a, h, rs, w, y, M, mrows, N, K, nt0, ntiles, s);
}
