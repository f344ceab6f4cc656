// Prefill GEMM for q4_k / q5_k / q6_k: y[M,N] = x[M,K] . W^T with M large, on the f16 matrix cores,
// exact in the weights (the B operand holds exact integers, see kq_mma.h).
//
// Activations are converted to f16 once by a prepass (scaled per row by a power of two so bf16
// inputs neither overflow nor lose bits) that also emits the sub-block sums of x as two f16 halves
// for the q4_k / q5_k minimum term.
//
// Tiling.  Workgroup = 4 or 8 waves, tile 64 or 128 (M) x 32 per wave (N), one 256-wide superblock of K per
// step; each wave owns all the tile's rows x 32 columns (2 or 4 accumulator tiles of
// v_mfma_f32_32x32x16_f16), so every weight is decoded by exactly one wave of the workgroup.  Wire bytes and activations are fetched
// with coalesced 16-byte loads into registers one step ahead and parked in LDS (activation rows
// padded by 16 bytes, wire rows an odd number of 16-byte pieces apart, which keeps the
// row-per-lane ds_read_b128 fragment fetch free of bank conflicts).
#include "kq_mma.h"

static int g_gemm_tile = 0;  // kq_set_gemm_tile_rows: 64, 128, 256, 512, 513, 1024 or 1025 forces the tile shape, 0 = automatic

namespace {

using namespace kqmma;

// ------------------------------------------------------------------ activation prepass
// One workgroup per row m (rows >= M are written as zeros): kqmma::prepass_row.
template <int DT>
__global__ __launch_bounds__(PP_THREADS) void gemm_prepass_kernel(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
                                                                  _Float16* __restrict__ xhl, float* __restrict__ rs,
                                                                  int M, int K) {
  __shared__ float red[PP_THREADS / 64];
  prepass_row<DT>(x, xh, xhl, rs, M, K, blockIdx.x, threadIdx.x, red);
}

// ------------------------------------------------------------------ main kernel
constexpr int BM = 128;
constexpr int A_STRIDE = 512 + 16;  // bytes per activation row of one K step in LDS

template <int C, int WAVES>
struct WireGeom : Wire<C> {
  static constexpr int THREADS = 64 * WAVES, BN = 32 * WAVES;
  static constexpr int PPR = Wire<C>::PP;                          // 16-byte pieces per row and step
  static constexpr int WPT = (BN * PPR + THREADS - 1) / THREADS;   // pieces per thread per step
};

// MT = 32-row activation blocks per workgroup tile (tile = 32 MT rows x 128 columns).  MT = 4 runs one
// workgroup per CU (one wave per SIMD) and is bound by LDS / MFMA latency it cannot hide; MT = 2 fits
// two workgroups per CU and measured 17 - 38 % faster although each decoded fragment feeds only two
// MFMAs (MT = 3 needs 256 registers and spills).
template <int C, int DT, int MT, int WAVES, bool DB>
__global__ __launch_bounds__(64 * WAVES, (MT == 4 || WAVES == 8) ? 1 : 2) void kquant_gemm_kernel(const _Float16* __restrict__ xh,
                                                                    const _Float16* __restrict__ xhl,
                                                                    const float* __restrict__ rs,
                                                                    const uint8_t* __restrict__ w,
                                                                    uint16_t* __restrict__ y, int M, int N, int K,
                                                                    int mtiles, int sb_per_split,
                                                                    float* __restrict__ part) {
  // part != null: grid y cuts the superblocks into ranges of sb_per_split, whose scaled f32 sums go to
  // part[range][M][N] and are added by gemm_splitk_reduce_kernel
  using G = WireGeom<C, WAVES>;
  constexpr int GM_THREADS = G::THREADS, BN = G::BN;
  constexpr int TM = 32 * MT;                   // activation rows per tile
  constexpr int A_BYTES = TM * A_STRIDE;
  constexpr int APT = TM * 32 / GM_THREADS;     // 16-byte activation pieces per thread per step
  constexpr int AROWS = GM_THREADS / 32;        // activation rows one pass of the workgroup covers
  static_assert(TM * 32 % GM_THREADS == 0 && 2 * TM <= GM_THREADS && BN <= GM_THREADS, "tile / thread count mismatch");
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // one stage: activations [TM][A_STRIDE] | wire [BN][LBPB] | X halves [TM][32] | side-channel d [BN] (q6_k);
  // DB keeps two stages so that the next step is parked while this one is multiplied
  constexpr int STAGE = A_BYTES + BN * G::LBPB + TM * 32 + BN * 2;
  static_assert(STAGE % 16 == 0, "stage size keeps 16-byte alignment");
  constexpr int B_OFF = A_BYTES, H_OFF = B_OFF + BN * G::LBPB, D_OFF = H_OFF + TM * 32;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, kg = lane >> 5;
  // consecutive workgroups share the weight columns (m fastest)
  const int mt = blockIdx.x % mtiles, nt = blockIdx.x / mtiles;
  const int m0 = mt * TM, n0 = nt * BN;
  const int nsb_all = K >> 8;
  const int sb0 = part ? (int)blockIdx.y * sb_per_split : 0;
  const int nsb = part ? (sb0 + sb_per_split < nsb_all ? sb_per_split : nsb_all - sb0) : nsb_all;  // steps of this workgroup
  const size_t row_bytes = (size_t)nsb_all * G::BPB;
  const int nrows = N - n0 < BN ? N - n0 : BN;

  // piece maps: activations piece i = tid + 256 t -> (row i / 32, piece i % 32); wire piece -> (row i / PPR, i % PPR)
  const int a_row = tid >> 5, a_pc = tid & 31;  // + AROWS rows per t
  uint32_t w_goff[G::WPT], w_loff[G::WPT];
  {
    int r = tid / G::PPR, pc = tid % G::PPR;
    StaticFor<G::WPT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      const bool ok = r < nrows;  // rows past N and the pieces past the tile re-read the tile start
      w_goff[T] = ok ? (uint32_t)r * (uint32_t)row_bytes + 16 * pc : 0;
      w_loff[T] = r < BN ? (uint32_t)r * G::LBPB + 16 * pc : 0xffffffffu;
      r += GM_THREADS / G::PPR;
      pc += GM_THREADS % G::PPR;
      if (pc >= G::PPR) {
        pc -= G::PPR;
        r++;
      }
    });
  }
  const uint8_t* wtile = w + (size_t)n0 * row_bytes + (size_t)sb0 * G::BPB;
  const _Float16* xtile = xh + (size_t)m0 * K + 256 * (size_t)sb0;
  const _Float16* htile = xhl + ((size_t)m0 * nsb_all + sb0) * 16;

  // side channel for the trailing 2-byte d of a q6_k block: thread -> row tid % BN
  const uint8_t* d_src = wtile + (size_t)((tid & (BN - 1)) < nrows ? (tid & (BN - 1)) : 0) * row_bytes + 208;
  u32x4 areg[APT], wreg[G::WPT], hreg;
  uint16_t dreg = 0;
  auto issue = [&](int sb) {
    StaticFor<APT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      areg[T] = *reinterpret_cast<const u32x4*>(xtile + (size_t)(a_row + AROWS * T) * K + 256 * sb + 8 * a_pc);
    });
    StaticFor<G::WPT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      wreg[T] = *reinterpret_cast<const typename G::piece_t*>(wtile + (size_t)sb * G::BPB + w_goff[T]);
    });
    if constexpr (G::SIDE_D) dreg = *reinterpret_cast<const uint16_t*>(d_src + (size_t)sb * G::BPB);
    // X halves: TM rows x 32 bytes = 2 TM pieces of 16 bytes (threads past them re-read the first rows)
    if constexpr (G::MINS)
      hreg = *reinterpret_cast<const u32x4*>(htile + ((size_t)((tid >> 1) < TM ? (tid >> 1) : 0) * nsb_all + sb) * 16 + 8 * (tid & 1));
  };
  auto park = [&](uint8_t* stage) {
    StaticFor<APT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      *reinterpret_cast<u32x4*>(stage + (a_row + AROWS * T) * A_STRIDE + 16 * a_pc) = areg[T];
    });
    StaticFor<G::WPT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      if (w_loff[T] != 0xffffffffu) *reinterpret_cast<u32x4*>(stage + B_OFF + w_loff[T]) = wreg[T];
    });
    if constexpr (G::MINS) {
      if (tid < 2 * TM) *reinterpret_cast<u32x4*>(stage + H_OFF + 16 * tid) = hreg;
    }
    if constexpr (G::SIDE_D) {
      if (tid < BN) reinterpret_cast<uint16_t*>(stage + D_OFF)[tid] = dreg;
    }
  };
  f32x16 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; t++) acc[t] = f32x16{0};

  auto multiply = [&](const uint8_t* stage) {
    const uint16_t d_side = G::SIDE_D ? reinterpret_cast<const uint16_t*>(stage + D_OFF)[wave * 32 + l32] : (uint16_t)0;
    superblock_mma<C, MT>(stage + B_OFF + (wave * 32 + l32) * G::LBPB, d_side, kg, stage + l32 * A_STRIDE + 32 * kg,
                         32 * A_STRIDE, stage + H_OFF + l32 * 32 + 16 * kg, 32 * 32, acc);
  };

  issue(0);
  if constexpr (DB) {
    // Two stages: step sb + 1 is parked into the idle stage (its loads were issued one whole step earlier),
    // the loads of step sb + 2 go out, then step sb is multiplied; ONE barrier per step tells everyone that
    // the stage just read may be overwritten and that the stage just written may be read.
    park(smem);
    if (nsb > 1) issue(1);
    lds_barrier();
    for (int sb = 0; sb < nsb; sb++) {
      uint8_t* cur = smem + (sb & 1) * STAGE;
      uint8_t* nxt = smem + ((sb + 1) & 1) * STAGE;
      if (sb + 1 < nsb) {
        park(nxt);
        if (sb + 2 < nsb) issue(sb + 2);
      }
      multiply(cur);
      lds_barrier();
    }
  } else {
    for (int sb = 0; sb < nsb; sb++) {
      if (sb > 0) lds_barrier();  // everyone is done reading the previous step
      park(smem);
      if (sb + 1 < nsb) issue(sb + 1);
      lds_barrier();
      multiply(smem);
    }
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
        if (part)
          part[((size_t)blockIdx.y * M + m) * N + n] = v;
        else
          y[(size_t)m * N + n] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
      }
    }
  }
}

// y[i] = round(sum over the K ranges of part[range][i]), ranges added in order
template <int DT>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(const float* __restrict__ part, uint16_t* __restrict__ y,
                                                                 size_t count, int splits) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  float v = 0.f;
  for (int sp = 0; sp < splits; sp++) v += part[(size_t)sp * count + i];
  y[i] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
}

// Superblocks per workgroup of a call on 64 x 128 tiles: K is cut while at most 512 workgroups exist (at least two
// superblocks each) and the partial sums stay within 8 MiB (their write and read cost about 0.5 us per MiB: cut in
// three, 128 rows on 14336 x 4096 went from 39 to 50 us); calls with 256 tiles or more run uncut (returns K / 256).
int gemm_sb_per_split(int M, int N, int K) {
  const int nsb = K >> 8;
  const int64_t tiles = (int64_t)((M + 63) / 64) * ((N + 127) / 128);
  if (tiles >= 256 || nsb < 4) return nsb;
  int64_t want = 512 / tiles;
  const int64_t cap = ((int64_t)8 << 20) / ((int64_t)M * N * 4);
  if (want > cap) want = cap;
  if (want > nsb / 2) want = nsb / 2;
  if (want < 2) return nsb;
  return (int)((nsb + want - 1) / want);
}

size_t gemm_base_bytes(int M, int K) {
  const size_t mpad = (size_t)((M + BM - 1) / BM) * BM;
  return mpad * K * 2 + mpad * (K >> 8) * 32 + mpad * 4 + 256;
}

template <int C, int DT, int MT, int WAVES, bool DB = false>
int launch_gemm_mt(const _Float16* xh, const _Float16* xhl, const float* rs, const uint8_t* w, void* y, int M, int N,
                   int K, hipStream_t s, int sb_per_split = 0, float* part = nullptr) {
  using G = WireGeom<C, WAVES>;
  constexpr int TM = 32 * MT, BN = G::BN;
  const int mtiles = (M + TM - 1) / TM, ntiles = (N + BN - 1) / BN;
  const size_t lds = (size_t)(TM * A_STRIDE + BN * G::LBPB + TM * 32 + BN * 2) * (DB ? 2 : 1);
  auto kern = kquant_gemm_kernel<C, DT, MT, WAVES, DB>;
  KQ_SET_MAX_LDS_ONCE((kern), lds);
  const int splits = part ? ((K >> 8) + sb_per_split - 1) / sb_per_split : 1;
  hipLaunchKernelGGL(kern, dim3(mtiles * ntiles, splits), dim3(G::THREADS), lds, s, xh, xhl, rs, w,
                     static_cast<uint16_t*>(y), M, N, K, mtiles, sb_per_split, part);
  if (part) {
    const size_t count = (size_t)M * N;
    hipLaunchKernelGGL((gemm_splitk_reduce_kernel<DT>), dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, part,
                       static_cast<uint16_t*>(y), count, splits);
  }
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}


int gemm_num_cus() {
  // compute units of the current device, looked up once per device
  static std::atomic<int> cus[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

template <int C, int DT>
int launch_gemm(const void* x, const uint8_t* w, void* y, int M, int N, int K, void* ws, size_t ws_bytes, hipStream_t s) {
  const int mpad = ((M + BM - 1) / BM) * BM, nsb = K >> 8;
  _Float16* xh = static_cast<_Float16*>(ws);
  _Float16* xhl = xh + (size_t)mpad * K;
  float* rs = reinterpret_cast<float*>(xhl + (size_t)mpad * nsb * 16);
  hipLaunchKernelGGL((gemm_prepass_kernel<DT>), dim3(mpad), dim3(PP_THREADS), 0, s, static_cast<const uint16_t*>(x), xh,
                     xhl, rs, M, K);
  KQ_HIP_CHECK(hipGetLastError());
  // Tile shapes (activation rows x weight rows): 64 x 128, one stage, two workgroups per CU: the default;
  // 128 x 128, one workgroup per CU: selectable only (measured slower);
  // 64 x 256 on 8 waves with two LDS stages (q4_k; q5_k would fit but measured slower, q6_k does not fit):
  // one barrier per step instead of two and the next step is parked while this one is multiplied, measured
  // 5 - 9 % faster once every CU gets 8 or more workgroups, slower below (fewer, longer workgroups).
  int tile = g_gemm_tile;
  // 128 x 256 tiles with 128-row wave tiles and direct-to-LDS loads (kq_gemm2.hip, q4_k / q5_k): one decoded
  // weight fragment feeds four MFMAs instead of two.  Taken when the matrix fills the 256 CUs with whole
  // workgroups of that size; `512` forces it, `513` its 128 x 128 / four-wave form.
  if constexpr (C != KQ_Q6_K) {
    // 256 x 256 tiles with 256-row wave tiles on one accumulator set (kq_gemm3.hip): a decoded fragment feeds eight
    // MFMAs.  Such tiles are few (2048 x 28672: 896 on 256 CUs), so they take the column tiles that fill whole rounds
    // of one workgroup per CU and the 128 x 256 kernel takes the rest (there: 96 + 16 column tiles = 3 + 1 rounds);
    // a matrix of less than one round runs on them whole when it fills three quarters of the CUs (512 x 28672: 224
    // workgroups, 10 % faster than 448 of the 128-row kernel).  `1024` forces them for every column tile, `512` /
    // `513` keep the 128-row kernels.
    const int nt256 = (N + 255) / 256;
    if (tile == 1024 && kq_gemm3_supported(M, mpad, N, K, C)) return kq_launch_gemm3(xh, xhl, rs, w, y, M, mpad, N, K, C, DT, 0, nt256, s);
    if (tile == 0 && M >= 256 && kq_gemm3_supported(M, mpad, N, K, C)) {
      const int mt256 = (M + 255) / 256, cus = gemm_num_cus();
      const int64_t tiles = (int64_t)mt256 * nt256;
      int tall = (int)((tiles / cus) * cus / mt256);  // column tiles in whole rounds
      if (tall == 0 && 4 * tiles >= 3 * (int64_t)cus) tall = nt256;
      if (tall > 0) {
        int rc = kq_launch_gemm3(xh, xhl, rs, w, y, M, mpad, N, K, C, DT, 0, tall, s);
        if (rc != KQ_OK || tall == nt256) return rc;
        rc = kq_launch_gemm2(xh, xhl, rs, w, y, M, N, K, C, DT, 0, s, tall, nt256 - tall);
        if (rc != KQ_ERR_UNSUPPORTED) return rc;
        return kq_launch_gemm3(xh, xhl, rs, w, y, M, mpad, N, K, C, DT, tall, nt256 - tall, s);
      }
    }
  }
  if constexpr (C == KQ_Q6_K) {
    // q6_k on the tiles of kq_gemm3.hip (two exact terms per weight: a decoded fragment feeds sixteen MFMAs on 256-row
    // tiles, eight on 128-row tiles).  One workgroup per CU, so a call costs whole rounds: a round of 256-row tiles
    // counts 200, a round of 128-row tiles 119 (measured: 0.59 of the taller tile's time), the 64-row kernel 167 per
    // 256 half-height tiles whatever their number (it runs at 0.6 of the rate and fills the chip with small
    // workgroups, K cut over the grid when they are few).  Candidates: every column tile on one tile height, or the
    // column tiles that fill whole rounds at 256 rows and the rest at whichever height is cheaper (2048 x 28672:
    // 96 + 16 column tiles = 3 rounds + 1 round of half-height tiles).  `1024` forces the 256-row form for every
    // column tile, `1025` the 128-row form.
    const int nt256 = (N + 255) / 256, mt256 = (M + 255) / 256, mt128 = (M + 127) / 128;
    const int64_t cus = gemm_num_cus();
    if ((tile == 1024 || tile == 1025) && kq_gemm3_supported(M, mpad, N, K, C))
      return kq_launch_gemm3(xh, xhl, rs, w, y, M, mpad, N, K, C, DT, 0, nt256, s, tile == 1025 ? 128 : 256);
    if (tile == 0 && M >= 128 && kq_gemm3_supported(M, mpad, N, K, C)) {
      auto rounds = [&](int64_t wgs) { return (wgs + cus - 1) / cus; };
      const int64_t c64 = (int64_t)mt128 * nt256 * 167 / cus;
      const int64_t c128 = rounds((int64_t)mt128 * nt256) * 119;
      const int64_t full = (int64_t)mt256 * nt256 / cus;      // whole rounds of 256-row tiles
      const int tall = full > 0 ? (int)(full * cus / mt256) : 0;  // column tiles in them
      const int rest = nt256 - tall;
      const int64_t rest256 = rounds((int64_t)mt256 * rest) * 200, rest128 = rounds((int64_t)mt128 * rest) * 119;
      const int64_t c256 = full * 200 + (rest128 < rest256 ? rest128 : rest256);
      if (c256 <= c128 && c256 < c64) {
        if (tall > 0) {
          const int rc = kq_launch_gemm3(xh, xhl, rs, w, y, M, mpad, N, K, C, DT, 0, tall, s);
          if (rc != KQ_OK || rest == 0) return rc;
        }
        return kq_launch_gemm3(xh, xhl, rs, w, y, M, mpad, N, K, C, DT, tall, rest, s, rest128 < rest256 ? 128 : 256);
      }
      if (c128 < c64) return kq_launch_gemm3(xh, xhl, rs, w, y, M, mpad, N, K, C, DT, 0, nt256, s, 128);
    }
  }
  if (tile == 512 || tile == 513 || (tile == 0 && M >= 256 && (int64_t)((M + 127) / 128) * ((N + 255) / 256) >= 256)) {
    const int rc = kq_launch_gemm2(xh, xhl, rs, w, y, M, N, K, C, DT, tile == 513 ? 1 : 0, s);
    if (rc != KQ_ERR_UNSUPPORTED) return rc;
  }
  if (tile == 512 || tile == 513 || tile == 1024 || tile == 1025) tile = 0;
  if (tile == 256 && C != KQ_Q4_K) tile = 0;
  if (tile == 0) {
    const int64_t wgs = (int64_t)((M + 63) / 64) * ((N + 255) / 256);
    tile = (C == KQ_Q4_K && wgs >= 8 * 256) ? 256 : 64;
  }
  if constexpr (C == KQ_Q4_K) {
    if (tile == 256) return launch_gemm_mt<C, DT, 2, 8, true>(xh, xhl, rs, w, y, M, N, K, s);
  }
  if (tile == 128) return launch_gemm_mt<C, DT, 4, 4>(xh, xhl, rs, w, y, M, N, K, s);
  // few tiles: cut K over the grid when the workspace also holds the partial sums
  const int per = g_gemm_tile == 0 ? gemm_sb_per_split(M, N, K) : nsb;
  if (per < nsb) {
    const size_t base = (gemm_base_bytes(M, K) + 255) & ~(size_t)255;
    const int splits = (nsb + per - 1) / per;
    if (ws_bytes >= base + (size_t)splits * M * N * 4)
      return launch_gemm_mt<C, DT, 2, 4>(xh, xhl, rs, w, y, M, N, K, s, per,
                                         reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + base));
  }
  return launch_gemm_mt<C, DT, 2, 4>(xh, xhl, rs, w, y, M, N, K, s);
}

}  // namespace

// Required part of the workspace: converted activations, block sums, row scales
size_t kq_gemm_workspace_min_bytes(int M, int K) { return gemm_base_bytes(M, K); }

// ... plus the f32 partial sums of a K range cut over the grid (calls with few tiles; optional: a call whose
// workspace holds only the required part runs uncut)
size_t kq_gemm_workspace_bytes(int M, int N, int K) {
  const size_t base = gemm_base_bytes(M, K);
  if (M <= 0 || N <= 0 || K < 256) return base;
  if (M >= 256 && (int64_t)((M + 127) / 128) * ((N + 255) / 256) >= 256) return base;
  const int nsb = K >> 8, per = gemm_sb_per_split(M, N, K);
  if (per >= nsb) return base;
  return ((base + 255) & ~(size_t)255) + (size_t)((nsb + per - 1) / per) * M * N * 4;
}

bool kq_gemm_supported(int M, int N, int K, int codec) {
  return (codec == KQ_Q4_K || codec == KQ_Q5_K || codec == KQ_Q6_K) && M > 8 && K > 0 && (K & 255) == 0 && N > 0;
}

int kq_launch_gemm(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                   size_t ws_bytes, hipStream_t s) {
  if (!kq_gemm_supported(M, N, K, codec)) return KQ_ERR_UNSUPPORTED;
  const uintptr_t wmask = codec == KQ_Q6_K ? 1 : 15;  // q6_k pieces are fetched with unaligned loads
  if ((reinterpret_cast<uintptr_t>(w) & wmask) || (reinterpret_cast<uintptr_t>(x) & 15) || (reinterpret_cast<uintptr_t>(ws) & 15))
    return KQ_ERR_UNSUPPORTED;
  if (codec == KQ_Q6_K)
    return dtype == KQ_F16 ? launch_gemm<KQ_Q6_K, KQ_F16>(x, w, y, M, N, K, ws, ws_bytes, s)
                           : launch_gemm<KQ_Q6_K, KQ_BF16>(x, w, y, M, N, K, ws, ws_bytes, s);
  if (codec == KQ_Q4_K)
    return dtype == KQ_F16 ? launch_gemm<KQ_Q4_K, KQ_F16>(x, w, y, M, N, K, ws, ws_bytes, s)
                           : launch_gemm<KQ_Q4_K, KQ_BF16>(x, w, y, M, N, K, ws, ws_bytes, s);
  return dtype == KQ_F16 ? launch_gemm<KQ_Q5_K, KQ_F16>(x, w, y, M, N, K, ws, ws_bytes, s)
                         : launch_gemm<KQ_Q5_K, KQ_BF16>(x, w, y, M, N, K, ws, ws_bytes, s);
}

int kq_launch_act_prepass(const void* x, void* xh, void* xhl, float* rs, int M, int K, int dtype, hipStream_t s) {
  if (M <= 0) return KQ_OK;
  if (dtype == KQ_F16)
    hipLaunchKernelGGL((gemm_prepass_kernel<KQ_F16>), dim3(M), dim3(PP_THREADS), 0, s, static_cast<const uint16_t*>(x),
                       static_cast<_Float16*>(xh), static_cast<_Float16*>(xhl), rs, M, K);
  else
    hipLaunchKernelGGL((gemm_prepass_kernel<KQ_BF16>), dim3(M), dim3(PP_THREADS), 0, s, static_cast<const uint16_t*>(x),
                       static_cast<_Float16*>(xh), static_cast<_Float16*>(xhl), rs, M, K);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

extern "C" void kq_set_gemm_tile_rows(int rows) {
  kq_gemm3b_force_tile(rows);
  kq_gemm3f_force_tile(rows);
  kq_gemm3i_force_tile(rows);
  g_gemm_tile = (rows == 64 || rows == 128 || rows == 256 || rows == 512 || rows == 513 || rows == 1024 || rows == 1025) ? rows : 0;
}
