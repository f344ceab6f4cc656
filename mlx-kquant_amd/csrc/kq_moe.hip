// Grouped MoE GEMM: the fused gate/up GLU op and the gathered down projection for many
// (token, expert) pairs.  Pairs are counting-sorted by expert on the device and cut into segments
// of at most 32 pairs of one expert; a workgroup multiplies one segment (the 32 activation rows of
// v_mfma_f32_32x32x16_f16) by a 128-row slab of that expert's weights, so an expert's wire bytes are
// streamed from HBM once per 32 pairs instead of once per pair.
//
// Workgroup = 4 waves.  Plain op: each wave owns 32 of the slab's 128 weight rows.  GLU: the slab
// is 64 gate rows + the same 64 up rows (waves 0/2 gate, 1/3 up); the up waves hand their
// accumulators to the gate waves through LDS and the epilogue act(g) * u runs before the single
// rounding.  K advances one 256-wide superblock per step; wire bytes and the gathered activation
// rows (converted to f16 by the activation prepass) are fetched one step ahead with coalesced
// 16-byte loads and parked in LDS.
#include "kq_epilogue.h"
#include "kq_mma.h"
#include "kq_moe_sort.h"

int kq_launch_act_prepass(const void* x, void* xh, void* xhl, float* rs, int M, int K, int dtype, hipStream_t s);

namespace {

using namespace kqmma;
using kqsort::moe_sort_body;
using kqsort::Segment;
using kqsort::SEG_M;
using kqsort::SORT_MAX_E;

constexpr int MOE_THREADS = 256;
constexpr int SLAB = 128;            // weight rows per workgroup (GLU: 64 gate + 64 up)
constexpr int A_STRIDE = 512 + 16;   // bytes per activation row of one K step in LDS
// LDS stages of the grouped kernel.  Two stages (next step parked while this one is multiplied, one barrier per
// step) cost a resident workgroup per CU and measured slower: 76.9 / 89.2 us against 72.7 / 64.7 us for the
// GLU / down ops at 256 tokens, 128 experts.
#ifndef KQ_MOE_STAGES
#define KQ_MOE_STAGES 1
#endif
constexpr int MOE_STAGES = KQ_MOE_STAGES;
constexpr int SORT_THREADS = 1024;

__global__ __launch_bounds__(SORT_THREADS) void moe_sort_kernel(const uint32_t* __restrict__ idx, int P, int E,
                                                               int* __restrict__ order, Segment* __restrict__ segs,
                                                               int* __restrict__ nseg_out) {
  __shared__ int cnt[SORT_MAX_E];     // pairs per expert, then the running cursor
  __shared__ int scan_p[SORT_THREADS], scan_s[SORT_THREADS];
  moe_sort_body<SORT_THREADS>(idx, P, E, order, segs, nseg_out, cnt, scan_p, scan_s);
}

// The pair sort and the activation prepass of one grouped launch in ONE kernel: workgroup 0 sorts the pairs, workgroups
// 1 .. rows convert one activation row each (neither depends on the other).  One launch fewer
// per op; at 256 tokens the op time measured the same as with two launches.
template <int DT>
__global__ __launch_bounds__(PP_THREADS) void moe_prologue_kernel(const uint16_t* __restrict__ x, _Float16* __restrict__ xh,
                                                                  _Float16* __restrict__ xhl, float* __restrict__ rs,
                                                                  int rows, int K, const uint32_t* __restrict__ idx, int P,
                                                                  int E, int* __restrict__ order,
                                                                  Segment* __restrict__ segs, int* __restrict__ nseg_out) {
  __shared__ int cnt[SORT_MAX_E];
  __shared__ int scan_p[PP_THREADS], scan_s[PP_THREADS];
  __shared__ float red[PP_THREADS / 64];
  if (blockIdx.x == 0)  // the sort is the longest workgroup of the launch (a chain of barriers): it goes first
    moe_sort_body<PP_THREADS>(idx, P, E, order, segs, nseg_out, cnt, scan_p, scan_s);
  else
    prepass_row<DT>(x, xh, xhl, rs, rows, K, blockIdx.x - 1, threadIdx.x, red);
}

// ------------------------------------------------------------------ row gather (batched gather_qmm)
// One workgroup per output row p = b*M + m: copies the K 16-bit activations of x[lhs[b]][m] to
// xg[p] and notes the row's expert, so that the grouped kernels below see a plain [P, K] matrix.
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint16_t* __restrict__ x, const uint32_t* __restrict__ lhs,
                                                          const uint32_t* __restrict__ rhs, uint16_t* __restrict__ xg,
                                                          uint32_t* __restrict__ idx_rows, int M, int K,
                                                          int64_t x_batch_stride) {
  const int p = blockIdx.x, b = p / M, m = p - b * M;
  const uint16_t* src = x + (size_t)(lhs ? lhs[b] : (uint32_t)b) * (size_t)x_batch_stride + (size_t)m * K;
  uint16_t* dst = xg + (size_t)p * K;
  for (int g = threadIdx.x; g < (K >> 3); g += 256)
    *reinterpret_cast<u32x4*>(dst + 8 * g) = *reinterpret_cast<const u32x4*>(src + 8 * g);
  if (threadIdx.x == 0) idx_rows[p] = rhs ? rhs[b] : 0u;
}

// idx2[t][s] = idx[t][s] for s < S - 1, expert 0 in the last slot (its product is overwritten later)
__global__ __launch_bounds__(256) void pad_idx_kernel(const uint32_t* __restrict__ idx, uint32_t* __restrict__ idx2, int T,
                                                      int S) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= T * S) return;
  const int t = i / S, s = i - t * S;
  idx2[i] = s < S - 1 ? idx[t * (S - 1) + s] : 0u;
}

// out[t][n] = T(sum_s scores[t][s] * yf[t][s][n]), f32, slots in order.  idx [T][routed]: the expert ids of the
// first `routed` slots; a slot whose id is >= E was skipped by the matmul kernels (its row of yf holds nothing)
// and adds nothing.
template <int DT>
__global__ __launch_bounds__(256) void mix_slots_kernel(const float* __restrict__ yf, const float* __restrict__ scores,
                                                        const uint32_t* __restrict__ idx, int routed, int E,
                                                        uint16_t* __restrict__ out, int T, int S, int N) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)T * N) return;
  const int t = (int)(i / N), n = (int)(i - (int64_t)t * N);
  float v = 0.f;
  for (int s = 0; s < S; s++) {
    if (s < routed && idx[(size_t)t * routed + s] >= (uint32_t)E) continue;
    v = fmaf(scores[t * S + s], yf[((size_t)t * S + s) * N + n], v);
  }
  out[i] = DT == KQ_F16 ? kq::f2f16(v) : kq::f2bf16(v);
}

// ------------------------------------------------------------------ expert tile map (sorted prefill GEMM)
// From expert-sorted routing indices, the (expert, first row, rows <= 64) tiles of every expert's run of rows;
// only the last tile of a run is partial.  One workgroup: each thread walks a contiguous chunk of rows (one
// binary search for the run its chunk starts in), a block scan numbers the tiles in row order, a second walk
// writes them.  Rows whose expert id is out of range belong to no tile.
constexpr int TILE_ROWS = 64;

__device__ __forceinline__ int first_row_of(const uint32_t* idx, int rows, uint32_t e) {  // lower bound
  int lo = 0, hi = rows;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (idx[mid] < e) lo = mid + 1; else hi = mid;
  }
  return lo;
}

__device__ __forceinline__ int end_row_of(const uint32_t* idx, int rows, uint32_t e) {  // upper bound
  int lo = 0, hi = rows;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (idx[mid] <= e) lo = mid + 1; else hi = mid;
  }
  return lo;
}

__global__ __launch_bounds__(SORT_THREADS) void expert_tile_map_kernel(const uint32_t* __restrict__ idx, int rows, int E,
                                                                      uint32_t* __restrict__ map, int cap,
                                                                      uint32_t* __restrict__ counts) {
  __shared__ int scan[SORT_THREADS];
  const int tid = threadIdx.x;
  const int ch = (rows + SORT_THREADS - 1) / SORT_THREADS;
  const int r0 = min(tid * ch, rows), r1 = min(r0 + ch, rows);
  int slot = 0;
  for (int pass = 0; pass < 2; pass++) {
    int n = 0, run_start = 0;
    uint32_t run_e = 0xffffffffu;
    for (int r = r0; r < r1; r++) {
      const uint32_t e = idx[r];
      if (r == r0 || e != run_e) {
        run_e = e;
        run_start = (r > r0) ? r : first_row_of(idx, rows, e);
      }
      if (e >= (uint32_t)E || (r - run_start) % TILE_ROWS) continue;
      if (pass == 1 && slot + n < cap) {
        const int left = end_row_of(idx, rows, e) - r;
        uint32_t* t = map + 3 * (size_t)(slot + n);
        t[0] = e;
        t[1] = (uint32_t)r;
        t[2] = (uint32_t)(left < TILE_ROWS ? left : TILE_ROWS);
      }
      n++;
    }
    if (pass == 1) break;
    scan[tid] = n;
    __syncthreads();
    for (int off = 1; off < SORT_THREADS; off <<= 1) {
      const int v = tid >= off ? scan[tid - off] : 0;
      __syncthreads();
      scan[tid] += v;
      __syncthreads();
    }
    slot = scan[tid] - n;
    if (tid == SORT_THREADS - 1) counts[0] = (uint32_t)(scan[tid] < cap ? scan[tid] : cap);
  }
}

// row_expert[r] = `none` everywhere, then the expert of the tile that covers row r
__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* __restrict__ p, int n, uint32_t v) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = v;
}

__global__ __launch_bounds__(TILE_ROWS) void tiles_to_rows_kernel(const uint32_t* __restrict__ map,
                                                                  const uint32_t* __restrict__ counts, int cap, int rows,
                                                                  int E, uint32_t* __restrict__ row_expert) {
  const int t = blockIdx.x;
  const uint32_t nt = counts[0];
  if ((uint32_t)t >= nt) return;
  const uint32_t e = map[3 * t], start = map[3 * t + 1], n = map[3 * t + 2];
  const uint32_t j = threadIdx.x;
  if (e >= (uint32_t)E || j >= n || start >= (uint32_t)rows || j >= (uint32_t)rows - start) return;
  row_expert[start + j] = e;
}

// ------------------------------------------------------------------ mxfp4: MLX packed layout <-> GGUF wire
// MLX keeps the 32 codes of a block in sequence (byte b = code 2b | code 2b+1 << 4, eight codes per uint32) and
// the e8m0 scale bytes in a tensor of their own; the GGUF block is the scale byte followed by 16 bytes holding
// code j in the low and code j + 16 in the high nibble.  One thread moves one block.
__global__ __launch_bounds__(256) void mxfp4_packed_to_wire_kernel(const uint32_t* __restrict__ packed,
                                                                   const uint8_t* __restrict__ scales,
                                                                   uint8_t* __restrict__ wire, int64_t nblocks) {
  const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (b >= nblocks) return;
  const u32x4 v = *reinterpret_cast<const u32x4*>(packed + 4 * b);
  const uint64_t lo = (uint64_t)v[0] | ((uint64_t)v[1] << 32), hi = (uint64_t)v[2] | ((uint64_t)v[3] << 32);
  uint8_t* o = wire + 17 * b;
  o[0] = scales[b];
#pragma unroll
  for (int j = 0; j < 16; j++) o[1 + j] = (uint8_t)(((lo >> (4 * j)) & 15) | (((hi >> (4 * j)) & 15) << 4));
}

__global__ __launch_bounds__(256) void mxfp4_wire_to_packed_kernel(const uint8_t* __restrict__ wire,
                                                                   uint32_t* __restrict__ packed,
                                                                   uint8_t* __restrict__ scales, int64_t nblocks) {
  const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (b >= nblocks) return;
  const uint8_t* in = wire + 17 * b;
  uint64_t lo = 0, hi = 0;
#pragma unroll
  for (int j = 0; j < 16; j++) {
    lo |= (uint64_t)(in[1 + j] & 15) << (4 * j);
    hi |= (uint64_t)(in[1 + j] >> 4) << (4 * j);
  }
  scales[b] = in[0];
  *reinterpret_cast<u32x4*>(packed + 4 * b) = u32x4{(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
}

// ------------------------------------------------------------------ grouped GEMM
struct MoeArgs {
  const _Float16* xh;   // [rows][K] f16 activations (prepass), row = pair / x_div
  const _Float16* xhl;  // [rows][K/256][16] X halves
  const float* rs;      // [rows] activation scale
  const uint8_t* w;
  const uint8_t* w2;    // up stack (GLU) or null
  void* y;              // [P][N]
  const int* order;
  const Segment* segs;
  const int* nseg;
  int N, K, x_div, act;
  int64_t w_expert_stride;
  float limit;
  KqOutMap om;
};

template <int C, int DT, bool GLU>
__global__ __launch_bounds__(MOE_THREADS, 3) void moe_grouped_kernel(MoeArgs a) {
  using G = Wire<C>;
  constexpr int WPT = (SLAB * G::PP + MOE_THREADS - 1) / MOE_THREADS;  // wire pieces per thread per step
  constexpr int APT = SEG_M * 32 / MOE_THREADS;                         // activation pieces per thread per step (4)
  constexpr int NCOLS = GLU ? SLAB / 2 : SLAB;                          // output columns per workgroup
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // two stages of: activations [32][A_STRIDE] | wire [128][LBPB] | X halves [32][32] | side-channel d [128]
  constexpr int B_OFF = SEG_M * A_STRIDE, H_OFF = B_OFF + SLAB * G::LBPB, D_OFF = H_OFF + SEG_M * 32;
  constexpr int STAGE = D_OFF + SLAB * 2;
  static_assert(STAGE % 16 == 0, "stages keep 16-byte alignment");
  int* pair_lds = reinterpret_cast<int*>(smem + MOE_STAGES * STAGE);  // [32] output row of each segment slot, -1 = none
  float* rs_lds = reinterpret_cast<float*>(pair_lds + SEG_M);         // [32]

  // Workgroups go to the 8 XCDs round-robin in launch order.  Launch position L = 8 j + c runs slab j % tiles of
  // segment 8 (j / tiles) + c: all slabs of a segment sit on one XCD, back to back, so the segment's activation
  // rows are fetched into one L2 once instead of into all eight (grid y is a multiple of 8).
  const int lin = blockIdx.x + gridDim.x * blockIdx.y;
  const int slab_id = (lin >> 3) % (int)gridDim.x;
  const int seg_id = ((lin >> 3) / (int)gridDim.x) * 8 + (lin & 7);
  if (seg_id >= *a.nseg) return;  // uniform: the grid is sized for the worst case
  const Segment seg = a.segs[seg_id];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, kg = lane >> 5;
  const int N = a.N, K = a.K, nsb = K >> 8;
  const size_t row_bytes = (size_t)nsb * G::BPB;
  const int n0 = slab_id * NCOLS;
  const int ncols = N - n0 < NCOLS ? N - n0 : NCOLS;
  const uint8_t* wtile = a.w + (size_t)seg.expert * (size_t)a.w_expert_stride + (size_t)n0 * row_bytes;
  const uint8_t* wtile2 = GLU ? a.w2 + (size_t)seg.expert * (size_t)a.w_expert_stride + (size_t)n0 * row_bytes : wtile;

  // slab row rr (= wave * 32 + l32 in the compute phase) -> (matrix, column): GLU waves alternate gate / up
  auto slab_col = [&](int rr, bool& up) {
    if constexpr (GLU) {
      const int wv = rr >> 5;
      up = wv & 1;
      return (wv >> 1) * 32 + (rr & 31);
    } else {
      up = false;
      return rr;
    }
  };

  if (tid < SEG_M) {
    const int pr = tid < seg.count ? a.order[seg.start + tid] : -1;
    pair_lds[tid] = pr;
    rs_lds[tid] = pr >= 0 ? a.rs[pr / a.x_div] : 0.f;
  }

  // piece maps.  Activations: piece i = tid + 256 t -> (slot i / 32, piece i % 32); spare slots of a
  // short segment re-read its first pair (their results are dropped).
  const int a_slot = tid >> 5, a_pc = tid & 31;  // + 8 slots per t
  size_t a_goff[APT];
  StaticFor<APT>::run([&](auto t) {
    constexpr int T = decltype(t)::value;
    const int slot = a_slot + 8 * T;
    const int pr = a.order[seg.start + (slot < seg.count ? slot : 0)];
    a_goff[T] = (size_t)(pr / a.x_div) * K + 8 * a_pc;
  });
  size_t h_goff;
  {
    const int slot = (tid & 63) >> 1;
    const int pr = a.order[seg.start + (slot < seg.count ? slot : 0)];
    h_goff = (size_t)(pr / a.x_div) * nsb * 16 + 8 * (tid & 1);
  }
  uint32_t w_goff[WPT], w_loff[WPT];
  bool w_up[WPT];
  {
    int r = tid / G::PP, pc = tid % G::PP;
    StaticFor<WPT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      bool up;
      const int col = slab_col(r < SLAB ? r : 0, up);
      const bool ok = r < SLAB && col < ncols;  // rows past N and pieces past the slab re-read the slab start
      w_up[T] = up;
      w_goff[T] = ok ? (uint32_t)col * (uint32_t)row_bytes + 16 * pc : 0;
      w_loff[T] = r < SLAB ? (uint32_t)r * G::LBPB + 16 * pc : 0xffffffffu;
      r += MOE_THREADS / G::PP;
      pc += MOE_THREADS % G::PP;
      if (pc >= G::PP) {
        pc -= G::PP;
        r++;
      }
    });
  }
  // side channel for the trailing 2-byte d of a q6_k block: thread -> slab row tid % 128
  const uint8_t* d_src;
  {
    bool up;
    const int col = slab_col(tid & (SLAB - 1), up);
    d_src = (up ? wtile2 : wtile) + (size_t)(col < ncols ? col : 0) * row_bytes + 208;
  }

  u32x4 areg[APT], wreg[WPT], hreg;
  uint16_t dreg = 0;
  auto issue = [&](int sb) {
    StaticFor<APT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      areg[T] = *reinterpret_cast<const u32x4*>(a.xh + a_goff[T] + 256 * sb);
    });
    StaticFor<WPT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      const uint8_t* base = (GLU && w_up[T]) ? wtile2 : wtile;
      wreg[T] = *reinterpret_cast<const typename G::piece_t*>(base + (size_t)sb * G::BPB + w_goff[T]);
    });
    if constexpr (G::SIDE_D) dreg = *reinterpret_cast<const uint16_t*>(d_src + (size_t)sb * G::BPB);
    if constexpr (G::MINS) hreg = *reinterpret_cast<const u32x4*>(a.xhl + h_goff + (size_t)sb * 16);
  };
  auto park = [&](uint8_t* stage) {
    StaticFor<APT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      *reinterpret_cast<u32x4*>(stage + (a_slot + 8 * T) * A_STRIDE + 16 * a_pc) = areg[T];
    });
    StaticFor<WPT>::run([&](auto t) {
      constexpr int T = decltype(t)::value;
      if (w_loff[T] != 0xffffffffu) *reinterpret_cast<u32x4*>(stage + B_OFF + w_loff[T]) = wreg[T];
    });
    if constexpr (G::MINS) {
      if (tid < 64) *reinterpret_cast<u32x4*>(stage + H_OFF + 16 * tid) = hreg;
    }
    if constexpr (G::SIDE_D) {
      if (tid < SLAB) reinterpret_cast<uint16_t*>(stage + D_OFF)[tid] = dreg;
    }
  };

  f32x16 acc[1] = {f32x16{0}};
  auto multiply = [&](const uint8_t* stage) {
    const uint16_t d_side = G::SIDE_D ? reinterpret_cast<const uint16_t*>(stage + D_OFF)[wave * 32 + l32] : (uint16_t)0;
    superblock_mma<C, 1>(stage + B_OFF + (wave * 32 + l32) * G::LBPB, d_side, kg, stage + l32 * A_STRIDE + 32 * kg, 0,
                        stage + H_OFF + l32 * 32 + 16 * kg, 0, acc);
  };

  issue(0);
  if constexpr (MOE_STAGES == 2) {
    // step sb + 1 is parked into the idle stage while step sb is multiplied; one barrier per step
    park(smem);
    if (nsb > 1) issue(1);
    lds_barrier();
    for (int sb = 0; sb < nsb; sb++) {
      if (sb + 1 < nsb) {
        park(smem + ((sb + 1) & 1) * STAGE);
        if (sb + 2 < nsb) issue(sb + 2);
      }
      multiply(smem + (sb & 1) * STAGE);
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

  // ---- epilogue: undo the activation scale, (GLU: combine gate and up,) round once, scatter rows
  if constexpr (GLU) {
    if constexpr (MOE_STAGES == 1) lds_barrier();  // the step buffers are free: reuse them for the up accumulators
    // The gate wave (even) and the up wave (odd) of a column block swap half of their accumulators and finish eight
    // outputs each: the gate wave registers 0 .. 7, the up wave 8 .. 15.
    float* ex = reinterpret_cast<float*>(smem);  // [2 column blocks][16][64]
    const int nb = wave >> 1;
    const bool upw = (wave & 1) != 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int give = upw ? i : 8 + i;  // the register the partner finishes
      ex[(nb * 16 + give) * 64 + lane] = upw ? acc[0][i] : acc[0][8 + i];
    }
    lds_barrier();
    const int col = nb * 32 + l32;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const int i = upw ? 8 + j : j;
      const int slot = 8 * (i >> 2) + 4 * kg + (i & 3);
      const int pr = pair_lds[slot];
      if (pr >= 0 && col < ncols) {
        const float r = rs_lds[slot];
        const float mine = (upw ? acc[0][8 + j] : acc[0][j]) * r, other = ex[(nb * 16 + i) * 64 + lane] * r;
        const float v = kq::glu_epilogue_fast(a.act, upw ? other : mine, upw ? mine : other, a.limit, 1.0f);
        kq::store_result<DT>(a.y, a.om, (size_t)kq::out_row(a.om, pr) * N + n0 + col, v);
      }
    }
  } else {
    const int col = wave * 32 + l32;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int slot = 8 * (i >> 2) + 4 * kg + (i & 3);
      const int pr = pair_lds[slot];
      if (pr >= 0 && col < ncols) {
        const float v = acc[0][i] * rs_lds[slot];
        kq::store_result<DT>(a.y, a.om, (size_t)kq::out_row(a.om, pr) * N + n0 + col, v);
      }
    }
  }
}

struct MoeWorkspace {
  _Float16* xh;
  _Float16* xhl;
  float* rs;
  int* order;
  Segment* segs;
  int* nseg;
  size_t bytes;
};

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

MoeWorkspace carve(void* ws, int rows, int P, int E, int K) {
  MoeWorkspace m;
  uint8_t* p = static_cast<uint8_t*>(ws);
  size_t o = 0;
  m.xh = reinterpret_cast<_Float16*>(p + o);
  o += align256((size_t)rows * K * 2);
  m.xhl = reinterpret_cast<_Float16*>(p + o);
  o += align256((size_t)rows * (K >> 8) * 32);
  m.rs = reinterpret_cast<float*>(p + o);
  o += align256((size_t)rows * 4);
  m.order = reinterpret_cast<int*>(p + o);
  o += align256((size_t)P * 4);
  const size_t maxseg = (size_t)E + P / SEG_M + 1;
  m.segs = reinterpret_cast<Segment*>(p + o);
  o += align256(maxseg * sizeof(Segment));
  m.nseg = reinterpret_cast<int*>(p + o);
  o += 256;
  m.bytes = o;
  return m;
}

template <int C, int DT, bool GLU>
int launch_grouped(const MoeArgs& a, int P, int E, hipStream_t s) {
  using G = Wire<C>;
  constexpr int NCOLS = GLU ? SLAB / 2 : SLAB;
  const int ntiles = (a.N + NCOLS - 1) / NCOLS;
  int maxseg = E + P / SEG_M;  // sum over experts of ceil(c_e / 32) <= E + P / 32
  if (maxseg > P) maxseg = P;
  maxseg = (maxseg + 7) & ~7;  // the kernel's launch-position map needs a multiple of 8
  const size_t lds = (size_t)MOE_STAGES * (SEG_M * A_STRIDE + SLAB * G::LBPB + SEG_M * 32 + SLAB * 2) + SEG_M * 8;
  auto kern = moe_grouped_kernel<C, DT, GLU>;
  hipLaunchKernelGGL(kern, dim3(ntiles, maxseg), dim3(MOE_THREADS), lds, s, a);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

template <bool GLU>
int launch_grouped_any(const MoeArgs& a, int P, int E, int codec, int dtype, hipStream_t s) {
  if (codec == KQ_Q4_K)
    return dtype == KQ_F16 ? launch_grouped<KQ_Q4_K, KQ_F16, GLU>(a, P, E, s)
                           : launch_grouped<KQ_Q4_K, KQ_BF16, GLU>(a, P, E, s);
  if (codec == KQ_Q5_K)
    return dtype == KQ_F16 ? launch_grouped<KQ_Q5_K, KQ_F16, GLU>(a, P, E, s)
                           : launch_grouped<KQ_Q5_K, KQ_BF16, GLU>(a, P, E, s);
  return dtype == KQ_F16 ? launch_grouped<KQ_Q6_K, KQ_F16, GLU>(a, P, E, s)
                         : launch_grouped<KQ_Q6_K, KQ_BF16, GLU>(a, P, E, s);
}

}  // namespace

int kq_launch_moe_sort(const uint32_t* idx, int P, int E, void* order, void* segs, void* nseg, hipStream_t s) {
  if (E > SORT_MAX_E) return KQ_ERR_UNSUPPORTED;
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(SORT_THREADS), 0, s, idx, P, E, static_cast<int*>(order),
                     static_cast<Segment*>(segs), static_cast<int*>(nseg));
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

int kq_launch_gather_rows(const void* x, const uint32_t* lhs, const uint32_t* rhs, void* xg, uint32_t* idx_rows, int B,
                          int M, int K, int64_t x_batch_stride, hipStream_t s) {
  if (B <= 0 || M <= 0) return KQ_OK;
  hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)B * (unsigned)M), dim3(256), 0, s, static_cast<const uint16_t*>(x),
                     lhs, rhs, static_cast<uint16_t*>(xg), idx_rows, M, K, x_batch_stride);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

int kq_launch_expert_tile_map(const uint32_t* idx, int rows, int E, uint32_t* map, int cap, uint32_t* counts,
                              hipStream_t s) {
  hipLaunchKernelGGL(expert_tile_map_kernel, dim3(1), dim3(SORT_THREADS), 0, s, idx, rows, E, map, cap, counts);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

// row_expert[r] = expert of the tile covering row r, `none` for rows no valid tile covers
int kq_launch_tiles_to_rows(const uint32_t* map, const uint32_t* counts, int cap, int rows, int E, uint32_t none,
                            uint32_t* row_expert, hipStream_t s) {
  if (rows <= 0 || cap <= 0) return KQ_OK;
  hipLaunchKernelGGL(fill_u32_kernel, dim3((rows + 255) / 256), dim3(256), 0, s, row_expert, rows, none);
  KQ_HIP_CHECK(hipGetLastError());
  hipLaunchKernelGGL(tiles_to_rows_kernel, dim3((unsigned)cap), dim3(TILE_ROWS), 0, s, map, counts, cap, rows, E,
                     row_expert);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

int kq_launch_mxfp4_repack(const void* packed, const void* scales, void* wire, int64_t nblocks, int to_wire,
                           hipStream_t s) {
  if (nblocks <= 0) return KQ_OK;
  const unsigned blocks = (unsigned)((nblocks + 255) / 256);
  if (to_wire)
    hipLaunchKernelGGL(mxfp4_packed_to_wire_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const uint32_t*>(packed),
                       static_cast<const uint8_t*>(scales), static_cast<uint8_t*>(wire), nblocks);
  else
    hipLaunchKernelGGL(mxfp4_wire_to_packed_kernel, dim3(blocks), dim3(256), 0, s, static_cast<const uint8_t*>(wire),
                       static_cast<uint32_t*>(const_cast<void*>(packed)), static_cast<uint8_t*>(const_cast<void*>(scales)),
                       nblocks);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

int kq_launch_pad_idx(const uint32_t* idx, uint32_t* idx2, int T, int S, hipStream_t s) {
  if (T <= 0 || S <= 0) return KQ_OK;
  hipLaunchKernelGGL(pad_idx_kernel, dim3((T * S + 255) / 256), dim3(256), 0, s, idx, idx2, T, S);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

int kq_launch_mix_slots(const float* yf, const float* scores, const uint32_t* idx, int routed, int E, void* out, int T,
                        int S, int N, int dtype, hipStream_t s) {
  if (T <= 0 || N <= 0) return KQ_OK;
  const unsigned blocks = (unsigned)(((int64_t)T * N + 255) / 256);
  if (dtype == KQ_F16)
    hipLaunchKernelGGL(mix_slots_kernel<KQ_F16>, dim3(blocks), dim3(256), 0, s, yf, scores, idx, routed, E,
                       static_cast<uint16_t*>(out), T, S, N);
  else
    hipLaunchKernelGGL(mix_slots_kernel<KQ_BF16>, dim3(blocks), dim3(256), 0, s, yf, scores, idx, routed, E,
                       static_cast<uint16_t*>(out), T, S, N);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

bool kq_moe_grouped_supported(int P, int E, int N, int K, int codec) {
  return (codec == KQ_Q4_K || codec == KQ_Q5_K || codec == KQ_Q6_K) && P > 16 && E <= SORT_MAX_E && K > 0 &&
         (K & 255) == 0 && N > 0 && (int64_t)E + P / SEG_M < 65535;
}

// rows = activation rows the prepass converts: T for the GLU op (x is [T,K]), T*R for the down op.
size_t kq_moe_grouped_workspace_bytes(int rows, int P, int E, int K) { return carve(nullptr, rows, P, E, K).bytes; }

// x: [rows][K] activations; pair p reads row p / x_div and expert idx[p]; out [P][N].
int kq_launch_moe_grouped(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* idx, void* out, int rows,
                          int P, int E, int N, int K, int x_div, int64_t w_expert_stride, int glu, int act,
                          float limit, int codec, int dtype, void* ws, KqOutMap om, hipStream_t s) {
  if (!kq_moe_grouped_supported(P, E, N, K, codec) || (glu && act == KQ_ACT_SWIGLU_CLAMP)) return KQ_ERR_UNSUPPORTED;
  const uintptr_t wmask = codec == KQ_Q6_K ? 1 : 15;  // q6_k pieces are fetched with unaligned loads
  if ((reinterpret_cast<uintptr_t>(w) & wmask) || (reinterpret_cast<uintptr_t>(w2) & wmask) ||
      ((uintptr_t)w_expert_stride & wmask) || (reinterpret_cast<uintptr_t>(x) & 15) ||
      (reinterpret_cast<uintptr_t>(ws) & 255))
    return KQ_ERR_UNSUPPORTED;
  const MoeWorkspace m = carve(ws, rows, P, E, K);
  if (dtype == KQ_F16)
    hipLaunchKernelGGL(moe_prologue_kernel<KQ_F16>, dim3(rows + 1), dim3(PP_THREADS), 0, s, static_cast<const uint16_t*>(x),
                       m.xh, m.xhl, m.rs, rows, K, idx, P, E, m.order, m.segs, m.nseg);
  else
    hipLaunchKernelGGL(moe_prologue_kernel<KQ_BF16>, dim3(rows + 1), dim3(PP_THREADS), 0, s, static_cast<const uint16_t*>(x),
                       m.xh, m.xhl, m.rs, rows, K, idx, P, E, m.order, m.segs, m.nseg);
  KQ_HIP_CHECK(hipGetLastError());
  MoeArgs a{};
  a.xh = m.xh;
  a.xhl = m.xhl;
  a.rs = m.rs;
  a.w = w;
  a.w2 = w2;
  a.y = out;
  a.order = m.order;
  a.segs = m.segs;
  a.nseg = m.nseg;
  a.N = N;
  a.K = K;
  a.x_div = x_div < 1 ? 1 : x_div;
  a.act = act;
  a.w_expert_stride = w_expert_stride;
  a.limit = limit;
  a.om = om;
  return glu ? launch_grouped_any<true>(a, P, E, codec, dtype, s) : launch_grouped_any<false>(a, P, E, codec, dtype, s);
}
