// Batched MoE on mxfp4 stacks with gfx950's block-scaled matrix instruction.
//
// v_mfma_scale_f32_16x16x128_f8f6f4 multiplies a 16 x 128 tile by a 128 x 16 tile whose elements are 4-, 6- or 8-bit
// floats and applies one e8m0 (power-of-two) scale per operand row and 32 elements: exactly the mxfp4 wire block, a
// scale byte and 32 e2m1 codes.  The weights therefore go from memory into the B operand as they are stored, no
// decode at all: lane (n, kb) of a 16-column tile loads block 4 s + kb of weight row n, its 16 code bytes as the
// operand and its scale byte as the scale.  (The reference's weight is 2^(e - 128) * (2 * e2m1), the instruction's
// 2^(e - 127) * e2m1: the same number; scale byte 255, which the instruction reads as NaN, is not a valid e8m0 scale.)
//
// Activations: a bf16 value has 8 significant bits, an e4m3 value 4, so x = hi + lo with two e4m3 terms that share
// a power-of-two scale per 32 values, those of a wire block (f16 inputs: three terms), written once per activation row by a prepass, and an
// MFMA per term.  Products are exact and summed in f32 by the matrix core.  A value more than 2^13 below the largest
// of its 32-group loses bits (an absolute error below 2^-16 of that largest value).
//
// Operand layout of the instruction (measured): B lane (n, kb) holds k = 32 kb .. 32 kb + 31 of column n, code i in
// nibble i; A lane (m, a) holds k = 16 a .. 16 a + 15 in bytes 0 .. 15 and k = 64 + 16 a .. + 15 in bytes 16 .. 31 of
// row m; the scale register (byte picked by op_sel) of lane (row, kb) applies to k = 32 kb .. 32 kb + 31 of that row,
// for A as for B (for A that is not the lane holding those values); D lane l holds column l % 16, rows 4 (l / 16) .. + 3.  A wire block keeps weight j in the low and weight j + 16 in the high nibble
// of byte j, so code i of a block is weight i / 2 (+ 16 for odd i): the prepass stores the activations in that order.
//
// Kernels: pairs sorted by expert into segments (the sort of kq_moe_sort.h); a workgroup of four waves takes one
// m-tile (16 pairs) of a segment and 64 output columns (fused gate / up: 64 weight rows of each matrix).  The weights
// go straight from global memory into registers (aligned dwords around each 17-byte block, the codes realigned with
// byte shifts): no LDS staging of weights.  fp4_grouped_kernel: the waves split K (steps of 128 dealt round-robin),
// every wave streams all column tiles of its steps one step ahead, the four partial sums meet in LDS (the plain op;
// two m-tiles on the same weight registers).  fp4_glu_tiles_kernel: the waves split the column tiles, a wave reads
// four consecutive steps of its gate and up tile per load group, one group ahead, and the activation terms of a step
// are loaded by one wave and shared through LDS (the fused op on one m-tile).
#include <atomic>
#include <type_traits>

#include "kq_common.h"
#include "kq_decode.h"
#include "kq_epilogue.h"
#include "kq_moe_sort.h"

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));

using kqsort::Segment;

// A pointer into device memory as such: the loads through it are global loads, not flat ones (a flat load also
// counts in the LDS counter, so a wait for an LDS result would wait for the prefetched step as well).
template <class T>
__device__ __forceinline__ const __attribute__((address_space(1))) T* in_global(const T* p) {
  return (const __attribute__((address_space(1))) T*)(uintptr_t)p;
}

constexpr int F4_THREADS = 256;  // four waves

template <int DT>
constexpr int f4_terms() { return DT == KQ_BF16 ? 2 : 3; }

struct F4Args {
  const uint8_t* xa;   // [rows][nsteps][NT][4][32] e4m3 terms in operand order
  const uint32_t* xs;  // [rows][nsteps][4]: byte t = e8m0 scale of term t
  const uint8_t* w;
  const uint8_t* w2;   // up stack (fused gate / up) or null
  const uint8_t* w_end;   // one past the last byte of the stacks: no load may reach beyond
  const uint8_t* w2_end;
  void* y;
  const float* bias;   // f32 [E][N] or null
  const float* bias2;
  const int* order;
  const Segment* segs;
  const int* nseg;
  int N, K, nsteps, x_div, act;
  int64_t w_expert_stride;
  float limit, alpha;
  KqOutMap om;
};

}  // namespace
namespace kq {
template <int N>
struct SForF4 {
  template <class F>
  __device__ __forceinline__ static void run(F&& f) {
    SForF4<N - 1>::run(f);
    f(std::integral_constant<int, N - 1>{});
  }
};
template <>
struct SForF4<0> {
  template <class F>
  __device__ __forceinline__ static void run(F&&) {}
};
}  // namespace kq
namespace {

__device__ __forceinline__ int in_vgpr(int v) {
  asm volatile("" : "+v"(v));
  return v;
}

// ------------------------------------------------------------------ activation prepass
// One workgroup per activation row (fp4_prologue_kernel); a thread writes the 32 operand bytes of one (step, lane block a): positions
// 8 (a & 1) .. + 7 and 16 + 8 (a & 1) .. + 7 of wire blocks a / 2 and 2 + a / 2 of the step, interleaved.  The scale
// belongs to the wire block (32 consecutive activations), so the thread looks at both whole blocks.
constexpr int F4_PRO_THREADS = 256;
template <int DT>
__device__ __forceinline__ void fp4_prepass_row(const uint16_t* __restrict__ x, uint8_t* __restrict__ xa,
                                                uint32_t* __restrict__ xs, int K, int nsteps, int row) {
  constexpr int NT = f4_terms<DT>();
  const uint16_t* xr = x + (size_t)row * K;
  for (int g = threadIdx.x; g < nsteps * 4; g += F4_PRO_THREADS) {
    const int s = g >> 2, a = g & 3;
    uint8_t* out = xa + ((size_t)(row * nsteps + s) * NT) * 128 + a * 32;
    u32x4 p[NT][2];
#pragma unroll
    for (int half = 0; half < 2; half++) {
      const int bw = 2 * half + (a >> 1), base = 128 * s + 32 * bw;
      u32x4 c[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
      if (base < K) {  // K is a multiple of 32: a wire block is inside or outside as a whole
#pragma unroll
        for (int i = 0; i < 4; i++) c[i] = *reinterpret_cast<const u32x4*>(xr + base + 8 * i);
      }
      auto val = [&](const u32x4& cc, int u) -> float {
        const uint32_t h = (cc[u >> 1] >> (16 * (u & 1))) & 0xffff;
        return DT == KQ_F16 ? kq::h2f((uint16_t)h) : __builtin_bit_cast(float, h << 16);
      };
      float amax = 0.f;
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int u = 0; u < 8; u++) amax = fmaxf(amax, fabsf(val(c[i], u)));
      // the block's largest magnitude lands in [128, 256): below e4m3's 448
      int eb = (int)((__builtin_bit_cast(uint32_t, amax) >> 23) & 0xff);
      if (eb == 0xff) eb = 0xfe;  // inf / nan inputs stay inf / nan through the products
      int sb = eb - 7;            // e8m0 byte of the first term: 2^(eb - 127 - 7)
      sb = sb < 1 ? 1 : sb;
      const float mul = __builtin_bit_cast(float, (uint32_t)(254 - sb) << 23);  // 2^(127 - sb), exact
      // this lane block's sixteen values of the block: 8 (a & 1) + u and 16 + 8 (a & 1) + u, interleaved
      float v[16];
      const u32x4 c0 = (a & 1) ? c[1] : c[0], c1 = (a & 1) ? c[3] : c[2];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        v[2 * u] = val(c0, u) * mul;
        v[2 * u + 1] = val(c1, u) * mul;
      }
      uint32_t sword = 0;
#pragma unroll
      for (int t = 0; t < NT; t++) {
        int tb = sb - 4 * t;  // every further term sits four bits lower
        const bool live = tb >= 1;
        tb = live ? tb : 1;
        sword |= (uint32_t)tb << (8 * t);
#pragma unroll
        for (int q = 0; q < 16; q += 4) {
          int pk = 0;
          pk = __builtin_amdgcn_cvt_pk_fp8_f32(v[q], v[q + 1], pk, false);
          pk = __builtin_amdgcn_cvt_pk_fp8_f32(v[q + 2], v[q + 3], pk, true);
          if (!live) pk = 0;
          // what is left, in units of the next term (exact: the remainder of a 4-bit rounding, times 16)
          v[q] = (v[q] - __builtin_amdgcn_cvt_f32_fp8(pk, 0)) * 16.0f;
          v[q + 1] = (v[q + 1] - __builtin_amdgcn_cvt_f32_fp8(pk, 1)) * 16.0f;
          v[q + 2] = (v[q + 2] - __builtin_amdgcn_cvt_f32_fp8(pk, 2)) * 16.0f;
          v[q + 3] = (v[q + 3] - __builtin_amdgcn_cvt_f32_fp8(pk, 3)) * 16.0f;
          p[t][half][q >> 2] = (uint32_t)pk;
        }
      }
      if ((a & 1) == 0) xs[(size_t)(row * nsteps + s) * 4 + bw] = sword;
    }
#pragma unroll
    for (int t = 0; t < NT; t++) {
      *reinterpret_cast<u32x4*>(out + t * 128) = p[t][0];
      *reinterpret_cast<u32x4*>(out + t * 128 + 16) = p[t][1];
    }
  }
}

// The pair sort and the activation prepass in ONE launch: workgroup 0 sorts the pairs by expert, workgroups 1 .. rows
// convert one activation row each (neither depends on the other).
template <int DT>
__global__ __launch_bounds__(F4_PRO_THREADS) void fp4_prologue_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ xa,
                                                                      uint32_t* __restrict__ xs, int K, int nsteps,
                                                                      const uint32_t* __restrict__ idx, int P, int E,
                                                                      int* __restrict__ order, Segment* __restrict__ segs,
                                                                      int* __restrict__ nseg_out) {
  __shared__ int cnt[kqsort::SORT_MAX_E];
  __shared__ int scan_p[F4_PRO_THREADS], scan_s[F4_PRO_THREADS];
  if (blockIdx.x == 0)  // the longest workgroup of the launch (a chain of barriers) goes first
    kqsort::moe_sort_body<F4_PRO_THREADS>(idx, P, E, order, segs, nseg_out, cnt, scan_p, scan_s);
  else
    fp4_prepass_row<DT>(x, xa, xs, K, nsteps, blockIdx.x - 1);
}

// ------------------------------------------------------------------ grouped kernel
// J = column tiles (of 16) a wave streams per step (8 or 4); MT = m-tiles (of 16 pairs) a workgroup multiplies with
// the same weight registers: 1 (grid z walks the m-tiles of a segment, the weights of a longer segment are read
// twice) or 2 (segments of up to 32 pairs in one pass, J = 4).
template <int DT, bool GLU, int J, int MT>
__global__ __launch_bounds__(F4_THREADS, 2) void fp4_grouped_kernel(F4Args a) {
  constexpr int NT = f4_terms<DT>();
  constexpr int JH = J / 2;                    // fused: gate tiles 0 .. JH - 1, up tiles JH .. J - 1
  constexpr int COLS = GLU ? 8 * J : 16 * J;  // output columns of a workgroup
  __shared__ v4f red[4][MT * J][64];
  const int nseg = *a.nseg;
  if ((int)blockIdx.y >= nseg) return;
  const Segment sg = a.segs[blockIdx.y];
  const int mt = MT == 1 ? blockIdx.z : 0;  // first m-tile (16 pairs) of this workgroup
  if (16 * mt >= sg.count) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, kb = lane >> 4;  // this lane's place in the operands: row / column r, block kb of the step
  // Its place in the loads.  With one m-tile the loads go in row order: four neighbouring lanes take the four blocks
  // of one row (68 contiguous bytes of weights, 64 of an activation term), so sixteen lanes touch 4 rows instead of
  // 16, and the loaded registers change lanes once (operand lane 16 p + 4 x + y reads what lane 16 x + 4 y + p
  // loaded).  With two m-tiles on the same weight registers the exchanged copies do not fit the register file and
  // the loads stay in operand order.
  constexpr bool COAL = MT == 1;
  const int rl = COAL ? lane >> 2 : r, kbl = COAL ? lane & 3 : kb;
  const int from_lane = 4 * (16 * ((lane >> 2) & 3) + 4 * (lane & 3) + (lane >> 4));
  const int N = a.N, nsteps = a.nsteps, nblk = a.K >> 5;
  const uint32_t row_bytes = (uint32_t)nblk * 17u;
  const int n0 = blockIdx.x * COLS;
  const int rows_here = sg.count - 16 * mt < 16 * MT ? sg.count - 16 * mt : 16 * MT;

  // Weight rows of this lane: tile j covers columns n0 + 16 j .. (fused: tiles JH .. are the same columns of the up
  // matrix); columns past N re-read the last one.  A row is addressed as a matrix pointer held in scalar registers
  // plus a 32-bit byte offset per lane (the pointer is taken four bytes low and the offset four bytes high: a
  // block's window starts up to three bytes before it).
  const int expert = __builtin_amdgcn_readfirstlane(sg.expert);
  const uint8_t* wmat[2];
  wmat[0] = a.w + (int64_t)expert * a.w_expert_stride - 4;
  wmat[1] = GLU ? a.w2 + (int64_t)expert * a.w_expert_stride - 4 : wmat[0];
  uint32_t woff[J];
  uint32_t row_meta = 0;  // bits 2 j, 2 j + 1: low address bits of row j; bit 16 + j: the row is the last of its stack
#pragma unroll
  for (int j = 0; j < J; j++) {
    int c = n0 + 16 * (GLU ? (j % JH) : j) + rl;
    c = c < N ? c : N - 1;
    woff[j] = (uint32_t)c * row_bytes + 4u;
    const uint8_t* base = wmat[(GLU && j >= JH) ? 1 : 0];
    row_meta |= (((uint32_t)reinterpret_cast<uintptr_t>(base) + woff[j]) & 3u) << (2 * j);
    row_meta |= (base + woff[j] + row_bytes == ((GLU && j >= JH) ? a.w2_end : a.w_end) ? 1u : 0u) << (16 + j);
  }
  // activation rows of this lane (rows past the segment re-read its last pair; their results are dropped)
  const uint8_t* arow[MT];
  const uint32_t* srow[MT];
#pragma unroll
  for (int m = 0; m < MT; m++) {
    const int mrow = 16 * m + rl < rows_here ? 16 * m + rl : rows_here - 1;
    const int xrow = in_global(a.order)[sg.start + 16 * mt + mrow] / a.x_div;
    arow[m] = a.xa + ((size_t)xrow * nsteps * NT) * 128 + kbl * 32;
    srow[m] = a.xs + (size_t)xrow * nsteps * 4 + kbl;
  }

  // A stage holds what the loads of a step return, untouched: anything computed from a loaded register at load
  // time would make the wave wait for the data there.
  struct Stage {
    u32x4 d[J];      // the four aligned dwords at and after a block's first byte
    uint32_t d4[J];  // the fifth
    v8i av[MT][NT];
    int sa[MT];
  };
  // The 17 bytes of a block (scale, 16 code bytes) sit at any byte offset: five aligned dwords around them, the codes
  // brought to dword boundaries by one byte permute per dword when the stage is used.  For the last block of a stack
  // the fifth dword would reach past the end: it is fetched 3 - sh bytes earlier and shifted back (the bytes past
  // the end are not part of the block); that arithmetic runs only in the work item that holds the stack's last row.
  auto window = [&](auto tail_c, int j, int s, uint32_t& sh, uint32_t& back, bool& live) {
    int blk = 4 * s + kbl;
    live = blk < nblk;  // past K: any block of the row with a neutral scale (the activations are zeros)
    blk = live ? blk : nblk - 1;
    const uint32_t off = (uint32_t)blk * 17u;
    sh = (((row_meta >> (2 * j)) & 3u) + off) & 3u;
    back = (decltype(tail_c)::value && ((row_meta >> (16 + j)) & 1u) && blk == nblk - 1) ? 3u - sh : 0u;
    return reinterpret_cast<uintptr_t>(wmat[(GLU && j >= JH) ? 1 : 0] + (woff[j] + off - sh));
  };
  auto fetch = [&](auto tail_c, Stage& st, int s) {
#pragma unroll
    for (int j = 0; j < J; j++) {
      uint32_t sh, back;
      bool live;
      const uintptr_t q = window(tail_c, j, s, sh, back, live);
      st.d[j] = *(const __attribute__((address_space(1))) u32x4_a4*)q;  // dword-aligned, no more
      typedef uint32_t u32_a1 __attribute__((aligned(1)));
      st.d4[j] = *(const __attribute__((address_space(1))) u32_a1*)(q + 16 - back);
    }
#pragma unroll
    for (int m = 0; m < MT; m++) {
#pragma unroll
      for (int t = 0; t < NT; t++) {
        const u32x4 lo = *in_global(reinterpret_cast<const u32x4*>(arow[m] + ((size_t)s * NT + t) * 128));
        const u32x4 hi = *in_global(reinterpret_cast<const u32x4*>(arow[m] + ((size_t)s * NT + t) * 128 + 16));
        st.av[m][t] = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
      }
      st.sa[m] = (int)in_global(srow[m])[(size_t)s * 4];
    }
  };
  v4f acc[MT][J];
#pragma unroll
  for (int m = 0; m < MT; m++)
#pragma unroll
    for (int j = 0; j < J; j++) acc[m][j] = v4f{0, 0, 0, 0};
  auto to_operand_lane = [&](int v) { return COAL ? __builtin_amdgcn_ds_bpermute(from_lane, v) : v; };
  auto multiply = [&](auto tail_c, const Stage& st, int s) {
    v8i av[MT][NT];
    int sav[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) {
#pragma unroll
      for (int t = 0; t < NT; t++)
#pragma unroll
        for (int i = 0; i < 8; i++) av[m][t][i] = to_operand_lane(st.av[m][t][i]);
      sav[m] = to_operand_lane(st.sa[m]);
    }
#pragma unroll
    for (int j = 0; j < J; j++) {
      uint32_t sh, back;
      bool live;
      window(tail_c, j, s, sh, back, live);
      const u32x4 d = st.d[j];
      const int sc = live ? (int)((d[0] >> (8 * sh)) & 0xff) : 127;
      // codes start at byte sh + 1 of the window: bytes sh + 1 .. sh + 4 of each pair of neighbouring dwords
      const uint32_t sel = 0x03020100u + 0x01010101u * (sh + 1u);
      const uint32_t dd[5] = {d[0], d[1], d[2], d[3], st.d4[j] >> (8 * back)};
      v8i bv = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < 4; i++) bv[i] = to_operand_lane((int)__builtin_amdgcn_perm(dd[i + 1], dd[i], sel));
      const int sb = in_vgpr(to_operand_lane(sc));
#pragma unroll
      for (int m = 0; m < MT; m++) {
        const int sa = in_vgpr(sav[m]);
        acc[m][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av[m][0], bv, acc[m][j], 0, 4, 0, sa, 0, sb);
        acc[m][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av[m][1], bv, acc[m][j], 0, 4, 1, sa, 0, sb);
        if constexpr (NT == 3)
          acc[m][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av[m][2], bv, acc[m][j], 0, 4, 2, sa, 0, sb);
      }
    }
  };

  // This wave's steps: wave, wave + 4, ...: two register stages, the loads of a step issued before the step before
  // it is multiplied.  The loop body holds no branch, so the wait before a multiply is for exactly the loads it
  // needs; the work item that holds the last row of a stack (a uniform condition) runs the form with the stack-end
  // arithmetic, every other item the form without.
  const int nq = wave < nsteps ? (nsteps - wave + 3) >> 2 : 0;  // steps of this wave
  auto stream = [&](auto tail_c) {
    if (nq == 0) return;
    Stage s0, s1;
    fetch(tail_c, s0, wave);
    int q = 0;
    while (q + 2 < nq) {
      fetch(tail_c, s1, wave + 4 * (q + 1));
      multiply(tail_c, s0, wave + 4 * q);
      fetch(tail_c, s0, wave + 4 * (q + 2));
      multiply(tail_c, s1, wave + 4 * (q + 1));
      q += 2;
    }
    if (q + 1 < nq) {
      fetch(tail_c, s1, wave + 4 * (q + 1));
      multiply(tail_c, s0, wave + 4 * q);
      multiply(tail_c, s1, wave + 4 * (q + 1));
    } else {
      multiply(tail_c, s0, wave + 4 * q);
    }
  };
  if (wmat[0] + 4 + (size_t)N * row_bytes == a.w_end && n0 + COLS >= N)
    stream(std::true_type{});
  else
    stream(std::false_type{});

  // ---- the four partial sums meet in LDS; wave w finishes J / 4 tiles (fused: gate tile w with up tile w)
#pragma unroll
  for (int m = 0; m < MT; m++)
#pragma unroll
    for (int j = 0; j < J; j++) red[wave][m * J + j][lane] = acc[m][j];
  __syncthreads();
  auto total = [&](int j) {
    v4f v = red[0][j][lane];
#pragma unroll
    for (int wv = 1; wv < 4; wv++) {
      const v4f o = red[wv][j][lane];
      v[0] += o[0];
      v[1] += o[1];
      v[2] += o[2];
      v[3] += o[3];
    }
    return v;
  };
  auto finish = [&](int m16, int col, const v4f& g, const v4f& u) {
    if (col >= N) return;
    const float gb = a.bias ? in_global(a.bias)[(size_t)expert * N + col] : 0.f;
    const float ub = (GLU && a.bias2) ? in_global(a.bias2)[(size_t)expert * N + col] : 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int m = 16 * m16 + 4 * kb + i;
      if (m < rows_here) {
        const int p = in_global(a.order)[sg.start + 16 * mt + m];
        float v = g[i] + gb;
        if constexpr (GLU) v = kq::glu_epilogue_fast(a.act, v, u[i] + ub, a.limit, a.alpha);
        kq::store_result<DT>(a.y, a.om, (size_t)kq::out_row(a.om, p) * N + col, v);
      }
    }
  };
#pragma unroll
  for (int m = 0; m < MT; m++) {
    if constexpr (GLU) {
      if (wave < JH) finish(m, n0 + 16 * wave + r, total(m * J + wave), total(m * J + wave + JH));
    } else {
      const v4f none = {0, 0, 0, 0};
#pragma unroll
      for (int t = 0; t < J / 4; t++) finish(m, n0 + 16 * (J / 4 * wave + t) + r, total(m * J + J / 4 * wave + t), none);
    }
  }
}

// ------------------------------------------------------------------ fused gate / up op, one m-tile, waves split the tiles
// One m-tile (16 pairs) of a segment and 64 output columns per workgroup, as in the kernel above with MT = 1, but the
// four waves split the column tiles instead of the K steps: wave v owns columns n0 + 16 v .. + 15 (that tile of the
// gate and of the up matrix) over all of K, so no partial sums meet at the end.  A wave's loads cover four
// consecutive steps of its rows at a time (272 contiguous bytes per row), the loads of the next four are issued
// before the present four are multiplied (two register stages; the loop body holds no branch, so the wait before
// a multiply is exact), and the loaded registers are used untouched until then (anything computed from them at
// load time would make the wave wait there).  The activation terms of a step are loaded once per workgroup -- wave v
// takes step 4 q + v of a group of four -- and shared through LDS in operand order, so they need no lane exchange
// and cost a fifth of the load instructions they cost when every wave fetches the terms of its own step.
// NW = waves per workgroup: four (64 columns), or two (32 columns, every wave loading the terms of two steps of a
// group) for calls of so few pairs that 64-column groups would leave CUs without a workgroup.
// (GLU = false, the plain op with one tile per wave, measured slower in this form than with the K steps split: 37.3
// us against 36.6 on 32 experts of 2880 x 2880 at 256 pairs; it stays on the kernel above and is not instantiated.)
template <int DT, bool GLU = true, int NW = 4>
__global__ __launch_bounds__(64 * NW, 2) void fp4_glu_tiles_kernel(F4Args a) {
  constexpr int NT = f4_terms<DT>();
  constexpr int TPW = GLU ? 2 : 1;  // tiles per wave: gate and up
  constexpr int SPG = 4;  // steps per group: a stage is eight blocks per lane
  constexpr int SPW = 4 / NW;  // steps of activation terms a wave loads per group
  constexpr int COLS = 16 * NW;  // output columns of a workgroup
  constexpr int A_STEP = NT * 2048 + 256;  // LDS bytes of a step's terms: [term][half][a][m][16] + scales [kb][m]
  __shared__ __attribute__((aligned(16))) uint8_t abuf[2][SPG][A_STEP];
  const int nseg = *in_global(a.nseg);
  if ((int)blockIdx.y >= nseg) return;
  const Segment sg = a.segs[blockIdx.y];
  const int mt = blockIdx.z;
  if (16 * mt >= sg.count) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, kb = lane >> 4;   // place in the operands
  const int rl = lane >> 2, kbl = lane & 3;  // place in the loads: four neighbouring lanes take the four blocks of a row
  const int from_lane = 4 * (16 * ((lane >> 2) & 3) + 4 * (lane & 3) + (lane >> 4));
  const int N = a.N, nsteps = a.nsteps, nblk = a.K >> 5;
  const uint32_t row_bytes = (uint32_t)nblk * 17u;
  const int n0 = blockIdx.x * COLS;
  const int rows_here = sg.count - 16 * mt < 16 ? sg.count - 16 * mt : 16;
  const int ngroups = (nsteps + SPG - 1) / SPG;

  // A row is addressed as a matrix pointer held in scalar registers plus a 32-bit byte offset per lane (the pointer
  // is taken four bytes low and the offset four bytes high: a block's window starts up to three bytes before it).
  const int expert = __builtin_amdgcn_readfirstlane(sg.expert);
  const uint8_t* wmat[TPW];
  uint32_t woff, wlow[TPW];  // the lane's row offset in both matrices; low address bits of its rows
  bool last_row[TPW];        // the row is the last of its stack
  {
    int c = n0 + 16 * wave + rl;
    c = c < N ? c : N - 1;  // columns past N re-read the last one (not stored)
    woff = (uint32_t)c * row_bytes + 4u;
  }
#pragma unroll
  for (int t = 0; t < TPW; t++) {
    wmat[t] = (t ? a.w2 : a.w) + (int64_t)expert * a.w_expert_stride - 4;
    wlow[t] = ((uint32_t)reinterpret_cast<uintptr_t>(wmat[t]) + woff) & 3u;
    last_row[t] = wmat[t] + woff + row_bytes == (t ? a.w2_end : a.w_end);
  }
  const int mrow = rl < rows_here ? rl : rows_here - 1;  // rows past the segment re-read its last pair (dropped)
  const int xrow = in_global(a.order)[sg.start + 16 * mt + mrow] / a.x_div;
  const uint8_t* arow = a.xa + ((size_t)xrow * nsteps * NT) * 128 + kbl * 32;
  const uint32_t* srow = a.xs + (size_t)xrow * nsteps * 4 + kbl;

  struct Stage {
    u32x4 d[TPW][SPG];      // the four aligned dwords at and after a block's first byte
    uint32_t d4[TPW][SPG];  // the fifth
    u32x4 lo[SPW][NT], hi[SPW][NT];
    uint32_t sa[SPW];
  };
  // the window of block (tile t, step s) of this lane: address of its first dword, the byte shift, and how many
  // bytes earlier the fifth dword is fetched (the last block of a stack: the dword would reach past the end)
  auto window = [&](auto tail_c, int t, int s, uint32_t& sh, uint32_t& back, bool& live) {
    int blk = 4 * s + kbl;
    live = blk < nblk;  // past K: any block of the row with a neutral scale (the activations are zeros)
    blk = live ? blk : nblk - 1;
    const uint32_t off = (uint32_t)blk * 17u;
    sh = (wlow[t] + off) & 3u;
    back = (decltype(tail_c)::value && last_row[t] && blk == nblk - 1) ? 3u - sh : 0u;
    return reinterpret_cast<uintptr_t>(wmat[t] + (woff + off - sh));
  };
  auto issue = [&](auto tail_c, Stage& st, int q) {  // group q: steps SPG q .. + SPG - 1 (past the last: the last once more, unused)
#pragma unroll
    for (int t = 0; t < TPW; t++)
#pragma unroll
      for (int g = 0; g < SPG; g++) {
        int s = SPG * q + g;
        s = s < nsteps ? s : nsteps - 1;
        uint32_t sh, back;
        bool live;
        const uintptr_t qa = window(tail_c, t, s, sh, back, live);
        st.d[t][g] = *(const __attribute__((address_space(1))) u32x4_a4*)qa;  // dword-aligned, no more
        typedef uint32_t u32_a1 __attribute__((aligned(1)));
        st.d4[t][g] = *(const __attribute__((address_space(1))) u32_a1*)(qa + 16 - back);
      }
#pragma unroll
    for (int i = 0; i < SPW; i++) {
      int s = SPG * q + NW * i + wave;
      s = s < nsteps ? s : nsteps - 1;
#pragma unroll
      for (int t = 0; t < NT; t++) {
        st.lo[i][t] = *in_global(reinterpret_cast<const u32x4*>(arow + ((size_t)s * NT + t) * 128));
        st.hi[i][t] = *in_global(reinterpret_cast<const u32x4*>(arow + ((size_t)s * NT + t) * 128 + 16));
      }
      st.sa[i] = in_global(srow)[(size_t)s * 4];
    }
  };
  v4f acc[TPW];
#pragma unroll
  for (int t = 0; t < TPW; t++) acc[t] = v4f{0, 0, 0, 0};
  auto consume = [&](auto tail_c, const Stage& st, int q) {
    // this wave's steps of activation terms into LDS: lane (row rl, block kbl) writes where operand lane
    // (m = rl, a = kbl) will read
#pragma unroll
    for (int i = 0; i < SPW; i++) {
      uint8_t* ab = abuf[q & 1][NW * i + wave];
#pragma unroll
      for (int t = 0; t < NT; t++) {
        *reinterpret_cast<u32x4*>(ab + (((t * 2 + 0) * 4 + kbl) * 16 + rl) * 16) = st.lo[i][t];
        *reinterpret_cast<u32x4*>(ab + (((t * 2 + 1) * 4 + kbl) * 16 + rl) * 16) = st.hi[i][t];
      }
      *reinterpret_cast<uint32_t*>(ab + NT * 2048 + (kbl * 16 + rl) * 4) = st.sa[i];
    }
    __syncthreads();  // two buffers in turn: a buffer is written again two groups later, past the next barrier
#pragma unroll
    for (int g = 0; g < SPG; g++) {
      const int s = SPG * q + g;
      if (s < nsteps) {  // uniform
        const uint8_t* ab = abuf[q & 1][g];
        v8i av[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) {
          const u32x4 l = *reinterpret_cast<const u32x4*>(ab + (((t * 2 + 0) * 4 + kb) * 16 + r) * 16);
          const u32x4 h = *reinterpret_cast<const u32x4*>(ab + (((t * 2 + 1) * 4 + kb) * 16 + r) * 16);
          av[t] = v8i{(int)l[0], (int)l[1], (int)l[2], (int)l[3], (int)h[0], (int)h[1], (int)h[2], (int)h[3]};
        }
        const int sa = in_vgpr(*reinterpret_cast<const int*>(ab + NT * 2048 + (kb * 16 + r) * 4));
#pragma unroll
        for (int t = 0; t < TPW; t++) {
          uint32_t sh, back;
          bool live;
          window(tail_c, t, s, sh, back, live);
          const u32x4 d = st.d[t][g];
          const int sc = live ? (int)((d[0] >> (8 * sh)) & 0xff) : 127;
          // codes start at byte sh + 1 of the window: bytes sh + 1 .. sh + 4 of each pair of neighbouring dwords
          const uint32_t sel = 0x03020100u + 0x01010101u * (sh + 1u);
          const uint32_t dd[5] = {d[0], d[1], d[2], d[3], st.d4[t][g] >> (8 * back)};
          v8i bv = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
          for (int i = 0; i < 4; i++)
            bv[i] = __builtin_amdgcn_ds_bpermute(from_lane, (int)__builtin_amdgcn_perm(dd[i + 1], dd[i], sel));
          const int sb = in_vgpr(__builtin_amdgcn_ds_bpermute(from_lane, sc));
          acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av[0], bv, acc[t], 0, 4, 0, sa, 0, sb);
          acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av[1], bv, acc[t], 0, 4, 1, sa, 0, sb);
          if constexpr (NT == 3)
            acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av[2], bv, acc[t], 0, 4, 2, sa, 0, sb);
        }
      }
    }
  };

  // The work item that holds the last row of a stack (a uniform condition) runs the form that can fetch a fifth
  // dword early; every other item the form without that arithmetic.
  auto stream = [&](auto tail_c) {
    Stage s0, s1;
    issue(tail_c, s0, 0);
    int q = 0;
    while (q + 2 < ngroups) {  // no branch inside: every wait is for exactly the loads it needs
      issue(tail_c, s1, q + 1);
      consume(tail_c, s0, q);
      issue(tail_c, s0, q + 2);
      consume(tail_c, s1, q + 1);
      q += 2;
    }
    if (q + 1 < ngroups) {
      issue(tail_c, s1, q + 1);
      consume(tail_c, s0, q);
      consume(tail_c, s1, q + 1);
    } else {
      consume(tail_c, s0, q);
    }
  };
  const uint8_t* after_tiles = wmat[0] + 4 + (size_t)N * row_bytes;
  if (after_tiles == a.w_end && n0 + COLS >= N)
    stream(std::true_type{});
  else
    stream(std::false_type{});

  // ---- epilogue: this wave's columns
  const int col = n0 + 16 * wave + r;
  if (col < N) {
    const float gb = a.bias ? in_global(a.bias)[(size_t)expert * N + col] : 0.f;
    const float ub = (GLU && a.bias2) ? in_global(a.bias2)[(size_t)expert * N + col] : 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int m = 4 * kb + i;
      if (m < rows_here) {
        const int p = in_global(a.order)[sg.start + 16 * mt + m];
        float v = acc[0][i] + gb;
        if constexpr (GLU) v = kq::glu_epilogue_fast(a.act, v, acc[TPW - 1][i] + ub, a.limit, a.alpha);
        kq::store_result<DT>(a.y, a.om, (size_t)kq::out_row(a.om, p) * N + col, v);
      }
    }
  }
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
int f4_num_cus() {
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
int f4_steps(int K) { return ((K >> 5) + 3) / 4; }

}  // namespace

// mxfp4 stacks: K a multiple of 32 (the block), N a multiple of 8 (the op's own rule)
bool kq_fp4_moe_supported(int P, int E, int N, int K, int codec) {
  // Up to 16 pairs the per-entry kernels are the alternative: the streamed one where K is a multiple of 256 (faster
  // there), the code-level one elsewhere, which this kernel passes at 8 pairs (32 experts of 2880 x 2880, fused +
  // plain op: 4 pairs 16.6 + 11.8 us entry by entry against 18.0 + 13.3 here, 8 pairs 27.1 + 17.5 against 24.8 + 16.6,
  // 16 pairs 49.0 + 29.8 against 34.6 + 20.3).
#ifndef KQ_FP4_MIN_PAIRS_TAIL
#define KQ_FP4_MIN_PAIRS_TAIL 8
#endif
  const int min_pairs = (K & 255) ? KQ_FP4_MIN_PAIRS_TAIL : 17;
  return codec == KQ_MXFP4 && P >= min_pairs && E > 0 && E <= 4096 && (int64_t)E + P / 32 < 65535 && N > 0 && K >= 32 &&
         (K & 31) == 0 && (int64_t)N * (K >> 5) * 17 < ((int64_t)1 << 32) - 64;
}

// Workspace: sorted pair list, segment table, segment count, then the prepass outputs for `rows` activation rows
// (three e4m3 terms at most: 384 bytes and four scale words per row and step of 128).
size_t kq_fp4_moe_workspace_bytes(int P, int E, int rows, int K) {
  const size_t rs = (size_t)rows * f4_steps(K);
  return align256((size_t)P * 4) + align256(((size_t)E + P / 32 + 1) * sizeof(Segment)) + 256 + align256(rs * 384) +
         align256(rs * 16);
}

// x: [rows][K] (rows = P / x_div); pair p reads row p / x_div and expert idx[p]; out rows through om.
int kq_launch_fp4_moe(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* idx, const float* bias,
                      const float* bias2, void* out, int P, int E, int N, int K, int x_div, int64_t w_expert_stride,
                      int glu, int act, float limit, float alpha, int codec, int dtype, void* ws, KqOutMap om,
                      hipStream_t s) {
  if (!kq_fp4_moe_supported(P, E, N, K, codec) || (reinterpret_cast<uintptr_t>(x) & 15) ||
      (reinterpret_cast<uintptr_t>(ws) & 255))
    return KQ_ERR_UNSUPPORTED;
  uint8_t* p = static_cast<uint8_t*>(ws);
  int* order = reinterpret_cast<int*>(p);
  Segment* segs = reinterpret_cast<Segment*>(p + align256((size_t)P * 4));
  int* nseg = reinterpret_cast<int*>(p + align256((size_t)P * 4) + align256(((size_t)E + P / 32 + 1) * sizeof(Segment)));
  x_div = x_div < 1 ? 1 : x_div;
  const int rows = glu ? P / x_div : P, nsteps = f4_steps(K);
  const size_t rs = (size_t)rows * nsteps;
  uint8_t* xa = reinterpret_cast<uint8_t*>(nseg) + 256;
  uint32_t* xs = reinterpret_cast<uint32_t*>(xa + align256(rs * 384));
  const uint16_t* xi = static_cast<const uint16_t*>(x);
  if (dtype == KQ_F16)
    hipLaunchKernelGGL((fp4_prologue_kernel<KQ_F16>), dim3(rows + 1), dim3(F4_PRO_THREADS), 0, s, xi, xa, xs, K, nsteps, idx, P,
                       E, order, segs, nseg);
  else
    hipLaunchKernelGGL((fp4_prologue_kernel<KQ_BF16>), dim3(rows + 1), dim3(F4_PRO_THREADS), 0, s, xi, xa, xs, K, nsteps, idx,
                       P, E, order, segs, nseg);
  KQ_HIP_CHECK(hipGetLastError());
  F4Args a{};
  a.xa = xa;
  a.xs = xs;
  a.w = w;
  a.w2 = w2;
  a.w_end = w + (int64_t)(E - 1) * w_expert_stride + (size_t)N * (K >> 5) * 17;
  a.w2_end = w2 ? w2 + (int64_t)(E - 1) * w_expert_stride + (size_t)N * (K >> 5) * 17 : nullptr;
  a.y = out;
  a.bias = bias;
  a.bias2 = bias2;
  a.order = order;
  a.segs = segs;
  a.nseg = nseg;
  a.N = N;
  a.K = K;
  a.nsteps = nsteps;
  a.x_div = x_div;
  a.act = act;
  a.w_expert_stride = w_expert_stride;
  a.limit = limit;
  a.alpha = alpha;
  a.om = om;
  int maxseg = E + P / 32;  // sum over experts of ceil(c_e / 32) <= E + P / 32
  if (maxseg > P) maxseg = P;
  // Shapes: the fused op streams 8 column tiles per wave and step (64 output columns per workgroup), the plain op 4
  // (64 columns: twice the workgroups of the 8-tile form, 50.7 -> 43.5 us on 32 experts of 2880 x 2880 at 256 pairs);
  // stacks whose experts see more than 12 pairs on average take both m-tiles of a segment in one pass, on 8 tiles
  // where the registers hold them (bf16: two activation terms; 1024 pairs: 160 + 83 -> 137 + 79 us), else on 4.
  const bool two = (int64_t)P > 12 * (int64_t)E;
#define KQ_F4_LAUNCH(DTV, GLUV, JV, MTV)                                                                         \
  hipLaunchKernelGGL((fp4_grouped_kernel<DTV, GLUV, JV, MTV>),                                                   \
                     dim3((N + (GLUV ? 8 * JV : 16 * JV) - 1) / (GLUV ? 8 * JV : 16 * JV), maxseg, MTV == 1 ? 2 : 1), \
                     dim3(F4_THREADS), 0, s, a)
#ifndef KQ_F4_TILES
#define KQ_F4_TILES 1
#endif
#define KQ_F4_LAUNCH_TILES(DTV, NWV)                                                                            \
  hipLaunchKernelGGL((fp4_glu_tiles_kernel<DTV, true, NWV>), dim3((N + 16 * NWV - 1) / (16 * NWV), maxseg, 2),   \
                     dim3(64 * NWV), 0, s, a)
  if (KQ_F4_TILES && glu && !two) {  // the fused op on one m-tile per pass: the waves split the column tiles
    // few pairs: 32-column workgroups of two waves where 64-column groups would leave most CUs one workgroup or none
    // (32 experts of 2880 x 2880: 8 pairs 25.5 -> 23.1 us; 12 pairs 27.6 -> 29.1 and 16 pairs 33.9 -> 36.2 the other way)
    const bool narrow = (int64_t)4 * P * ((N + 63) / 64) < (int64_t)7 * f4_num_cus();
    if (dtype == KQ_F16) { if (narrow) KQ_F4_LAUNCH_TILES(KQ_F16, 2); else KQ_F4_LAUNCH_TILES(KQ_F16, 4); }
    else { if (narrow) KQ_F4_LAUNCH_TILES(KQ_BF16, 2); else KQ_F4_LAUNCH_TILES(KQ_BF16, 4); }
  } else if (glu) {
    if (dtype == KQ_F16) { if (two) KQ_F4_LAUNCH(KQ_F16, true, 4, 2); else KQ_F4_LAUNCH(KQ_F16, true, 8, 1); }
    else { if (two) KQ_F4_LAUNCH(KQ_BF16, true, 8, 2); else KQ_F4_LAUNCH(KQ_BF16, true, 8, 1); }
  } else {
    if (dtype == KQ_F16) { if (two) KQ_F4_LAUNCH(KQ_F16, false, 4, 2); else KQ_F4_LAUNCH(KQ_F16, false, 4, 1); }
    else { if (two) KQ_F4_LAUNCH(KQ_BF16, false, 8, 2); else KQ_F4_LAUNCH(KQ_BF16, false, 4, 1); }
  }
#undef KQ_F4_LAUNCH_TILES
#undef KQ_F4_LAUNCH
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}
