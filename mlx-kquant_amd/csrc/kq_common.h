// Shared host/device definitions: codec ids and block geometry, error plumbing, small
// bit helpers.  Codec order follows the reference registry (src/kquant_codec.cpp:12-37).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "kq.h"

enum KqCodec : int {
  KQ_Q2_K = 0, KQ_Q3_K, KQ_Q4_K, KQ_Q5_K, KQ_Q6_K, KQ_Q4_0, KQ_Q4_1, KQ_Q5_0, KQ_Q5_1, KQ_Q8_0,
  KQ_IQ4_NL, KQ_IQ4_XS, KQ_IQ3_S, KQ_IQ3_XXS, KQ_IQ2_XXS, KQ_IQ2_XS, KQ_IQ2_S, KQ_IQ1_S, KQ_IQ1_M,
  KQ_MXFP4, KQ_NVFP4
};

struct KqGeom {
  int wpb;  // weights per block
  int bpb;  // bytes per block
};

__host__ __device__ constexpr KqGeom kq_geom(int c) {
  constexpr KqGeom g[KQ_NUM_CODECS] = {
      {256, 84},  {256, 110}, {256, 144}, {256, 176}, {256, 210}, {32, 18},  {32, 20},
      {32, 22},   {32, 24},   {32, 34},   {32, 18},   {256, 136}, {256, 110}, {256, 98},
      {256, 66},  {256, 74},  {256, 82},  {256, 50},  {256, 56},  {32, 17},  {64, 36}};
  return g[c];
}

// Offsets of the IQ codebooks inside the device copy of the grid blob
// (iq2xxs u64[256] | iq2xs u64[512] | iq2s u64[1024] | iq1s u64[2048] | iq3xxs u32[256] |
// iq3s u32[512]).
#define KQ_GRID_IQ2XXS 0
#define KQ_GRID_IQ2XS 2048
#define KQ_GRID_IQ2S 6144
#define KQ_GRID_IQ1S 14336
#define KQ_GRID_IQ3XXS 30720
#define KQ_GRID_IQ3S 31744
#define KQ_GRID_BYTES 33792

// Where the gathered / grouped kernels put the result of pair p: output row (p / in) * out + p % in + off,
// as 16-bit values of the activation dtype or (f32 != 0) as float.  The default {1, 1, 0, 0} is row p,
// activation dtype.  The fused MoE ops that interleave a shared-expert slot or mix the slots in f32 pass
// another map to the launchers (kq_api.cpp).
struct KqOutMap {
  int in, out, off, f32;
};
constexpr KqOutMap KQ_OUT_ROWS = {1, 1, 0, 0};

// ---- host-side plumbing (kq_api.cpp) ----
int kq_set_error(int code, const char* fmt, ...);
// Device copy of the IQ codebooks for the current device (uploaded once per device).
const uint8_t* kq_device_grids(void);

#define KQ_HIP_CHECK(expr)                                                              \
  do {                                                                                  \
    hipError_t _e = (expr);                                                             \
    if (_e != hipSuccess)                                                               \
      return kq_set_error(KQ_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(_e));  \
  } while (0)

// hipFuncSetAttribute applies to the current device only: one flag per (call site = kernel instantiation, device).
// Two host threads may both set the attribute the first time; the call is idempotent.
#define KQ_SET_MAX_LDS_ONCE(kern, bytes)                                                          \
  do {                                                                                            \
    static std::atomic<uint64_t> _kq_done{0};                                                     \
    int _kq_dev = 0;                                                                              \
    KQ_HIP_CHECK(hipGetDevice(&_kq_dev));                                                         \
    const uint64_t _kq_bit = 1ull << (_kq_dev & 63);                                              \
    if (!(_kq_done.load(std::memory_order_acquire) & _kq_bit)) {                                  \
      KQ_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                       \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)(bytes))); \
      _kq_done.fetch_or(_kq_bit, std::memory_order_release);                                      \
    }                                                                                             \
  } while (0)

// ---- per-op launchers implemented in the .hip files ----
int kq_launch_dequantize(const uint8_t* w, void* out, uint64_t num_blocks, int codec, int out_dtype,
                         hipStream_t s);
int kq_launch_gemv_generic(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype,
                           hipStream_t s);
int kq_launch_gemm_nt_generic(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec,
                              int dtype, hipStream_t s);
int kq_launch_gather_nt_generic(const void* x, const uint8_t* w, const uint32_t* lhs, const uint32_t* rhs, void* out,
                                int B, int M, int E, int N, int K, int64_t x_batch_stride, int64_t w_expert_stride,
                                int codec, int dtype, hipStream_t s);
// kq_nt.hip: transpose = false on the matrix cores (dense: lhs = rhs = null, B = E = 1); KQ_ERR_UNSUPPORTED when
// the output is not 16-byte aligned.  Dense calls with few tiles cut K when given kq_nt_workspace_bytes of workspace.
size_t kq_nt_workspace_bytes(int M, int N, int K);
int kq_launch_nt_mfma(const void* x, const uint8_t* w, const uint32_t* lhs, const uint32_t* rhs, void* out, int B,
                      int M, int E, int N, int K, int64_t x_batch_stride, int64_t w_expert_stride, int codec, int dtype,
                      void* ws, size_t ws_bytes, hipStream_t s);
int kq_launch_gather_generic(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* lhs,
                             const uint32_t* rhs, const float* bias, const float* bias2, void* out, int B, int M,
                             int N, int K, int x_div, int64_t x_batch_stride, int64_t w_expert_stride, int glu,
                             int act, float limit, float alpha, int codec, int dtype, int E, KqOutMap om,
                             hipStream_t s);
// Score-weighted slot sum in one launch (kq_generic.hip): decode-sized gather_qmv_mix calls.
int kq_launch_gather_mix_generic(const void* x, const uint8_t* w, const uint8_t* shexp_w, const uint32_t* idx,
                                 const float* scores, const float* bias, void* out, int T, int S, int E, int N, int K,
                                 int64_t w_expert_stride, int codec, int shexp_codec, int dtype, hipStream_t s);
// Tuned path: returns KQ_ERR_UNSUPPORTED (without touching the error text) when no tuned kernel
// covers the request, so the caller can fall through to the generic kernels.
// A null / short workspace is allowed: the call then runs without its split-K plan.
size_t kq_qmm_tuned_workspace_bytes(int M, int N, int K, int codec);
int kq_launch_qmm_tuned(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                        size_t ws_bytes, hipStream_t s);
// Streamed skinny kernel (direct-to-LDS weight stream, q4_k / q5_k / q6_k, M <= 4): same fall-through contract.
// Needs its split-K workspace when its plan splits K (K > 4096 or few row tiles); without it the call is declined.
bool kq_stream_supported(int M, int N, int K, int codec, const void* x, const void* w);
size_t kq_stream_workspace_bytes(int M, int N, int K, int codec);
int kq_launch_qmm_stream(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                         size_t ws_bytes, hipStream_t s, const void* bias = nullptr);
// Gathered matvec (MoE decode, one activation row per entry) on the streamed kernel; UNSUPPORTED -> older kernels.
// Entry p reads activation row p / x_div of x, or (lhs != null) the row at x + lhs[p] * x_row_stride.  bias / bias2:
// null, or f32 [E][N] added to the gate (or plain) and up sums; alpha: the sigmoid slope of swiglu_clamp.
int kq_launch_gather_stream(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* lhs, const uint32_t* rhs,
                            void* out, int entries, int N, int K, int x_div, int64_t x_row_stride,
                            int64_t w_expert_stride, int act, float limit, float alpha, const float* bias,
                            const float* bias2, int codec, int dtype, int E, KqOutMap om, hipStream_t s);
// Whether kq_launch_gather_stream takes a call of this shape and alignment (strided_x: rows addressed through lhs
// with x_row_stride); the most entries it takes.
bool kq_gather_stream_takes(const void* x, const void* w, const void* w2, int entries, int N, int K, bool strided_x,
                            int64_t x_row_stride, int64_t w_expert_stride, bool second_bias_without_glu, int codec);
int kq_gather_stream_max_entries();
// codecs whose gathered calls the streamed kernel also takes with biases and swiglu_clamp (the fp4 stacks that carry
// them, and the two codecs that share their unit)
inline bool kq_stream_full_epilogue(int codec) {
  return codec == KQ_MXFP4 || codec == KQ_NVFP4 || codec == KQ_IQ4_NL || codec == KQ_Q4_0;
}
// Tuned gathered GEMV (items = (activation matrix, expert) pairs, M <= 8 rows each; with glu the
// gate/up pair and the fused epilogue, M = 1): same fall-through contract as kq_launch_qmm_tuned.
// The per-entry gather launchers take the stack height E and skip entries whose expert id is >= E.
int kq_launch_gather_tuned(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* lhs,
                           const uint32_t* rhs, void* out, int B, int M, int N, int K, int x_div,
                           int64_t x_batch_stride, int64_t w_expert_stride, int glu, int act, float limit, int codec,
                           int dtype, int E, KqOutMap om, hipStream_t s);
// Prefill GEMM (q4_k / q5_k / q6_k, M > 8): needs kq_gemm_workspace_min_bytes(M, K) bytes of device workspace
// (converted activations); with kq_gemm_workspace_bytes(M, N, K) a call with few tiles cuts K over the grid.
size_t kq_gemm_workspace_min_bytes(int M, int K);
size_t kq_gemm_workspace_bytes(int M, int N, int K);
bool kq_gemm_supported(int M, int N, int K, int codec);
int kq_launch_gemm(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                   size_t ws_bytes, hipStream_t s);
// 128 x 256-tile prefill GEMM (q4_k / q5_k) on the outputs of the activation prepass (rows padded to 128).
bool kq_gemm2_supported(int M, int N, int K, int codec);
int kq_launch_gemm2(const void* xh, const void* xhl, const float* rs, const uint8_t* w, void* y, int M, int N, int K,
                    int codec, int dtype, int shape, hipStream_t s, int nt0 = 0, int ntiles = -1);
// 256 x 256-tile prefill GEMM (q4_k / q5_k, 256-row wave tiles on one accumulator set) on the same prepass outputs
// (mrows >= M prepared rows): column tiles nt0 .. nt0 + ntiles - 1 of 256 weight rows each.
bool kq_gemm3_supported(int M, int mrows, int N, int K, int codec);
int kq_launch_gemm3(const void* xh, const void* xhl, const float* rs, const uint8_t* w, void* y, int M, int mrows, int N,
                    int K, int codec, int dtype, int nt0, int ntiles, hipStream_t s, int tile_rows = 256);
// 256-row / 128-row wave tiles for the 32-weight-block codecs with an f16 scale (q8_0, q4_0): every weight as two
// exact f16 terms (kq_gemm3b.hip).  Runs its own activation prepass into ws (kq_gemm3b_workspace_bytes).
bool kq_gemm3b_supported(int M, int N, int K, int codec);
size_t kq_gemm3b_workspace_bytes(int M, int K);
void kq_gemm3b_force_tile(int rows);
int kq_launch_gemm3b(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                     hipStream_t s);
// The same tiles for the fp4 codecs (mxfp4, nvfp4): one exact f16 term per weight, converted from the wire nibbles by
// the hardware's fp4 -> f16 instruction (kq_gemm3f.hip).  Runs its own activation prepass into ws.
bool kq_gemm3f_supported(int M, int N, int K, int codec);
size_t kq_gemm3f_workspace_bytes(int M, int K);
void kq_gemm3f_force_tile(int rows);
int kq_launch_gemm3f(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                     hipStream_t s);
// The same tiles for the codebook codecs (iq2_xxs, iq2_xs, iq2_s, iq3_xxs, iq3_s, iq1_s, iq1_m): one exact f16 term per
// weight (the reference-order decoder with d = 1), d in the unit of the running sums (kq_gemm3i.hip).  Runs its own
// activation prepass into ws.
bool kq_gemm3i_supported(int M, int N, int K, int codec);
size_t kq_gemm3i_workspace_bytes(int M, int K);
void kq_gemm3i_force_tile(int rows);
int kq_launch_gemm3i(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                     hipStream_t s);
// The same tile kernel for q2_k / q3_k (M >= 256, tiles filling the chip): runs its own activation prepass.
bool kq_gemm2_low_supported(int M, int N, int K, int codec);
size_t kq_gemm2_low_workspace_bytes(int M, int K);
int kq_launch_gemm2_low(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype, void* ws,
                        hipStream_t s);
// Batched MoE path (q4_k / q5_k / q6_k, more than 16 pairs): pairs sorted by expert, one MFMA GEMM
// per segment of <= 32 pairs.  rows = activation rows (T for the GLU op, T*R for the down op).
bool kq_moe_grouped_supported(int P, int E, int N, int K, int codec);
size_t kq_moe_grouped_workspace_bytes(int rows, int P, int E, int K);
int kq_launch_moe_grouped(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* idx, void* out, int rows,
                          int P, int E, int N, int K, int x_div, int64_t w_expert_stride, int glu, int act,
                          float limit, int codec, int dtype, void* ws, KqOutMap om, hipStream_t s);
// Gathered activations of a batched gather_qmm: xg[b*M + m][:] = x[lhs[b]][m][:], idx_rows[b*M + m] = rhs[b]
// (16-bit elements; K a multiple of 8, x and xg 16-byte aligned).  lhs == null: b; rhs == null: 0.
int kq_launch_gather_rows(const void* x, const uint32_t* lhs, const uint32_t* rhs, void* xg, uint32_t* idx_rows, int B,
                          int M, int K, int64_t x_batch_stride, hipStream_t s);
// Skinny-M (M <= 8) matrix-core kernel of the legacy / IQ / fp4 codecs: exact f16 codes in, block scales
// applied to the f32 partial sums.  Same fall-through contract as kq_launch_qmm_tuned; no workspace.
bool kq_codes_supported(int M, int N, int K, int codec);
// bias: [N] in the activation dtype (added in f32 before the single rounding) or null
int kq_launch_codes_skinny(const void* x, const uint8_t* w, const void* bias, void* y, int M, int N, int K, int codec,
                           int dtype, hipStream_t s);
// Batched MoE of the same codecs (more than 16 pairs; biases and every activation): pairs sorted by expert,
// 32-pair segments x 128-row slabs.  Workspace layout and size as the any-codec path below.
bool kq_codes_gather_supported(int M, int N, int K, int codec);
bool kq_codes_moe_supported(int P, int E, int N, int K, int codec);
size_t kq_codes_moe_workspace_bytes(int P, int E, int rows, int K);
int kq_launch_codes_moe(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* idx, const float* bias,
                        const float* bias2, void* out, int P, int E, int N, int K, int x_div, int64_t w_expert_stride,
                        int glu, int act, float limit, float alpha, int codec, int dtype, void* ws, KqOutMap om,
                        hipStream_t s);
// Batched MoE of mxfp4 stacks on the block-scaled matrix instruction (wire blocks undecoded, activations as e4m3
// terms); same contract and workspace layout idea as kq_launch_codes_moe.
bool kq_fp4_moe_supported(int P, int E, int N, int K, int codec);
size_t kq_fp4_moe_workspace_bytes(int P, int E, int rows, int K);
int kq_launch_fp4_moe(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* idx, const float* bias,
                      const float* bias2, void* out, int P, int E, int N, int K, int x_div, int64_t w_expert_stride,
                      int glu, int act, float limit, float alpha, int codec, int dtype, void* ws, KqOutMap om,
                      hipStream_t s);
// Helpers of the slot-mixing ops: idx [T][S-1] -> idx2 [T][S] (last slot = expert 0), and
// out[t][n] = T(sum_s scores[t][s] * yf[t][s][n]).
int kq_launch_pad_idx(const uint32_t* idx, uint32_t* idx2, int T, int S, hipStream_t s);
int kq_launch_codes_gather(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* lhs, const uint32_t* rhs,
                           const float* bias, const float* bias2, void* out, int B, int M, int N, int K, int x_div,
                           int64_t x_batch_stride, int64_t w_expert_stride, int glu, int act, float limit, float alpha,
                           int codec, int dtype, int E, KqOutMap om, hipStream_t s);
bool kq_encode_dev_supported(int codec);
int kq_launch_encode(const void* w, int dtype, const float* im, uint8_t* wire, int64_t rows, int64_t K, int codec,
                     hipStream_t s);
int kq_launch_mxfp4_repack(const void* packed, const void* scales, void* wire, int64_t nblocks, int to_wire, hipStream_t s);
int kq_launch_expert_tile_map(const uint32_t* idx, int rows, int E, uint32_t* map, int cap, uint32_t* counts,
                              hipStream_t s);
int kq_launch_tiles_to_rows(const uint32_t* map, const uint32_t* counts, int cap, int rows, int E, uint32_t none,
                            uint32_t* row_expert, hipStream_t s);
int kq_launch_mix_slots(const float* yf, const float* scores, const uint32_t* idx, int routed, int E, void* out, int T,
                        int S, int N, int dtype, hipStream_t s);
// Matrix-core GEMM for every codec (two-term bf16 split of the reference-order decoded weights):
// prefill, and the batched MoE ops with biases and every activation.
bool kq_anymma_supported(int M, int N, int K, int codec);
size_t kq_anymma_dense_workspace_bytes(int M, int N, int K, int dtype);
int kq_launch_anymma_dense(const void* x, const uint8_t* w, void* y, int M, int N, int K, int codec, int dtype,
                           void* ws, size_t ws_bytes, hipStream_t s);
bool kq_anymma_moe_supported(int P, int E, int N, int K, int codec);
size_t kq_anymma_moe_workspace_bytes(int P, int E);
int kq_launch_anymma_moe(const void* x, const uint8_t* w, const uint8_t* w2, const uint32_t* idx, const float* bias,
                         const float* bias2, void* out, int P, int E, int N, int K, int x_div, int64_t w_expert_stride,
                         int glu, int act, float limit, float alpha, int codec, int dtype, void* ws, KqOutMap om,
                        hipStream_t s);
// Router top-k (one workgroup per token): see kq_moe_router_topk in include/kq.h.
int kq_launch_router_topk(const void* logits, int dtype, int T, int E, int top_k, int norm, int shared, const float* pes,
                          const float* bias, int scoring, float scale, uint32_t* indices, float* scores, hipStream_t s);
