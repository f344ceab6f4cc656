// C ABI of libkq (declared in include/kq.h): argument validation, error reporting, the device copy of the
// IQ codebooks and routing to the HIP launchers.  Compiled by hipcc as HIP (the codebooks are a __device__ array).
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "kq_common.h"

// IQ codebooks (33,792 bytes of ggml constants) as device-resident storage: part of the code object, so no
// entry point allocates or copies anything for them.  The initialiser is the data file
// data/kq_iq_grids.bin written out as a byte list by build.py (kq_iq_grids.inc in the object directory).
// (not const: a const device array has internal linkage and cannot be looked up by symbol)
__device__ __attribute__((aligned(16))) uint8_t kq_grid_blob_dev[KQ_GRID_BYTES] = {
#include "kq_iq_grids.inc"
};
// host copy of the same bytes (the host encoders search the codebooks)
extern "C" __attribute__((visibility("hidden"))) const uint8_t kq_grid_blob_host[KQ_GRID_BYTES] = {
#include "kq_iq_grids.inc"
};

// Workspace of kq_qmm_noalloc: device-resident storage inside the code object.  In host code this name is only
// a handle for hipGetSymbolAddress; kernels get the per-device address that call returns.
static __device__ __attribute__((aligned(256))) uint8_t kq_noalloc_scratch[KQ_NOALLOC_SCRATCH_BYTES];

namespace {

thread_local char g_err[512] = "";

// Reference registry, src/kquant_codec.cpp:12-37.
const kq_codec_info kCodecs[KQ_NUM_CODECS] = {
    {"q2_k", 256, 84, 2, 1, 1, 1, 0},    {"q3_k", 256, 110, 3, 1, 1, 1, 0},
    {"q4_k", 256, 144, 4, 1, 1, 1, 0},   {"q5_k", 256, 176, 5, 1, 1, 1, 0},
    {"q6_k", 256, 210, 6, 1, 1, 1, 0},   {"q4_0", 32, 18, 4, 1, 1, 1, 0},
    {"q4_1", 32, 20, 4, 1, 1, 1, 0},     {"q5_0", 32, 22, 5, 1, 1, 1, 0},
    {"q5_1", 32, 24, 5, 1, 1, 1, 0},     {"q8_0", 32, 34, 8, 1, 1, 1, 0},
    {"iq4_nl", 32, 18, 4, 1, 1, 1, 0},   {"iq4_xs", 256, 136, 4, 1, 1, 1, 0},
    {"iq3_s", 256, 110, 3, 1, 1, 1, 0},  {"iq3_xxs", 256, 98, 3, 1, 1, 1, 0},
    {"iq2_xxs", 256, 66, 2, 1, 1, 1, 1}, {"iq2_xs", 256, 74, 2, 1, 1, 1, 1},
    {"iq2_s", 256, 82, 2, 1, 1, 1, 0},   {"iq1_s", 256, 50, 1, 1, 1, 1, 1},
    {"iq1_m", 256, 56, 1, 1, 1, 1, 0},   {"mxfp4", 32, 17, 4, 1, 0, 0, 0},
    {"nvfp4", 64, 36, 4, 1, 0, 0, 0},
};

constexpr int kMaxDevices = 64;
std::mutex g_grid_mu;
const uint8_t* g_grids[kMaxDevices] = {};
void* g_scratch[kMaxDevices] = {};  // per-device address of kq_noalloc_scratch

bool codec_ok(int c) { return c >= 0 && c < KQ_NUM_CODECS; }
bool half_dtype(int dt) { return dt == KQ_F16 || dt == KQ_BF16; }

}  // namespace

int kq_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

const uint8_t* kq_device_grids(void) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    kq_set_error(KQ_ERR_HIP, "no usable HIP device: %s", hipGetErrorString(e));
    return nullptr;
  }
  std::lock_guard<std::mutex> lk(g_grid_mu);
  if (!g_grids[dev]) {
    // every device holds its own copy of the array at its own address
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(kq_grid_blob_dev));
    if (e != hipSuccess || !p) {
      kq_set_error(KQ_ERR_HIP, "codebook lookup failed: %s", hipGetErrorString(e));
      return nullptr;
    }
    g_grids[dev] = static_cast<const uint8_t*>(p);
  }
  return g_grids[dev];
}

extern "C" {

const char* kq_last_error(void) { return g_err; }
const char* kq_version(void) { return "kq-mi355x 0.1 (gfx950)"; }
int kq_codec_count(void) { return KQ_NUM_CODECS; }

int kq_codec_id(const char* name) {
  if (!name) return -1;
  for (int i = 0; i < KQ_NUM_CODECS; i++)
    if (std::strcmp(kCodecs[i].name, name) == 0) return i;
  return -1;
}

int kq_codec_get(int codec, kq_codec_info* out) {
  if (!codec_ok(codec) || !out) return kq_set_error(KQ_ERR_INVALID, "codec id %d out of range", codec);
  *out = kCodecs[codec];
  return KQ_OK;
}

int kq_codec_has_moe_glu(int codec) { return codec_ok(codec) ? 1 : 0; }

int kq_dequantize(const void* w_dev, void* out_dev, uint64_t num_weights, int codec, int out_dtype, void* stream) {
  if (!codec_ok(codec)) return kq_set_error(KQ_ERR_INVALID, "dequantize: unknown codec id %d", codec);
  if (out_dtype < KQ_F32 || out_dtype > KQ_BF16)
    return kq_set_error(KQ_ERR_INVALID, "dequantize: only real floating output dtypes are supported");
  const int wpb = kCodecs[codec].weights_per_block;
  if (num_weights % (uint64_t)wpb)
    return kq_set_error(KQ_ERR_INVALID, "dequantize: num_weights (%llu) is not a whole number of %d-weight blocks",
                        (unsigned long long)num_weights, wpb);
  if (num_weights == 0) return KQ_OK;
  if (!w_dev || !out_dev) return kq_set_error(KQ_ERR_INVALID, "dequantize: null buffer");
  return kq_launch_dequantize(static_cast<const uint8_t*>(w_dev), out_dev, num_weights / wpb, codec, out_dtype,
                              static_cast<hipStream_t>(stream));
}

size_t kq_qmm_workspace_size(int M, int N, int K, int transpose, int codec, int dtype) {
  (void)dtype;
  if (!codec_ok(codec)) return 0;
  if (!transpose) return kq_nt_workspace_bytes(M, N, K);  // optional: partial sums of a K range cut over the grid
  if (kq_gemm_supported(M, N, K, codec)) return kq_gemm_workspace_bytes(M, N, K);
  // split-K partial sums (optional) of whichever skinny kernel takes the call
  const size_t tuned = kq_qmm_tuned_workspace_bytes(M, N, K, codec);
  size_t any = (M > 8 && kq_anymma_supported(M, N, K, codec)) ? kq_anymma_dense_workspace_bytes(M, N, K, dtype) : 0;
  if (kq_gemm2_low_supported(M, N, K, codec) && kq_gemm2_low_workspace_bytes(M, K) > any) any = kq_gemm2_low_workspace_bytes(M, K);
  if (kq_gemm3b_supported(M, N, K, codec) && kq_gemm3b_workspace_bytes(M, K) > any) any = kq_gemm3b_workspace_bytes(M, K);
  if (kq_gemm3f_supported(M, N, K, codec) && kq_gemm3f_workspace_bytes(M, K) > any) any = kq_gemm3f_workspace_bytes(M, K);
  if (kq_gemm3i_supported(M, N, K, codec) && kq_gemm3i_workspace_bytes(M, K) > any) any = kq_gemm3i_workspace_bytes(M, K);
  return tuned > any ? tuned : any;
}

int kq_qmm(const void* x_dev, const void* w_dev, void* y_dev, int M, int N, int K, int transpose, int codec,
           int dtype, void* workspace_dev, size_t workspace_bytes, void* stream) {
  if (!codec_ok(codec)) return kq_set_error(KQ_ERR_INVALID, "quantized_matmul: unknown codec id %d", codec);
  if (!half_dtype(dtype))
    return kq_set_error(KQ_ERR_INVALID, "quantized_matmul: activations must be float16 or bfloat16");
  if (M < 0 || N < 0 || K < 0) return kq_set_error(KQ_ERR_INVALID, "quantized_matmul: negative dimension");
  const int wpb = kCodecs[codec].weights_per_block;
  const int inner = transpose ? K : N;
  if (inner % wpb)
    return kq_set_error(KQ_ERR_INVALID, "quantized_matmul: quantized row length %d is not a multiple of %d", inner,
                        wpb);
  if (M == 0 || N == 0) return KQ_OK;
  if (!x_dev || !w_dev || !y_dev) return kq_set_error(KQ_ERR_INVALID, "quantized_matmul: null buffer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!transpose) {
    const int rcn = kq_launch_nt_mfma(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, nullptr, y_dev, 1, M, 1, N, K,
                                      0, 0, codec, dtype, workspace_dev, workspace_bytes, s);
    if (rcn != KQ_ERR_UNSUPPORTED) return rcn;
    return kq_launch_gemm_nt_generic(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, M, N, K, codec, dtype, s);
  }
  if (kq_gemm_supported(M, N, K, codec)) {
    const size_t need = kq_gemm_workspace_min_bytes(M, K);
    if (!workspace_dev || workspace_bytes < need)
      return kq_set_error(KQ_ERR_WORKSPACE, "quantized_matmul: workspace of %zu bytes required (got %zu)", need,
                          workspace_bytes);
    int rcg = kq_launch_gemm(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, M, N, K, codec, dtype, workspace_dev,
                             workspace_bytes, s);
    if (rcg != KQ_ERR_UNSUPPORTED) return rcg;
  }
  if (kq_gemm2_low_supported(M, N, K, codec) && workspace_dev && workspace_bytes >= kq_gemm2_low_workspace_bytes(M, K)) {
    const int rcl = kq_launch_gemm2_low(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, M, N, K, codec, dtype, workspace_dev, s);
    if (rcl != KQ_ERR_UNSUPPORTED) return rcl;
  }
  if (kq_gemm3b_supported(M, N, K, codec) && workspace_dev && workspace_bytes >= kq_gemm3b_workspace_bytes(M, K)) {
    const int rcb = kq_launch_gemm3b(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, M, N, K, codec, dtype, workspace_dev, s);
    if (rcb != KQ_ERR_UNSUPPORTED) return rcb;
  }
  if (kq_gemm3f_supported(M, N, K, codec) && workspace_dev && workspace_bytes >= kq_gemm3f_workspace_bytes(M, K)) {
    const int rcf = kq_launch_gemm3f(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, M, N, K, codec, dtype, workspace_dev, s);
    if (rcf != KQ_ERR_UNSUPPORTED) return rcf;
  }
  if (kq_gemm3i_supported(M, N, K, codec) && workspace_dev && workspace_bytes >= kq_gemm3i_workspace_bytes(M, K)) {
    const int rci = kq_launch_gemm3i(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, M, N, K, codec, dtype, workspace_dev, s);
    if (rci != KQ_ERR_UNSUPPORTED) return rci;
  }
  if (M > 8) {
    const int rca = kq_launch_anymma_dense(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, M, N, K, codec, dtype,
                                           workspace_dev, workspace_bytes, s);
    if (rca != KQ_ERR_UNSUPPORTED) return rca;
  }
  int rc = kq_launch_qmm_tuned(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, M, N, K, codec, dtype, workspace_dev,
                               workspace_bytes, s);
  if (rc != KQ_ERR_UNSUPPORTED) return rc;
  rc = kq_launch_codes_skinny(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, y_dev, M, N, K, codec, dtype, s);
  if (rc != KQ_ERR_UNSUPPORTED) return rc;
  return kq_launch_gemv_generic(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, M, N, K, codec, dtype, s);
}

int kq_qmm_noalloc(const void* x_dev, const void* w_dev, void* y_dev, int M, int N, int K, int codec, int dtype,
                   void* stream) {
  if (!codec_ok(codec)) return kq_set_error(KQ_ERR_INVALID, "quantized_matmul: unknown codec id %d", codec);
  // what the call cannot run without (the prefill GEMM's converted activations); partial sums of a K range cut
  // over the grid are optional and are left out when they do not fit
  const size_t need = kq_gemm_supported(M, N, K, codec) ? kq_gemm_workspace_min_bytes(M, K) : 0;
  if (need > KQ_NOALLOC_SCRATCH_BYTES)
    return kq_set_error(KQ_ERR_WORKSPACE,
                        "quantized_matmul (no-allocation entry): this shape needs %zu bytes of workspace, the built-in "
                        "buffer holds %u; call kq_qmm with a caller-owned workspace",
                        need, (unsigned)KQ_NOALLOC_SCRATCH_BYTES);
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return kq_set_error(KQ_ERR_HIP, "no usable HIP device: %s", hipGetErrorString(e));
  void* scratch = nullptr;
  {
    std::lock_guard<std::mutex> lk(g_grid_mu);
    if (!g_scratch[dev]) {
      // once per device, with that device current: every GPU holds its own copy of the array
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(kq_noalloc_scratch));
      if (e != hipSuccess || !p)
        return kq_set_error(KQ_ERR_HIP, "scratch lookup failed: %s", hipGetErrorString(e));
      g_scratch[dev] = p;
    }
    scratch = g_scratch[dev];
  }
  return kq_qmm(x_dev, w_dev, y_dev, M, N, K, 1, codec, dtype, scratch, KQ_NOALLOC_SCRATCH_BYTES, stream);
}

int kq_qmv_bias(const void* x_dev, const void* w_dev, const void* bias_dev, void* y_dev, int N, int K, int codec,
                int dtype, void* stream) {
  const char* op = "quantized_matmul_qmv_bias";
  if (codec != KQ_Q8_0) return kq_set_error(KQ_ERR_INVALID, "%s: only kquant_type 'q8_0' is wired", op);
  if (!half_dtype(dtype)) return kq_set_error(KQ_ERR_INVALID, "%s: activations must be float16 or bfloat16", op);
  if (N < 0 || K < 0 || K % kCodecs[codec].weights_per_block)
    return kq_set_error(KQ_ERR_INVALID, "%s: bad dimension", op);
  if (N == 0) return KQ_OK;
  if (!x_dev || !w_dev || !bias_dev || !y_dev) return kq_set_error(KQ_ERR_INVALID, "%s: null buffer", op);
  // the streamed kernel where its plan needs no K split (this op has no workspace), else the code-level kernel
  const int rcs = kq_launch_qmm_stream(x_dev, static_cast<const uint8_t*>(w_dev), y_dev, 1, N, K, codec, dtype, nullptr, 0,
                                       static_cast<hipStream_t>(stream), bias_dev);
  if (rcs != KQ_ERR_UNSUPPORTED) return rcs;
  const int rc = kq_launch_codes_skinny(x_dev, static_cast<const uint8_t*>(w_dev), bias_dev, y_dev, 1, N, K, codec, dtype,
                                        static_cast<hipStream_t>(stream));
  if (rc == KQ_ERR_UNSUPPORTED) return kq_set_error(KQ_ERR_UNSUPPORTED, "%s: x must be 16-byte aligned", op);
  return rc;
}

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// Batched gather_qmm: B * M output rows, gathered into a dense [P, K] matrix + a per-row expert id.
static bool gather_batched_shape(int B, int M, int E, int N, int K, int transpose, int codec, int64_t* P_out) {
  const int64_t P = (int64_t)B * M;
  *P_out = P;
  if (!transpose || E <= 0 || P <= 16 || P > 0x7fffffff || (K & 7)) return false;
  return kq_moe_grouped_supported((int)P, E, N, K, codec) || kq_anymma_moe_supported((int)P, E, N, K, codec);
}

size_t kq_gather_qmm_workspace_size(int B, int M, int E, int N, int K, int transpose, int codec, int dtype) {
  int64_t P;
  if (B <= 0 || M <= 0 || !codec_ok(codec) || !gather_batched_shape(B, M, E, N, K, transpose, codec, &P)) return 0;
  return align256((size_t)P * K * 2) + align256((size_t)P * 4) + kq_moe_workspace_size((int)P, 1, E, N, K, 0, codec, dtype);
}

static int try_moe_grouped(const char* op, const void* x, const void* w, const void* w2, const uint32_t* idx,
                           const float* bias, const float* bias2, void* out, int T, int R, int E, int N, int K,
                           int64_t estride, int glu, int act, float limit, float alpha, int codec, int dtype, void* ws,
                           size_t ws_bytes, KqOutMap om, hipStream_t s, int entry_rows = 1);
static bool per_entry_route(int64_t P, int entry_rows, bool has_bias, int glu, int act, int codec, int E, int N, int K,
                            bool stream_takes);

int kq_gather_qmm(const void* x_dev, const void* w_dev, const uint32_t* lhs_idx_dev, const uint32_t* rhs_idx_dev,
                  void* out_dev, int B, int M, int E, int N, int K, int64_t x_batch_stride,
                  int64_t w_expert_stride_bytes, int transpose, int rhs_sorted, int codec, int dtype,
                  void* workspace_dev, size_t workspace_bytes, void* stream) {
  (void)rhs_sorted;
  if (!codec_ok(codec)) return kq_set_error(KQ_ERR_INVALID, "gather_qmm: unknown codec id %d", codec);
  if (!half_dtype(dtype)) return kq_set_error(KQ_ERR_INVALID, "gather_qmm: activations must be float16 or bfloat16");
  if (B < 0 || M < 0 || N < 0 || K < 0 || E < 0) return kq_set_error(KQ_ERR_INVALID, "gather_qmm: negative dimension");
  const int inner = transpose ? K : N;  // the quantized (row) dimension of the expert matrices
  if (inner % kCodecs[codec].weights_per_block)
    return kq_set_error(KQ_ERR_INVALID, "gather_qmm: quantized row length %d is not a multiple of %d", inner,
                        kCodecs[codec].weights_per_block);
  if (B == 0 || M == 0 || N == 0) return KQ_OK;
  if (!x_dev || !w_dev || !out_dev || !lhs_idx_dev || !rhs_idx_dev)
    return kq_set_error(KQ_ERR_INVALID, "gather_qmm: null buffer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!transpose) {
    const int rcn = kq_launch_nt_mfma(x_dev, static_cast<const uint8_t*>(w_dev), lhs_idx_dev, rhs_idx_dev, out_dev, B, M,
                                      E, N, K, x_batch_stride, w_expert_stride_bytes, codec, dtype, nullptr, 0, s);
    if (rcn != KQ_ERR_UNSUPPORTED) return rcn;
    return kq_launch_gather_nt_generic(x_dev, static_cast<const uint8_t*>(w_dev), lhs_idx_dev, rhs_idx_dev, out_dev, B,
                                       M, E, N, K, x_batch_stride, w_expert_stride_bytes, codec, dtype, s);
  }
  // many output rows: gather them into a dense matrix and run the expert-grouped kernels
  int64_t P;
  if (workspace_dev && gather_batched_shape(B, M, E, N, K, transpose, codec, &P) &&
      !per_entry_route(P, M, false, 0, 0, codec, E, N, K,
                       kq_gather_stream_takes(x_dev, w_dev, nullptr, (int)(P > 0x7fffffff ? 0x7fffffff : P), N, K, true,
                                              x_batch_stride, w_expert_stride_bytes, false, codec)) &&
      !(reinterpret_cast<uintptr_t>(workspace_dev) & 255) && !(reinterpret_cast<uintptr_t>(x_dev) & 15) &&
      !(x_batch_stride & 7)) {
    const size_t need = kq_gather_qmm_workspace_size(B, M, E, N, K, transpose, codec, dtype);
    if (workspace_bytes >= need) {
      uint8_t* wsb = static_cast<uint8_t*>(workspace_dev);
      void* xg = wsb;
      uint32_t* idx_rows = reinterpret_cast<uint32_t*>(wsb + align256((size_t)P * K * 2));
      const size_t used = align256((size_t)P * K * 2) + align256((size_t)P * 4);
      const int rcr = kq_launch_gather_rows(x_dev, lhs_idx_dev, rhs_idx_dev, xg, idx_rows, B, M, K, x_batch_stride, s);
      if (rcr) return rcr;
      const int rcg = try_moe_grouped("gather_qmm", xg, w_dev, nullptr, idx_rows, nullptr, nullptr, out_dev, (int)P, 1, E,
                                      N, K, w_expert_stride_bytes, 0, 0, 0.f, 0.f, codec, dtype, wsb + used,
                                      workspace_bytes - used, KQ_OUT_ROWS, s, M);
      if (rcg != KQ_ERR_UNSUPPORTED) return rcg;
    }
  }
  {
    const int rct = kq_launch_gather_tuned(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, lhs_idx_dev, rhs_idx_dev,
                                           out_dev, B, M, N, K, 1, x_batch_stride, w_expert_stride_bytes, 0, 0, 0.f,
                                           codec, dtype, E, KQ_OUT_ROWS, s);
    if (rct != KQ_ERR_UNSUPPORTED) return rct;
  }
  {
    // legacy / IQ / fp4 stacks, one row per entry: the code-level skinny kernel, one entry per grid row
    const int rcc = kq_launch_codes_gather(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, lhs_idx_dev, rhs_idx_dev,
                                  nullptr, nullptr, out_dev, B, M, N, K, 1, x_batch_stride, w_expert_stride_bytes, 0,
                                  0, 0.f, 0.f, codec, dtype, E, KQ_OUT_ROWS, s);
    if (rcc != KQ_ERR_UNSUPPORTED) return rcc;
  }
  return kq_launch_gather_generic(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, lhs_idx_dev, rhs_idx_dev,
                                  nullptr, nullptr, out_dev, B, M, N, K, 1, x_batch_stride, w_expert_stride_bytes, 0,
                                  0, 0.f, 0.f, codec, dtype, E, KQ_OUT_ROWS, s);
}

static int check_moe(const char* op, int T, int R, int E, int N, int K, int codec, int dtype) {
  if (!codec_ok(codec)) return kq_set_error(KQ_ERR_INVALID, "%s: codec id %d has no fused MoE kernel", op, codec);
  if (!half_dtype(dtype)) return kq_set_error(KQ_ERR_INVALID, "%s: x must be float16 or bfloat16", op);
  if (T < 0 || R < 0 || E <= 0 || N < 0 || K < 0) return kq_set_error(KQ_ERR_INVALID, "%s: bad dimension", op);
  if (K % kCodecs[codec].weights_per_block)
    return kq_set_error(KQ_ERR_INVALID, "%s: weight trailing dim does not match K for '%s'", op, kCodecs[codec].name);
  if (N % 8) return kq_set_error(KQ_ERR_INVALID, "%s: N must be a multiple of 8", op);
  return KQ_OK;
}

size_t kq_moe_workspace_size(int T, int R, int E, int N, int K, int glu, int codec, int dtype) {
  (void)dtype;
  if (T <= 0 || R <= 0 || !codec_ok(codec)) return 0;
  const int64_t P = (int64_t)T * R;
  if (P > 0x7fffffff) return 0;
  if (kq_moe_grouped_supported((int)P, E, N, K, codec)) return kq_moe_grouped_workspace_bytes(glu ? T : (int)P, (int)P, E, K);
  if (kq_fp4_moe_supported((int)P, E, N, K, codec)) {  // mxfp4: block-scaled MFMA path, else the code-level kernel
    const size_t a = kq_fp4_moe_workspace_bytes((int)P, E, glu ? T : (int)P, K);
    const size_t b = kq_codes_moe_supported((int)P, E, N, K, codec) ? kq_codes_moe_workspace_bytes((int)P, E, glu ? T : (int)P, K) : 0;
    return a > b ? a : b;
  }
  if (kq_codes_moe_supported((int)P, E, N, K, codec)) return kq_codes_moe_workspace_bytes((int)P, E, glu ? T : (int)P, K);
  if (kq_anymma_moe_supported((int)P, E, N, K, codec)) return kq_anymma_moe_workspace_bytes((int)P, E);
  return 0;
}

// Batched MoE path: returns KQ_ERR_UNSUPPORTED (error text untouched) when it does not apply.
//
// Entry by entry or grouped.  A call of P (token, expert) pairs can run entry by entry (one grid row per pair, every
// pair streams its expert's matrix) or sorted by expert (one prologue launch, then every expert's matrix once for all
// of its pairs).  Entry by entry saves the prologue and the mostly empty 32-row segments; it pays by reading a
// matrix once per pair instead of once per call.  The crossover was measured per codec family on the reference stack
// (128 experts of 2048 <-> 768, top-8, fused gate / up + down, us entry by entry against grouped):
//   q4_k / q5_k / q6_k (streamed kernel against the grouped K-quant kernel): 24 pairs 17.5 + 16.3 against
//     28.0 + 20.5, 48 pairs 25.2 + 27.3 against 28.3 + 27.4, 64 pairs 30.0 + 33.7 against 35.1 + 32.9      -> 48
//   q2_k / q3_k (streamed against the any-codec kernel): 64 pairs 21.9 + 20.1 against 87.9 + 47.6 (q2_k), 256 pairs
//     67 + 61 against 154 + 76 and 126 + 76 against 200 + 106, 512 pairs 125 + 116 against 156 + 86        -> 256
//   q8_0 (streamed against the code-level grouped kernel): 64 pairs 38.8 + 28.0 against 55.7 + 36.8, 128 pairs
//     74.3 + 53.0 against 71.4 + 48.6                                                                        -> 64
//   iq4_nl / q4_0 / mxfp4 with K a multiple of 256 (streamed against code-level grouped): mxfp4 64 pairs 37.2 + 30.1
//     against 50.1 + 30.5, 96 pairs 54.5 + 43.7 against 58.3 + 37.3; q4_0 64 pairs 33.3 + 28.3 against 48.0 + 25.8 -> 64
//   iq4_xs / iq3_s / iq2_xxs (streamed against code-level grouped)                                          -> 64
//   nvfp4 with K a multiple of 256 (streamed against the any-codec kernel): 160 pairs 87 + 72 against 187 + 92,
//     256 pairs 138 + 113 against 213 + 105; the streamed kernel stops at 256 entries                       -> 256
//   the same codecs where the streamed kernel does not apply, and the other legacy / IQ codecs (code-level per-entry
//     kernel against code-level grouped): mxfp4 32 pairs 24.9 + 21.0 against 37.4 + 22.7, 64 pairs 41.2 + 36.1
//     against 53.8 + 34.1; iq2_xs 48 pairs 33.6 + 29.8 against 40.7 + 26.6                                  -> 48
//   nvfp4 there (against the any-codec kernel): 64 pairs 68 + 51 against 128 + 71, 128 pairs 127 + 96 against
//     158 + 96                                                                                               -> 128
// A family's figure is a crossover on that stack only.  What it stands for is carried to other stacks in three
// bounds, all of which a call must meet to run entry by entry:
//   pairs:             P <= the figure (more pairs were not measured to pay on any stack);
//   pairs per expert:  P / E <= figure / 128 (the saving of the grouped route grows with the pairs that share an
//                      expert: 32 experts of 3072 x 3072 in mxfp4, 64 pairs, 188 + 81 us entry by entry against
//                      118 + 68 grouped);
//   bytes read again:  (P - D(P, E)) x bytes of one expert's matrices <= the same expression on the reference stack
//                      at the figure, D(P, E) = E (1 - exp(-P / E)) being the distinct experts P uniform pairs hit:
//                      the bytes a call reads beyond the grouped route's are what it pays for skipping the prologue,
//                      and larger matrices reach that price with fewer repeated experts.
struct EntryFamily {
  int pairs;  // crossover on the reference stack
};
static constexpr EntryFamily kEntryKQuant{48}, kEntryLowK{256}, kEntryQ8{64}, kEntryNibStreamed{64}, kEntryIq{64},
    kEntryNvfp4Streamed{256}, kEntryCodes{48}, kEntryNvfp4Codes{128};
static constexpr int kEntryRefExperts = 128;
static constexpr double kEntryRefWeights = 768.0 * 2048.0;  // weights of one matrix of the reference stack

static double distinct_experts(double pairs, double experts) { return experts * (1.0 - std::exp(-pairs / experts)); }

static bool entry_by_entry_pays(EntryFamily f, int64_t P, int E, int N, int K) {
  if (P > f.pairs) return false;
  if (P * kEntryRefExperts > (int64_t)f.pairs * E) return false;
  // bytes per weight and the fused form's second matrix scale both sides alike
  const double again = ((double)P - distinct_experts((double)P, E)) * (double)N * (double)K;
  const double again_ref = (f.pairs - distinct_experts(f.pairs, kEntryRefExperts)) * kEntryRefWeights;
  return again <= again_ref;
}

// True when a call of P (token, expert) pairs is better served entry by entry than by the sorted, expert-grouped
// kernels.  entry_rows = activation rows per entry of the caller's per-entry fallback (1 for the MoE ops; gather_qmm's
// M): the per-entry kernels take one row per entry, the older K-quant ones up to eight.  stream_takes: the streamed
// gathered kernel accepts the call's shape and alignment; where it does not, the families measured on it keep the
// grouped route (the older per-entry kernels behind it are 2 - 4 x slower at these pair counts).
static bool per_entry_route(int64_t P, int entry_rows, bool has_bias, int glu, int act, int codec, int E, int N, int K,
                            bool stream_takes) {
  if (P <= 16) return false;  // the callers never reach the grouped route with so few pairs
  const bool grouped_codec = codec == KQ_Q4_K || codec == KQ_Q5_K || codec == KQ_Q6_K;
  const bool low_codec = codec == KQ_Q2_K || codec == KQ_Q3_K;  // their batched route is the any-codec kernel
  const bool iq_codec = codec == KQ_IQ4_XS || codec == KQ_IQ3_S || codec == KQ_IQ2_XXS;
  const bool q8 = codec == KQ_Q8_0;  // per-entry kernel: the streamed one; batched: the code-level grouped kernel
  // iq4_nl / q4_0 / mxfp4 / nvfp4 entries the streamed kernel takes (biases and swiglu_clamp included); the others
  // fall to the code-level rule below
  if ((codec == KQ_IQ4_NL || codec == KQ_Q4_0 || codec == KQ_MXFP4) && stream_takes && entry_rows == 1 &&
      entry_by_entry_pays(kEntryNibStreamed, P, E, N, K))
    return true;
  if (codec == KQ_NVFP4 && stream_takes && entry_rows == 1 && entry_by_entry_pays(kEntryNvfp4Streamed, P, E, N, K))
    return true;
  // the other codecs' per-entry kernel is the code-level one, which takes biases and every activation
  if (!grouped_codec && !low_codec && !iq_codec && !q8)
    return entry_rows == 1 && entry_by_entry_pays(codec == KQ_NVFP4 ? kEntryNvfp4Codes : kEntryCodes, P, E, N, K) &&
           kq_codes_gather_supported(1, N, K, codec);
  if (!stream_takes || has_bias || (glu && act == KQ_ACT_SWIGLU_CLAMP)) return false;
  if (grouped_codec) return entry_rows <= 8 && entry_by_entry_pays(kEntryKQuant, P, E, N, K);
  return entry_rows == 1 && entry_by_entry_pays(low_codec ? kEntryLowK : q8 ? kEntryQ8 : kEntryIq, P, E, N, K);
}

static int try_moe_grouped(const char* op, const void* x, const void* w, const void* w2, const uint32_t* idx,
                           const float* bias, const float* bias2, void* out, int T, int R, int E, int N, int K,
                           int64_t estride, int glu, int act, float limit, float alpha, int codec, int dtype, void* ws,
                           size_t ws_bytes, KqOutMap om, hipStream_t s, int entry_rows) {
  // entry_rows: activation rows per entry of the CALLER's per-entry fallback (1 for the MoE ops; gather_qmm's M)
  const int64_t P = (int64_t)T * R;
  if (P > 0x7fffffff) return KQ_ERR_UNSUPPORTED;
  // few entries: the per-entry kernels (the caller tries them next) beat the prologue + grouped-kernel pair
  const bool stream_takes = kq_gather_stream_takes(x, w, w2, (int)P, N, K, false, K, estride, false, codec);
  if (per_entry_route(P, entry_rows, bias || bias2, glu, act, codec, E, N, K, stream_takes)) return KQ_ERR_UNSUPPORTED;
  if (!kq_moe_grouped_supported((int)P, E, N, K, codec)) {
    // mxfp4: the wire blocks go into the block-scaled matrix instruction undecoded (kq_fp4.hip).  The plain op on
    // stacks whose K ends inside a 256-weight unit stays entry by entry on the streamed kernel up to 11 pairs (32
    // experts of 2880 x 2880: 8 pairs 14.6 us against 16.6 here, 16 pairs 24.9 against 20.3).
    if (codec == KQ_MXFP4 && !glu && (K & 255) && P < 12 && entry_rows == 1 && stream_takes) return KQ_ERR_UNSUPPORTED;
    if (kq_fp4_moe_supported((int)P, E, N, K, codec)) {
      const size_t need = kq_fp4_moe_workspace_bytes((int)P, E, glu ? T : (int)P, K);
      if (!ws || ws_bytes < need)
        return kq_set_error(KQ_ERR_WORKSPACE, "%s: workspace of %zu bytes required (got %zu)", op, need, ws ? ws_bytes : 0);
      const int rcf = kq_launch_fp4_moe(x, static_cast<const uint8_t*>(w), static_cast<const uint8_t*>(w2), idx, bias, bias2,
                                        out, (int)P, E, N, K, glu ? R : 1, estride, glu, act, limit, alpha, codec, dtype, ws,
                                        om, s);
      if (rcf != KQ_ERR_UNSUPPORTED) return rcf;
    }
    // legacy / IQ / fp4 codecs (biases and every activation included): code-level grouped kernel
    if (kq_codes_moe_supported((int)P, E, N, K, codec)) {
      const size_t need = kq_codes_moe_workspace_bytes((int)P, E, glu ? T : (int)P, K);
      if (!ws || ws_bytes < need)
        return kq_set_error(KQ_ERR_WORKSPACE, "%s: workspace of %zu bytes required (got %zu)", op, need, ws ? ws_bytes : 0);
      const int rcc = kq_launch_codes_moe(x, static_cast<const uint8_t*>(w), static_cast<const uint8_t*>(w2), idx, bias,
                                          bias2, out, (int)P, E, N, K, glu ? R : 1, estride, glu, act, limit, alpha, codec,
                                          dtype, ws, om, s);
      if (rcc != KQ_ERR_UNSUPPORTED) return rcc;
    }
    // q2_k / q3_k, and q4_k ... q6_k with biases or swiglu_clamp: the any-codec matrix-core path
    if (!kq_anymma_moe_supported((int)P, E, N, K, codec)) return KQ_ERR_UNSUPPORTED;
    const size_t need = kq_anymma_moe_workspace_bytes((int)P, E);
    if (!ws || ws_bytes < need)
      return kq_set_error(KQ_ERR_WORKSPACE, "%s: workspace of %zu bytes required (got %zu)", op, need, ws ? ws_bytes : 0);
    return kq_launch_anymma_moe(x, static_cast<const uint8_t*>(w), static_cast<const uint8_t*>(w2), idx, bias, bias2, out,
                                (int)P, E, N, K, glu ? R : 1, estride, glu, act, limit, alpha, codec, dtype, ws, om, s);
  }
  const int rows = glu ? T : (int)P;
  const size_t need = kq_moe_grouped_workspace_bytes(rows, (int)P, E, K);
  if (!ws || ws_bytes < need)
    return kq_set_error(KQ_ERR_WORKSPACE, "%s: workspace of %zu bytes required (got %zu)", op, need, ws ? ws_bytes : 0);
  return kq_launch_moe_grouped(x, static_cast<const uint8_t*>(w), static_cast<const uint8_t*>(w2), idx, out, rows,
                               (int)P, E, N, K, glu ? R : 1, estride, glu, act, limit, codec, dtype, ws, om, s);
}

// om: where the result of pair (t, r) goes; the exported op writes row t R + r of a 16-bit matrix
static int moe_glu_gather_impl(const void* x_dev, const void* gate_w_dev, const void* up_w_dev, const uint32_t* idx_dev,
                               const float* gate_bias_dev, const float* up_bias_dev, void* out_dev, int T, int R, int E,
                               int N, int K, int act, float limit, float alpha, int codec, int dtype, void* workspace_dev,
                               size_t workspace_bytes, KqOutMap om, void* stream) {
  const char* op = "moe_glu_gather_kq";
  int rc = check_moe(op, T, R, E, N, K, codec, dtype);
  if (rc) return rc;
  if (act < KQ_ACT_SILU || act > KQ_ACT_SWIGLU_CLAMP)
    return kq_set_error(KQ_ERR_INVALID, "%s: act must be 'silu', 'gelu', 'silu_limit' or 'swiglu_clamp'", op);
  if (act == KQ_ACT_SILU_LIMIT && !(limit > 0.f))
    return kq_set_error(KQ_ERR_INVALID, "%s: act 'silu_limit' requires limit > 0", op);
  const bool biased = gate_bias_dev || up_bias_dev;
  if (act == KQ_ACT_SWIGLU_CLAMP) {
    if (!gate_bias_dev || !up_bias_dev || !(limit > 0.f) || !(alpha > 0.f))
      return kq_set_error(KQ_ERR_INVALID, "%s: act 'swiglu_clamp' requires gate_bias, up_bias, limit > 0 and alpha > 0",
                          op);
    if (codec != KQ_MXFP4 && codec != KQ_NVFP4)
      return kq_set_error(KQ_ERR_INVALID, "%s: biased kernels are instantiated for mxfp4/nvfp4 only", op);
  } else if (biased) {
    return kq_set_error(KQ_ERR_INVALID, "%s: gate_bias/up_bias require act 'swiglu_clamp'", op);
  }
  if (T == 0 || R == 0 || N == 0) return KQ_OK;
  if (!x_dev || !gate_w_dev || !up_w_dev || !idx_dev || !out_dev)
    return kq_set_error(KQ_ERR_INVALID, "%s: null buffer", op);
  const int64_t estride = (int64_t)N * (K / kCodecs[codec].weights_per_block) * kCodecs[codec].bytes_per_block;
  {
    const int rcg = try_moe_grouped(op, x_dev, gate_w_dev, up_w_dev, idx_dev, gate_bias_dev, up_bias_dev, out_dev, T, R, E,
                                    N, K, estride, 1, act, limit, alpha, codec, dtype, workspace_dev, workspace_bytes, om,
                                    static_cast<hipStream_t>(stream));
    if (rcg != KQ_ERR_UNSUPPORTED) return rcg;
  }
  if (kq_stream_full_epilogue(codec) && (biased || act == KQ_ACT_SWIGLU_CLAMP)) {
    // fp4 stacks with biases / swiglu_clamp: the streamed kernel's gathered mode carries both
    const int rcs = kq_launch_gather_stream(x_dev, static_cast<const uint8_t*>(gate_w_dev),
                                            static_cast<const uint8_t*>(up_w_dev), nullptr, idx_dev, out_dev, T * R, N, K,
                                            R, K, estride, act, limit, alpha, gate_bias_dev, up_bias_dev, codec, dtype, E,
                                            om, static_cast<hipStream_t>(stream));
    if (rcs != KQ_ERR_UNSUPPORTED) return rcs;
  }
  if (!biased) {
    const int rct = kq_launch_gather_tuned(x_dev, static_cast<const uint8_t*>(gate_w_dev),
                                           static_cast<const uint8_t*>(up_w_dev), nullptr, idx_dev, out_dev, T * R, 1, N,
                                           K, R, K, estride, 1, act, limit, codec, dtype, E, om,
                                           static_cast<hipStream_t>(stream));
    if (rct != KQ_ERR_UNSUPPORTED) return rct;
  }
  {
    // legacy / IQ / fp4 stacks, one row per entry: the code-level skinny kernel, one entry per grid row
    const int rcc = kq_launch_codes_gather(x_dev, static_cast<const uint8_t*>(gate_w_dev),
                                  static_cast<const uint8_t*>(up_w_dev), nullptr, idx_dev, gate_bias_dev, up_bias_dev,
                                  out_dev, T * R, 1, N, K, R, K, estride, 1, act, limit, alpha, codec, dtype, E, om,
                                  static_cast<hipStream_t>(stream));
    if (rcc != KQ_ERR_UNSUPPORTED) return rcc;
  }
  return kq_launch_gather_generic(x_dev, static_cast<const uint8_t*>(gate_w_dev),
                                  static_cast<const uint8_t*>(up_w_dev), nullptr, idx_dev, gate_bias_dev, up_bias_dev,
                                  out_dev, T * R, 1, N, K, R, K, estride, 1, act, limit, alpha, codec, dtype, E, om,
                                  static_cast<hipStream_t>(stream));
}

int kq_moe_glu_gather(const void* x_dev, const void* gate_w_dev, const void* up_w_dev, const uint32_t* idx_dev,
                      const float* gate_bias_dev, const float* up_bias_dev, void* out_dev, int T, int R, int E, int N,
                      int K, int act, float limit, float alpha, int codec, int dtype, void* workspace_dev,
                      size_t workspace_bytes, void* stream) {
  return moe_glu_gather_impl(x_dev, gate_w_dev, up_w_dev, idx_dev, gate_bias_dev, up_bias_dev, out_dev, T, R, E, N, K, act,
                             limit, alpha, codec, dtype, workspace_dev, workspace_bytes, KQ_OUT_ROWS, stream);
}

static int gather_qmv_impl(const void* x_dev, const void* w_dev, const uint32_t* idx_dev, const float* bias_dev,
                           void* out_dev, int T, int R, int E, int N, int K, int codec, int dtype, void* workspace_dev,
                           size_t workspace_bytes, KqOutMap om, void* stream) {
  const char* op = "gather_qmv_kq";
  int rc = check_moe(op, T, R, E, N, K, codec, dtype);
  if (rc) return rc;
  if (bias_dev && codec != KQ_MXFP4 && codec != KQ_NVFP4)
    return kq_set_error(KQ_ERR_INVALID, "%s: biased kernels are instantiated for mxfp4/nvfp4 only", op);
  if (T == 0 || R == 0 || N == 0) return KQ_OK;
  if (!x_dev || !w_dev || !idx_dev || !out_dev) return kq_set_error(KQ_ERR_INVALID, "%s: null buffer", op);
  const int64_t estride = (int64_t)N * (K / kCodecs[codec].weights_per_block) * kCodecs[codec].bytes_per_block;
  {
    const int rcg = try_moe_grouped(op, x_dev, w_dev, nullptr, idx_dev, bias_dev, nullptr, out_dev, T, R, E, N, K, estride,
                                    0, 0, 0.f, 0.f, codec, dtype, workspace_dev, workspace_bytes, om,
                                    static_cast<hipStream_t>(stream));
    if (rcg != KQ_ERR_UNSUPPORTED) return rcg;
  }
  if (bias_dev && kq_stream_full_epilogue(codec)) {
    const int rcs = kq_launch_gather_stream(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, nullptr, idx_dev, out_dev,
                                            T * R, N, K, 1, K, estride, 0, 0.f, 1.0f, bias_dev, nullptr, codec, dtype, E, om,
                                            static_cast<hipStream_t>(stream));
    if (rcs != KQ_ERR_UNSUPPORTED) return rcs;
  }
  if (!bias_dev) {
    const int rct = kq_launch_gather_tuned(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, nullptr, idx_dev, out_dev,
                                           T * R, 1, N, K, 1, K, estride, 0, 0, 0.f, codec, dtype, E, om,
                                           static_cast<hipStream_t>(stream));
    if (rct != KQ_ERR_UNSUPPORTED) return rct;
  }
  {
    // legacy / IQ / fp4 stacks, one row per entry: the code-level skinny kernel, one entry per grid row
    const int rcc = kq_launch_codes_gather(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, nullptr, idx_dev, bias_dev,
                                  nullptr, out_dev, T * R, 1, N, K, 1, K, estride, 0, 0, 0.f, 0.f, codec, dtype, E, om,
                                  static_cast<hipStream_t>(stream));
    if (rcc != KQ_ERR_UNSUPPORTED) return rcc;
  }
  return kq_launch_gather_generic(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, nullptr, idx_dev, bias_dev,
                                  nullptr, out_dev, T * R, 1, N, K, 1, K, estride, 0, 0, 0.f, 0.f, codec, dtype, E, om,
                                  static_cast<hipStream_t>(stream));
}

int kq_gather_qmv(const void* x_dev, const void* w_dev, const uint32_t* idx_dev, const float* bias_dev, void* out_dev,
                  int T, int R, int E, int N, int K, int codec, int dtype, void* workspace_dev, size_t workspace_bytes,
                  void* stream) {
  return gather_qmv_impl(x_dev, w_dev, idx_dev, bias_dev, out_dev, T, R, E, N, K, codec, dtype, workspace_dev,
                         workspace_bytes, KQ_OUT_ROWS, stream);
}


// ------------------------------------------------------------------ sorted-segment prefill GEMM
int64_t kq_expert_tile_map_cap(int64_t rows, int n_experts) {
  if (rows < 1 || n_experts < 1) return 1;
  const int64_t c = rows / 64 + (rows < n_experts ? rows : (int64_t)n_experts);
  return c > 1 ? c : 1;
}

int kq_expert_tile_map(const uint32_t* indices_dev, int64_t rows, int n_experts, uint32_t* map_dev, int64_t cap,
                       uint32_t* counts_dev, void* stream) {
  const char* op = "expert_tile_map";
  if (rows < 1 || n_experts < 1)
    return kq_set_error(KQ_ERR_INVALID, "%s: indices must be non-empty and n_experts positive", op);
  if (rows > 0x7fffffff) return kq_set_error(KQ_ERR_INVALID, "%s: too many rows", op);
  if (cap < kq_expert_tile_map_cap(rows, n_experts))
    return kq_set_error(KQ_ERR_INVALID, "%s: map holds %lld tiles, %lld may be needed", op, (long long)cap,
                        (long long)kq_expert_tile_map_cap(rows, n_experts));
  if (!indices_dev || !map_dev || !counts_dev) return kq_set_error(KQ_ERR_INVALID, "%s: null buffer", op);
  return kq_launch_expert_tile_map(indices_dev, (int)rows, n_experts, map_dev, (int)(cap > 0x7fffffff ? 0x7fffffff : cap),
                                   counts_dev, static_cast<hipStream_t>(stream));
}

size_t kq_gather_qmm_seg_workspace_size(int64_t rows, int E, int N, int K, int codec, int dtype) {
  if (rows <= 0 || rows > 0x7fffffff) return 0;
  return align256((size_t)rows * 4) + kq_moe_workspace_size((int)rows, 1, E, N, K, 0, codec, dtype);
}

int kq_gather_qmm_seg(const void* x_dev, const void* w_dev, const uint32_t* map_dev, const uint32_t* counts_dev,
                      void* out_dev, int64_t rows, int64_t n_tiles, int E, int N, int K, int codec, int dtype,
                      void* workspace_dev, size_t workspace_bytes, void* stream) {
  const char* op = "gather_qmm_seg";
  if (rows < 0 || rows > 0x7fffffff || n_tiles > 0x7fffffff) return kq_set_error(KQ_ERR_INVALID, "%s: bad dimension", op);
  int rc = check_moe(op, (int)rows, 1, E, N, K, codec, dtype);
  if (rc) return rc;
  if (n_tiles < 1) return kq_set_error(KQ_ERR_INVALID, "%s: map must hold at least one tile row", op);
  if (rows == 0 || N == 0) return KQ_OK;
  if (!x_dev || !w_dev || !map_dev || !counts_dev || !out_dev) return kq_set_error(KQ_ERR_INVALID, "%s: null buffer", op);
  const size_t need = kq_gather_qmm_seg_workspace_size(rows, E, N, K, codec, dtype);
  if (!workspace_dev || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace_dev) & 255))
    return kq_set_error(KQ_ERR_WORKSPACE, "%s: a 256-byte aligned workspace of %zu bytes is required (got %zu)", op, need,
                        workspace_dev ? workspace_bytes : 0);
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint8_t* wsb = static_cast<uint8_t*>(workspace_dev);
  uint32_t* row_expert = reinterpret_cast<uint32_t*>(wsb);
  const size_t used = align256((size_t)rows * 4);
  // rows no tile covers carry an expert id outside the stack, which every kernel below leaves out
  rc = kq_launch_tiles_to_rows(map_dev, counts_dev, (int)n_tiles, (int)rows, E, 0xffffffffu, row_expert, s);
  if (rc) return rc;
  const int64_t estride = (int64_t)N * (K / kCodecs[codec].weights_per_block) * kCodecs[codec].bytes_per_block;
  if (kq_moe_workspace_size((int)rows, 1, E, N, K, 0, codec, dtype) > 0) {
    const int rcg = try_moe_grouped(op, x_dev, w_dev, nullptr, row_expert, nullptr, nullptr, out_dev, (int)rows, 1, E, N, K,
                                    estride, 0, 0, 0.f, 0.f, codec, dtype, wsb + used, workspace_bytes - used, KQ_OUT_ROWS, s);
    if (rcg != KQ_ERR_UNSUPPORTED) return rcg;
  }
  const int rct = kq_launch_gather_tuned(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, nullptr, row_expert, out_dev,
                                         (int)rows, 1, N, K, 1, K, estride, 0, 0, 0.f, codec, dtype, E, KQ_OUT_ROWS, s);
  if (rct != KQ_ERR_UNSUPPORTED) return rct;
  {
    // legacy / IQ / fp4 stacks, one row per entry: the code-level skinny kernel, one entry per grid row
    const int rcc = kq_launch_codes_gather(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, nullptr, row_expert, nullptr,
                                  nullptr, out_dev, (int)rows, 1, N, K, 1, K, estride, 0, 0, 0.f, 0.f, codec, dtype, E, KQ_OUT_ROWS, s);
    if (rcc != KQ_ERR_UNSUPPORTED) return rcc;
  }
  return kq_launch_gather_generic(x_dev, static_cast<const uint8_t*>(w_dev), nullptr, nullptr, row_expert, nullptr,
                                  nullptr, out_dev, (int)rows, 1, N, K, 1, K, estride, 0, 0, 0.f, 0.f, codec, dtype, E, KQ_OUT_ROWS, s);
}

}  // extern "C"

// ------------------------------------------------------------------ shared-expert / slot-mixing MoE ops
static bool shexp_combo_ok(int codec, int shexp_codec) {
  return codec_ok(codec) && codec_ok(shexp_codec) && (shexp_codec == codec || shexp_codec == KQ_Q6_K || shexp_codec == KQ_Q8_0);
}

size_t kq_moe_glu_gather_shexp_workspace_size(int T, int R, int E, int N, int K, int codec, int shexp_codec, int dtype) {
  if (T <= 0 || R <= 0) return 0;
  const size_t a = kq_moe_workspace_size(T, R, E, N, K, 1, codec, dtype);
  const size_t b = kq_moe_workspace_size(T, 1, 1, N, K, 1, shexp_codec, dtype);
  return align256((size_t)T * 4) + (a > b ? a : b);
}

int kq_moe_glu_gather_shexp(const void* x_dev, const void* gate_w_dev, const void* up_w_dev, const void* shexp_gate_w_dev,
                            const void* shexp_up_w_dev, const uint32_t* idx_dev, void* out_dev, int T, int R, int E, int N,
                            int K, int act, int codec, int shexp_codec, int dtype, void* workspace_dev,
                            size_t workspace_bytes, void* stream) {
  const char* op = "moe_glu_gather_shexp_kq";
  if (!shexp_combo_ok(codec, shexp_codec))
    return kq_set_error(KQ_ERR_INVALID, "%s: no fused kernel for this expert / shared-expert codec pair", op);
  if (act != KQ_ACT_SILU && act != KQ_ACT_GELU) return kq_set_error(KQ_ERR_INVALID, "%s: act must be 'silu' or 'gelu'", op);
  int rc = check_moe(op, T, R, E, N, K, codec, dtype);
  if (rc) return rc;
  rc = check_moe(op, T, 1, 1, N, K, shexp_codec, dtype);
  if (rc) return rc;
  if (T == 0 || N == 0) return KQ_OK;
  if (!shexp_gate_w_dev || !shexp_up_w_dev) return kq_set_error(KQ_ERR_INVALID, "%s: null buffer", op);
  const size_t need = kq_moe_glu_gather_shexp_workspace_size(T, R, E, N, K, codec, shexp_codec, dtype);
  if (!workspace_dev || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace_dev) & 255))
    return kq_set_error(KQ_ERR_WORKSPACE, "%s: 256-byte aligned workspace of %zu bytes required", op, need);
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint8_t* wsb = static_cast<uint8_t*>(workspace_dev);
  uint32_t* idx0 = reinterpret_cast<uint32_t*>(wsb);  // [T] zeros: the shared expert is a one-matrix stack
  uint8_t* sub = wsb + align256((size_t)T * 4);
  const size_t sub_bytes = workspace_bytes - align256((size_t)T * 4);
  if (R > 0) {
    // slot r of token t -> row t (R + 1) + r
    rc = moe_glu_gather_impl(x_dev, gate_w_dev, up_w_dev, idx_dev, nullptr, nullptr, out_dev, T, R, E, N, K, act, 0.f, 0.f,
                             codec, dtype, sub, sub_bytes, KqOutMap{R, R + 1, 0, 0}, stream);
    if (rc) return rc;
  }
  rc = kq_launch_pad_idx(nullptr, idx0, T, 1, s);  // S = 1: every entry is the padded slot, i.e. 0
  if (rc) return rc;
  // token t -> row t (R + 1) + R
  return moe_glu_gather_impl(x_dev, shexp_gate_w_dev, shexp_up_w_dev, idx0, nullptr, nullptr, out_dev, T, 1, 1, N, K, act,
                             0.f, 0.f, shexp_codec, dtype, sub, sub_bytes, KqOutMap{1, R + 1, R, 0}, stream);
}

// Decode-sized calls run as one kernel (a workgroup per output element, the slots spread over its waves): one token,
// or up to three when there is a shared expert (whose other form takes six launches against two); measured at
// 128 experts of 2048 x 768 q6_k, top-8: 14.4 against 14.1 us without and 15.5 against 25.2 us with a shared
// expert at one token.  Larger calls run the gathered matmul kernels into f32 slot rows and mix those.
#ifndef KQ_MIX_SINGLE_TOKENS
#define KQ_MIX_SINGLE_TOKENS 1
#endif
static bool mix_single_launch(int T, int S, bool shared) {
  return KQ_MIX_SINGLE_TOKENS > 0 && S <= 32 && T <= (shared ? 3 * KQ_MIX_SINGLE_TOKENS : KQ_MIX_SINGLE_TOKENS);
}

size_t kq_gather_qmv_mix_workspace_size(int T, int S, int E, int N, int K, int codec, int shexp_codec, int dtype) {
  if (T <= 0 || S <= 0) return 0;
  if (mix_single_launch(T, S, shexp_codec >= 0)) return 0;
  size_t fixed = align256((size_t)T * S * N * 4);  // f32 slot results
  size_t sub = kq_moe_workspace_size(T, S, E, N, K, 0, codec, dtype);
  if (shexp_codec >= 0) {
    fixed += align256((size_t)T * S * 4) + align256((size_t)T * 4) + align256((size_t)T * K * 2);
    const size_t b = kq_moe_workspace_size(T, 1, 1, N, K, 0, shexp_codec, dtype);
    if (b > sub) sub = b;
  }
  return fixed + sub;
}

static int gather_qmv_mix_impl(const char* op, const void* x_dev, const void* w_dev, const void* shexp_w_dev,
                               const float* bias_dev, const uint32_t* idx_dev, const float* scores_dev, void* out_dev, int T,
                               int S, int E, int N, int K, int codec, int shexp_codec, int dtype, void* workspace_dev,
                               size_t workspace_bytes, void* stream) {
  const bool shared = shexp_w_dev != nullptr;
  if (shared && !shexp_combo_ok(codec, shexp_codec))
    return kq_set_error(KQ_ERR_INVALID, "%s: no fused kernel for this expert / shared-expert codec pair", op);
  if (S < (shared ? 2 : 1)) return kq_set_error(KQ_ERR_INVALID, "%s: bad slot count", op);
  int rc = check_moe(op, T, S, E, N, K, codec, dtype);
  if (rc) return rc;
  if (shared) {
    rc = check_moe(op, T, 1, 1, N, K, shexp_codec, dtype);
    if (rc) return rc;
  }
  if (T == 0 || N == 0) return KQ_OK;
  if (!x_dev || !w_dev || !idx_dev || !scores_dev || !out_dev) return kq_set_error(KQ_ERR_INVALID, "%s: null buffer", op);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (mix_single_launch(T, S, shared)) {
    const int64_t expert_stride = (int64_t)N * (K / kCodecs[codec].weights_per_block) * kCodecs[codec].bytes_per_block;
    rc = kq_launch_gather_mix_generic(x_dev, static_cast<const uint8_t*>(w_dev), static_cast<const uint8_t*>(shexp_w_dev),
                                      idx_dev, scores_dev, bias_dev, out_dev, T, S, E, N, K, expert_stride, codec,
                                      shared ? shexp_codec : codec, dtype, s);
    return rc == KQ_OK ? KQ_OK : kq_set_error(rc, "%s: launch failed", op);
  }
  const size_t need = kq_gather_qmv_mix_workspace_size(T, S, E, N, K, codec, shared ? shexp_codec : -1, dtype);
  if (!workspace_dev || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace_dev) & 255))
    return kq_set_error(KQ_ERR_WORKSPACE, "%s: 256-byte aligned workspace of %zu bytes required", op, need);
  uint8_t* wsb = static_cast<uint8_t*>(workspace_dev);
  float* yf = reinterpret_cast<float*>(wsb);
  size_t o = align256((size_t)T * S * N * 4);
  const uint32_t* idx_all = idx_dev;
  uint32_t* idx0 = nullptr;
  void* xs = nullptr;
  if (shared) {
    uint32_t* idx2 = reinterpret_cast<uint32_t*>(wsb + o);
    o += align256((size_t)T * S * 4);
    idx0 = reinterpret_cast<uint32_t*>(wsb + o);
    o += align256((size_t)T * 4);
    xs = wsb + o;
    o += align256((size_t)T * K * 2);
    rc = kq_launch_pad_idx(idx_dev, idx2, T, S, s);  // the shared slot rides along as expert 0; overwritten below
    if (rc) return rc;
    idx_all = idx2;
  }
  uint8_t* sub = wsb + o;
  const size_t sub_bytes = workspace_bytes - o;
  // f32 slot results [T][S][N]
  rc = gather_qmv_impl(x_dev, w_dev, idx_all, bias_dev, yf, T, S, E, N, K, codec, dtype, sub, sub_bytes,
                       KqOutMap{1, 1, 0, 1}, stream);
  if (rc) return rc;
  if (shared) {
    // rows x[t][S - 1] -> dense [T][K], expert ids 0; the shared expert is a one-matrix stack
    rc = kq_launch_gather_rows(static_cast<const uint16_t*>(x_dev) + (size_t)(S - 1) * K, nullptr, nullptr, xs, idx0, T, 1, K,
                               (int64_t)S * K, s);
    if (rc) return rc;
    // token t -> slot row t S + S - 1, f32
    rc = gather_qmv_impl(xs, shexp_w_dev, idx0, nullptr, yf, T, 1, 1, N, K, shexp_codec, dtype, sub, sub_bytes,
                         KqOutMap{1, S, S - 1, 1}, stream);
    if (rc) return rc;
  }
  return kq_launch_mix_slots(yf, scores_dev, idx_dev, shared ? S - 1 : S, E, out_dev, T, S, N, dtype, s);
}

int kq_gather_qmv_mix(const void* x_dev, const void* w_dev, const void* shexp_w_dev, const uint32_t* idx_dev,
                      const float* scores_dev, void* out_dev, int T, int S, int E, int N, int K, int codec,
                      int shexp_codec, int dtype, void* workspace_dev, size_t workspace_bytes, void* stream) {
  return gather_qmv_mix_impl(shexp_w_dev ? "gather_qmv_mix_kq" : "gather_qmv_mix_ns_kq", x_dev, w_dev, shexp_w_dev, nullptr,
                             idx_dev, scores_dev, out_dev, T, S, E, N, K, codec, shexp_codec, dtype, workspace_dev,
                             workspace_bytes, stream);
}

int kq_gather_qmv_mix_bias(const void* x_dev, const void* w_dev, const float* bias_dev, const uint32_t* idx_dev,
                           const float* scores_dev, void* out_dev, int T, int S, int E, int N, int K, int codec, int dtype,
                           void* workspace_dev, size_t workspace_bytes, void* stream) {
  const char* op = "gather_qmv_mix_bias";
  if (!bias_dev) return kq_set_error(KQ_ERR_INVALID, "%s: null bias", op);
  return gather_qmv_mix_impl(op, x_dev, w_dev, nullptr, bias_dev, idx_dev, scores_dev, out_dev, T, S, E, N, K, codec, -1,
                             dtype, workspace_dev, workspace_bytes, stream);
}

int kq_quantize_dev_supported(int codec) { return codec_ok(codec) && kq_encode_dev_supported(codec) ? 1 : 0; }

int kq_quantize_dev(const void* w_dev, int w_dtype, const float* imatrix_dev, void* wire_dev, int64_t rows, int64_t K,
                    int codec, void* stream) {
  if (!codec_ok(codec)) return kq_set_error(KQ_ERR_INVALID, "quantize: unknown codec id %d", codec);
  if (!kq_encode_dev_supported(codec))
    return kq_set_error(KQ_ERR_UNSUPPORTED, "quantize: '%s' has no device encoder (use the host encoder)", kCodecs[codec].name);
  if (w_dtype != KQ_F32 && w_dtype != KQ_F16 && w_dtype != KQ_BF16)
    return kq_set_error(KQ_ERR_INVALID, "quantize: w must be float32, float16 or bfloat16");
  const int wpb = kCodecs[codec].weights_per_block;
  if (rows < 0 || K < 0 || K % wpb)
    return kq_set_error(KQ_ERR_INVALID, "quantize: K (%lld) is not a multiple of %d", (long long)K, wpb);
  if (rows == 0 || K == 0) return KQ_OK;
  if (!w_dev || !wire_dev) return kq_set_error(KQ_ERR_INVALID, "quantize: null buffer");
  return kq_launch_encode(w_dev, w_dtype, imatrix_dev, static_cast<uint8_t*>(wire_dev), rows, K, codec,
                          static_cast<hipStream_t>(stream));
}

int kq_mxfp4_packed_to_wire(const void* packed_dev, const void* scales_dev, void* wire_dev, int64_t num_blocks,
                            void* stream) {
  if (num_blocks < 0) return kq_set_error(KQ_ERR_INVALID, "mxfp4_packed_to_wire: negative block count");
  if (num_blocks == 0) return KQ_OK;
  if (!packed_dev || !scales_dev || !wire_dev) return kq_set_error(KQ_ERR_INVALID, "mxfp4_packed_to_wire: null buffer");
  if (reinterpret_cast<uintptr_t>(packed_dev) & 15)
    return kq_set_error(KQ_ERR_INVALID, "mxfp4_packed_to_wire: packed codes must be 16-byte aligned");
  return kq_launch_mxfp4_repack(packed_dev, scales_dev, wire_dev, num_blocks, 1, static_cast<hipStream_t>(stream));
}

int kq_mxfp4_wire_to_packed(const void* wire_dev, void* packed_dev, void* scales_dev, int64_t num_blocks, void* stream) {
  if (num_blocks < 0) return kq_set_error(KQ_ERR_INVALID, "mxfp4_wire_to_packed: negative block count");
  if (num_blocks == 0) return KQ_OK;
  if (!packed_dev || !scales_dev || !wire_dev) return kq_set_error(KQ_ERR_INVALID, "mxfp4_wire_to_packed: null buffer");
  if (reinterpret_cast<uintptr_t>(packed_dev) & 15)
    return kq_set_error(KQ_ERR_INVALID, "mxfp4_wire_to_packed: packed codes must be 16-byte aligned");
  return kq_launch_mxfp4_repack(packed_dev, scales_dev, const_cast<void*>(wire_dev), num_blocks, 0,
                                static_cast<hipStream_t>(stream));
}

int kq_moe_router_topk(const void* logits_dev, int dtype, int T, int E, int top_k, int norm_topk_prob, int shared_gate,
                       const float* per_expert_scale_dev, const float* bias_dev, int scoring, float scale,
                       uint32_t* indices_dev, float* scores_dev, void* stream) {
  const char* op = "moe_router_topk";
  if (scoring != 0 && scoring != 1) return kq_set_error(KQ_ERR_INVALID, "%s: scoring must be softmax or sqrtsoftplus", op);
  if (scoring == 1 && !norm_topk_prob) return kq_set_error(KQ_ERR_INVALID, "%s: sqrtsoftplus requires norm_topk_prob", op);
  if (dtype != KQ_F32 && dtype != KQ_F16 && dtype != KQ_BF16)
    return kq_set_error(KQ_ERR_INVALID, "%s: logits must be float32/float16/bfloat16", op);
  if (T < 0 || E < 1) return kq_set_error(KQ_ERR_INVALID, "%s: bad dimension", op);
  if (top_k < 1 || top_k > 16 || top_k > E) return kq_set_error(KQ_ERR_INVALID, "%s: top_k must be in [1, min(E, 16)]", op);
  if (E > 1024) return kq_set_error(KQ_ERR_INVALID, "%s: requires E <= 1024", op);
  if (T == 0) return KQ_OK;
  if (!logits_dev || !indices_dev || !scores_dev) return kq_set_error(KQ_ERR_INVALID, "%s: null buffer", op);
  return kq_launch_router_topk(logits_dev, dtype, T, E, top_k, norm_topk_prob, shared_gate, per_expert_scale_dev,
                               bias_dev, scoring, scale, indices_dev, scores_dev, static_cast<hipStream_t>(stream));
}
