// Device-side wire encoder behind kq_quantize_dev: the legacy 32-weight codecs and the K-quant superblock
// codecs, one thread per block running the very block encoders the host uses (kq_encode_blocks.h), so the
// bytes equal kq_quantize's.  The searches are sequential per block and keep their working arrays in
// per-lane scratch memory; the parallelism is across blocks (a 14336 x 4096 matrix has 229,376 superblocks).
// The reference's GPU encoders cover the same codecs (metal/.../kq_quantized_encode.h); its IQ encoders are
// CPU-only (src/kquant_ops.cpp:602-606), as here.
#include "kq_common.h"
#include "kq_decode.h"
#include "kq_encode_blocks.h"

namespace {

template <int C>
__device__ __forceinline__ void encode_block(const float* x, const float* im, uint8_t* b) {
  if constexpr (C == KQ_Q8_0) kqenc::enc_q8_0(x, b);
  else if constexpr (C == KQ_Q4_0) kqenc::enc_legacy<false, 4>(x, b);
  else if constexpr (C == KQ_Q4_1) kqenc::enc_legacy<true, 4>(x, b);
  else if constexpr (C == KQ_Q5_0) kqenc::enc_legacy<false, 5>(x, b);
  else if constexpr (C == KQ_Q5_1) kqenc::enc_legacy<true, 5>(x, b);
  else if constexpr (C == KQ_Q2_K) kqenc::enc_q2_k(x, im, b);
  else if constexpr (C == KQ_Q3_K) kqenc::enc_q3_k(x, im, b);
  else if constexpr (C == KQ_Q4_K) kqenc::enc_q45_k<4>(x, im, b);
  else if constexpr (C == KQ_Q5_K) kqenc::enc_q45_k<5>(x, im, b);
  else kqenc::enc_q6_k(x, im, b);
}

constexpr int ENC_THREADS = 64;

template <int C>
__global__ __launch_bounds__(ENC_THREADS) void encode_kernel(const void* __restrict__ w, int dtype,
                                                             const float* __restrict__ imatrix,
                                                             uint8_t* __restrict__ wire, int64_t nblocks,
                                                             int64_t blocks_per_row) {
  constexpr int WPB = kq_geom(C).wpb, BPB = kq_geom(C).bpb;
  const int64_t blk = (int64_t)blockIdx.x * ENC_THREADS + threadIdx.x;
  if (blk >= nblocks) return;
  float x[WPB];
  if (dtype == KQ_F32) {
    const float* src = static_cast<const float*>(w) + blk * WPB;
    for (int i = 0; i < WPB; i++) x[i] = src[i];
  } else {
    const uint16_t* src = static_cast<const uint16_t*>(w) + blk * WPB;
    for (int i = 0; i < WPB; i++) x[i] = dtype == KQ_F16 ? kq::h2f(src[i]) : __builtin_bit_cast(float, (uint32_t)src[i] << 16);
  }
  const float* im = (imatrix && WPB == 256) ? imatrix + (blk % blocks_per_row) * WPB : nullptr;
  uint8_t out[BPB];
  encode_block<C>(x, im, out);
  uint8_t* dst = wire + blk * BPB;
  for (int i = 0; i < BPB; i++) dst[i] = out[i];
}

template <int C>
int launch(const void* w, int dtype, const float* im, uint8_t* wire, int64_t nblocks, int64_t bpr, hipStream_t s) {
  const int64_t wgs = (nblocks + ENC_THREADS - 1) / ENC_THREADS;
  if (wgs > 0x7fffffff) return kq_set_error(KQ_ERR_INVALID, "quantize: tensor too large for one launch");
  hipLaunchKernelGGL(encode_kernel<C>, dim3((unsigned)wgs), dim3(ENC_THREADS), 0, s, w, dtype, im, wire, nblocks, bpr);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}

}  // namespace

bool kq_encode_dev_supported(int codec) {
  switch (codec) {
    case KQ_Q8_0: case KQ_Q4_0: case KQ_Q4_1: case KQ_Q5_0: case KQ_Q5_1:
    case KQ_Q2_K: case KQ_Q3_K: case KQ_Q4_K: case KQ_Q5_K: case KQ_Q6_K:
      return true;
  }
  return false;
}

int kq_launch_encode(const void* w, int dtype, const float* im, uint8_t* wire, int64_t rows, int64_t K, int codec,
                     hipStream_t s) {
  const KqGeom g = kq_geom(codec);
  const int64_t bpr = K / g.wpb, nblocks = rows * bpr;
  switch (codec) {
    case KQ_Q8_0: return launch<KQ_Q8_0>(w, dtype, im, wire, nblocks, bpr, s);
    case KQ_Q4_0: return launch<KQ_Q4_0>(w, dtype, im, wire, nblocks, bpr, s);
    case KQ_Q4_1: return launch<KQ_Q4_1>(w, dtype, im, wire, nblocks, bpr, s);
    case KQ_Q5_0: return launch<KQ_Q5_0>(w, dtype, im, wire, nblocks, bpr, s);
    case KQ_Q5_1: return launch<KQ_Q5_1>(w, dtype, im, wire, nblocks, bpr, s);
    case KQ_Q2_K: return launch<KQ_Q2_K>(w, dtype, im, wire, nblocks, bpr, s);
    case KQ_Q3_K: return launch<KQ_Q3_K>(w, dtype, im, wire, nblocks, bpr, s);
    case KQ_Q4_K: return launch<KQ_Q4_K>(w, dtype, im, wire, nblocks, bpr, s);
    case KQ_Q5_K: return launch<KQ_Q5_K>(w, dtype, im, wire, nblocks, bpr, s);
    case KQ_Q6_K: return launch<KQ_Q6_K>(w, dtype, im, wire, nblocks, bpr, s);
  }
  return KQ_ERR_UNSUPPORTED;
}
