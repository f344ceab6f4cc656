/* kq_oracle.h -- C interface of the CPU oracle (test infrastructure, never shipped).
 * dtype codes: 0 = float32, 1 = float16, 2 = bfloat16 (half types passed as uint16 bits). */
#ifndef KQ_ORACLE_H
#define KQ_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define KQ_ORACLE_NUM_CODECS 21
typedef struct {
  const char* name;
  int weights_per_block, bytes_per_block, bits;
  int has_matmul, has_encode, has_nax, requires_imatrix;
} kq_oracle_codec_t;

enum { KQ_ORACLE_ACT_SILU = 0, KQ_ORACLE_ACT_GELU = 1, KQ_ORACLE_ACT_SILU_LIMIT = 2, KQ_ORACLE_ACT_SWIGLU_CLAMP = 3 };

int kq_oracle_codec_id(const char* name);
const kq_oracle_codec_t* kq_oracle_codec(int id);
void kq_oracle_set_threads(int n);
int kq_oracle_threads(void);

float kq_oracle_f16_to_f32(uint16_t h);
uint16_t kq_oracle_f32_to_f16(float f);
float kq_oracle_bf16_to_f32(uint16_t h);
uint16_t kq_oracle_f32_to_bf16(float f);

int kq_oracle_dequantize(int codec, const uint8_t* w, void* out, uint64_t num_weights, int out_dtype);
int kq_oracle_qmm_f32(int codec, float* out, const float* xf, const uint8_t* w, int M, int N, int K, int transpose);
int kq_oracle_qmm(int codec, void* out, const void* x, const uint8_t* w, int M, int N, int K, int transpose, int dtype);
int kq_oracle_gather_qmm(int codec, void* out, const void* x, const uint8_t* w, const uint32_t* lhs,
                         const uint32_t* rhs, int B, int M, int N, int K, int64_t x_batch_stride,
                         int64_t w_expert_stride_bytes, int transpose, int dtype);
float kq_oracle_glu_epilogue(int act, float g, float u, float limit, float alpha);
int kq_oracle_moe_glu_gather(int codec, void* out, const void* x, const uint8_t* gate_w, const uint8_t* up_w,
                             const uint32_t* idx, const float* gate_bias, const float* up_bias, int T, int R,
                             int N, int K, int act, float limit, float alpha, int dtype);
int kq_oracle_gather_qmv(int codec, void* out, const void* x, const uint8_t* w, const uint32_t* idx,
                         const float* bias, int T, int R, int N, int K, int dtype);
/* moe_glu_gather with the shared expert as slot R: out [T][R + 1][N]. */
int kq_oracle_moe_glu_gather_shexp(int codec, int shexp_codec, void* out, const void* x, const uint8_t* gate_w,
                                   const uint8_t* up_w, const uint8_t* shexp_gate_w, const uint8_t* shexp_up_w,
                                   const uint32_t* idx, int T, int R, int N, int K, int act, int dtype);
/* out[t][:] = T(sum_s scores[t][s] * x[t][s][:] . W_s^T); shexp_w != NULL: idx [T][S-1], slot S-1 uses shexp_w. */
int kq_oracle_gather_qmv_mix(int codec, int shexp_codec, void* out, const void* x, const uint8_t* w,
                             const uint8_t* shexp_w, const uint32_t* idx, const float* scores, int T, int S, int N,
                             int K, int dtype);
/* Router: scores (softmax = 0, sqrt(softplus) = 1) over E logit columns, top_k by score (+ bias), smallest
 * index first on ties; logits [T][E + shared] in `dtype`, indices [T][top_k], scores f32 [T][top_k + shared]. */
int kq_oracle_router_topk(const void* logits, int dtype, int T, int E, int top_k, int norm, int shared,
                          const float* per_expert_scale, const float* bias, int scoring, float scale,
                          uint32_t* indices, float* scores);
#ifdef __cplusplus
}
#endif
#endif
