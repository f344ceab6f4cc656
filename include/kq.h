/*
 * kq.h -- C ABI of libkq: GGUF K-quant / legacy / IQ / fp4 wire-byte kernels for AMD
 * Instinct MI355X (gfx950).
 *
 * Conventions
 *   - every `*_dev` pointer is DEVICE memory on the current HIP device; the caller
 *     owns every buffer (inputs, outputs, workspace) and keeps it alive until the
 *     stream has run the call;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); device
 *     entry points enqueue work and return without synchronising;
 *   - return value 0 = success, negative = error (KQ_ERR_*); the message of the last
 *     error on the calling thread is returned by kq_last_error();
 *   - dtype codes: KQ_F32 / KQ_F16 / KQ_BF16.  Wire bytes are the unchanged GGUF block
 *     layout (uint8), rows packed back to back: bytes_per_row = K / weights_per_block
 *     * bytes_per_block;
 *   - there is no CPU fallback: a call on a machine without a usable GPU fails with
 *     KQ_ERR_HIP.
 */
#ifndef KQ_H
#define KQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KQ_NUM_CODECS 21

enum { KQ_F32 = 0, KQ_F16 = 1, KQ_BF16 = 2 };
enum { KQ_ACT_SILU = 0, KQ_ACT_GELU = 1, KQ_ACT_SILU_LIMIT = 2, KQ_ACT_SWIGLU_CLAMP = 3 };
enum {
  KQ_OK = 0,
  KQ_ERR_INVALID = -1,     /* bad argument (maps to the reference's std::invalid_argument) */
  KQ_ERR_UNSUPPORTED = -2, /* valid request this build has no kernel for (std::runtime_error) */
  KQ_ERR_HIP = -3,         /* HIP runtime failure (std::runtime_error) */
  KQ_ERR_WORKSPACE = -4    /* workspace missing or too small */
};

/* Replaces struct KQuantCodec, reference src/kquant_codec.h:10-19. */
typedef struct kq_codec_info {
  char name[16];
  int weights_per_block;
  int bytes_per_block;
  int bits;
  int has_matmul_kernel;
  int has_encode;
  int has_nax_kernel;
  int requires_imatrix;
} kq_codec_info;

/* Registry, in the reference's canonical order.
 * Replaces codec_by_name / codec_names, reference src/kquant_codec.cpp:12-57. */
int kq_codec_count(void);
int kq_codec_id(const char* name);               /* -1 if unknown */
int kq_codec_get(int codec, kq_codec_info* out); /* KQ_ERR_INVALID if out of range */
/* Replaces codec_has_moe_glu, reference src/kquant_moe_glu.cpp:792-798. */
int kq_codec_has_moe_glu(int codec);

const char* kq_last_error(void);
const char* kq_version(void);

/* out[i] = T(decode(w)[i]) for i < num_weights (num_weights a whole number of blocks).
 * f32 results are bit-identical to the reference's scalar decoders; f16/bf16 are one
 * round-to-nearest-even of that f32 value.
 * Replaces kquant_dequantize_parallel<T>, reference src/kquant_cpu_decode.h:37-52 /
 * src/kquant_cpu_decode.cpp:1189-1207 (called by KQuantDequantize::eval_cpu,
 * src/kquant_dequantize.cpp:59-91). */
int kq_dequantize(const void* w_dev, void* out_dev, uint64_t num_weights, int codec, int out_dtype,
                  void* stream);

/* y[M,N] = x[M,K] . W^T  (transpose != 0, W decodes to [N,K])  or  x[M,K] . W (transpose == 0,
 * W decodes to [K,N]).  x and y have dtype `dtype` (KQ_F16 / KQ_BF16; the op layer casts f32
 * activations to bf16 first, as the reference does); accumulation is f32 with one rounding
 * to `dtype`.  Workspace: kq_qmm_workspace_size bytes of device memory (may be 0).  With transpose == 0 the
 * workspace is optional (f32 partial sums of a K range cut over the grid, for calls with few output tiles;
 * without it the call runs uncut), the weights are split into two bf16 terms (16 significant bits) and the
 * op is the reference's qmm_n, src/kquant_matmul.cpp:455-527.
 * Replaces kquant_qmm_cpu<T>, reference src/kquant_cpu_decode.h:54-70 /
 * src/kquant_cpu_decode.cpp:1209-1359 (called by KQuantMatmul::eval_cpu,
 * src/kquant_matmul.cpp:1104-1164). */
size_t kq_qmm_workspace_size(int M, int N, int K, int transpose, int codec, int dtype);
int kq_qmm(const void* x_dev, const void* w_dev, void* y_dev, int M, int N, int K, int transpose,
           int codec, int dtype, void* workspace_dev, size_t workspace_bytes, void* stream);

/* kq_qmm for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): transpose is implied, and the workspace is a buffer of
 * KQ_NOALLOC_SCRATCH_BYTES that lives inside the library's code object on every GPU (no hipMalloc, hipFree
 * or other allocating call is made).  A call that cannot run in that size (the prefill GEMM of q4_k / q5_k /
 * q6_k keeps its converted activations there: about 2.2 * M * K bytes) is rejected with KQ_ERR_WORKSPACE; the
 * optional part of kq_qmm_workspace_size (partial sums of a K range cut over the grid) is used when it fits
 * and left out otherwise.  All calls on one GPU share that GPU's buffer: calls that overlap in time on the same
 * GPU (different streams or threads) race; the buffer keeps the last call's contents, and the kernels write
 * every element they later read, so nothing needs clearing between calls.  The first call of a shape on a
 * device looks the buffer's address up and sets kernel attributes: make one eager call of each shape before
 * capturing it into a HIP graph.
 * No counterpart in the reference. */
#define KQ_NOALLOC_SCRATCH_BYTES (4u << 20)
int kq_qmm_noalloc(const void* x_dev, const void* w_dev, void* y_dev, int M, int N, int K, int codec, int dtype,
                   void* stream);

/* Decode-only matvec with the layer bias fused in: y[n] = T(x . W[n]^T + float(bias[n])), one activation row,
 * bias [N] in the activation dtype, q8_0 only (as wired in the reference).
 * Replaces KQuantQmvBias (op quantized_matmul_qmv_bias), reference src/kquant_ops.cpp:185-270. */
int kq_qmv_bias(const void* x_dev, const void* w_dev, const void* bias_dev, void* y_dev, int N, int K, int codec,
                int dtype, void* stream);

/* Tuning hook without a counterpart in the reference: workgroup tile of the prefill GEMM.  64 = 64
 * activation rows x 128 weight rows, 128 = 128 x 128, 256 = 64 x 256 on eight waves with two LDS stages
 * (q4_k only; other codecs fall back to automatic), 512 = 128 x 256 on eight waves with 128-row wave tiles and
 * direct-to-LDS loads (q2_k / q3_k / q4_k / q5_k / iq4_xs; 513 = the same kernel as 128 x 128 on four waves),
 * 1024 = 256 x 256 on eight waves with 256-row wave tiles on one accumulator set (q4_k / q5_k / q6_k) for every
 * column tile, 1025 = the 128 x 256 form of that kernel (q6_k only; other codecs fall back to automatic); for
 * q8_0 / q4_0 / q4_1 / q5_0 / q5_1 / iq4_nl / mxfp4 / nvfp4 and the codebook codecs (iq1 / iq2 / iq3), 1024 / 1025 force the 256- / 128-row form of their tall-tile kernels on any
 * shape of 128 rows or more and 64 keeps them on the any-codec kernel;
 * anything else restores the automatic choice (q4_k / q5_k / q6_k with 256 rows or more: the 256 x 256 kernel on the
 * column tiles that fill whole rounds of one workgroup per CU, a 128 x 256 kernel on the rest; q6_k matrices of
 * few tiles stay on the 64-row kernel).
 * Process-wide, not thread-safe. */
void kq_set_gemm_tile_rows(int rows);
/* Tuning hook without a counterpart in the reference: which skinny-M kernel dense calls use.
 * 0 = default: the streamed kernel (direct-to-LDS weight loads) for up to 8 activation rows of every codec it
 * has a unit for (q2_k ... q6_k, iq4_xs, iq3_s, iq2_xxs, q8_0, q4_0, iq4_nl, mxfp4, nvfp4); calls it declines (a
 * split plan without workspace, unaligned activations) fall to the older K-quant kernels: decoupled-wave up to
 * 4 rows, diagonal for 5 - 8.  The other values pin one of those older kernels for q2_k ... q6_k so that tests
 * reach them: 1 = workgroup-synchronous kernel (the one multi-row gathered entries use), 2 = decoupled-wave
 * kernel always, 3 = decoupled-wave kernel with two-superblock units, 4 = diagonal kernel wherever K allows it;
 * 5 = same as 0.  Process-wide, not thread-safe. */
void kq_set_skinny_variant(int variant);

/* out[b] = x[lhs[b]] . W[rhs[b]]^T for b < B; x batches are [M,K] matrices
 * `x_batch_stride` elements apart, experts are [N, bytes_per_row] wire matrices
 * `w_expert_stride_bytes` apart (64-bit, so strided / >2 GiB stacks work); out is
 * [B, M, N] dense.  `E` = number of matrices in the stack (entries whose rhs index is >= E are
 * skipped by the batched path and must not occur).  `rhs_sorted` != 0 promises rhs is
 * non-decreasing.  With a workspace of kq_gather_qmm_workspace_size bytes and more than 16 output
 * rows (B * M) the entries are grouped by expert on the device, so an expert's wire bytes are
 * streamed once per 32 rows instead of once per entry; without one every entry is computed on its own.
 * Replaces KQuantGatherQMM::eval_cpu, reference src/kquant_gather.cpp:470-746
 * (kquant_qmm_cpu_batch, src/kquant_cpu_decode.cpp:1361-1527). */
size_t kq_gather_qmm_workspace_size(int B, int M, int E, int N, int K, int transpose, int codec, int dtype);
int kq_gather_qmm(const void* x_dev, const void* w_dev, const uint32_t* lhs_idx_dev,
                  const uint32_t* rhs_idx_dev, void* out_dev, int B, int M, int E, int N, int K,
                  int64_t x_batch_stride, int64_t w_expert_stride_bytes, int transpose, int rhs_sorted,
                  int codec, int dtype, void* workspace_dev, size_t workspace_bytes, void* stream);

/* Device workspace (bytes, 256-byte aligned, may be 0) of the two MoE ops below: `glu` != 0 for
 * kq_moe_glu_gather, 0 for kq_gather_qmv.  The batched path sorts the pairs by expert and keeps converted
 * activations there.  It takes calls of more than 16 (token, expert) pairs unless the per-entry kernels are ahead,
 * which a codec family's measured figure decides (48 pairs for q4_k / q5_k / q6_k and the legacy / fp4 / other IQ
 * stacks, 64 for iq4_xs / iq3_s / iq2_xxs / q8_0 / iq4_nl / q4_0 / mxfp4 on the streamed kernel, 256 for q2_k / q3_k /
 * nvfp4), carried to the call's stack as three bounds: that many pairs, that many pairs per 128 experts, and no more
 * bytes read again than on the stack the figure was measured on (128 experts of 2048 x 768); mxfp4 stacks go to the
 * block-scaled kernel from 8 pairs where K is no multiple of 256.  The reference allocates its own
 * temporaries inside eval_gpu (src/kquant_moe_glu.cpp:277-382); here the caller owns them. */
size_t kq_moe_workspace_size(int T, int R, int E, int N, int K, int glu, int codec, int dtype);

/* out[t,r,:] = T(act(x[t] . G_e^T (+gb_e), x[t] . U_e^T (+ub_e))), e = idx[t,r]; f32 throughout,
 * one rounding.  x [T,K], gate/up stacks [E,N,bytes_per_row] dense, idx [T,R] uint32,
 * biases f32 [E,N] or NULL, out [T,R,N].
 * Replaces KQuantMoEGLUKQ (op moe_glu_gather_kq), reference src/kquant_moe_glu.cpp:1070-1157,
 * dispatch :277-329, epilogue metal/mlx/backend/metal/kernels/kq_moe_glu_kq.h:34-60. */
int kq_moe_glu_gather(const void* x_dev, const void* gate_w_dev, const void* up_w_dev,
                      const uint32_t* idx_dev, const float* gate_bias_dev, const float* up_bias_dev,
                      void* out_dev, int T, int R, int E, int N, int K, int act, float limit, float alpha,
                      int codec, int dtype, void* workspace_dev, size_t workspace_bytes, void* stream);

/* out[t,r,:] = T(x[t,r,:] . W_e^T (+ bias_e)), e = idx[t,r].  x [T,R,K], w [E,N,bytes_per_row].
 * Replaces KQuantGatherQMVKQ (op gather_qmv_kq), reference src/kquant_moe_glu.cpp:1159-1210,
 * dispatch :331-382, kernels kq_moe_glu_kq.h:933-999. */
int kq_gather_qmv(const void* x_dev, const void* w_dev, const uint32_t* idx_dev, const float* bias_dev,
                  void* out_dev, int T, int R, int E, int N, int K, int codec, int dtype, void* workspace_dev,
                  size_t workspace_bytes, void* stream);

/* Tile map of expert-sorted routing indices, built on the device without a host sync: map uint32 [cap][3] rows
 * of (expert, first row, rows <= 64) cutting every expert's run of rows into 64-row tiles of which only the last
 * may be partial, in row order; counts[0] = number of valid tiles (slots past it are left untouched).
 * cap = kq_expert_tile_map_cap(rows, n_experts) = max(rows / 64 + min(n_experts, rows), 1) bounds the tile
 * count.  Rows whose index is >= n_experts belong to no tile.
 * Replaces expert_tile_map (KQuantExpertTileMap), reference src/kquant.h:102-109, src/kquant_ops.cpp:422-447,
 * src/kquant_gather.cpp:1010-1042; host-built equivalent mlx_kquant/nn.py:33-47. */
int64_t kq_expert_tile_map_cap(int64_t rows, int n_experts);
int kq_expert_tile_map(const uint32_t* indices_dev, int64_t rows, int n_experts, uint32_t* map_dev, int64_t cap,
                       uint32_t* counts_dev, void* stream);

/* Sorted-segment GEMM for MoE prefill: for every valid tile (expert e, first row r, n rows) of the map,
 * out[r : r + n] = T(x[r : r + n] . W_e^T).  x [rows, K] sorted by expert, w [E, N, bytes_per_row] dense,
 * map uint32 [n_tiles][3] and counts uint32 [1] as kq_expert_tile_map writes them (or host-built; tiles of at
 * most 64 rows that never span experts and cover every row once).  Rows no valid tile covers hold unspecified
 * values afterwards.  The tiles are turned into a per-row expert list on the device and the rows run through
 * the expert-grouped kernels of kq_gather_qmv, so the workspace is kq_gather_qmm_seg_workspace_size bytes.
 * Replaces gather_qmm_seg (KQuantGatherQMMSeg), reference src/kquant.h:111-128, src/kquant_ops.cpp:466-548,
 * src/kquant_gather.cpp:1044-1092. */
size_t kq_gather_qmm_seg_workspace_size(int64_t rows, int E, int N, int K, int codec, int dtype);
int kq_gather_qmm_seg(const void* x_dev, const void* w_dev, const uint32_t* map_dev, const uint32_t* counts_dev,
                      void* out_dev, int64_t rows, int64_t n_tiles, int E, int N, int K, int codec, int dtype,
                      void* workspace_dev, size_t workspace_bytes, void* stream);

/* out[t, r < R] as kq_moe_glu_gather (act silu or gelu, no biases); out[t, R] = the same GLU of x[t] against
 * the block's shared expert, two single [N, bytes_per_row] matrices in `shexp_codec` (the expert codec, or
 * q6_k / q8_0).  out [T, R + 1, N].  The workspace (kq_moe_glu_gather_shexp_workspace_size bytes, 256-byte
 * aligned) is required.
 * Replaces KQuantMoEGLUShexpKQ (op moe_glu_gather_shexp_kq), reference src/kquant_moe_glu.cpp:1212-1272. */
size_t kq_moe_glu_gather_shexp_workspace_size(int T, int R, int E, int N, int K, int codec, int shexp_codec, int dtype);
int kq_moe_glu_gather_shexp(const void* x_dev, const void* gate_w_dev, const void* up_w_dev,
                            const void* shexp_gate_w_dev, const void* shexp_up_w_dev, const uint32_t* idx_dev,
                            void* out_dev, int T, int R, int E, int N, int K, int act, int codec, int shexp_codec,
                            int dtype, void* workspace_dev, size_t workspace_bytes, void* stream);

/* Down projection with the routing mix folded in: out[t, :] = T(sum_s scores[t, s] * (x[t, s, :] . W_s^T)),
 * f32 accumulation over the S slots, one rounding.  x [T, S, K], scores f32 [T, S], out [T, N].
 * shexp_w_dev != NULL: idx is [T, S - 1], slot S - 1 multiplies the shared expert's single matrix (codec
 * `shexp_codec`: the expert codec, or q6_k / q8_0) -- op gather_qmv_mix_kq; shexp_w_dev == NULL: idx is
 * [T, S] and every slot gathers from the stack -- op gather_qmv_mix_ns_kq (pass shexp_codec = -1 to the
 * size query).  Decode-sized calls (one token; up to three with a shared expert; S <= 32) run as one kernel and
 * need no workspace (the size query returns 0, any pointer is accepted); larger calls need the 256-byte aligned
 * workspace.  Entries whose expert id is >= E add nothing.
 * Replaces KQuantGatherQMVMixKQ / KQuantGatherQMVMixNSKQ, reference src/kquant_moe_glu.cpp:1274-1364. */
size_t kq_gather_qmv_mix_workspace_size(int T, int S, int E, int N, int K, int codec, int shexp_codec, int dtype);
int kq_gather_qmv_mix(const void* x_dev, const void* w_dev, const void* shexp_w_dev, const uint32_t* idx_dev,
                      const float* scores_dev, void* out_dev, int T, int S, int E, int N, int K, int codec,
                      int shexp_codec, int dtype, void* workspace_dev, size_t workspace_bytes, void* stream);

/* kq_gather_qmv_mix without a shared expert and with the expert bias (f32 [E, N]) added to every slot's product
 * before the mix: out[t, :] = T(sum_s scores[t, s] * (x[t, s, :] . W_s^T + bias_s)).  mxfp4 / nvfp4 stacks only, as
 * kq_gather_qmv's bias.  Workspace: kq_gather_qmv_mix_workspace_size(..., shexp_codec = -1, ...).
 * Replaces gather_qmv_mix_bias (packed-layout op, reference src/kquant.h:321-333) once the stack is in wire form
 * (kq_mxfp4_packed_to_wire). */
int kq_gather_qmv_mix_bias(const void* x_dev, const void* w_dev, const float* bias_dev, const uint32_t* idx_dev,
                           const float* scores_dev, void* out_dev, int T, int S, int E, int N, int K, int codec,
                           int dtype, void* workspace_dev, size_t workspace_bytes, void* stream);

/* mxfp4 between the MLX packed layout (uint32 codes [.., K/8], eight sequential 4-bit codes per word, 16-byte
 * aligned; e8m0 scale bytes [.., K/32] in a tensor of their own) and the GGUF wire (17-byte blocks: scale byte,
 * then code j in the low and code j + 16 in the high nibble of byte j).  num_blocks = number of 32-weight
 * blocks.  The packed-layout ops of the reference (moe_glu_gather, gather_qmv_bias, gather_qmv_mix_bias,
 * src/kquant.h:291-333) are served by converting a stack once and calling the wire-form ops. */
int kq_mxfp4_packed_to_wire(const void* packed_dev, const void* scales_dev, void* wire_dev, int64_t num_blocks,
                            void* stream);
int kq_mxfp4_wire_to_packed(const void* wire_dev, void* packed_dev, void* scales_dev, int64_t num_blocks,
                            void* stream);

/* Router: expert scores over the E logit columns (scoring 0 = softmax, 1 = sqrt(softplus(x))), the top_k
 * largest by score (+ bias[e] when given; smallest index first on ties) and their mixing weights:
 * score / (sum of the picked scores (+ 1e-20 for scoring 1) if norm_topk_prob else the softmax sum)
 * * per_expert_scale[e] * scale.  With shared_gate logits are [T, E + 1] and sigmoid(column E) is
 * appended: scores [T, top_k + 1].  logits in `dtype` (0 / 1 / 2 = f32 / f16 / bf16), all math f32;
 * indices uint32 [T, top_k], scores f32.  E <= 1024, top_k <= min(E, 16); scoring 1 needs norm_topk_prob.
 * Replaces KQuantMoERouterTopK (op moe_router_topk), reference src/kquant_moe_glu.cpp:1366-1441, kernel
 * metal/mlx/backend/metal/kernels/kq_moe_glu_kq.h:1215-1358. */
int kq_moe_router_topk(const void* logits_dev, int dtype, int T, int E, int top_k, int norm_topk_prob,
                       int shared_gate, const float* per_expert_scale_dev, const float* bias_dev, int scoring,
                       float scale, uint32_t* indices_dev, float* scores_dev, void* stream);

/* HOST function: wire = encode(w[rows, K] f32) (imatrix f32 [K] or NULL), rows * bytes_per_row
 * bytes written to wire_host.  Runs on the calling thread's CPU cores like the reference's
 * encoder (which is CPU-only for the IQ codecs and serial).
 * Replaces kquant_quantize_dispatch, reference src/kquant_cpu_encode.h:25-31 /
 * src/kquant_cpu_encode.cpp:824-859 (op quantize, src/kquant_ops.cpp:550-631). */
int kq_quantize(const float* w_host, const float* imatrix_host, uint8_t* wire_host, int64_t rows, int64_t K,
                int codec);

/* The same encoding on the device for the codecs the reference encodes on the GPU (q8_0, q4_0/1, q5_0/1,
 * q2_k ... q6_k; KQ_ERR_UNSUPPORTED for the IQ codecs, whose encoder is host-only there and here):
 * w_dev [rows, K] in `w_dtype` (0 / 1 / 2 = f32 / f16 / bf16), imatrix_dev f32 [K] or NULL, wire_dev
 * rows * bytes_per_row bytes.  One thread per block runs the host encoder's code, so the bytes equal
 * kq_quantize's on the same values.  kq_quantize_dev_supported tells which codecs qualify.
 * Replaces KQuantQuantize::eval_gpu (kernels metal/mlx/backend/metal/kernels/kq_quantized_encode.h),
 * reference src/kquant_ops.cpp:550-631. */
int kq_quantize_dev_supported(int codec);
int kq_quantize_dev(const void* w_dev, int w_dtype, const float* imatrix_dev, void* wire_dev, int64_t rows,
                    int64_t K, int codec, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KQ_H */
