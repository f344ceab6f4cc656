// Router top-k: expert scores from the router logits, the top_k picks and their mixing weights in one
// launch -- the inputs of the fused MoE ops.  One workgroup (256 threads) per token; the E <= 1024 scores
// live in LDS; every pick is a workgroup arg-max (largest score + bias, smallest index on ties) after
// which the winner leaves the pool.  All math in f32.  Semantics of the reference's kq_moe_router_topk
// (metal/mlx/backend/metal/kernels/kq_moe_glu_kq.h:1215-1358; op contract src/kquant_moe_glu.cpp:1366-1441).
#include "kq_decode.h"

namespace {

constexpr int RT_THREADS = 256;
constexpr int RT_WAVES = RT_THREADS / 64;
constexpr int RT_MAX_E = 1024;
constexpr int RT_MAX_R = 16;

struct RouterArgs {
  const void* logits;  // [T][E + shared]
  uint32_t* indices;   // [T][R]
  float* scores;       // [T][R + shared]
  const float* pes;    // per-expert scale [E] or null
  const float* bias;   // selection bias [E] or null
  int E, R, norm, shared, scoring;
  float scale;
};

template <int DT>
__device__ __forceinline__ float load_logit(const void* p, size_t i) {
  if constexpr (DT == KQ_F32) return static_cast<const float*>(p)[i];
  const uint16_t h = static_cast<const uint16_t*>(p)[i];
  return DT == KQ_F16 ? kq::h2f(h) : kq::bf162f(h);
}

template <int DT>
__global__ __launch_bounds__(RT_THREADS) void router_topk_kernel(RouterArgs a) {
  __shared__ float p[RT_MAX_E];
  __shared__ float red_v[RT_WAVES];
  __shared__ uint32_t red_i[RT_WAVES];
  __shared__ float win_v[RT_MAX_R];
  __shared__ uint32_t win_i[RT_MAX_R];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int E = a.E, R = a.R;
  const size_t row = (size_t)blockIdx.x * (E + a.shared);

  float gsum = 1.0f;
  if (a.scoring == 1) {
    for (int e = tid; e < E; e += RT_THREADS) {
      const float x = load_logit<DT>(a.logits, row + e);
      // stable softplus: max(x, 0) + log1p(exp(-|x|)), series where log(1 + z) loses bits
      const float z = expf(-fabsf(x));
      const float l1p = z < 1e-4f ? fmaf(-0.5f * z, z, z) : logf(1.0f + z);
      p[e] = sqrtf(fmaxf(x, 0.0f) + l1p);
    }
    __syncthreads();
  } else {
    float m = -INFINITY;
    for (int e = tid; e < E; e += RT_THREADS) m = fmaxf(m, load_logit<DT>(a.logits, row + e));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if (lane == 0) red_v[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red_v[0], red_v[1]), fmaxf(red_v[2], red_v[3]));
    __syncthreads();
    float s = 0.f;
    for (int e = tid; e < E; e += RT_THREADS) {
      const float v = expf(load_logit<DT>(a.logits, row + e) - m);
      p[e] = v;
      s += v;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off);
    if (lane == 0) red_v[wave] = s;
    __syncthreads();
    gsum = (red_v[0] + red_v[1]) + (red_v[2] + red_v[3]);
    __syncthreads();
  }

  for (int r = 0; r < R; r++) {
    float bv = -INFINITY;
    uint32_t bi = 0xffffffffu;
    for (int e = tid; e < E; e += RT_THREADS) {
      float v = p[e];
      if (a.bias) v += a.bias[e];
      if (v > bv || (v == bv && (uint32_t)e < bi)) {
        bv = v;
        bi = (uint32_t)e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off);
      const uint32_t oi = __shfl_xor(bi, off);
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    }
    if (lane == 0) {
      red_v[wave] = bv;
      red_i[wave] = bi;
    }
    __syncthreads();
    if (tid == 0) {
      float wv = red_v[0];
      uint32_t wi = red_i[0];
      for (int i = 1; i < RT_WAVES; i++) {
        if (red_v[i] > wv || (red_v[i] == wv && red_i[i] < wi)) {
          wv = red_v[i];
          wi = red_i[i];
        }
      }
      if (wi == 0xffffffffu) wi = 0;  // every value NaN: keep the index in range
      a.indices[(size_t)blockIdx.x * R + r] = wi;
      win_v[r] = p[wi];  // the emitted score is the unbiased one
      win_i[r] = wi;
      p[wi] = -INFINITY;
    }
    __syncthreads();
  }

  if (tid == 0) {
    float ps = 0.f;
    for (int r = 0; r < R; r++) ps += win_v[r];
    const float denom = a.norm ? (a.scoring == 1 ? ps + 1e-20f : ps) : gsum;
    float* srow = a.scores + (size_t)blockIdx.x * (R + a.shared);
    for (int r = 0; r < R; r++) {
      float sv = win_v[r] / denom;
      if (a.pes) sv *= a.pes[win_i[r]];
      srow[r] = sv * a.scale;
    }
    if (a.shared) srow[R] = 1.0f / (1.0f + expf(-load_logit<DT>(a.logits, row + E)));
  }
}

}  // namespace

int kq_launch_router_topk(const void* logits, int dtype, int T, int E, int top_k, int norm, int shared, const float* pes,
                          const float* bias, int scoring, float scale, uint32_t* indices, float* scores, hipStream_t s) {
  if (T <= 0) return KQ_OK;
  RouterArgs a{logits, indices, scores, pes, bias, E, top_k, norm, shared ? 1 : 0, scoring, scale};
  if (dtype == KQ_F32)
    hipLaunchKernelGGL(router_topk_kernel<KQ_F32>, dim3(T), dim3(RT_THREADS), 0, s, a);
  else if (dtype == KQ_F16)
    hipLaunchKernelGGL(router_topk_kernel<KQ_F16>, dim3(T), dim3(RT_THREADS), 0, s, a);
  else
    hipLaunchKernelGGL(router_topk_kernel<KQ_BF16>, dim3(T), dim3(RT_THREADS), 0, s, a);
  KQ_HIP_CHECK(hipGetLastError());
  return KQ_OK;
}
