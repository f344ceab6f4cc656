// Fused gate/up epilogue of the MoE GLU ops, shared by the generic and the tuned kernels
// (metal/mlx/backend/metal/kernels/kq_moe_glu_kq.h:34-60 of the reference).
#pragma once

#include "kq_common.h"
#include "kq_decode.h"

namespace kq {
__device__ __forceinline__ float glu_epilogue(int act, float g, float u, float limit, float alpha) {
  if (act == KQ_ACT_GELU) {
    const float g3 = 0.044715f * g * g * g;
    const float t = tanhf(0.7978845608028654f * (g + g3));
    return (0.5f * g * (1.0f + t)) * u;
  }
  if (act == KQ_ACT_SWIGLU_CLAMP) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    const float sig = 1.0f / (1.0f + expf(-alpha * g));
    return (g * sig) * (u + 1.0f);
  }
  if (act == KQ_ACT_SILU_LIMIT) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  const float sig = 1.0f / (1.0f + expf(-g));
  return (g * sig) * u;
}

// The same epilogue on the hardware's exp2 and reciprocal instructions (about 1 ulp each; the result is rounded
// to a 16-bit type right after): the grouped kernels run it on up to sixteen accumulators per lane, where the
// range-reduced expf, the IEEE division and tanhf of the form above are a fifth of the kernel's vector work.
__device__ __forceinline__ float fast_sigmoid(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}
__device__ __forceinline__ float glu_epilogue_fast(int act, float g, float u, float limit, float alpha) {
  if (act == KQ_ACT_GELU) {
    const float g3 = 0.044715f * g * g * g;
    const float z = 0.7978845608028654f * (g + g3);
    // 0.5 (1 + tanh z) = sigmoid(2 z)
    return (g * fast_sigmoid(2.0f * z)) * u;
  }
  if (act == KQ_ACT_SWIGLU_CLAMP) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return (g * fast_sigmoid(alpha * g)) * (u + 1.0f);
  }
  if (act == KQ_ACT_SILU_LIMIT) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  return (g * fast_sigmoid(g)) * u;
}

__device__ __forceinline__ int out_row(const KqOutMap& m, int p) {
  return m.in == m.out ? p + m.off : (p / m.in) * m.out + (p % m.in) + m.off;
}
// one rounding to the activation dtype (DT = KQ_F16 / KQ_BF16), or the f32 value itself
template <int DT>
__device__ __forceinline__ void store_result(void* y, const KqOutMap& m, size_t off, float v) {
  if (m.f32)
    static_cast<float*>(y)[off] = v;
  else
    static_cast<uint16_t*>(y)[off] = DT == KQ_F16 ? f2f16(v) : f2bf16(v);
}

}  // namespace kq
