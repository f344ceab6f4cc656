// Fused gate/up epilogue of the MoE GLU ops, shared by the generic and the tuned kernels
// (metal/mlx/backend/metal/kernels/kq_moe_glu_kq.h:34-60 of the reference).
#pragma once

#include "kq_common.h"

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

}  // namespace kq
