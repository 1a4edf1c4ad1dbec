// The gate functions of gated feed-forwards, shared by the activation kernel and by product kernels that apply the
// activation in their epilogue.  Everything is float32.
#pragma once
#include "common.h"

enum { QIL_ACT_SILU = 0, QIL_ACT_CLAMPED = 1 };

//   QIL_ACT_SILU     g * sigmoid(g) * u
//   QIL_ACT_CLAMPED  g' = min(g, limit), u' = clamp(u, -limit, limit):  g' * sigmoid(alpha * g') * (u' + 1)
__device__ __forceinline__ float gated_act(float g, float u, int act, float limit, float alpha) {
  if (act == QIL_ACT_CLAMPED) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return (g / (1.f + expf(-alpha * g))) * (u + 1.f);
  }
  return (g / (1.f + expf(-g))) * u;
}
