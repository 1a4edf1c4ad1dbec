// Activations of gated feed-forwards over the gate and up halves of one product, by code:
//   0  silu(g) * u
//   1  g' = min(g, limit), u' = clamp(u, -limit, limit):  g' * sigmoid(alpha * g') * (u' + 1)
// The halves of a row of gate_up [n, 2 inner] are stacked (gate columns first) or interleaved in tiles of 16 columns.
#include "common.h"
#include "partials.h"
#include "gated_act.h"

template <typename TD, typename T>
__global__ void gated_act_kernel(const TD* __restrict__ gate_up, int splits, size_t split_stride, T* __restrict__ out,
                                 int inner, size_t total, int interleaved, int act, float limit, float alpha) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t n = idx / inner;
  const int i = (int)(idx - n * inner);
  const size_t at = n * 2 * (size_t)inner + (interleaved ? (size_t)(i >> 4) * 32 + (i & 15) : (size_t)i);
  const float g = parts_sum(gate_up, at, splits, split_stride);
  const float u = parts_sum(gate_up, at + (interleaved ? 16 : inner), splits, split_stride);
  st(out + idx, gated_act(g, u, act, limit, alpha));
}

extern "C" {

// gate_up: in_dtype QIL_BF16 [n, 2 inner] or QIL_F32 [splits][n][2 inner] partial sums.
int qil_gated_act(const void* gate_up, int in_dtype, int splits, void* out, int n, int inner, int out_dtype,
                  int interleaved, int act, float limit, float alpha, hipStream_t s) {
  const size_t total = (size_t)n * inner;
  if (total == 0) return 0;
  if (splits < 1 || (in_dtype == QIL_BF16 && splits != 1) || (interleaved && inner % 16) || act < 0 || act > 1) return -1;
  const size_t stride = (size_t)n * 2 * inner;
  const unsigned blocks = (unsigned)((total + 255) / 256);
#define QIL_ACT_CASE(TD, T)                                                                                            \
  hipLaunchKernelGGL((gated_act_kernel<TD, T>), dim3(blocks), dim3(256), 0, s, (const TD*)gate_up, splits, stride,      \
                     (T*)out, inner, total, interleaved, act, limit, alpha)
  if (out_dtype == QIL_F32) {
    if (in_dtype != QIL_F32) return -1;
    QIL_ACT_CASE(float, float);
  } else if (in_dtype == QIL_F32) {
    QIL_ACT_CASE(float, bf16_t);
  } else {
    QIL_ACT_CASE(bf16_t, bf16_t);
  }
#undef QIL_ACT_CASE
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
