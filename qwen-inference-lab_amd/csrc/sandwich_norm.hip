// A sub-layer output that is RMS-normed (weight of its own) before it joins the residual stream, fused with the
// norm that follows:
//     t = delta * rsqrt(mean(delta^2) + post_eps) * post_weight
//     x = stream[r] + t;  if (update) stream[r] = x
//     out[m] = round_T(round_T(x * rsqrt(mean(x^2) + eps)) * weight)
// r = rows ? rows[m] : m.  delta arrives in the model's type or as float32 partial sums [splits][rows][width] of a
// K-split product (added in split order), or as complete float32 rows (splits == 1), or as what a routed
// feed-forward leaves before its weighted sum (`Routed`: every (token, slot) pair's float32 row, the slots' weights and
// experts, and the feed-forward's input for the identity experts; the sum runs in slot order as `moe_combine_kernel`
// makes it).  Everything between the loads and the final rounding is float32: t is never rounded, and the stream keeps
// the unrounded sum.
// One block a row; the row of delta and then the row of x wait in LDS between the two passes each norm needs.
#include "common.h"

template <typename TD>
__device__ __forceinline__ float load_sum(const TD* __restrict__ base, size_t index, int splits, size_t stride) {
  float v = 0.f;
  for (int s0 = 0; s0 < splits; s0 += 8) {
    float part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) part[u] = s0 + u < splits ? ld(base + (s0 + u) * stride + index) : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) v += part[u];
  }
  return v;
}

struct Routed {
  const float* pairs;                                      // [tokens * top][width]; null: delta is an array
  const float* weights;                                    // [tokens][top]
  const int* chosen;                                       // [tokens][top]
  const void* input;                                       // [tokens][width], the out type's elements
  int top, experts;
};

template <typename TD, typename T>
__global__ void post_norm_add_norm_kernel(float* __restrict__ stream, const TD* __restrict__ delta, int splits,
                                          size_t split_stride, const float* __restrict__ post_weight, float post_eps,
                                          const int* __restrict__ rows, const float* __restrict__ weight,
                                          T* __restrict__ out, int width, float eps, int update, Routed routed) {
  extern __shared__ float row[];                       // [width]
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t r = rows ? (size_t)rows[m] : (size_t)m;
  float* x = stream + r * width;
  float squares = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float d = 0.f;
    if (routed.pairs) {
      for (int slot = 0; slot < routed.top; ++slot) {
        const size_t pair = r * routed.top + slot;
        const float value = routed.chosen[pair] >= routed.experts ? ld(reinterpret_cast<const T*>(routed.input) + r * width + i)
                                                                  : routed.pairs[pair * width + i];
        d += routed.weights[pair] * value;
      }
    } else {
      d = load_sum(delta, r * width + i, splits, split_stride);
    }
    row[i] = d;
    squares += d * d;
  }
  squares = block_sum(squares, scratch);
  const float post = rsqrtf(squares / (float)width + post_eps);
  float sum = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {     // (a thread meets its own elements again: no barrier)
    const float v = x[i] + row[i] * post * post_weight[i];
    if (update) x[i] = v;
    row[i] = v;
    sum += v * v;
  }
  sum = block_sum(sum, scratch);
  const float rstd = rsqrtf(sum / (float)width + eps);
  T* y = out + (size_t)m * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) st(y + i, round_to<T>(row[i] * rstd) * weight[i]);
}

extern "C" {

// delta_dtype QIL_BF16 (one array, splits == 1) or QIL_F32 ([splits][delta_rows][width]).  out_dtype: type of `out`.
static int post_norm_launch(float* stream, const void* delta, int delta_dtype, int splits, int delta_rows,
                            const float* post_weight, float post_eps, const int* rows, const float* weight, void* out,
                            int n_out, int width, float eps, int update, int out_dtype, Routed routed, hipStream_t s) {
  if (n_out == 0) return 0;
  if ((!delta && !routed.pairs) || !post_weight || !weight || splits < 1 || (delta_dtype == QIL_BF16 && splits != 1) || width < 1 ||
      (size_t)width * sizeof(float) > 96 * 1024)
    return -1;
  const size_t stride = (size_t)delta_rows * width, lds = (size_t)width * sizeof(float);
  const int threads = width >= 4096 ? 1024 : width >= 1024 ? 512 : width >= 256 ? 256 : 64;
#define QIL_SANDWICH(TD, T)                                                                                          \
  do {                                                                                                               \
    if (lds > 48 * 1024) {                                                                                           \
      hipError_t e = hipFuncSetAttribute((const void*)post_norm_add_norm_kernel<TD, T>,                              \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                      \
      if (e != hipSuccess) return (int)e;                                                                            \
    }                                                                                                                \
    hipLaunchKernelGGL((post_norm_add_norm_kernel<TD, T>), dim3(n_out), dim3(threads), lds, s, stream,               \
                       (const TD*)delta, splits, stride, post_weight, post_eps, rows, weight, (T*)out, width, eps,   \
                       update, routed);                                                                              \
  } while (0)
  if (out_dtype == QIL_F32) {
    if (delta_dtype != QIL_F32) return -1;
    QIL_SANDWICH(float, float);
  } else if (delta_dtype == QIL_F32) {
    QIL_SANDWICH(float, bf16_t);
  } else {
    QIL_SANDWICH(bf16_t, bf16_t);
  }
#undef QIL_SANDWICH
  QIL_RETURN_LAUNCH_STATUS();
}

int qil_post_norm_add_norm(float* stream, const void* delta, int delta_dtype, int splits, int delta_rows,
                           const float* post_weight, float post_eps, const int* rows, const float* weight, void* out,
                           int n_out, int width, float eps, int update, int out_dtype, hipStream_t s) {
  const Routed none = {};
  return post_norm_launch(stream, delta, delta_dtype, splits, delta_rows, post_weight, post_eps, rows, weight, out, n_out,
                          width, eps, update, out_dtype, none, s);
}

// The same with the weighted sum of a routed feed-forward's pairs in the place of delta: pairs float32
// [tokens * top][width], weights and chosen [tokens][top], input [tokens][width] of the out type (what an identity
// expert, an index from `experts` on, passes).
int qil_post_norm_add_norm_routed(float* stream, const float* pairs, const float* weights, const int* chosen,
                                  const void* input, int top, int experts, const float* post_weight, float post_eps,
                                  const int* rows, const float* weight, void* out, int n_out, int width, float eps,
                                  int update, int out_dtype, hipStream_t s) {
  if (!pairs || !weights || !chosen || !input || top < 1) return -1;
  const Routed routed = {pairs, weights, chosen, input, top, experts};
  return post_norm_launch(stream, nullptr, out_dtype == QIL_F32 ? QIL_F32 : QIL_BF16, 1, 0, post_weight, post_eps, rows,
                          weight, out, n_out, width, eps, update, out_dtype, routed, s);
}

}  // extern "C"
