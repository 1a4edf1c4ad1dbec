// A product's result as its consumers read it: one array of the model's type, or float32 partial sums of a product
// whose K was split over blocks, [splits][rows][width], added in split order.
#pragma once
#include "common.h"

template <typename TD>
__device__ __forceinline__ float parts_sum(const TD* __restrict__ base, size_t index, int splits, size_t stride) {
  float v = 0.f;
  for (int s = 0; s < splits; ++s) v += ld(base + s * stride + index);
  return v;
}
