// An operand that is either one array of the model's type or float32 partial sums of a product split over K
// ([splits][rows][columns], added here in split order): what a consumer of ``ops.linear``'s results reads.
#pragma once
#include "common.h"

struct Operand {
  const void* data;
  int code;            // QIL_F32 | QIL_BF16
  int splits;          // float32 only; 1 for a plain array
  size_t stride;       // elements between two splits
};

__device__ __forceinline__ float operand_at(const Operand& x, size_t index) {
  if (x.code == QIL_BF16) return bf16_to_f32(reinterpret_cast<const bf16_t*>(x.data)[index]);
  const float* base = reinterpret_cast<const float*>(x.data) + index;
  float v = 0.f;
  for (int s0 = 0; s0 < x.splits; s0 += 4) {             // four splits' loads in flight; the additions stay in split order
    float part[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) part[k] = s0 + k < x.splits ? base[(size_t)(s0 + k) * x.stride] : 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) v += part[k];
  }
  return v;
}
