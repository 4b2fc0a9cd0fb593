// Activations of feed-forwards without a gate branch, applied to one product, by code:
//   0  xielu with two stored numbers (p, q):  z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1 / 2 + softplus(q)) (exp(z) - 1 - z) + z / 2
//   1  gelu_tanh:  z / 2 (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))
// The input is one array of the model's type or float32 partial sums; the arithmetic is float32, the result is
// rounded once.
#include "common.h"
#include "partials.h"

enum { QIL_PLAIN_XIELU = 0, QIL_PLAIN_GELU_TANH = 1 };

__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }

__device__ __forceinline__ float plain_act(float z, int act, float a_pos, float a_neg) {
  if (act == QIL_PLAIN_GELU_TANH) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return z > 0.f ? a_pos * z * z + 0.5f * z : a_neg * (expm1f(z) - z) + 0.5f * z;
}

template <typename TD, typename T>
__global__ void plain_act_kernel(const TD* __restrict__ x, int splits, size_t split_stride, T* __restrict__ out,
                                 size_t total, int act, const float* __restrict__ params) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float a_pos = 0.f, a_neg = 0.f;
  if (act == QIL_PLAIN_XIELU) {
    a_pos = softplus_f(params[0]);
    a_neg = 0.5f + softplus_f(params[1]);
  }
  st(out + idx, plain_act(parts_sum(x, idx, splits, split_stride), act, a_pos, a_neg));
}

extern "C" {

// x: in_dtype QIL_BF16 [n, inner] or QIL_F32 [splits][n][inner] partial sums; params: float32 [2] for xielu.
int qil_plain_act(const void* x, int in_dtype, int splits, void* out, int n, int inner, int out_dtype, int act,
                  const float* params, hipStream_t s) {
  const size_t total = (size_t)n * inner;
  if (total == 0) return 0;
  if (splits < 1 || (in_dtype == QIL_BF16 && splits != 1) || act < 0 || act > 1 || (act == QIL_PLAIN_XIELU && !params))
    return -1;
  const unsigned blocks = (unsigned)((total + 255) / 256);
#define QIL_PLAIN_CASE(TD, T)                                                                                         \
  hipLaunchKernelGGL((plain_act_kernel<TD, T>), dim3(blocks), dim3(256), 0, s, (const TD*)x, splits, total, (T*)out,   \
                     total, act, params)
  if (out_dtype == QIL_F32) {
    if (in_dtype != QIL_F32) return -1;
    QIL_PLAIN_CASE(float, float);
  } else if (in_dtype == QIL_F32) {
    QIL_PLAIN_CASE(float, bf16_t);
  } else {
    QIL_PLAIN_CASE(bf16_t, bf16_t);
  }
#undef QIL_PLAIN_CASE
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
