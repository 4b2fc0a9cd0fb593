// Activations of feed-forwards without a gate branch, applied to one product, by code:
//   0  xielu with two stored numbers (p, q):  z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1 / 2 + softplus(q)) (exp(z) - 1 - z) + z / 2
//   1  gelu_tanh:  z / 2 (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))
// The input is one array of the model's type or float32 partial sums; the arithmetic is float32, the result is
// rounded once.  A thread takes four neighbouring elements (one 8- or 16-byte access) where the sizes allow.
#include "common.h"
#include "partials.h"

enum { QIL_PLAIN_XIELU = 0, QIL_PLAIN_GELU_TANH = 1 };

__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }

__device__ __forceinline__ float plain_act(float z, int act, float a_pos, float a_neg) {
  if (act == QIL_PLAIN_GELU_TANH) return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  return z > 0.f ? a_pos * z * z + 0.5f * z : a_neg * (expm1f(z) - z) + 0.5f * z;
}

template <typename TD, typename T, int V>
__global__ void plain_act_kernel(const TD* __restrict__ x, int splits, size_t split_stride, T* __restrict__ out,
                                 size_t total, int act, const float* __restrict__ params) {
  const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
  if (idx >= total) return;
  float a_pos = 0.f, a_neg = 0.f;
  if (act == QIL_PLAIN_XIELU) {
    a_pos = softplus_f(params[0]);
    a_neg = 0.5f + softplus_f(params[1]);
  }
  if (V == 4) {
    float4 z = ld4(x + idx);
    for (int s = 1; s < splits; ++s) {
      const float4 more = ld4(x + s * split_stride + idx);
      z.x += more.x, z.y += more.y, z.z += more.z, z.w += more.w;
    }
    st4(out + idx, make_float4(plain_act(z.x, act, a_pos, a_neg), plain_act(z.y, act, a_pos, a_neg),
                               plain_act(z.z, act, a_pos, a_neg), plain_act(z.w, act, a_pos, a_neg)));
  } else {
    st(out + idx, plain_act(parts_sum(x, idx, splits, split_stride), act, a_pos, a_neg));
  }
}

extern "C" {

// x: in_dtype QIL_BF16 [n, inner] or QIL_F32 [splits][n][inner] partial sums; params: float32 [2] for xielu.
int qil_plain_act(const void* x, int in_dtype, int splits, void* out, int n, int inner, int out_dtype, int act,
                  const float* params, hipStream_t s) {
  const size_t total = (size_t)n * inner;
  if (total == 0) return 0;
  if (splits < 1 || (in_dtype == QIL_BF16 && splits != 1) || act < 0 || act > 1 || (act == QIL_PLAIN_XIELU && !params))
    return -1;
  const bool vec = total % 4 == 0 && (((uintptr_t)x | (uintptr_t)out) % 16) == 0;
  const size_t threads = vec ? total / 4 : total;
  const unsigned blocks = (unsigned)((threads + 255) / 256);
#define QIL_PLAIN_LAUNCH(TD, T, V)                                                                                    \
  hipLaunchKernelGGL((plain_act_kernel<TD, T, V>), dim3(blocks), dim3(256), 0, s, (const TD*)x, splits, total, (T*)out, \
                     total, act, params)
#define QIL_PLAIN_CASE(TD, T) do { if (vec) QIL_PLAIN_LAUNCH(TD, T, 4); else QIL_PLAIN_LAUNCH(TD, T, 1); } while (0)
  if (out_dtype == QIL_F32) {
    if (in_dtype != QIL_F32) return -1;
    QIL_PLAIN_CASE(float, float);
  } else if (in_dtype == QIL_F32) {
    QIL_PLAIN_CASE(float, bf16_t);
  } else {
    QIL_PLAIN_CASE(bf16_t, bf16_t);
  }
#undef QIL_PLAIN_CASE
#undef QIL_PLAIN_LAUNCH
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
