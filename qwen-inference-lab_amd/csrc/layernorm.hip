// Norms fused with a scaled residual add: layer norm (mean removed, weight, optional bias) and RMS norm.
// The residual stream is float32; statistics, the sum and the weight product are float32, the result is rounded once.
#include "common.h"
#include "partials.h"

template <typename TD>
__device__ __forceinline__ float row_value(const float* __restrict__ x, const TD* __restrict__ delta, size_t at, int i,
                                           int splits, size_t stride, float delta_scale) {
  float v = x[i];
  if (delta) v = v + delta_scale * parts_sum(delta, at + i, splits, stride);
  return v;
}

// One block per output row m; r = rows ? rows[m] : m.
//   v = stream[r] + delta_scale * delta[r];  if (update) stream[r] = v;
//   CENTRE: out[m] = (v - mean(v)) / sqrt(mean((v - mean(v))^2) + eps) * weight (+ bias)
//   else:   out[m] = v / sqrt(mean(v^2) + eps) * weight (+ bias)
template <typename TD, typename T, int CENTRE>
__global__ void add_norm_kernel(float* __restrict__ stream, const TD* __restrict__ delta, int splits, size_t split_stride,
                                float delta_scale, const int* __restrict__ rows, const float* __restrict__ weight,
                                const float* __restrict__ bias, T* __restrict__ out, int width, float eps, int update) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const size_t r = rows ? (size_t)rows[m] : (size_t)m;
  float* x = stream + r * width;
  const size_t at = r * width;
  float sum = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = row_value(x, delta, at, i, splits, split_stride, delta_scale);
    if (delta && update) x[i] = v;
    sum += v;
  }
  const TD* later = update ? nullptr : delta;          // after the update the stream holds the sum already
  float mean = 0.f;
  if (CENTRE) mean = block_sum(sum, scratch) / (float)width;
  float squares = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float c = row_value(x, later, at, i, splits, split_stride, delta_scale) - mean;
    squares += c * c;
  }
  squares = block_sum(squares, scratch);
  const float scale = 1.f / sqrtf(squares / (float)width + eps);
  T* y = out + (size_t)m * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float c = row_value(x, later, at, i, splits, split_stride, delta_scale) - mean;
    st(y + i, c * scale * weight[i] + (bias ? bias[i] : 0.f));
  }
}

extern "C" {

// delta: null, or the sub-layer output to add: delta_dtype QIL_BF16 (one array, splits == 1) or QIL_F32
// ([splits][delta_rows][width] partial sums).  centre: 1 layer norm, 0 RMS norm.  bias: float32 [width] or null.
// out_dtype: type of `out`.
int qil_add_norm(float* stream, const void* delta, int delta_dtype, int splits, int delta_rows, float delta_scale,
                 const int* rows, const float* weight, const float* bias, void* out, int n_out, int width, float eps, int update, int centre,
                 int out_dtype, hipStream_t s) {
  if (n_out == 0) return 0;
  if (width < 1 || splits < 1 || (delta_dtype == QIL_BF16 && splits != 1)) return -1;
  const size_t stride = (size_t)delta_rows * width;
  const int threads = width >= 2048 ? 512 : width >= 512 ? 256 : width >= 128 ? 128 : 64;
#define QIL_NORM_LAUNCH(TD, T, C)                                                                                    \
  hipLaunchKernelGGL((add_norm_kernel<TD, T, C>), dim3(n_out), dim3(threads), 0, s, stream, (const TD*)delta, splits, \
                     stride, delta_scale, rows, weight, bias, (T*)out, width, eps, update)
#define QIL_NORM_CASE(TD, T) do { if (centre) QIL_NORM_LAUNCH(TD, T, 1); else QIL_NORM_LAUNCH(TD, T, 0); } while (0)
  if (out_dtype == QIL_F32) {
    if (delta_dtype != QIL_F32) return -1;
    QIL_NORM_CASE(float, float);
  } else if (delta_dtype == QIL_F32) {
    QIL_NORM_CASE(float, bf16_t);
  } else {
    QIL_NORM_CASE(bf16_t, bf16_t);
  }
#undef QIL_NORM_CASE
#undef QIL_NORM_LAUNCH
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
