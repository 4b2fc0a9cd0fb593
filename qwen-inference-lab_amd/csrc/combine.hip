// Small float32 steps between the products of a mixer or at the model's end:
//   scaled sum     out[n, c] = a_scale * a[n, c] + b_scale * b[n, c]      (two branches joined; float32 result)
//   sigmoid gate   out[n, c] = x[n, c] * sigmoid(source[n, offset + c])   (an output gate made from the mixer's input)
//   soft cap       x <- cap * tanh(x / cap), in place                     (the logits' cap)
// a, b and source are arrays of the model's type or float32 partial sums of a product split over K (operand.h).
#include "common.h"
#include "operand.h"

__global__ void scaled_sum_kernel(Operand a, Operand b, float a_scale, float b_scale, float* __restrict__ out, size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) out[i] = a_scale * operand_at(a, i) + b_scale * operand_at(b, i);
}

template <typename T>
__global__ void sigmoid_gate_kernel(const T* __restrict__ x, Operand source, int source_columns, int offset,
                                    T* __restrict__ out, int n, int columns) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)n * columns) return;
  const size_t row = i / columns, c = i - row * columns;
  const float g = operand_at(source, row * source_columns + offset + c);
  st(out + i, ld(x + i) / (1.f + expf(-g)));
}

__global__ void soft_cap_kernel(float* __restrict__ x, float cap, size_t count) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" {

// a, b: [n * columns] elements each (code QIL_F32 with `splits` partial sums, or QIL_BF16 with one array).
int qil_scaled_sum(const void* a, int a_code, int a_splits, const void* b, int b_code, int b_splits, float a_scale,
                   float b_scale, float* out, int n, int columns, hipStream_t s) {
  const size_t count = (size_t)n * columns;
  if (count == 0) return 0;
  if (a_splits < 1 || b_splits < 1 || (a_code == QIL_BF16 && a_splits != 1) || (b_code == QIL_BF16 && b_splits != 1)) return -1;
  const Operand oa{a, a_code, a_splits, count}, ob{b, b_code, b_splits, count};
  hipLaunchKernelGGL(scaled_sum_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, oa, ob, a_scale, b_scale,
                     out, count);
  QIL_RETURN_LAUNCH_STATUS();
}

// x, out: [n, columns] of dtype (out may be x); source: [n, source_columns], the gate's logits from column `offset` on.
int qil_sigmoid_gate(const void* x, const void* source, int source_code, int source_splits, int source_columns, int offset,
                     void* out, int n, int columns, int dtype, hipStream_t s) {
  const size_t count = (size_t)n * columns;
  if (count == 0) return 0;
  if (source_splits < 1 || (source_code == QIL_BF16 && source_splits != 1) || offset < 0 ||
      offset + columns > source_columns) return -1;
  const Operand src{source, source_code, source_splits, (size_t)n * source_columns};
  const dim3 grid((unsigned)((count + 255) / 256));
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, grid, dim3(256), 0, s, (const float*)x, src, source_columns, offset,
                       (float*)out, n, columns);
  else
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, grid, dim3(256), 0, s, (const bf16_t*)x, src, source_columns, offset,
                       (bf16_t*)out, n, columns);
  QIL_RETURN_LAUNCH_STATUS();
}

int qil_soft_cap(float* x, float cap, size_t count, hipStream_t s) {
  if (count == 0) return 0;
  if (!(cap > 0.f)) return -1;
  hipLaunchKernelGGL(soft_cap_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, x, cap, count);
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
