// A sub-layer's output that joins the float32 residual stream as its norm, scaled per channel, and optionally a
// weighted average over the results of all layers so far:
//
//   z      = norm(y) * w + b                 norm: (y - mean) / sqrt(mean((y - mean)^2) + eps) (CENTRE), or
//                                            y / sqrt(mean(y^2) + eps); w, b, the channel scale ls: float32 or absent
//   X      = stream + ls * z                 the layer's result so far
//   depth > 0:  history[depth - 1] = X;  stream = sum_(j < depth) mix[j] * history[j]   (the new X is the last term)
//   else:       stream = X
//   out    = stream rounded to T             (if asked for: what the next sub-layer's products read)
//
// y: one array of the model's type or float32 partial sums [splits][rows][width]; everything else is float32.  In
// the place of y a routed feed-forward's pairs can stand (`Routed`): y is then the weighted sum of a token's pairs in
// slot order, made while the row is loaded (an identity expert's pair is the token's own input).
// One block per row; the row of y is held in LDS between the passes (statistics in two passes: the variance is that
// of the deviations); a thread takes four neighbouring elements at a time where the rows allow.
#include "common.h"
#include "partials.h"

struct RoutedPairs {
  const float* pairs;                                      // [tokens * top][width]; null: y is an array
  const float* weights;                                    // [tokens][top]
  const int* chosen;                                       // [tokens][top]
  const void* input;                                       // [tokens][width] of input_dtype
  int input_dtype, top, experts;
};

// V elements of a token's weighted sum of pairs, from element i of its row.
template <int V>
__device__ __forceinline__ void routed_row(const RoutedPairs& routed, size_t token, int width, int i, float* v) {
#pragma unroll
  for (int e = 0; e < V; ++e) v[e] = 0.f;
  for (int slot = 0; slot < routed.top; ++slot) {
    const size_t pair = token * routed.top + slot;
    const float w = routed.weights[pair];
    float in[V];
    if (routed.chosen[pair] >= routed.experts) {           // an identity expert passes the token's input
      const size_t from = token * width + i;
#pragma unroll
      for (int e = 0; e < V; ++e)
        in[e] = routed.input_dtype == QIL_F32 ? reinterpret_cast<const float*>(routed.input)[from + e]
                                              : ld(reinterpret_cast<const bf16_t*>(routed.input) + from + e);
    } else if (V == 4) {
      const float4 a = ld4(routed.pairs + pair * width + i);
      in[0] = a.x, in[1] = a.y, in[2] = a.z, in[3] = a.w;
    } else {
      in[0] = routed.pairs[pair * width + i];
    }
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] += w * in[e];
  }
}

template <typename TD, typename T, int CENTRE, int V>
__global__ void post_norm_scale_add_kernel(float* __restrict__ stream, const TD* __restrict__ y, int splits, size_t split_stride,
                                           const float* __restrict__ weight, const float* __restrict__ bias,
                                           const float* __restrict__ channel_scale, float eps, T* __restrict__ out,
                                           float* __restrict__ history, size_t history_stride, int depth,
                                           const float* __restrict__ mix, int width, RoutedPairs routed) {
  extern __shared__ __align__(16) float row[];        // [width]
  __shared__ float scratch[16];
  const size_t at = (size_t)blockIdx.x * width;
  const int step = blockDim.x * V;
  float sum = 0.f;
  for (int i = threadIdx.x * V; i < width; i += step) {          // a thread rereads only what it wrote
    if (routed.pairs) {
      float v[V];
      routed_row<V>(routed, blockIdx.x, width, i, v);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        row[i + e] = v[e];
        sum += v[e];
      }
    } else if (V == 4) {
      float4 v = ld4(y + at + i);
      for (int s = 1; s < splits; ++s) {
        const float4 more = ld4(y + s * split_stride + at + i);
        v.x += more.x, v.y += more.y, v.z += more.z, v.w += more.w;
      }
      st4(row + i, v);
      sum += (v.x + v.y) + (v.z + v.w);
    } else {
      const float v = parts_sum(y, at + i, splits, split_stride);
      row[i] = v;
      sum += v;
    }
  }
  float mean = 0.f;
  if (CENTRE) mean = block_sum(sum, scratch) / (float)width;
  float squares = 0.f;
  for (int i = threadIdx.x * V; i < width; i += step)
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const float c = row[i + e] - mean;
      squares += c * c;
    }
  squares = block_sum(squares, scratch);
  const float scale = 1.f / sqrtf(squares / (float)width + eps);
  float* x = stream + at;
  for (int i = threadIdx.x * V; i < width; i += step) {
    float v[V], mixed[V];
    if (V == 4) { const float4 a = ld4(x + i); v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w; } else v[0] = x[i];
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float z = (row[i + e] - mean) * scale;
      if (weight) z *= weight[i + e];
      if (bias) z += bias[i + e];
      if (channel_scale) z *= channel_scale[i + e];
      v[e] += z;
      mixed[e] = 0.f;
    }
    if (depth > 0) {
      float* mine = history + (size_t)(depth - 1) * history_stride + at + i;
      if (V == 4) st4(mine, make_float4(v[0], v[1], v[2], v[3])); else *mine = v[0];
#pragma unroll 4
      for (int j = 0; j + 1 < depth; ++j) {
        const float* theirs = history + (size_t)j * history_stride + at + i;
        const float m = mix[j];
        if (V == 4) {
          const float4 a = ld4(theirs);
          mixed[0] += m * a.x, mixed[1] += m * a.y, mixed[2] += m * a.z, mixed[3] += m * a.w;
        } else {
          mixed[0] += m * *theirs;
        }
      }
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = mixed[e] + mix[depth - 1] * v[e];
    }
    if (V == 4) {
      st4(x + i, make_float4(v[0], v[1], v[2], v[3]));
      if (out) st4(out + at + i, make_float4(v[0], v[1], v[2], v[3]));
    } else {
      x[i] = v[0];
      if (out) st(out + at + i, v[0]);
    }
  }
}

extern "C" {

// stream float32 [n, width], changed in place.  y: y_dtype QIL_BF16 (one array, splits == 1) or QIL_F32
// ([splits][n][width] partial sums).  weight, bias, channel_scale: float32 [width] or null.  out: null, or [n, width] of
// out_dtype (the new stream, rounded).  history: null (depth 0), or float32 [>= depth][n][width] whose entries
// 0 .. depth - 2 are read and whose entry depth - 1 is written; mix float32 [depth].
static int post_norm_scale_add_launch(float* stream, const void* y, int y_dtype, int splits, const float* weight,
                                      const float* bias, const float* channel_scale, float eps, int centre, void* out,
                                      int out_dtype, float* history, int depth, const float* mix, int n, int width,
                                      RoutedPairs routed, hipStream_t s) {
  if (n == 0) return 0;
  if ((!y && !routed.pairs) || width < 1 || splits < 1 || (y_dtype == QIL_BF16 && splits != 1) || depth < 0 || (depth > 0 && (!history || !mix)) ||
      (size_t)width * sizeof(float) > 64 * 1024)
    return -1;
  const size_t stride = (size_t)n * width, lds = (size_t)width * sizeof(float);
  // four neighbouring elements a thread (one 8- or 16-byte access) where the rows allow
  const bool vec = width % 4 == 0 &&
                   (((uintptr_t)stream | (uintptr_t)y | (uintptr_t)out | (uintptr_t)history | (uintptr_t)routed.pairs) % 16) == 0;
  const int lanes = vec ? width / 4 : width;
  const int threads = lanes >= 512 ? 512 : lanes >= 256 ? 256 : lanes >= 128 ? 128 : 64;
#define QIL_POST_LAUNCH(TD, T, C, V)                                                                                   \
  hipLaunchKernelGGL((post_norm_scale_add_kernel<TD, T, C, V>), dim3(n), dim3(threads), lds, s, stream, (const TD*)y, \
                     splits, stride, weight, bias, channel_scale, eps, (T*)out, history, stride, depth, mix, width, routed)
#define QIL_POST_CASE(TD, T)                                                                                          \
  do {                                                                                                                \
    if (centre) { if (vec) QIL_POST_LAUNCH(TD, T, 1, 4); else QIL_POST_LAUNCH(TD, T, 1, 1); }                          \
    else { if (vec) QIL_POST_LAUNCH(TD, T, 0, 4); else QIL_POST_LAUNCH(TD, T, 0, 1); }                                 \
  } while (0)
  if (out_dtype == QIL_F32) {
    if (y_dtype == QIL_F32) QIL_POST_CASE(float, float); else QIL_POST_CASE(bf16_t, float);
  } else {
    if (y_dtype == QIL_F32) QIL_POST_CASE(float, bf16_t); else QIL_POST_CASE(bf16_t, bf16_t);
  }
#undef QIL_POST_CASE
#undef QIL_POST_LAUNCH
  QIL_RETURN_LAUNCH_STATUS();
}

int qil_post_norm_scale_add(float* stream, const void* y, int y_dtype, int splits, const float* weight, const float* bias,
                            const float* channel_scale, float eps, int centre, void* out, int out_dtype, float* history,
                            int depth, const float* mix, int n, int width, hipStream_t s) {
  const RoutedPairs none = {nullptr, nullptr, nullptr, nullptr, 0, 0, 0};
  return post_norm_scale_add_launch(stream, y, y_dtype, splits, weight, bias, channel_scale, eps, centre, out, out_dtype,
                                    history, depth, mix, n, width, none, s);
}

// The same with the weighted sum of a routed feed-forward's pairs in the place of y: pairs float32 [n * top][width],
// weights and chosen [n][top], input [n][width] of input_dtype (what a chosen index from `experts` on passes).
int qil_post_norm_scale_add_routed(float* stream, const float* pairs, const float* weights, const int* chosen,
                                   const void* input, int input_dtype, int top, int experts, const float* weight,
                                   const float* bias, const float* channel_scale, float eps, int centre, void* out,
                                   int out_dtype, float* history, int depth, const float* mix, int n, int width,
                                   hipStream_t s) {
  if (!pairs || !weights || !chosen || !input || top < 1) return -1;
  const RoutedPairs routed = {pairs, weights, chosen, input, input_dtype, top, experts};
  return post_norm_scale_add_launch(stream, nullptr, QIL_F32, 1, weight, bias, channel_scale, eps, centre, out, out_dtype,
                                    history, depth, mix, n, width, routed, s);
}

}  // extern "C"
