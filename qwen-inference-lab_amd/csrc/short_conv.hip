// A short causal convolution over time on every channel, added to its input:
//
//   h_t = x_t + sum_(j < taps) w[j, c] * x_(t - taps + 1 + j)      (inputs before a sequence's start are zero)
//
// x is the float32 residual stream of the step's rows (packed sequence after sequence); w holds a tap's factors side
// by side, [taps][width]; the last taps - 1 inputs of a sequence are its state between steps, state[slot][k] = the
// input at position (cached length) - (taps - 1) + k, float32.  Everything is float32; the result is rounded once to T.
//
// grid (groups of rows, pieces of the width): a thread takes V neighbouring channels (V = 4: one 16-byte access an
// input) of `rows_each` consecutive rows.  With one to four taps (TAPS) the factors and the last taps - 1 inputs stay
// in registers while the thread walks its rows, so a row costs one load of x beyond the first; more taps (TAPS = 0)
// load every input where it is used.  Only a sequence's first taps - 1 rows of a step read the state; the thread that
// has its first row computes them all and then writes the state's new contents, for its own channels, so every read
// of a state element comes before its write without a barrier or a second launch (rows 1 .. taps - 2 are skipped
// where they come up).  The new state is written in ascending order: entry k takes what entry k + rows held (or a
// row of this step), and k + rows > k.
#include "common.h"

template <int V> struct conv_vec;
template <> struct conv_vec<1> {
  float v[1];
  __device__ __forceinline__ void load(const float* p) { v[0] = *p; }
  __device__ __forceinline__ void store(float* p) const { *p = v[0]; }
  __device__ __forceinline__ void store(bf16_t* p) const { *p = f32_to_bf16(v[0]); }
};
template <> struct conv_vec<4> {
  float v[4];
  __device__ __forceinline__ void load(const float* p) { const float4 a = ld4(p); v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w; }
  __device__ __forceinline__ void store(float* p) const { st4(p, make_float4(v[0], v[1], v[2], v[3])); }
  __device__ __forceinline__ void store(bf16_t* p) const { st4(p, make_float4(v[0], v[1], v[2], v[3])); }
};

template <typename T, int V, int TAPS>
__global__ void short_conv_kernel(const float* __restrict__ x, const float* __restrict__ w, float* state,
                                  const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts,
                                  const int* __restrict__ seq_slots, const int* __restrict__ row_seq, T* __restrict__ out,
                                  int n_rows, int width, int taps_given, int rows_each) {
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * V;
  if (c >= width) return;
  const int taps = TAPS ? TAPS : taps_given, keep = taps - 1;
  conv_vec<V> factor[TAPS ? TAPS : 1], before[TAPS > 1 ? TAPS - 1 : 1];      // before: x rows have - keep .. have - 1
  if (TAPS) {
#pragma unroll
    for (int j = 0; j < TAPS; ++j) factor[j].load(w + (size_t)j * width + c);
  }
  int have = -1;
  const int first = blockIdx.x * rows_each, last = min(first + rows_each, n_rows);
  for (int n = first; n < last; ++n) {
    const int s = row_seq[n], row0 = cu_seqlens[s], t = n - row0;
    if (t > 0 && t < keep) continue;                  // computed with the sequence's first row
    if (t == 0 || !TAPS) {
      const int rows = cu_seqlens[s + 1] - row0, start = seq_starts[s];
      float* held = state ? state + (size_t)seq_slots[s] * keep * width : nullptr;
      const int upto = t == 0 ? min(rows, max(keep, 1)) : t + 1;        // rows t .. upto - 1 of the sequence
      for (int r = t; r < upto; ++r) {
        conv_vec<V> own, acc;
        own.load(x + (size_t)(row0 + r) * width + c);
#pragma unroll
        for (int e = 0; e < V; ++e) acc.v[e] = own.v[e];
#pragma unroll
        for (int j = 0; j < taps; ++j) {
          const int source = r - keep + j;            // the input's row within the sequence's rows of this step
          conv_vec<V> in, f;
          if (source == r) in = own;
          else if (source >= 0) in.load(x + (size_t)(row0 + source) * width + c);
          else if (start + source >= 0) in.load(held + (size_t)(keep + source) * width + c);
          else continue;
          if (TAPS) f = factor[j]; else f.load(w + (size_t)j * width + c);
#pragma unroll
          for (int e = 0; e < V; ++e) acc.v[e] += f.v[e] * in.v[e];
        }
        acc.store(out + (size_t)(row0 + r) * width + c);
      }
      if (t == 0 && held) {
        for (int k = 0; k < keep; ++k) {
          const int source = rows - keep + k;
          conv_vec<V> in;
#pragma unroll
          for (int e = 0; e < V; ++e) in.v[e] = 0.f;
          if (source >= 0) in.load(x + (size_t)(row0 + source) * width + c);
          else if (start + source >= 0) in.load(held + (size_t)(k + rows) * width + c);
          in.store(held + (size_t)k * width + c);
        }
      }
      have = -1;
      continue;
    }
    // every input is a row of this step: the rows before this one are at hand unless the walk just began or skipped
    if (TAPS > 1 && have != n) {
#pragma unroll
      for (int j = 0; j < TAPS - 1; ++j) before[j].load(x + (size_t)(n - (TAPS - 1) + j) * width + c);
    }
    conv_vec<V> own, acc;
    own.load(x + (size_t)n * width + c);
#pragma unroll
    for (int e = 0; e < V; ++e) acc.v[e] = own.v[e] + factor[TAPS ? TAPS - 1 : 0].v[e] * own.v[e];
    if (TAPS > 1) {
#pragma unroll
      for (int j = 0; j < TAPS - 1; ++j)
#pragma unroll
        for (int e = 0; e < V; ++e) acc.v[e] += factor[j].v[e] * before[j].v[e];
#pragma unroll
      for (int j = 0; j + 1 < TAPS - 1; ++j) before[j] = before[j + 1];
      before[TAPS - 2 > 0 ? TAPS - 2 : 0] = own;
    }
    acc.store(out + (size_t)n * width + c);
    have = n + 1;
  }
}

extern "C" {

// x float32 [n, width]; w float32 [taps, width]; state float32 [slots][taps - 1][width] (null: nothing is kept and every
// sequence is taken to begin in this step); the step's rows by cu_seqlens [n_seqs + 1], seq_starts, seq_slots [n_seqs],
// row_seq [n]; out [n, width] of out_dtype.
int qil_short_conv(const float* x, const float* w, float* state, const int* cu_seqlens, const int* seq_starts,
                   const int* seq_slots, const int* row_seq, void* out, int out_dtype, int n, int width, int taps,
                   hipStream_t s) {
  if (n == 0) return 0;
  if (width < 1 || taps < 1 || (taps > 1 && !state)) return -1;
  const bool vec = width % 4 == 0 && (((uintptr_t)x | (uintptr_t)w | (uintptr_t)out | (uintptr_t)state) % 16) == 0;
  const int lanes = vec ? width / 4 : width, most = vec ? 128 : 256;
  const int threads = lanes >= most ? most : (lanes + 63) / 64 * 64;
  const int rows_each = taps <= 4 && n >= 1024 ? 4 : 1;      // many rows: a thread walks four with the inputs at hand
  const dim3 grid((n + rows_each - 1) / rows_each, (lanes + threads - 1) / threads);
#define QIL_CONV(T, V, TAPS)                                                                                         \
  hipLaunchKernelGGL((short_conv_kernel<T, V, TAPS>), grid, dim3(threads), 0, s, x, w, state, cu_seqlens, seq_starts, \
                     seq_slots, row_seq, (T*)out, n, width, taps, rows_each)
#define QIL_CONV_TAPS(T, V)                                                                                          \
  switch (taps) {                                                                                                    \
    case 1: QIL_CONV(T, V, 1); break;                                                                                \
    case 2: QIL_CONV(T, V, 2); break;                                                                                \
    case 3: QIL_CONV(T, V, 3); break;                                                                                \
    case 4: QIL_CONV(T, V, 4); break;                                                                                \
    default: QIL_CONV(T, V, 0);                                                                                      \
  }
  if (out_dtype == QIL_F32) { if (vec) QIL_CONV_TAPS(float, 4) else QIL_CONV_TAPS(float, 1) }
  else { if (vec) QIL_CONV_TAPS(bf16_t, 4) else QIL_CONV_TAPS(bf16_t, 1) }
#undef QIL_CONV_TAPS
#undef QIL_CONV
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
