// A short causal convolution over time on every channel, added to its input:
//
//   h_t = x_t + sum_(j < taps) w[c, j] * x_(t - taps + 1 + j)      (inputs before a sequence's start are zero)
//
// x is the float32 residual stream of the step's rows (packed sequence after sequence); the last taps - 1 inputs of a
// sequence are its state between steps, state[slot][k] = the input at position (cached length) - (taps - 1) + k,
// float32.  Everything is float32; the result is rounded once to T.
//
// grid (rows, pieces of the width): a thread takes V neighbouring channels of one row (V = 4: one 16-byte access an
// input).  Only a sequence's first taps - 1 rows of a step read the state; the threads of its first row compute them
// all and then write the state's new contents, each thread for its own channels, so every read of a state element
// comes before its write without a barrier or a second launch (the threads of rows 1 .. taps - 2 have nothing left
// to do).  The new state is written in ascending order: entry k takes what entry k + rows held (or a row of this
// step), and k + rows > k.
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

template <typename T, int V>
__global__ void short_conv_kernel(const float* __restrict__ x, const float* __restrict__ w, float* state,
                                  const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts,
                                  const int* __restrict__ seq_slots, const int* __restrict__ row_seq, T* __restrict__ out,
                                  int width, int taps) {
  const int n = blockIdx.x, c = (blockIdx.y * blockDim.x + threadIdx.x) * V;
  if (c >= width) return;
  const int s = row_seq[n], row0 = cu_seqlens[s], t = n - row0, keep = taps - 1;
  if (t > 0 && t < keep) return;                      // computed by the threads of the sequence's first row
  const int rows = cu_seqlens[s + 1] - row0, start = seq_starts[s];
  float* held = state ? state + (size_t)seq_slots[s] * keep * width : nullptr;
  const int last = t == 0 ? min(rows, max(keep, 1)) : t + 1;          // these threads compute rows t .. last - 1
  for (int r = t; r < last; ++r) {
    conv_vec<V> own, acc;
    own.load(x + (size_t)(row0 + r) * width + c);
#pragma unroll
    for (int e = 0; e < V; ++e) acc.v[e] = own.v[e];
    for (int j = 0; j < taps; ++j) {
      const int source = r - keep + j;                // the input's row within the sequence's rows of this step
      conv_vec<V> in;
      if (source == r) in = own;
      else if (source >= 0) in.load(x + (size_t)(row0 + source) * width + c);
      else if (start + source >= 0) in.load(held + (size_t)(keep + source) * width + c);
      else continue;
#pragma unroll
      for (int e = 0; e < V; ++e) acc.v[e] += w[(size_t)(c + e) * taps + j] * in.v[e];
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
}

extern "C" {

// x float32 [n, width]; w float32 [width, taps]; state float32 [slots][taps - 1][width] (null: nothing is kept and every
// sequence is taken to begin in this step); the step's rows by cu_seqlens [n_seqs + 1], seq_starts, seq_slots [n_seqs],
// row_seq [n]; out [n, width] of out_dtype.
int qil_short_conv(const float* x, const float* w, float* state, const int* cu_seqlens, const int* seq_starts,
                   const int* seq_slots, const int* row_seq, void* out, int out_dtype, int n, int width, int taps,
                   hipStream_t s) {
  if (n == 0) return 0;
  if (width < 1 || taps < 1 || (taps > 1 && !state)) return -1;
  const bool vec = width % 4 == 0 && (((uintptr_t)x | (uintptr_t)out | (uintptr_t)state) % 16) == 0;
  const int lanes = vec ? width / 4 : width;
  const int threads = lanes >= 256 ? 256 : (lanes + 63) / 64 * 64;
  const dim3 grid(n, (lanes + threads - 1) / threads);
#define QIL_CONV(T, V)                                                                                              \
  hipLaunchKernelGGL((short_conv_kernel<T, V>), grid, dim3(threads), 0, s, x, w, state, cu_seqlens, seq_starts,      \
                     seq_slots, row_seq, (T*)out, width, taps)
  if (out_dtype == QIL_F32) { if (vec) QIL_CONV(float, 4); else QIL_CONV(float, 1); }
  else { if (vec) QIL_CONV(bf16_t, 4); else QIL_CONV(bf16_t, 1); }
#undef QIL_CONV
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
