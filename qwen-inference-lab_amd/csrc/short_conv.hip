// A short causal convolution over time on every channel, added to its input:
//
//   h_t = x_t + sum_(j < taps) w[c, j] * x_(t - taps + 1 + j)      (inputs before a sequence's start are zero)
//
// x is the float32 residual stream of the step's rows (packed sequence after sequence); the last taps - 1 inputs of a
// sequence are its state between steps, state[slot][k] = the input at position (cached length) - (taps - 1) + k,
// float32.  Everything is float32; the result is rounded once to T.
//
// One block per row, a thread per channel (in turns).  Only a sequence's first taps - 1 rows of a step read the
// state; the block of its first row computes them all and then writes the state's new contents, channel by channel
// in the same thread, so every read of a state element comes before its write without a barrier or a second
// launch (the blocks of rows 1 .. taps - 2 have nothing left to do).  The new state is written in ascending order:
// entry k takes what entry k + rows held (or a row of this step), and k + rows > k.
#include "common.h"

template <typename T>
__global__ void short_conv_kernel(const float* __restrict__ x, const float* __restrict__ w, float* __restrict__ state,
                                  const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts,
                                  const int* __restrict__ seq_slots, const int* __restrict__ row_seq, T* __restrict__ out,
                                  int width, int taps) {
  const int n = blockIdx.x, s = row_seq[n], row0 = cu_seqlens[s], t = n - row0, keep = taps - 1;
  if (t > 0 && t < keep) return;                      // computed by the block of the sequence's first row
  const int rows = cu_seqlens[s + 1] - row0, start = seq_starts[s];
  float* held = state ? state + (size_t)seq_slots[s] * keep * width : nullptr;
  const int last = t == 0 ? min(rows, max(keep, 1)) : t + 1;          // this block computes rows t .. last - 1
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float* wc = w + (size_t)c * taps;
    for (int r = t; r < last; ++r) {
      float acc = 0.f;
      for (int j = 0; j < taps; ++j) {
        const int source = r - keep + j;              // the input's row within the sequence's rows of this step
        float v = 0.f;
        if (source >= 0) v = x[(size_t)(row0 + source) * width + c];
        else if (start + source >= 0) v = held[(size_t)(keep + source) * width + c];
        acc += wc[j] * v;
      }
      st(out + (size_t)(row0 + r) * width + c, x[(size_t)(row0 + r) * width + c] + acc);
    }
    if (t == 0 && held) {
      for (int k = 0; k < keep; ++k) {
        const int source = rows - keep + k;
        float v = 0.f;
        if (source >= 0) v = x[(size_t)(row0 + source) * width + c];
        else if (start + source >= 0) v = held[(size_t)(k + rows) * width + c];
        held[(size_t)k * width + c] = v;
      }
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
  const int threads = width >= 1024 ? 256 : width >= 128 ? 128 : 64;
  if (out_dtype == QIL_F32)
    hipLaunchKernelGGL(short_conv_kernel<float>, dim3(n), dim3(threads), 0, s, x, w, state, cu_seqlens, seq_starts, seq_slots,
                       row_seq, (float*)out, width, taps);
  else
    hipLaunchKernelGGL(short_conv_kernel<bf16_t>, dim3(n), dim3(threads), 0, s, x, w, state, cu_seqlens, seq_starts,
                       seq_slots, row_seq, (bf16_t*)out, width, taps);
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
