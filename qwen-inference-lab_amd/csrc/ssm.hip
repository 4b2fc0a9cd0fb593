// A selective state-space mixer's two steps between its products.
//
// 1. The short causal convolution per channel with a bias and an activation:
//      u[t, c] = act(b[c] + sum_(j < taps) w[j, c] * x[t - taps + 1 + j, c])       (inputs before a sequence's start: 0)
//    x: the first `channels` columns of the rows of a product ([n, x_columns]; the model's type, or float32 partial
//    sums).  The last taps - 1 inputs of a sequence are its state between steps, state[slot][k] = the input at
//    position (cached length) - (taps - 1) + k, float32.  grid (rows, pieces of the channels); the thread of a
//    sequence's first row computes its first taps - 1 rows and then writes the state's new contents for its channel
//    (ascending: entry k takes what entry k + rows held, or a row of this step), so every read of a state element
//    comes before its write; the threads of rows 1 .. taps - 2 leave at once.
//
// 2. The scan, a sequence's rows in order:
//      dt = softplus(dt_raw[t, c] + dt_bias[c])
//      S[c, n] <- exp(dt * A[c, n]) * S[c, n] + dt * u[t, c] * B[t, n]
//      y[t, c] = (sum_n S[c, n] * C[t, n] + D[c] * u[t, c]) * silu(z[t, c])
//    S float32 [slots][channels][states], read unless the sequence starts at position 0 and written back at the end.
//    grid (groups of 16 channels, sequences), 256 threads: a channel takes 16 lanes (one row of the data-parallel
//    moves), lane l holds the states l, l + 16, ...; the sum over the states is four such moves.  The loads of a
//    token do not depend on the state, so four tokens' loads go out before their updates run.
//    Everything from dt on is float32; u, B, C, z and dt_raw come as the products left them.
#include "common.h"
#include "operand.h"

__device__ __forceinline__ float silu_f(float v) { return v / (1.f + expf(-v)); }
__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }

template <typename T>
__global__ void channel_conv_kernel(Operand x, int x_columns, const float* __restrict__ w, const float* __restrict__ bias,
                                    float* state, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts,
                                    const int* __restrict__ seq_slots, const int* __restrict__ row_seq,
                                    T* __restrict__ out, int channels, int taps, int act) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x, n = blockIdx.x;
  if (c >= channels) return;
  const int keep = taps - 1;
  const int s = row_seq[n], row0 = cu_seqlens[s], t = n - row0;
  if (t > 0 && t < keep) return;                       // computed with the sequence's first row
  const int rows = cu_seqlens[s + 1] - row0, start = seq_starts[s];
  float* held = state ? state + (size_t)seq_slots[s] * keep * channels : nullptr;
  const int upto = t == 0 ? min(rows, max(keep, 1)) : t + 1;
  const float b = bias ? bias[c] : 0.f;
  for (int r = t; r < upto; ++r) {
    float acc = b;
    for (int j = 0; j < taps; ++j) {
      const int source = r - keep + j;                 // the input's row within the sequence's rows of this step
      float in;
      if (source >= 0) in = operand_at(x, (size_t)(row0 + source) * x_columns + c);
      else if (held && start + source >= 0) in = held[(size_t)(keep + source) * channels + c];
      else continue;
      acc += w[(size_t)j * channels + c] * in;
    }
    st(out + (size_t)(row0 + r) * channels + c, act ? silu_f(acc) : acc);
  }
  if (t == 0 && held) {
    for (int k = 0; k < keep; ++k) {
      const int source = rows - keep + k;
      float in = 0.f;
      if (source >= 0) in = operand_at(x, (size_t)(row0 + source) * x_columns + c);
      else if (start + source >= 0) in = held[(size_t)(k + rows) * channels + c];
      held[(size_t)k * channels + c] = in;
    }
  }
}

__device__ __forceinline__ float row16_total(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
  return v;
}

#define SCAN_AHEAD 4

template <typename T, int NPER>
__global__ void __launch_bounds__(256)
selective_scan_kernel(const T* __restrict__ u, Operand dt_raw, const float* __restrict__ dt_bias,
                      const float* __restrict__ a, Operand bc, const float* __restrict__ d, Operand gate, int gate_columns,
                      int gate_offset, float* state, const int* __restrict__ cu_seqlens,
                      const int* __restrict__ seq_starts, const int* __restrict__ seq_slots, T* __restrict__ y,
                      int channels, int states) {
  const int lane = threadIdx.x & 15;
  const int c = blockIdx.x * 16 + (threadIdx.x >> 4);
  const int seq = blockIdx.y;
  const bool live = c < channels;
  const int cc = live ? c : channels - 1;              // lanes past the end compute a copy and store nothing
  const int first = cu_seqlens[seq], last = cu_seqlens[seq + 1];
  float* held = state + ((size_t)seq_slots[seq] * channels + cc) * states;
  const bool continues = seq_starts[seq] > 0;
  float decay[NPER], S[NPER];
#pragma unroll
  for (int j = 0; j < NPER; ++j) {
    const int n = lane + 16 * j;
    decay[j] = n < states ? a[(size_t)cc * states + n] : 0.f;
    S[j] = (continues && n < states) ? held[n] : 0.f;
  }
  const float bias = dt_bias[cc], skip = d[cc];
  for (int t0 = first; t0 < last; t0 += SCAN_AHEAD) {
    float dt[SCAN_AHEAD], uv[SCAN_AHEAD], zv[SCAN_AHEAD], B[SCAN_AHEAD][NPER], C[SCAN_AHEAD][NPER];
#pragma unroll
    for (int k = 0; k < SCAN_AHEAD; ++k) {
      const int t = min(t0 + k, last - 1);
      dt[k] = operand_at(dt_raw, (size_t)t * channels + cc);
      uv[k] = ld(u + (size_t)t * channels + cc);
      zv[k] = operand_at(gate, (size_t)t * gate_columns + gate_offset + cc);
#pragma unroll
      for (int j = 0; j < NPER; ++j) {
        const int n = lane + 16 * j;
        B[k][j] = n < states ? operand_at(bc, (size_t)t * 2 * states + n) : 0.f;
        C[k][j] = n < states ? operand_at(bc, (size_t)t * 2 * states + states + n) : 0.f;
      }
    }
#pragma unroll
    for (int k = 0; k < SCAN_AHEAD; ++k) {
      if (t0 + k < last) {
        const float step = softplus_f(dt[k] + bias), in = step * uv[k];
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < NPER; ++j) {
          S[j] = expf(step * decay[j]) * S[j] + in * B[k][j];
          acc += S[j] * C[k][j];
        }
        acc = row16_total(acc);
        if (lane == 0 && live) st(y + (size_t)(t0 + k) * channels + c, (acc + skip * uv[k]) * silu_f(zv[k]));
      }
    }
  }
  if (live) {
#pragma unroll
    for (int j = 0; j < NPER; ++j) {
      const int n = lane + 16 * j;
      if (n < states) held[n] = S[j];
    }
  }
}

extern "C" {

int qil_selective_scan_takes(int channels, int states, int taps) {
  return channels >= 1 && states >= 1 && states <= 256 && taps >= 1 && taps <= 64;
}

// x: [n, x_columns] (x_code QIL_F32 with x_splits partial sums, or QIL_BF16), its first `channels` columns are the
// convolution's input; w float32 [taps, channels]; bias float32 [channels] or null; state float32 [slots][taps - 1]
// [channels] (null only for one tap); out [n, channels] of out_dtype; act: 0 none, 1 silu.
int qil_channel_conv(const void* x, int x_code, int x_splits, int x_columns, const float* w, const float* bias, float* state,
                     const int* cu_seqlens, const int* seq_starts, const int* seq_slots, const int* row_seq, void* out,
                     int out_dtype, int n, int channels, int taps, int act, hipStream_t s) {
  if (n == 0) return 0;
  if (channels < 1 || channels > x_columns || taps < 1 || (taps > 1 && !state) || x_splits < 1 ||
      (x_code == QIL_BF16 && x_splits != 1)) return -1;
  const Operand in{x, x_code, x_splits, (size_t)n * x_columns};
  const int threads = channels >= 256 ? 256 : (channels + 63) / 64 * 64;
  const dim3 grid(n, (channels + threads - 1) / threads);
  if (out_dtype == QIL_F32)
    hipLaunchKernelGGL(channel_conv_kernel<float>, grid, dim3(threads), 0, s, in, x_columns, w, bias, state, cu_seqlens,
                       seq_starts, seq_slots, row_seq, (float*)out, channels, taps, act);
  else
    hipLaunchKernelGGL(channel_conv_kernel<bf16_t>, grid, dim3(threads), 0, s, in, x_columns, w, bias, state, cu_seqlens,
                       seq_starts, seq_slots, row_seq, (bf16_t*)out, channels, taps, act);
  QIL_RETURN_LAUNCH_STATUS();
}

// u, y: [n, channels] of dtype; dt_raw [n, channels], bc [n, 2 * states] (B then C), gate [n, gate_columns] with z from
// column gate_offset on: each QIL_BF16, or QIL_F32 with so many partial sums; dt_bias, d float32 [channels]; a float32
// [channels, states]; state float32 [slots][channels][states].
int qil_selective_scan(const void* u, const void* dt_raw, int dt_code, int dt_splits, const float* dt_bias, const float* a,
                       const void* bc, int bc_code, int bc_splits, const float* d, const void* gate, int gate_code,
                       int gate_splits, int gate_columns, int gate_offset, float* state, const int* cu_seqlens,
                       const int* seq_starts, const int* seq_slots, void* y, int dtype, int n, int n_seqs, int channels,
                       int states, hipStream_t s) {
  if (n == 0 || n_seqs == 0) return 0;
  if (!qil_selective_scan_takes(channels, states, 1) || !state || gate_offset < 0 || gate_offset + channels > gate_columns ||
      dt_splits < 1 || bc_splits < 1 || gate_splits < 1 || (dt_code == QIL_BF16 && dt_splits != 1) ||
      (bc_code == QIL_BF16 && bc_splits != 1) || (gate_code == QIL_BF16 && gate_splits != 1) || n_seqs > 65535) return -1;
  const Operand odt{dt_raw, dt_code, dt_splits, (size_t)n * channels}, obc{bc, bc_code, bc_splits, (size_t)n * 2 * states},
      og{gate, gate_code, gate_splits, (size_t)n * gate_columns};
  const dim3 grid((channels + 15) / 16, n_seqs);
  const int per = (states + 15) / 16;
#define QIL_SCAN(T, NPER)                                                                                             \
  hipLaunchKernelGGL((selective_scan_kernel<T, NPER>), grid, dim3(256), 0, s, (const T*)u, odt, dt_bias, a, obc, d, og, \
                     gate_columns, gate_offset, state, cu_seqlens, seq_starts, seq_slots, (T*)y, channels, states)
#define QIL_SCAN_T(T)                                                                                                 \
  do {                                                                                                                \
    if (per <= 1) QIL_SCAN(T, 1); else if (per <= 2) QIL_SCAN(T, 2); else if (per <= 4) QIL_SCAN(T, 4);                \
    else if (per <= 8) QIL_SCAN(T, 8); else QIL_SCAN(T, 16);                                                          \
  } while (0)
  if (dtype == QIL_F32) QIL_SCAN_T(float); else QIL_SCAN_T(bf16_t);
#undef QIL_SCAN_T
#undef QIL_SCAN
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
