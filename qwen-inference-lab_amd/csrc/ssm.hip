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
//
//    Up to 32 states the scan runs with a thread a channel and the channel's states in registers
//    (scan_chunk_kernel): no sum across lanes, dt and u are loaded once a channel and token in whole lines, and B and
//    C, which all channels share, are staged in LDS a tile of 64 tokens at a time.  A step whose sequences bring at
//    most 64 rows walks each from its stored state in one launch.  Longer portions are cut into chunks of 64 tokens
//    that run side by side: the recurrence is linear in the state, S_end = P S_in + E with P = exp(A * sum of the
//    chunk's dt) and E the chunk's end state from zero, so (1) every chunk is walked from zero and leaves E and its
//    sum of dt, (2) a small kernel walks a sequence's chunks in order, leaves every chunk's S_in where its E was and
//    the sequence's last state in its slot, (3) every chunk is walked again from its S_in and writes y.  The bfloat16
//    model takes exp(dt A) as the hardware's exp2 of dt * (A log2 e); the float32 model calls expf.
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


// The same with V neighbouring channels a thread (V = 8 for a bfloat16 input, 4 for float32 partial sums: 16-byte
// loads of the input, the factors and the state), for sizes and addresses that allow it.
template <typename TI, int V> struct conv_in;
template <> struct conv_in<bf16_t, 8> {
  static __device__ __forceinline__ void load(const bf16_t* base, size_t index, int, size_t, float* out) { ld8(base + index, out); }
};
template <> struct conv_in<float, 4> {
  static __device__ __forceinline__ void load(const float* base, size_t index, int splits, size_t stride, float* out) {
    float4 v = ld4(base + index);
    for (int s = 1; s < splits; ++s) {
      const float4 w = ld4(base + (size_t)s * stride + index);
      v.x += w.x; v.y += w.y; v.z += w.z; v.w += w.w;
    }
    out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
  }
};
template <int V> __device__ __forceinline__ void load_floats(const float* p, float* out) {
#pragma unroll
  for (int e = 0; e < V; e += 4) { const float4 v = ld4(p + e); out[e] = v.x; out[e + 1] = v.y; out[e + 2] = v.z; out[e + 3] = v.w; }
}
template <int V> __device__ __forceinline__ void store_floats(float* p, const float* v) {
#pragma unroll
  for (int e = 0; e < V; e += 4) st4(p + e, make_float4(v[e], v[e + 1], v[e + 2], v[e + 3]));
}
template <int V> __device__ __forceinline__ void store_floats(bf16_t* p, const float* v) {
#pragma unroll
  for (int e = 0; e < V; e += 4) st4(p + e, make_float4(v[e], v[e + 1], v[e + 2], v[e + 3]));
}

template <typename TI, typename T, int V>
__global__ void channel_conv_vec_kernel(const TI* __restrict__ x, int splits, size_t split_stride, int x_columns,
                                        const float* __restrict__ w, const float* __restrict__ bias, float* state,
                                        const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts,
                                        const int* __restrict__ seq_slots, const int* __restrict__ row_seq,
                                        T* __restrict__ out, int channels, int taps, int act) {
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * V, n = blockIdx.x;
  if (c >= channels) return;
  const int keep = taps - 1;
  const int s = row_seq[n], row0 = cu_seqlens[s], t = n - row0;
  if (t > 0 && t < keep) return;                       // computed with the sequence's first row
  const int rows = cu_seqlens[s + 1] - row0, start = seq_starts[s];
  float* held = state ? state + (size_t)seq_slots[s] * keep * channels : nullptr;
  const int upto = t == 0 ? min(rows, max(keep, 1)) : t + 1;
  float b[V];
#pragma unroll
  for (int e = 0; e < V; ++e) b[e] = 0.f;
  if (bias) load_floats<V>(bias + c, b);
  for (int r = t; r < upto; ++r) {
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = b[e];
    for (int j = 0; j < taps; ++j) {
      const int source = r - keep + j;
      float in[V], f[V];
      if (source >= 0) conv_in<TI, V>::load(x, (size_t)(row0 + source) * x_columns + c, splits, split_stride, in);
      else if (held && start + source >= 0) load_floats<V>(held + (size_t)(keep + source) * channels + c, in);
      else continue;
      load_floats<V>(w + (size_t)j * channels + c, f);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] += f[e] * in[e];
    }
    if (act) {
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = silu_f(acc[e]);
    }
    store_floats<V>(out + (size_t)(row0 + r) * channels + c, acc);
  }
  if (t == 0 && held) {
    for (int k = 0; k < keep; ++k) {
      const int source = rows - keep + k;
      float in[V];
#pragma unroll
      for (int e = 0; e < V; ++e) in[e] = 0.f;
      if (source >= 0) conv_in<TI, V>::load(x, (size_t)(row0 + source) * x_columns + c, splits, split_stride, in);
      else if (start + source >= 0) load_floats<V>(held + (size_t)(k + rows) * channels + c, in);
      store_floats<V>(held + (size_t)k * channels + c, in);
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


#define SCAN_L 64                      // tokens a chunk, and a tile of B and C in LDS
#define SCAN_THREADS 256

template <bool FAST> __device__ __forceinline__ float scan_decay(float step, float rate) {
  return FAST ? __builtin_amdgcn_exp2f(step * rate) : expf(step * rate);          // FAST: rate = A * log2(e)
}
template <bool FAST> __device__ __forceinline__ float scan_softplus(float v) {
  if (v > 20.f) return v;
  return FAST ? __logf(1.f + __expf(v)) : log1pf(expf(v));
}
template <bool FAST> __device__ __forceinline__ float scan_silu(float v) {
  return FAST ? v * __builtin_amdgcn_rcpf(1.f + __expf(-v)) : v / (1.f + expf(-v));
}

// PHASE 0: a sequence's rows from its stored state, y and the new state written.  PHASE 1: a chunk from zero; its end
// state goes to carry[seq * max_chunks + chunk][channel][NS] and its sum of steps to sums[..][channel].  PHASE 2: a
// chunk from the state that the carry kernel left in carry[..]; y written.
// DIRECT: dt_raw, bc and gate are plain arrays of T (what the products of many rows leave): typed loads, no branches.
template <bool DIRECT, typename T> __device__ __forceinline__ float scan_fetch(const Operand& x, size_t index) {
  if (DIRECT) return ld(reinterpret_cast<const T*>(x.data) + index);
  return operand_at(x, index);
}

template <typename T, int NS, int PHASE, bool DIRECT>
__global__ void __launch_bounds__(SCAN_THREADS)
scan_chunk_kernel(const T* __restrict__ u, Operand dt_raw, const float* __restrict__ dt_bias,
                  const float* __restrict__ a, Operand bc, const float* __restrict__ d, Operand gate, int gate_columns,
                  int gate_offset, float* state, const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts,
                  const int* __restrict__ seq_slots, T* __restrict__ y, int channels, int states, float* carry,
                  float* sums, int max_chunks) {
  constexpr bool FAST = sizeof(T) == 2;
  __shared__ float tile[SCAN_L * 2 * NS];
  const int c = blockIdx.x * SCAN_THREADS + threadIdx.x, seq = blockIdx.y, chunk = PHASE == 0 ? 0 : blockIdx.z;
  const bool live = c < channels;
  const int cc = live ? c : channels - 1;              // threads past the end walk a copy and store nothing
  int first = cu_seqlens[seq], last = cu_seqlens[seq + 1];
  if (PHASE != 0) {
    first += chunk * SCAN_L;
    if (first >= last) return;                         // (the whole block)
    last = min(last, first + SCAN_L);
  }
  const size_t cell = (size_t)seq * max_chunks + chunk;
  float rate[NS], S[NS];
#pragma unroll
  for (int n = 0; n < NS; ++n) {
    const float an = n < states ? a[(size_t)cc * states + n] : 0.f;
    rate[n] = FAST ? an * 1.44269504088896f : an;
    S[n] = 0.f;
  }
  if (PHASE == 0 && seq_starts[seq] > 0) {
    const float* held = state + ((size_t)seq_slots[seq] * channels + cc) * states;
#pragma unroll
    for (int n = 0; n < NS; ++n) if (n < states) S[n] = held[n];
  }
  if (PHASE == 2) {
#pragma unroll
    for (int n = 0; n < NS; ++n) S[n] = carry[(cell * channels + cc) * NS + n];
  }
  const float bias = dt_bias[cc], skip = d[cc];
  float total = 0.f;
  for (int t0 = first; t0 < last; t0 += SCAN_L) {
    const int rows = min(SCAN_L, last - t0);
    __syncthreads();                                   // the tile before this one has been used
    for (int i = threadIdx.x; i < rows * 2 * NS; i += SCAN_THREADS) {
      const int r = i / (2 * NS), k = i - r * 2 * NS, half = k / NS, n = k - half * NS;
      tile[i] = n < states ? scan_fetch<DIRECT, T>(bc, (size_t)(t0 + r) * 2 * states + half * states + n) : 0.f;
    }
    __syncthreads();
    for (int r0 = 0; r0 < rows; r0 += 8) {
      float dt[8], uv[8], zv[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const size_t t = min(t0 + r0 + k, last - 1);
        dt[k] = scan_fetch<DIRECT, T>(dt_raw, t * channels + cc);
        uv[k] = ld(u + t * channels + cc);
        zv[k] = PHASE == 1 ? 0.f : scan_fetch<DIRECT, T>(gate, t * gate_columns + gate_offset + cc);
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        if (r0 + k < rows) {
          const float step = scan_softplus<FAST>(dt[k] + bias), in = step * uv[k];
          const float* B = tile + (r0 + k) * 2 * NS;
          float acc = 0.f;
#pragma unroll
          for (int n = 0; n < NS; ++n) {
            S[n] = scan_decay<FAST>(step, rate[n]) * S[n] + in * B[n];
            if (PHASE != 1) acc += S[n] * B[NS + n];
          }
          if (PHASE == 1) total += step;
          else if (live) st(y + (size_t)(t0 + r0 + k) * channels + c, (acc + skip * uv[k]) * scan_silu<FAST>(zv[k]));
        }
      }
    }
  }
  if (!live) return;
  if (PHASE == 0) {
    float* held = state + ((size_t)seq_slots[seq] * channels + c) * states;
#pragma unroll
    for (int n = 0; n < NS; ++n) if (n < states) held[n] = S[n];
  }
  if (PHASE == 1) {
#pragma unroll
    for (int n = 0; n < NS; ++n) carry[(cell * channels + c) * NS + n] = S[n];
    sums[cell * channels + c] = total;
  }
}

// A sequence's chunks in order, a thread a (channel, state): every chunk's end state from zero is replaced by the state
// it starts from, and the sequence's last state goes to its slot.
__global__ void scan_carry_kernel(float* carry, const float* __restrict__ sums, const float* __restrict__ a, float* state,
                                  const int* __restrict__ cu_seqlens, const int* __restrict__ seq_starts,
                                  const int* __restrict__ seq_slots, int channels, int states, int NS, int max_chunks) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x, seq = blockIdx.y;
  if (i >= channels * states) return;
  const int c = i / states, n = i - c * states;
  const int chunks = (cu_seqlens[seq + 1] - cu_seqlens[seq] + SCAN_L - 1) / SCAN_L;
  float* held = state + ((size_t)seq_slots[seq] * channels + c) * states + n;
  float S = seq_starts[seq] > 0 ? *held : 0.f;
  const float an = a[(size_t)c * states + n];
  for (int chunk = 0; chunk < chunks; ++chunk) {
    const size_t cell = (size_t)seq * max_chunks + chunk;
    float* at = carry + (cell * channels + c) * NS + n;
    const float end = *at;
    *at = S;
    S = expf(an * sums[cell * channels + c]) * S + end;
  }
  *held = S;
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
  const int V = x_code == QIL_BF16 ? 8 : 4;
  if (channels % V == 0 && x_columns % V == 0 &&
      (((uintptr_t)x | (uintptr_t)w | (uintptr_t)bias | (uintptr_t)state | (uintptr_t)out) % 16) == 0 &&
      !(x_code == QIL_BF16 && out_dtype == QIL_F32)) {
    const int lanes = channels / V;
    const int threads = lanes >= 128 ? 128 : (lanes + 63) / 64 * 64;
    const dim3 grid(n, (lanes + threads - 1) / threads);
    const size_t stride = (size_t)n * x_columns;
    if (x_code == QIL_BF16)
      hipLaunchKernelGGL((channel_conv_vec_kernel<bf16_t, bf16_t, 8>), grid, dim3(threads), 0, s, (const bf16_t*)x, 1, stride,
                         x_columns, w, bias, state, cu_seqlens, seq_starts, seq_slots, row_seq, (bf16_t*)out, channels, taps, act);
    else if (out_dtype == QIL_F32)
      hipLaunchKernelGGL((channel_conv_vec_kernel<float, float, 4>), grid, dim3(threads), 0, s, (const float*)x, x_splits, stride,
                         x_columns, w, bias, state, cu_seqlens, seq_starts, seq_slots, row_seq, (float*)out, channels, taps, act);
    else
      hipLaunchKernelGGL((channel_conv_vec_kernel<float, bf16_t, 4>), grid, dim3(threads), 0, s, (const float*)x, x_splits, stride,
                         x_columns, w, bias, state, cu_seqlens, seq_starts, seq_slots, row_seq, (bf16_t*)out, channels, taps, act);
    QIL_RETURN_LAUNCH_STATUS();
  }
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

// Bytes of float32 workspace the scan needs for a step whose longest sequence brings max_query rows (0: none).
size_t qil_selective_scan_workspace(int n_seqs, int max_query, int channels, int states) {
  const int chunks = (max_query + SCAN_L - 1) / SCAN_L;
  if (states > 32 || chunks <= 1) return 0;
  return (size_t)n_seqs * chunks * channels * ((states + 7) / 8 * 8 + 1) * sizeof(float);
}

// u, y: [n, channels] of dtype; dt_raw [n, channels], bc [n, 2 * states] (B then C), gate [n, gate_columns] with z from
// column gate_offset on: each QIL_BF16, or QIL_F32 with so many partial sums; dt_bias, d float32 [channels]; a float32
// [channels, states]; state float32 [slots][channels][states].  max_query: the most rows of one sequence; workspace:
// qil_selective_scan_workspace bytes (may be null when that is 0).
int qil_selective_scan(const void* u, const void* dt_raw, int dt_code, int dt_splits, const float* dt_bias, const float* a,
                       const void* bc, int bc_code, int bc_splits, const float* d, const void* gate, int gate_code,
                       int gate_splits, int gate_columns, int gate_offset, float* state, const int* cu_seqlens,
                       const int* seq_starts, const int* seq_slots, void* y, int dtype, int n, int n_seqs, int channels,
                       int states, int max_query, float* workspace, hipStream_t s) {
  if (n == 0 || n_seqs == 0) return 0;
  if (!qil_selective_scan_takes(channels, states, 1) || !state || gate_offset < 0 || gate_offset + channels > gate_columns ||
      dt_splits < 1 || bc_splits < 1 || gate_splits < 1 || (dt_code == QIL_BF16 && dt_splits != 1) ||
      (bc_code == QIL_BF16 && bc_splits != 1) || (gate_code == QIL_BF16 && gate_splits != 1) || n_seqs > 65535) return -1;
  const Operand odt{dt_raw, dt_code, dt_splits, (size_t)n * channels}, obc{bc, bc_code, bc_splits, (size_t)n * 2 * states},
      og{gate, gate_code, gate_splits, (size_t)n * gate_columns};
  if (states <= 32) {                                  // a thread a channel, the states in registers
    const int chunks = (max_query + SCAN_L - 1) / SCAN_L;
    if (max_query < 1 || (chunks > 1 && !workspace) || chunks > 65535) return -1;
    const dim3 blocks((channels + SCAN_THREADS - 1) / SCAN_THREADS, n_seqs, chunks);
    float* carry = workspace;
    const int ns = (states + 7) / 8 * 8;
    float* sums = workspace ? workspace + (size_t)n_seqs * chunks * channels * ns : nullptr;
    const bool direct = dt_code == dtype && bc_code == dtype && gate_code == dtype && dt_splits == 1 && bc_splits == 1 &&
                        gate_splits == 1;
#define QIL_CHUNK_D(T, NS, PHASE, DIRECT)                                                                             \
  hipLaunchKernelGGL((scan_chunk_kernel<T, NS, PHASE, DIRECT>), blocks, dim3(SCAN_THREADS), 0, s, (const T*)u, odt,    \
                     dt_bias, a, obc, d, og, gate_columns, gate_offset, state, cu_seqlens, seq_starts, seq_slots, (T*)y, \
                     channels, states, carry, sums, chunks)
#define QIL_CHUNK(T, NS, PHASE)                                                                                       \
  do { if (direct) QIL_CHUNK_D(T, NS, PHASE, true); else QIL_CHUNK_D(T, NS, PHASE, false); } while (0)
#define QIL_CHUNK_NS(T, PHASE)                                                                                        \
  do {                                                                                                                \
    if (ns == 8) QIL_CHUNK(T, 8, PHASE); else if (ns == 16) QIL_CHUNK(T, 16, PHASE);                                   \
    else if (ns == 24) QIL_CHUNK(T, 24, PHASE); else QIL_CHUNK(T, 32, PHASE);                                          \
  } while (0)
#define QIL_CHUNK_T(PHASE)                                                                                            \
  do { if (dtype == QIL_F32) QIL_CHUNK_NS(float, PHASE); else QIL_CHUNK_NS(bf16_t, PHASE); } while (0)
    if (chunks == 1) {
      QIL_CHUNK_T(0);
      QIL_RETURN_LAUNCH_STATUS();
    }
    QIL_CHUNK_T(1);
    const int pairs = channels * states;
    hipLaunchKernelGGL(scan_carry_kernel, dim3((pairs + 255) / 256, n_seqs), dim3(256), 0, s, carry, sums, a, state,
                       cu_seqlens, seq_starts, seq_slots, channels, states, ns, chunks);
    QIL_CHUNK_T(2);
#undef QIL_CHUNK_T
#undef QIL_CHUNK_NS
#undef QIL_CHUNK
#undef QIL_CHUNK_D
    QIL_RETURN_LAUNCH_STATUS();
  }
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
