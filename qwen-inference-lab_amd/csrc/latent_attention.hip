// Attention over a cached low-rank latent (one per token, shared by all heads) with a rotated key part shared by all
// heads and a per-head sink logit in the softmax's denominator.
//
// The cache of a token is c [rank] (normalised latent) and kr [rot] (rotated key part).  A head's key is W_uk c and
// its value W_uv c; neither is ever made.  Instead the query is taken into the latent's space,
//     qa_h = W_uk,h^T q_h          (q_h the head's unrotated part),
// so that score(h, j) = scale * (qa_h . c_j + qr_h . kr_j), and the weighted sum runs over the latents themselves,
//     u_h = sum_j p(h, j) c_j,     value_h = W_uv,h u_h.
// Every head reads the same cached row: one staged tile of keys serves all heads of a block.
// The sink: a logit s_h with no key and no value; it enters the running maximum and the denominator once
// (running state starts at maximum s_h, sum 1, result 0).
// A window w > 0: the row at position p sees the keys j with 0 <= p - j < w only (w <= 0: every key j <= p).
// An output gate: head h's result of row n is multiplied by gate[n, h] (a float32 factor per row and head, made by
// the prepare kernel as the sigmoid of `gates` more columns of the stacked down product); a factor per head commutes
// with W_uv,h, so it is applied here, to the weighted sum of latents.
#include "common.h"
#include "partials.h"

// ---------------------------------------------------------------------------------------------------------------
// Step 1 of the mixer, after the stacked down products x = [W_dq h ; W_dkv h] (q_rank + rank + rot columns):
//   cq = x[:q_rank] / sqrt(mean(.^2) + eps) * wq                     -> cq_out (T)
//   c  = x[q_rank : q_rank + rank] / sqrt(mean(.^2) + eps) * wc      -> latent cache at the row's slot
//   kr = rotate(x[q_rank + rank : q_rank + rank + rot], position)    -> rope cache at the row's slot
//   g  = sigmoid(x[q_rank + rank + rot :])   (`gates` columns, if any)  -> gate_out [n, gates] float32
// Rotation of a vector of `rot` elements: element i pairs with i + rot / 2, angle position * freq[i].
template <typename TD, typename T>
__global__ void latent_prepare_kernel(const TD* __restrict__ x, int splits, size_t split_stride, const float* __restrict__ wq,
                                      const float* __restrict__ wc, const float* __restrict__ freq,
                                      const int* __restrict__ positions, const int* __restrict__ slots, T* __restrict__ cq_out,
                                      T* __restrict__ latent, T* __restrict__ rope, float* __restrict__ gate_out, int q_rank,
                                      int rank, int rot, int gates, float eps, int held) {
  extern __shared__ float sums[];                     // [q_rank + rank + rot + gates] when `held`: the row, its partial sums added
  __shared__ float scratch[16];
  const int n = blockIdx.x, total = q_rank + rank + rot + gates;
  const size_t at = (size_t)n * total;
  if (held) {                                         // every element is read from memory once, all reads side by side
    for (int i = threadIdx.x; i < total; i += blockDim.x) sums[i] = parts_sum(x, at + i, splits, split_stride);
    __syncthreads();
  }
  auto value = [&](int i) { return held ? sums[i] : parts_sum(x, at + i, splits, split_stride); };
  float sq = 0.f, sc = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) { const float v = value(i); sq += v * v; }
  for (int i = threadIdx.x; i < rank; i += blockDim.x) { const float v = value(q_rank + i); sc += v * v; }
  sq = block_sum(sq, scratch);
  sc = block_sum(sc, scratch);
  const float rq = 1.f / sqrtf(sq / (float)q_rank + eps), rc = 1.f / sqrtf(sc / (float)rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) st(cq_out + (size_t)n * q_rank + i, value(i) * rq * wq[i]);
  for (int i = threadIdx.x; i < gates; i += blockDim.x)
    gate_out[(size_t)n * gates + i] = 1.f / (1.f + expf(-value(q_rank + rank + rot + i)));
  if (!slots) return;
  const size_t slot = (size_t)slots[n];
  for (int i = threadIdx.x; i < rank; i += blockDim.x) st(latent + slot * rank + i, value(q_rank + i) * rc * wc[i]);
  const int half = rot / 2;
  const float p = (float)positions[n];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float u = value(q_rank + rank + i);
    const float v = value(q_rank + rank + half + i);
    float sn, cs;
    sincosf(p * freq[i], &sn, &cs);
    st(rope + slot * rot + i, u * cs - v * sn);
    st(rope + slot * rot + half + i, v * cs + u * sn);
  }
}

// ---------------------------------------------------------------------------------------------------------------
// A product per head: out[n, h, o] = sum_k W[h, k, o] x[n, h, k]   (W "k-major": the outputs of one k side by side).
// x: row stride x_row, head stride x_head (elements); out likewise.  A block takes ROWS rows of one head and 256
// outputs; x passes through LDS, every W element is read once a block.
template <typename TX, typename TW, typename TO, int ROWS>
__global__ void head_product_kernel(const TX* __restrict__ x, int x_row, int x_head, const TW* __restrict__ w,
                                    TO* __restrict__ out, int out_row, int out_head, int n_rows, int k_dim, int o_dim) {
  extern __shared__ float xs[];                       // [ROWS][k_dim]
  const int row0 = blockIdx.x * ROWS, h = blockIdx.y, o = blockIdx.z * blockDim.x + threadIdx.x;
  for (int idx = threadIdx.x; idx < ROWS * k_dim; idx += blockDim.x) {
    const int r = idx / k_dim, k = idx - r * k_dim;
    xs[idx] = row0 + r < n_rows ? ld(x + (size_t)(row0 + r) * x_row + (size_t)h * x_head + k) : 0.f;
  }
  __syncthreads();
  if (o >= o_dim) return;
  float acc[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) acc[r] = 0.f;
  const TW* wh = w + (size_t)h * k_dim * o_dim + o;
  for (int k = 0; k < k_dim; ++k) {
    const float wv = ld(wh + (size_t)k * o_dim);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) acc[r] += wv * xs[r * k_dim + k];
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r)
    if (row0 + r < n_rows) st(out + (size_t)(row0 + r) * out_row + (size_t)h * out_head + o, acc[r]);
}

// The same product for few rows (decoding): the weights of a head are then read by too few blocks for the chip, so a
// block takes 8 rows, OT * 8 outputs (OT = 8, or 4 where that still leaves few blocks) and splits k 256 / OT ways: a
// thread reads 8 consecutive outputs of every (256 / OT)th k (16 bytes of bfloat16), and the partial sums meet by
// shuffles in a wave and through LDS between the four waves.  Takes o_dim % 8 == 0 and w aligned to 8 elements.
template <typename TX, typename TW, typename TO, int OT>
__global__ void __launch_bounds__(256)
head_product_few_kernel(const TX* __restrict__ x, int x_row, int x_head, const TW* __restrict__ w, TO* __restrict__ out,
                        int out_row, int out_head, int n_rows, int k_dim, int o_dim) {
  constexpr int OB = OT * 8, KG = 256 / OT;           // outputs a block, k groups
  extern __shared__ float xs[];                       // [8][k_dim], then [4 waves][8 rows][OB outputs]
  float* sums = xs + 8 * k_dim;
  const int row0 = blockIdx.x * 8, h = blockIdx.y, tid = threadIdx.x, to = tid % OT, kg = tid / OT;
  const int o0 = blockIdx.z * OB + to * 8;
#pragma unroll 4
  for (int idx = tid; idx < 8 * k_dim; idx += 256) {
    const int r = idx / k_dim, k = idx - r * k_dim;
    xs[idx] = row0 + r < n_rows ? ld(x + (size_t)(row0 + r) * x_row + (size_t)h * x_head + k) : 0.f;
  }
  __syncthreads();
  float acc[8][8] = {};
  if (o0 < o_dim) {
    const TW* wh = w + (size_t)h * k_dim * o_dim + o0;
#pragma unroll 4                                      // four weight reads on their way at a time
    for (int k = kg; k < k_dim; k += KG) {
      float wv[8];
      ld8(wh + (size_t)k * o_dim, wv);
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const float xv = xs[r * k_dim + k];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[r][j] += xv * wv[j];
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 8; ++r)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float v = acc[r][j];
#pragma unroll
      for (int step = OT; step < QIL_WAVE; step *= 2) v += __shfl_xor(v, step, QIL_WAVE);
      acc[r][j] = v;
    }
  const int wave = tid >> 6;
  if ((tid & 63) < OT) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
#pragma unroll
      for (int j = 0; j < 8; ++j) sums[(wave * 8 + r) * OB + to * 8 + j] = acc[r][j];
  }
  __syncthreads();
  for (int idx = tid; idx < 8 * OB; idx += 256) {
    const int r = idx / OB, j = idx % OB, o = blockIdx.z * OB + j;
    if (row0 + r < n_rows && o < o_dim)
      st(out + (size_t)(row0 + r) * out_row + (size_t)h * out_head + o,
         sums[r * OB + j] + sums[(8 + r) * OB + j] + sums[(16 + r) * OB + j] + sums[(24 + r) * OB + j]);
  }
}

// The rotated tail of every head's query: out[n, h, i] = rotate(q[n, h, offset + i], position), i < rot.
template <typename TX>
__global__ void rotate_tail_kernel(const TX* __restrict__ q, int q_row, int q_head, int offset, const float* __restrict__ freq,
                                   const int* __restrict__ positions, float* __restrict__ out, int out_row, int out_head,
                                   int out_offset, int rot) {
  const int n = blockIdx.x, h = blockIdx.y, half = rot / 2;
  const float p = (float)positions[n];
  const TX* src = q + (size_t)n * q_row + (size_t)h * q_head + offset;
  float* dst = out + (size_t)n * out_row + (size_t)h * out_head + out_offset;
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float u = ld(src + i), v = ld(src + half + i);
    float sn, cs;
    sincosf(p * freq[i], &sn, &cs);
    dst[i] = u * cs - v * sn;
    dst[half + i] = v * cs + u * sn;
  }
}

// ---------------------------------------------------------------------------------------------------------------
// The general kernel: one block per (row, group of heads), any sizes, float32 arithmetic on the vector units.
//   Q [N, H, D] float32, D = rank + rot (qa then the rotated part); caches latent [slots, rank], rope [slots, rot] (TC);
//   out [N, H, rank] float32 = sum_j p(h, j) c_j.
// Keys come in tiles of KT (<= 64) rows staged in LDS as float32; a wave makes one head's softmax step with a lane
// per key; a thread owns up to ACC elements (h, c) of the group's results.
#define LA_THREADS 256
#define LA_ACC 16
template <typename TC>
__global__ void __launch_bounds__(LA_THREADS)
latent_attention_kernel(const float* __restrict__ q, const TC* __restrict__ latent, const TC* __restrict__ rope,
                        const int* __restrict__ tables, int table_stride, const int* __restrict__ row_seq,
                        const int* __restrict__ positions, const float* __restrict__ sink, const float* __restrict__ gate,
                        float* __restrict__ out, int heads, int group, int rank, int rot, int page_size, int kt, float scale,
                        int window) {
  extern __shared__ float lds[];
  const int d = rank + rot, pad = d + 1;
  float* qs = lds;                                   // [group][d]
  float* ks = qs + group * d;                        // [kt][pad]
  float* ps = ks + kt * pad;                         // [group][kt]
  float* top = ps + group * kt;                      // [group]
  float* den = top + group;                          // [group]
  float* shrink = den + group;                       // [group]
  const int n = blockIdx.x, h0 = blockIdx.y * group;
  const int live = min(group, heads - h0);
  const int position = positions[n];
  const int* table = tables + (size_t)row_seq[n] * table_stride;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  for (int idx = tid; idx < live * d; idx += LA_THREADS) qs[idx] = q[((size_t)n * heads + h0) * d + idx];
  if (tid < live) { top[tid] = sink ? sink[h0 + tid] : -INFINITY; den[tid] = sink ? 1.f : 0.f; }
  float acc[LA_ACC];
#pragma unroll
  for (int a = 0; a < LA_ACC; ++a) acc[a] = 0.f;
  const int owned = live * rank;

  const int first = window > 0 ? max(0, position - window + 1) : 0;     // the oldest key the row sees
  for (int j0 = first; j0 <= position; j0 += kt) {
    const int keys = min(kt, position + 1 - j0);
    __syncthreads();                                 // the last tile's reads are done (and qs / top / den are written)
    for (int idx = tid; idx < keys * d; idx += LA_THREADS) {
      const int j = idx / d, i = idx - j * d;
      const int key = j0 + j;
      const size_t slot = (size_t)table[key / page_size] * page_size + key % page_size;
      ks[j * pad + i] = i < rank ? ld(latent + slot * rank + i) : ld(rope + slot * rot + (i - rank));
    }
    __syncthreads();
    for (int pair = tid; pair < live * kt; pair += LA_THREADS) {
      const int h = pair / kt, j = pair - h * kt;
      float s = -INFINITY;
      if (j < keys) {
        const float* qh = qs + h * d;
        const float* kj = ks + j * pad;
        float dot = 0.f;
        for (int i = 0; i < d; ++i) dot += qh[i] * kj[i];
        s = dot * scale;
      }
      ps[pair] = s;
    }
    __syncthreads();
    for (int h = wave; h < live; h += LA_THREADS / 64) {
      const float s = lane < kt ? ps[h * kt + lane] : -INFINITY;
      const float old = top[h];
      const float now = fmaxf(old, wave_max(s));
      const float p = (lane < keys && now > -INFINITY) ? expf(s - now) : 0.f;
      const float total = wave_sum(p);
      if (lane < kt) ps[h * kt + lane] = p;
      if (lane == 0) {
        const float f = now > -INFINITY ? expf(old - now) : 1.f;
        shrink[h] = f;
        den[h] = den[h] * f + total;
        top[h] = now;
      }
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < LA_ACC; ++a) {
      const int e = tid + a * LA_THREADS;
      if (e < owned) {
        const int h = e / rank, c = e - h * rank;
        float v = acc[a] * shrink[h];
        const float* ph = ps + h * kt;
        for (int j = 0; j < keys; ++j) v += ph[j] * ks[j * pad + c];
        acc[a] = v;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int a = 0; a < LA_ACC; ++a) {
    const int e = tid + a * LA_THREADS;
    if (e < owned) {
      const int h = e / rank, c = e - h * rank;
      const float factor = gate ? gate[(size_t)n * heads + h0 + h] : 1.f;
      out[((size_t)n * heads + h0 + h) * rank + c] = acc[a] / den[h] * factor;
    }
  }
}

// Heads a block of the general kernel takes, and the keys of a staged tile, for these sizes.
static void latent_plan(int heads, int rank, int rot, int* group, int* kt, size_t* lds) {
  const int d = rank + rot;
  int g = LA_ACC * LA_THREADS / rank;
  if (g > heads) g = heads;
  while (g > 1 && (size_t)g * d * 4 > 24 * 1024) --g;
  int t = 64;
  while (t > 1 && (size_t)t * (d + 1) * 4 > 32 * 1024) t /= 2;
  *group = g;
  *kt = t;
  *lds = ((size_t)g * d + (size_t)t * (d + 1) + (size_t)g * t + 3 * (size_t)g) * sizeof(float);
}

extern "C" {

int qil_latent_prepare(const void* x, int x_dtype, int splits, const float* wq, const float* wc, const float* freq,
                       const int* positions, const int* slots, void* cq_out, void* latent, void* rope, float* gate_out,
                       int n, int q_rank, int rank, int rot, int gates, float eps, int dtype, hipStream_t s) {
  if (n == 0) return 0;
  if (q_rank < 1 || rank < 1 || rot < 2 || rot % 2 || splits < 1 || (x_dtype == QIL_BF16 && splits != 1) || gates < 0 ||
      (gates > 0 && !gate_out))
    return -1;
  const size_t stride = (size_t)n * (q_rank + rank + rot + gates);
  const size_t row_bytes = (size_t)(q_rank + rank + rot + gates) * sizeof(float);
  const int held = row_bytes <= 48 * 1024;            // the row's sums fit in LDS
  // a thread's loads of the row come one after the other: with few rows (too few blocks to hide that) wide rows get
  // more threads, not more turns
  const int total = q_rank + rank + rot + gates, threads = n > 64 ? 256 : total >= 2048 ? 1024 : total >= 1024 ? 512 : 256;
#define QIL_LP(TD, T)                                                                                               \
  hipLaunchKernelGGL((latent_prepare_kernel<TD, T>), dim3(n), dim3(threads), held ? row_bytes : 0, s, (const TD*)x, splits, \
                     stride, wq, wc, freq, positions, slots, (T*)cq_out, (T*)latent, (T*)rope, gate_out, q_rank, rank, rot, gates, eps, held)
  if (dtype == QIL_F32) {
    if (x_dtype != QIL_F32) return -1;
    QIL_LP(float, float);
  } else if (x_dtype == QIL_F32) {
    QIL_LP(float, bf16_t);
  } else {
    QIL_LP(bf16_t, bf16_t);
  }
#undef QIL_LP
  QIL_RETURN_LAUNCH_STATUS();
}

// out[n, h, o] = sum_k w[h, k, o] x[n, h, k]; x_dtype / w_dtype / out_dtype element codes; strides in elements.
// Combinations: all float32; x bfloat16, w bfloat16, out float32; x float32, w bfloat16, out bfloat16.
int qil_head_product(const void* x, int x_dtype, int x_row, int x_head, const void* w, int w_dtype, void* out,
                     int out_dtype, int out_row, int out_head, int n, int heads, int k_dim, int o_dim, hipStream_t s) {
  if (n == 0 || heads == 0 || o_dim == 0) return 0;
  if (k_dim < 1) return -1;
  const int rows = 8;
  const size_t lds = (size_t)rows * k_dim * sizeof(float);
  if (lds > 64 * 1024) return -1;
  const int threads = o_dim >= 256 ? 256 : (o_dim + 63) / 64 * 64;
  dim3 grid((n + rows - 1) / rows, heads, (o_dim + threads - 1) / threads);
  const size_t w_bytes = w_dtype == QIL_F32 ? 4 : 2;
  const bool few = n <= 32 && o_dim % 8 == 0 && (size_t)w % (8 * w_bytes) == 0 && lds + 4 * 8 * 64 * sizeof(float) <= 64 * 1024;
  const dim3 grid_few((n + 7) / 8, heads, (o_dim + 63) / 64);
  const bool narrow = grid_few.x * grid_few.y * grid_few.z < 128;      // few blocks: 32 outputs a block, k split 64 ways
  const dim3 grid_narrow((n + 7) / 8, heads, (o_dim + 31) / 32);
#define QIL_HP(TX, TW, TO)                                                                                            \
  do {                                                                                                                  \
    if (few && narrow)                                                                                                  \
      hipLaunchKernelGGL((head_product_few_kernel<TX, TW, TO, 4>), grid_narrow, dim3(256), lds + 4 * 8 * 32 * sizeof(float), s, \
                         (const TX*)x, x_row, x_head, (const TW*)w, (TO*)out, out_row, out_head, n, k_dim, o_dim);       \
    else if (few)                                                                                                       \
      hipLaunchKernelGGL((head_product_few_kernel<TX, TW, TO, 8>), grid_few, dim3(256), lds + 4 * 8 * 64 * sizeof(float), s, \
                         (const TX*)x, x_row, x_head, (const TW*)w, (TO*)out, out_row, out_head, n, k_dim, o_dim);       \
    else                                                                                                                \
      hipLaunchKernelGGL((head_product_kernel<TX, TW, TO, 8>), grid, dim3(threads), lds, s, (const TX*)x, x_row, x_head, \
                         (const TW*)w, (TO*)out, out_row, out_head, n, k_dim, o_dim);                                    \
  } while (0)
  if (x_dtype == QIL_F32 && w_dtype == QIL_F32 && out_dtype == QIL_F32) QIL_HP(float, float, float);
  else if (x_dtype == QIL_BF16 && w_dtype == QIL_BF16 && out_dtype == QIL_F32) QIL_HP(bf16_t, bf16_t, float);
  else if (x_dtype == QIL_F32 && w_dtype == QIL_BF16 && out_dtype == QIL_BF16) QIL_HP(float, bf16_t, bf16_t);
  else return -1;
#undef QIL_HP
  QIL_RETURN_LAUNCH_STATUS();
}

// out[n, h, out_offset + i] = rotate(q[n, h, offset + i], positions[n]) for i < rot; out float32.
int qil_rotate_tail(const void* q, int q_dtype, int q_row, int q_head, int offset, const float* freq, const int* positions,
                    float* out, int out_row, int out_head, int out_offset, int n, int heads, int rot, hipStream_t s) {
  if (n == 0 || heads == 0) return 0;
  if (rot < 2 || rot % 2) return -1;
  if (q_dtype == QIL_F32)
    hipLaunchKernelGGL(rotate_tail_kernel<float>, dim3(n, heads), dim3(64), 0, s, (const float*)q, q_row, q_head, offset,
                       freq, positions, out, out_row, out_head, out_offset, rot);
  else
    hipLaunchKernelGGL(rotate_tail_kernel<bf16_t>, dim3(n, heads), dim3(64), 0, s, (const bf16_t*)q, q_row, q_head, offset,
                       freq, positions, out, out_row, out_head, out_offset, rot);
  QIL_RETURN_LAUNCH_STATUS();
}

// Whether the general kernel takes these sizes.
int qil_latent_attention_takes(int heads, int rank, int rot) {
  if (heads < 1 || rank < 1 || rot < 0 || rank > LA_ACC * LA_THREADS) return 0;
  int group, kt;
  size_t lds;
  latent_plan(heads, rank, rot, &group, &kt, &lds);
  return group >= 1 && kt >= 1 && (size_t)group * (rank + rot) * 4 <= 24 * 1024 && lds <= 64 * 1024;
}

int qil_latent_attention(const float* q, const void* latent, const void* rope, const int* tables, int table_stride,
                         const int* row_seq, const int* positions, const float* sink, const float* gate, float* out, int n,
                         int heads, int rank, int rot, int page_size, float scale, int window, int cache_dtype,
                         hipStream_t s) {
  if (n == 0) return 0;
  if (!qil_latent_attention_takes(heads, rank, rot) || page_size < 1) return -1;
  int group, kt;
  size_t lds;
  latent_plan(heads, rank, rot, &group, &kt, &lds);
  dim3 grid(n, (heads + group - 1) / group);
  if (cache_dtype == QIL_F32)
    hipLaunchKernelGGL(latent_attention_kernel<float>, grid, dim3(LA_THREADS), lds, s, q, (const float*)latent,
                       (const float*)rope, tables, table_stride, row_seq, positions, sink, gate, out, heads, group, rank,
                       rot, page_size, kt, scale, window);
  else
    hipLaunchKernelGGL(latent_attention_kernel<bf16_t>, grid, dim3(LA_THREADS), lds, s, q, (const bf16_t*)latent,
                       (const bf16_t*)rope, tables, table_stride, row_seq, positions, sink, gate, out, heads, group, rank,
                       rot, page_size, kt, scale, window);
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
