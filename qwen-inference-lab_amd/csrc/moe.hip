// A routed feed-forward (mixture of experts): the router, the grouping of (token, chosen expert) pairs by expert, the
// experts' two products on the matrix cores, and the weighted sum.
//
//   route    (two kernels: the logits, then the choice) per token: logits z = W_r h (+ a stored bias) in float32 (W_r float32, h as it comes), scores s = softmax(z) over all
//            outputs; choice scores c = s + correction (without a correction the choice goes by the logits themselves,
//            which order the outputs as their scores do and do not underflow); the outputs form `groups` equal groups of neighbours, a
//            group's score is its largest c, and only the `keep` best groups stay (the others' c count as -inf);
//            the `top` largest c are chosen (lowest index first among equals); the weights are their s, optionally
//            divided by their sum.  The last `identity` outputs are experts without tensors that pass their input.
//   align    pairs (token, slot) whose expert has tensors are put in the order of their experts, every expert's run
//            cut into tiles of TM pairs: tile -> (expert, first place, pairs), a fixed number of tiles of which the
//            unused ones hold no pair.  One block; the order inside an expert's run is whatever the atomics give,
//            which no result depends on (every pair's row is a product of its own).
//   gate_up  hidden[place] = act(W_gate,e h, W_up,e h) for the pairs of a tile, one wave per 16 hidden columns
//   down     y[pair] = W_down,e hidden[place], float32
//   combine  out[token] = sum over the token's slots, in slot order, of weight * (y[pair], or h for an identity expert)
//
// The products read their operands from memory in the matrix cores' own layout, 16 bytes a lane (a row's 8 bfloat16
// or 4 float32 at k0 + 8 or 4 * (lane / 16)): v_mfma_f32_16x16x32_bf16, or four v_mfma_f32_16x16x4_f32 whose k runs
// over the lanes' 4 elements in turn (true float32 products and sums).  A wave owns its output columns' weights, so a
// block reads every weight once; the tile's rows of h are read by each wave again (from the caches).
#include "common.h"
#include "gated_act.h"

typedef __bf16 moe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float moe_f32x4 __attribute__((ext_vector_type(4)));

#define MOE_MAX_OUTPUTS 1024          // experts + identity experts the router takes
#define MOE_ROUTE_THREADS 256

// ------------------------------------------------------------------------------------------------ route
__device__ __forceinline__ void wave_argmax(float& v, int& at) {          // the largest value, the lowest index among equals
#pragma unroll
  for (int o = QIL_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, QIL_WAVE);
    const int oa = __shfl_xor(at, o, QIL_WAVE);
    if (ov > v || (ov == v && oa < at)) { v = ov; at = oa; }
  }
}

// logits[n, e] = sum_i x[n, i] w[e, i] in float32.  grid (rows / 8, outputs / 4): a wave makes one output of eight rows, its
// lanes along the width (a router row is read once for the eight); no LDS, no barrier.
__device__ __forceinline__ float4 moe_load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 moe_load4(const bf16_t* p) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                     __uint_as_float(raw.y & 0xffff0000u));
}
template <typename T, bool VEC>
__global__ void __launch_bounds__(MOE_ROUTE_THREADS)
moe_logits_kernel(const T* __restrict__ x, int n, int width, const float* __restrict__ w_router, int outputs,
                  float* __restrict__ logits) {
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  const int e = blockIdx.y * 4 + wave, row0 = blockIdx.x * 8;
  if (e >= outputs) return;
  const float* w = w_router + (size_t)e * width;
  const T* rows[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) rows[r] = x + (size_t)min(row0 + r, n - 1) * width;
  float acc[8] = {};
  if (VEC) {
    for (int i = lane * 4; i < width; i += QIL_WAVE * 4) {
      const float4 wv = moe_load4(w + i);
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const float4 xv = moe_load4(rows[r] + i);
        acc[r] += xv.x * wv.x + xv.y * wv.y + xv.z * wv.z + xv.w * wv.w;
      }
    }
  } else {
    for (int i = lane; i < width; i += QIL_WAVE) {
      const float wv = w[i];
#pragma unroll
      for (int r = 0; r < 8; ++r) acc[r] += ld(rows[r] + i) * wv;
    }
  }
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const float total = wave_sum(acc[r]);
    if (lane == 0 && row0 + r < n) logits[(size_t)(row0 + r) * outputs + e] = total;
  }
}

// The choice from the logits: a wave a row, four rows a block (every wave walks the same steps, so the barriers
// between a wave's writes to its part of LDS and its reads are met by all).
__global__ void __launch_bounds__(MOE_ROUTE_THREADS)
moe_select_kernel(const float* __restrict__ logits, int n, const float* __restrict__ bias,
                  const float* __restrict__ correction, int outputs, int groups,
                  int keep, int top, int renormalize, int* __restrict__ chosen, float* __restrict__ weights,
                  int sigmoid_scores, int group_top2, float weight_scale, float renormalize_eps) {
  extern __shared__ float lds[];                        // per wave: [outputs] scores, [outputs] choice scores, [groups]
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  float* score = lds + (size_t)wave * (2 * outputs + groups);
  float* choice = score + outputs;
  float* group_best = choice + outputs;
  const int n_row = blockIdx.x * (MOE_ROUTE_THREADS / QIL_WAVE) + wave;
  const bool live = n_row < n;
  const float* z = logits + (size_t)min(n_row, n - 1) * outputs;
  auto logit = [&](int e) { return z[e] + (bias ? bias[e] : 0.f); };
  if (sigmoid_scores) {                                 // every output by itself; the choice goes by the score
    for (int e = lane; e < outputs; e += QIL_WAVE) {
      const float s = 1.f / (1.f + expf(-logit(e)));
      score[e] = s;
      choice[e] = correction ? s + correction[e] : s;
    }
  } else {
    float top_logit = -INFINITY;
    for (int e = lane; e < outputs; e += QIL_WAVE) top_logit = fmaxf(top_logit, logit(e));
    top_logit = wave_max(top_logit);
    float total = 0.f;
    for (int e = lane; e < outputs; e += QIL_WAVE) total += expf(logit(e) - top_logit);
    total = wave_sum(total);
    for (int e = lane; e < outputs; e += QIL_WAVE) {
      const float s = expf(logit(e) - top_logit) / total;
      score[e] = s;
      choice[e] = correction ? s + correction[e] : logit(e);
    }
  }
  __syncthreads();
  if (groups > 1 && keep < groups) {
    const int size = outputs / groups;
    for (int g = lane; g < groups; g += QIL_WAVE) {
      float best = -INFINITY, second = -INFINITY;
      for (int e = g * size; e < (g + 1) * size; ++e) {
        const float v = choice[e];
        if (v > best) { second = best; best = v; }
        else if (v > second) second = v;
      }
      group_best[g] = group_top2 && size > 1 ? best + second : best;     // its largest, or the sum of its two largest
    }
    __syncthreads();
    // the `keep` best groups are marked by +inf in their place, one after the other
    for (int round = 0; round < keep; ++round) {
      float v = -INFINITY;
      int at = 0x7fffffff;
      for (int g = lane; g < groups; g += QIL_WAVE) {
        const float gv = group_best[g];
        if (gv != INFINITY && (gv > v || at == 0x7fffffff)) { v = gv; at = g; }
      }
      wave_argmax(v, at);
      __syncthreads();
      if (lane == 0 && at != 0x7fffffff) group_best[at] = INFINITY;
      __syncthreads();
    }
    for (int e = lane; e < outputs; e += QIL_WAVE)
      if (group_best[e / size] != INFINITY) choice[e] = -INFINITY;
    __syncthreads();
  }
  float sum = 0.f, mine = 0.f;
  for (int round = 0; round < top; ++round) {
    float v = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < outputs; e += QIL_WAVE) {
      const float c = choice[e];
      if (c == c && c != INFINITY && (c > v || at == 0x7fffffff)) { v = c; at = e; }   // +inf marks what is taken
    }
    wave_argmax(v, at);
    if (at == 0x7fffffff) at = 0;
    const float s = score[at];
    sum += s;
    if (lane == round) mine = s;
    __syncthreads();
    if (lane == 0) {
      if (live) chosen[(size_t)n_row * top + round] = at;
      choice[at] = INFINITY;
    }
    __syncthreads();
  }
  if (live && lane < top)
    weights[(size_t)n_row * top + lane] = (renormalize ? mine / (sum + renormalize_eps) : mine) * weight_scale;
}

// ------------------------------------------------------------------------------------------------ align
// tiles: [3][max_tiles] expert, first place, pairs.  places: [pairs] the pair at every place.
__global__ void __launch_bounds__(1024)
moe_align_kernel(const int* __restrict__ chosen, int pairs, int experts, int tile_rows, int max_tiles,
                 int* __restrict__ tiles, int* __restrict__ places) {
  __shared__ int count[MOE_MAX_OUTPUTS], first[MOE_MAX_OUTPUTS], first_tile[MOE_MAX_OUTPUTS + 1];
  const int tid = threadIdx.x;
  for (int e = tid; e < experts; e += blockDim.x) count[e] = 0;
  __syncthreads();
  for (int p = tid; p < pairs; p += blockDim.x) {
    const int e = chosen[p];
    if (e < experts) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int place = 0, tile = 0;
    for (int e = 0; e < experts; ++e) {
      first[e] = place;
      first_tile[e] = tile;
      place += count[e];
      tile += (count[e] + tile_rows - 1) / tile_rows;
    }
    first_tile[experts] = tile;
  }
  __syncthreads();
  for (int t = tid; t < max_tiles; t += blockDim.x) tiles[2 * max_tiles + t] = 0;
  __syncthreads();
  for (int e = tid; e < experts; e += blockDim.x) {
    const int n_tiles = first_tile[e + 1] - first_tile[e];
    for (int t = 0; t < n_tiles; ++t) {
      const int at = first_tile[e] + t;
      tiles[at] = e;
      tiles[max_tiles + at] = first[e] + t * tile_rows;
      tiles[2 * max_tiles + at] = min(tile_rows, count[e] - t * tile_rows);
    }
    count[e] = 0;                                       // from here on: the places of the expert's run already given out
  }
  __syncthreads();
  for (int p = tid; p < pairs; p += blockDim.x) {
    const int e = chosen[p];
    if (e < experts) places[first[e] + atomicAdd(&count[e], 1)] = p;
  }
}

// ------------------------------------------------------------------------------------------------ products
template <typename T> struct Frag;
template <> struct Frag<bf16_t> {
  static constexpr int EPL = 8;                         // elements a lane holds of a row
  typedef qil_u32x4 raw;
  static __device__ __forceinline__ void mma(moe_f32x4& acc, const raw& a, const raw& b) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(moe_bf16x8, a), __builtin_bit_cast(moe_bf16x8, b), acc, 0, 0, 0);
  }
};
template <> struct Frag<float> {
  static constexpr int EPL = 4;
  typedef moe_f32x4 raw;
  static __device__ __forceinline__ void mma(moe_f32x4& acc, const raw& a, const raw& b) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[i], acc, 0, 0, 0);
  }
};

// A lane's 16 bytes of a row at element k (zeros from `length` on; rows that are 16-byte aligned with a length that is
// a multiple of EPL take one vector load, others go element by element).
template <typename T, bool ALIGNED>
__device__ __forceinline__ typename Frag<T>::raw load_frag(const T* __restrict__ row_ptr, int k, int length) {
  typename Frag<T>::raw out;
  if (ALIGNED) {
    if (k < length) return *reinterpret_cast<const typename Frag<T>::raw*>(row_ptr + k);
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = 0;
    return out;
  }
  T e[Frag<T>::EPL];
#pragma unroll
  for (int i = 0; i < Frag<T>::EPL; ++i) e[i] = k + i < length ? row_ptr[k + i] : (T)0;
  return __builtin_bit_cast(typename Frag<T>::raw, e);
}

// grid (tiles, ceil(ff / 64)); a wave: the tile's rows by 16 gate and the same 16 up columns.
// w: [experts][2][ff][width] (an expert's gate rows, then its up rows).  hidden: [places][ff].
template <typename T, int MT, bool ALIGNED>
__global__ void __launch_bounds__(256)
moe_gate_up_kernel(const T* __restrict__ x, int width, const T* __restrict__ w, int ff, const int* __restrict__ tiles,
                   int max_tiles, const int* __restrict__ places, int top, T* __restrict__ hidden, int act, float limit,
                   float alpha) {
  constexpr int EPL = Frag<T>::EPL, KC = 4 * EPL;
  const int tile = blockIdx.x, rows = tiles[2 * max_tiles + tile];
  if (rows == 0) return;
  const int e = tiles[tile], begin = tiles[max_tiles + tile];
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  const int col0 = (blockIdx.y * 4 + wave) * 16;
  if (col0 >= ff) return;
  const int r = lane & 15, kq = lane >> 4;
  const T* a_row[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int local = m * 16 + r;
    a_row[m] = x + (size_t)(places[begin + min(local, rows - 1)] / top) * width;
  }
  const int col = min(col0 + r, ff - 1);
  const T* g_row = w + ((size_t)e * 2 * ff + col) * width;
  const T* u_row = g_row + (size_t)ff * width;
  moe_f32x4 acc_g[MT], acc_u[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc_g[m] = acc_u[m] = (moe_f32x4){0.f, 0.f, 0.f, 0.f};
  // the fragments of the next step are on their way while this step's products run
  typename Frag<T>::raw bg = load_frag<T, ALIGNED>(g_row, kq * EPL, width), bu = load_frag<T, ALIGNED>(u_row, kq * EPL, width);
  typename Frag<T>::raw a[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) a[m] = load_frag<T, ALIGNED>(a_row[m], kq * EPL, width);
  for (int k0 = 0; k0 < width; k0 += KC) {
    const int k = k0 + KC + kq * EPL;                    // (past the end: zeros, never used)
    const typename Frag<T>::raw bg_next = load_frag<T, ALIGNED>(g_row, k, width), bu_next = load_frag<T, ALIGNED>(u_row, k, width);
    typename Frag<T>::raw a_next[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) a_next[m] = load_frag<T, ALIGNED>(a_row[m], k, width);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      Frag<T>::mma(acc_g[m], a[m], bg);
      Frag<T>::mma(acc_u[m], a[m], bu);
    }
    bg = bg_next;
    bu = bu_next;
#pragma unroll
    for (int m = 0; m < MT; ++m) a[m] = a_next[m];
  }
  if (col0 + r >= ff) return;
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int local = m * 16 + 4 * kq + i;
      if (local < rows) st(hidden + (size_t)(begin + local) * ff + col0 + r, gated_act(acc_g[m][i], acc_u[m][i], act, limit, alpha));
    }
}

// grid (tiles, ceil(width / 128)); a wave: the tile's rows by 32 output columns.  w: [experts][width][ff].
// y: [pairs][width] float32, a pair's row at the pair's own index.
template <typename T, int MT, bool ALIGNED>
__global__ void __launch_bounds__(256)
moe_down_kernel(const T* __restrict__ hidden, int ff, const T* __restrict__ w, int width, const int* __restrict__ tiles,
                int max_tiles, const int* __restrict__ places, float* __restrict__ y) {
  constexpr int EPL = Frag<T>::EPL, KC = 4 * EPL;
  const int tile = blockIdx.x, rows = tiles[2 * max_tiles + tile];
  if (rows == 0) return;
  const int e = tiles[tile], begin = tiles[max_tiles + tile];
  const int lane = threadIdx.x & (QIL_WAVE - 1), wave = threadIdx.x / QIL_WAVE;
  const int col0 = (blockIdx.y * 4 + wave) * 32;
  if (col0 >= width) return;
  const int r = lane & 15, kq = lane >> 4;
  const T* a_row[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) a_row[m] = hidden + (size_t)(begin + min(m * 16 + r, rows - 1)) * ff;
  const T* b_row[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) b_row[t] = w + ((size_t)e * width + min(col0 + t * 16 + r, width - 1)) * ff;
  moe_f32x4 acc[MT][2];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m][0] = acc[m][1] = (moe_f32x4){0.f, 0.f, 0.f, 0.f};
  typename Frag<T>::raw b0 = load_frag<T, ALIGNED>(b_row[0], kq * EPL, ff), b1 = load_frag<T, ALIGNED>(b_row[1], kq * EPL, ff);
  typename Frag<T>::raw a[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) a[m] = load_frag<T, ALIGNED>(a_row[m], kq * EPL, ff);
  for (int k0 = 0; k0 < ff; k0 += KC) {
    const int k = k0 + KC + kq * EPL;
    const typename Frag<T>::raw b0_next = load_frag<T, ALIGNED>(b_row[0], k, ff), b1_next = load_frag<T, ALIGNED>(b_row[1], k, ff);
    typename Frag<T>::raw a_next[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) a_next[m] = load_frag<T, ALIGNED>(a_row[m], k, ff);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      Frag<T>::mma(acc[m][0], a[m], b0);
      Frag<T>::mma(acc[m][1], a[m], b1);
    }
    b0 = b0_next;
    b1 = b1_next;
#pragma unroll
    for (int m = 0; m < MT; ++m) a[m] = a_next[m];
  }
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int local = m * 16 + 4 * kq + i;
      if (local >= rows) continue;
      float* out = y + (size_t)places[begin + local] * width;
#pragma unroll
      for (int t = 0; t < 2; ++t)
        if (col0 + t * 16 + r < width) out[col0 + t * 16 + r] = acc[m][t][i];
    }
}

// The two products for steps with many pairs an expert (bfloat16, tiles of 64 pairs, rows of whole 16-byte pieces): a
// block of eight waves makes 64 pairs by 256 result columns, a wave 32 by 64 (8 tiles of 16 x 16,
// v_mfma_f32_16x16x32_bf16).  A stage is 64 columns of K: every thread fetches its 16-byte pieces of the stage's A rows
// (64 x 128 bytes) and B rows (256 x 128 bytes: whole cache lines) into registers while the two stages before are
// multiplied, then the block puts them into LDS
// (rows 144 bytes apart, so that the 16 rows of a fragment read fall on all banks) and the waves read their fragments
// from there: a weight is read from memory once a block, a pair's row once a block.
// GATED: A rows are the pairs' rows of x, the result columns are 128 gate columns and the same 128 up columns of the
// expert (a wave owns 32 of each), and the block writes act(gate, up) for 128 hidden columns.  Otherwise A rows are the
// places' rows of hidden, the result columns are 256 of the expert's down matrix, written to the pairs' rows of y.
#define MOE_TILE_ROW 144                                  // bytes of a staged row: 128 and 16 to spread the banks
#define MOE_TILE_LDS ((64 + 256) * MOE_TILE_ROW)
#define MOE_TILE_THREADS 512
struct MoeFetched { qil_u32x4 a, b[4]; };                 // a thread's pieces of one stage: one of A, four of B
template <bool GATED>
__global__ void __launch_bounds__(MOE_TILE_THREADS, 2)
moe_tile_kernel(const bf16_t* __restrict__ a_base, const bf16_t* __restrict__ w, int K, int columns,
                const int* __restrict__ tiles, int max_tiles, const int* __restrict__ places, int top,
                bf16_t* __restrict__ hidden, float* __restrict__ y, int act, float limit, float alpha, int column_blocks) {
  extern __shared__ __align__(16) unsigned char tile_lds[];
  unsigned char* a_lds = tile_lds;
  unsigned char* b_lds = tile_lds + 64 * MOE_TILE_ROW;
  // Blocks go to the chip's 8 XCDs in turn, and every XCD has an L2 of its own: the block numbers are turned so that
  // an XCD works through a run of (column block, tile) pairs with the tile moving fastest.  The tiles of one expert
  // follow each other, so its weights come from memory once an XCD and from that XCD's L2 for the expert's other tiles
  // (numbered in launch order, every XCD fetched every expert's weights: 2.2 GB through the fabric for 0.6 GB of weights).
  const int per_xcd = gridDim.x / 8;
  const int turned = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (turned >= max_tiles * column_blocks) return;
  const int tile = turned % max_tiles, column_block = turned / max_tiles;
  const int rows = tiles[2 * max_tiles + tile];
  if (rows == 0) return;
  const int e = tiles[tile], begin = tiles[max_tiles + tile];
  const int tid = threadIdx.x, lane = tid & (QIL_WAVE - 1), wave = tid / QIL_WAVE;
  const int r = lane & 15, kq = lane >> 4;
  const int half = wave >> 2, quarter = wave & 3;         // the wave's 32 of the 64 pairs, its 64 of the 256 columns
  const int c0 = column_block * (GATED ? 128 : 256);      // first hidden column, or first output column
  // what this thread fetches of a stage: piece tid % 8 of row tid / 8 of A and of the rows tid / 8 + 64 j of B
  const int piece = tid & 7, row0 = tid >> 3;
  const int local0 = min(row0, rows - 1);
  const bf16_t* a_src = GATED ? a_base + (size_t)(places[begin + local0] / top) * K : a_base + (size_t)(begin + local0) * K;
  const bf16_t* b_src[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int rb = row0 + 64 * j;
    if (GATED) b_src[j] = w + ((size_t)(e * 2 + (rb >> 7)) * columns + min(c0 + (rb & 127), columns - 1)) * K;
    else b_src[j] = w + ((size_t)e * columns + min(c0 + rb, columns - 1)) * K;
  }
  auto fetch = [&](MoeFetched& f, int k0) {
    const int k = k0 + piece * 8;
    const bool inside = k < K;
    f.a = inside ? *reinterpret_cast<const qil_u32x4*>(a_src + k) : (qil_u32x4){0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 4; ++j)
      f.b[j] = inside ? *reinterpret_cast<const qil_u32x4*>(b_src[j] + k) : (qil_u32x4){0u, 0u, 0u, 0u};
  };
  auto put = [&](const MoeFetched& f) {
    *reinterpret_cast<qil_u32x4*>(a_lds + row0 * MOE_TILE_ROW + piece * 16) = f.a;
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<qil_u32x4*>(b_lds + (row0 + 64 * j) * MOE_TILE_ROW + piece * 16) = f.b[j];
  };
  // the rows of B whose tiles this wave multiplies: GATED 32 gate rows and the 32 up rows of the same columns
  int b_tile[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) b_tile[t] = GATED ? (t >> 1) * 128 + quarter * 32 + (t & 1) * 16 : quarter * 64 + t * 16;
  moe_f32x4 acc[2][4];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[m][t] = (moe_f32x4){0.f, 0.f, 0.f, 0.f};
  auto multiply = [&]() {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      qil_u32x4 a[2], b[4];
#pragma unroll
      for (int m = 0; m < 2; ++m)
        a[m] = *reinterpret_cast<const qil_u32x4*>(a_lds + (half * 32 + m * 16 + r) * MOE_TILE_ROW + ks * 64 + kq * 16);
#pragma unroll
      for (int t = 0; t < 4; ++t)
        b[t] = *reinterpret_cast<const qil_u32x4*>(b_lds + (b_tile[t] + r) * MOE_TILE_ROW + ks * 64 + kq * 16);
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int t = 0; t < 4; ++t) Frag<bf16_t>::mma(acc[m][t], a[m], b[t]);
    }
  };
  // two stages are on their way while a stage is multiplied (a trip to memory takes longer than one stage's products)
  MoeFetched even, odd;
  fetch(even, 0);
  fetch(odd, 64);
  for (int k0 = 0; k0 < K; k0 += 128) {
    __syncthreads();                                      // the stage before has been read
    put(even);
    __syncthreads();
    fetch(even, k0 + 128);                                // (past the end: zeros, no access)
    multiply();
    if (k0 + 64 < K) {
      __syncthreads();
      put(odd);
      __syncthreads();
      fetch(odd, k0 + 192);
      multiply();
    }
  }
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int local = half * 32 + m * 16 + 4 * kq + i;
      if (local >= rows) continue;
      if (GATED) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int col = c0 + quarter * 32 + t * 16 + r;
          if (col < columns) st(hidden + (size_t)(begin + local) * columns + col, gated_act(acc[m][t][i], acc[m][2 + t][i], act, limit, alpha));
        }
      } else {
        float* out = y + (size_t)places[begin + local] * columns;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int col = c0 + quarter * 64 + t * 16 + r;
          if (col < columns) out[col] = acc[m][t][i];
        }
      }
    }
}

// out[n, c] = sum over slots, in slot order, of weight * (identity expert ? x[n, c] : y[n * top + slot, c])
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ x, const float* __restrict__ y, const int* __restrict__ chosen,
                                   const float* __restrict__ weights, int experts, int top, int width,
                                   float* __restrict__ out) {
  const int n = blockIdx.x;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float sum = 0.f;
    for (int slot = 0; slot < top; ++slot) {
      const size_t pair = (size_t)n * top + slot;
      const float value = chosen[pair] >= experts ? ld(x + (size_t)n * width + c) : y[pair * width + c];
      sum += weights[pair] * value;
    }
    out[(size_t)n * width + c] = sum;
  }
}

extern "C" {

int qil_moe_takes(int width, int outputs, int experts, int groups, int keep, int top) {
  return width >= 1 && outputs >= 1 && outputs <= MOE_MAX_OUTPUTS && experts >= 0 && experts <= outputs && groups >= 1 &&
         outputs % groups == 0 && keep >= 1 && keep <= groups && top >= 1 && top <= outputs && top <= QIL_WAVE &&
         (size_t)(MOE_ROUTE_THREADS / QIL_WAVE) * (2 * outputs + groups) * sizeof(float) <= 64 * 1024;
}

// x [n, width] (dtype), w_router float32 [outputs, width], bias and correction float32 [outputs] or null -> chosen
// int32 [n, top], weights float32 [n, top].  logits: float32 scratch [n, outputs].
// sigmoid_scores: scores are sigmoid(logit) instead of the softmax over all outputs.  group_top2: a group's score is
// the sum of its two largest choice scores instead of its largest.  The weights are the chosen scores, divided by
// (their sum + renormalize_eps) if renormalize, times weight_scale.
int qil_moe_route(const void* x, int dtype, const float* w_router, const float* bias, const float* correction,
                  float* logits, int* chosen,
                  float* weights, int n, int width, int outputs, int groups, int keep, int top, int renormalize,
                  int sigmoid_scores, int group_top2, float weight_scale, float renormalize_eps, hipStream_t s) {
  if (n == 0) return 0;
  if (!qil_moe_takes(width, outputs, 0, groups, keep, top) || !logits) return -1;
  const dim3 g_logits((n + 7) / 8, (outputs + 3) / 4);
  const bool vec = width % 4 == 0 && (((uintptr_t)x | (uintptr_t)w_router) % 16) == 0;
#define QIL_LOGITS(T, VEC)                                                                                            \
  hipLaunchKernelGGL((moe_logits_kernel<T, VEC>), g_logits, dim3(MOE_ROUTE_THREADS), 0, s, (const T*)x, n, width,      \
                     w_router, outputs, logits)
  if (dtype == QIL_F32) { if (vec) QIL_LOGITS(float, true); else QIL_LOGITS(float, false); }
  else { if (vec) QIL_LOGITS(bf16_t, true); else QIL_LOGITS(bf16_t, false); }
#undef QIL_LOGITS
  const int per_block = MOE_ROUTE_THREADS / QIL_WAVE;
  const size_t lds = (size_t)per_block * (2 * outputs + groups) * sizeof(float);
  hipLaunchKernelGGL(moe_select_kernel, dim3((n + per_block - 1) / per_block), dim3(MOE_ROUTE_THREADS), lds, s, logits, n,
                     bias, correction, outputs, groups, keep, top, renormalize, chosen, weights, sigmoid_scores, group_top2,
                     weight_scale, renormalize_eps);
  QIL_RETURN_LAUNCH_STATUS();
}

// Rows a tile of pairs holds for a step of `pairs` pairs over `experts` experts: 16, or 64 when an expert's share
// fills such tiles.
int qil_moe_tile_rows(int pairs, int experts) { return experts > 0 && pairs / experts >= 48 ? 64 : 16; }
int qil_moe_max_tiles(int pairs, int experts, int tile_rows) { return (pairs + tile_rows - 1) / tile_rows + experts; }

// The experts' work on the routed pairs: x [n, width], chosen/weights [n, top]; w_gate_up [experts][2][ff][width],
// w_down [experts][width][ff] (dtype); scratch: tiles int32 [3 * max_tiles], places int32 [n * top], hidden (dtype)
// [n * top, ff], y float32 [n * top, width].  out float32 [n, width], or null: the pairs' rows stay in y for a consumer
// that makes the weighted sum itself.
int qil_moe_experts(const void* x, int dtype, const int* chosen, const float* weights, const void* w_gate_up,
                    const void* w_down, int* tiles, int* places, void* hidden, float* y, float* out, int n, int width,
                    int ff, int experts, int top, int tile_rows, int max_tiles, int act, float limit, float alpha,
                    hipStream_t s) {
  if (n == 0) return 0;
  const int pairs = n * top;
  if (experts > MOE_MAX_OUTPUTS || (tile_rows != 16 && tile_rows != 64) ||
      max_tiles < qil_moe_max_tiles(pairs, experts, tile_rows) || width < 1 || ff < 1)
    return -1;
  if (experts > 0) {
    hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), 0, s, chosen, pairs, experts, tile_rows, max_tiles, tiles,
                       places);
    const int epl = dtype == QIL_F32 ? 4 : 8;
    const bool aligned = width % epl == 0 && ff % epl == 0 &&
                         (((uintptr_t)x | (uintptr_t)w_gate_up | (uintptr_t)w_down | (uintptr_t)hidden) % 16) == 0;
    const dim3 g_up(max_tiles, (ff + 63) / 64), g_down(max_tiles, (width + 127) / 128);
    if (dtype == QIL_BF16 && tile_rows == 64 && aligned && width % 8 == 0 && ff % 8 == 0) {
      static bool granted = false;                        // (both instantiations, once)
      if (!granted) {
        hipError_t a = hipFuncSetAttribute((const void*)moe_tile_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, MOE_TILE_LDS);
        hipError_t b = hipFuncSetAttribute((const void*)moe_tile_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, MOE_TILE_LDS);
        if (a != hipSuccess || b != hipSuccess) return (int)(a != hipSuccess ? a : b);
        granted = true;
      }
      const int up_blocks = (ff + 127) / 128, down_blocks = (width + 255) / 256;
      hipLaunchKernelGGL(moe_tile_kernel<true>, dim3(((size_t)max_tiles * up_blocks + 7) / 8 * 8), dim3(MOE_TILE_THREADS),
                         MOE_TILE_LDS, s, (const bf16_t*)x, (const bf16_t*)w_gate_up, width, ff, tiles, max_tiles, places,
                         top, (bf16_t*)hidden, (float*)nullptr, act, limit, alpha, up_blocks);
      hipLaunchKernelGGL(moe_tile_kernel<false>, dim3(((size_t)max_tiles * down_blocks + 7) / 8 * 8), dim3(MOE_TILE_THREADS),
                         MOE_TILE_LDS, s, (const bf16_t*)hidden, (const bf16_t*)w_down, ff, width, tiles, max_tiles, places,
                         top, (bf16_t*)nullptr, y, act, limit, alpha, down_blocks);
    } else {
#define QIL_MOE(T, MT, ALIGNED)                                                                                       \
  do {                                                                                                                \
    hipLaunchKernelGGL((moe_gate_up_kernel<T, MT, ALIGNED>), g_up, dim3(256), 0, s, (const T*)x, width,                \
                       (const T*)w_gate_up, ff, tiles, max_tiles, places, top, (T*)hidden, act, limit, alpha);         \
    hipLaunchKernelGGL((moe_down_kernel<T, MT, ALIGNED>), g_down, dim3(256), 0, s, (const T*)hidden, ff,               \
                       (const T*)w_down, width, tiles, max_tiles, places, y);                                          \
  } while (0)
#define QIL_MOE_T(T)                                                                                                  \
  do {                                                                                                                \
    if (tile_rows == 64) { if (aligned) QIL_MOE(T, 4, true); else QIL_MOE(T, 4, false); }                              \
    else { if (aligned) QIL_MOE(T, 1, true); else QIL_MOE(T, 1, false); }                                              \
  } while (0)
    if (dtype == QIL_F32) QIL_MOE_T(float); else QIL_MOE_T(bf16_t);
#undef QIL_MOE_T
#undef QIL_MOE
    }
  }
  if (!out) QIL_RETURN_LAUNCH_STATUS();                  // the caller's next norm makes the weighted sum itself
  const int threads = width >= 1024 ? 256 : 64;
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, dim3(n), dim3(threads), 0, s, (const float*)x, y, chosen, weights,
                       experts, top, width, out);
  else
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, dim3(n), dim3(threads), 0, s, (const bf16_t*)x, y, chosen, weights,
                       experts, top, width, out);
  QIL_RETURN_LAUNCH_STATUS();
}

// The weighted sum alone (what qil_moe_experts ends with when it is given an `out`).
int qil_moe_combine(const void* x, int dtype, const float* y, const int* chosen, const float* weights, float* out, int n,
                    int width, int experts, int top, hipStream_t s) {
  if (n == 0) return 0;
  const int threads = width >= 1024 ? 256 : 64;
  if (dtype == QIL_F32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, dim3(n), dim3(threads), 0, s, (const float*)x, y, chosen, weights,
                       experts, top, width, out);
  else
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, dim3(n), dim3(threads), 0, s, (const bf16_t*)x, y, chosen, weights,
                       experts, top, width, out);
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
