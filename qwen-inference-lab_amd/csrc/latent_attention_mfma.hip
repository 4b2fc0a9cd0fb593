// Attention over a cached latent on the matrix cores (bfloat16 caches): the arithmetic of latent_attention.hip,
//     score(h, j) = scale * (qa_h . c_j + qr_h . kr_j),   u_h = sum_j p(h, j) c_j,   a sink logit in the denominator,
// with v_mfma_f32_16x16x32_bf16.  Every head reads the same cached row [c_j ; kr_j], so a block stages a tile of 32
// keys in LDS once and serves up to 64 query columns with it: a column is a (row, head) pair, the block's columns
// are `rt` consecutive rows of one sequence times `hb` heads.  A wave owns 16 columns:
//
//   S^T[key, column] = sum_dim K[key, dim] Q[column, dim]       A = staged key rows, B = the wave's queries (registers)
//   U^T[dim, column] = sum_key C^T[dim, key] P^T[key, column]    A = the tile's latents transposed, B = probabilities
//
// The value of a key is its own latent, so the same staged tile feeds both products; the second needs it with the
// keys along a row, and the staging writes that transposed copy beside the plain one.  Row r of a 16-key score
// sub-tile is key 8 (r / 4) + 4 jt + r % 4 of the 32-key step, so that a lane's eight scores are the eight consecutive
// keys 8 kb .. 8 kb + 7 and go into the second product's B operand as they are.  Scores, maxima, exponentials, sums
// and results are float32; probabilities enter the second product as bfloat16.
//
// With few blocks the keys go in parts (grid.z): a block leaves (reference, sum, unnormalised result) per column and
// part, and latent_merge_kernel finishes, which is also where the sink enters then.
// A window w > 0 hides the keys j <= position - w of a row: a block begins at the oldest key its first row sees, a
// part that no row of the block sees is left out, and the merge reads the parts between a row's oldest key and its
// position.  An output gate (a float32 factor per row and head) multiplies the finished column.
//
// Takes rank % 16 == 0, rot % 8 == 0, rank + rot <= 640, rank <= 512; other sizes run on the general kernel.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define LM_THREADS 256
#define LM_KEYS 32
#define LM_VROW (LM_KEYS + 8)                               // elements of a row of the transposed tile (80 bytes)
#define LOG2E 1.44269504088896f
#define LM_AHEAD 8                                          // LDS fragments asked for ahead of the product that takes them
#define LM_SLACK 5.5f                                      // how far a score may pass the exponentials' reference

// EXACT: the sizes are the template's (rank + rot == 32 QF up to padding, rank == 16 VT): no size guards the products.
// SPLIT (steps of single rows): the block's columns are at most 16, one wave's; every wave takes the scores of all of
// them and a quarter of the latent's dims in the second product, so that four waves work where one would, each holds
// a quarter of the sums, and two blocks fit a compute unit.
template <int QF, int VT, bool EXACT, bool SPLIT>
__global__ void __launch_bounds__(LM_THREADS, SPLIT ? 2 : 1)
latent_mfma_kernel(const float* __restrict__ q, const bf16_t* __restrict__ latent, const bf16_t* __restrict__ rope,
                   const int* __restrict__ tables, int table_stride, const int* __restrict__ cu_seqlens,
                   const int* __restrict__ seq_starts, int n_seqs, int single, const float* __restrict__ sink,
                   const float* __restrict__ gate, float* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_m,
                   float* __restrict__ part_l, int heads, int rank, int rot, int page_size, float scale, int rt, int hb,
                   int P, int parts, int window) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int d = rank + rot;
  const int qf = EXACT ? QF : (d + 31) / 32, vt = EXACT ? VT : rank / 16;
  const int dp = qf * 32, krow = dp + 8;
  bf16_t* ks = reinterpret_cast<bf16_t*>(smem);            // [32 keys][krow]: c then kr then zeros
  bf16_t* vts = ks + LM_KEYS * krow;                        // [rank][LM_VROW]: the latents, keys along a row

  // which rows: tile `tile` of rt rows of sequence s
  int s = 0, tile = gridDim.x - 1 - blockIdx.x;             // the last tiles see the most keys: they start first
  if (single) {
    s = blockIdx.x;
    tile = 0;
  } else {
    for (; s < n_seqs; ++s) {
      const int tiles = (cu_seqlens[s + 1] - cu_seqlens[s] + rt - 1) / rt;
      if (tile < tiles) break;
      tile -= tiles;
    }
  }
  if (s >= n_seqs) return;
  const int seq_row0 = cu_seqlens[s], seq_rows = cu_seqlens[s + 1] - seq_row0, start = seq_starts[s];
  const int r0 = tile * rt, rows_here = min(rt, seq_rows - r0);
  const int last_pos = start + r0 + rows_here - 1;
  const int h0 = blockIdx.y * hb, heads_here = min(hb, heads - h0);
  const int part = blockIdx.z;
  const int oldest = window > 0 ? max(0, start + r0 - window + 1) : 0;     // of the tile's first row, which sees furthest back
  const int begin = max(part * P, oldest), end = min((part + 1) * P, last_pos + 1);
  if (begin >= end) return;                                 // no row of the tile sees this part; the merge does not read it
  const int* table = tables + (size_t)s * table_stride;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, kb = lane >> 4;
  const int column = (SPLIT ? 0 : wave * 16) + r, ci = column / hb, ch = column - ci * hb;
  const bool valid = ci < rows_here && ch < heads_here && column < rt * hb;
  const bool working = SPLIT || wave * 16 < rt * hb;        // wave-uniform: this wave has columns at all
  constexpr int VTW = SPLIT ? VT / 4 : VT;                  // tiles of 16 dims of the sums that this wave holds
  const int t0 = SPLIT ? wave * VTW : 0;
  const int grow = seq_row0 + r0 + (valid ? ci : 0), head = h0 + (valid ? ch : 0);
  const int pos = valid ? start + r0 + ci : -1;
  const int low = window > 0 ? pos - window + 1 : 0;        // the column's oldest visible key (<= 0: from the start)
  const size_t gcol = (size_t)grow * heads + head;

  bf16x8 qb[QF];
  {
    const float* qrow = q + gcol * d;
    const bool wide = d % 4 == 0;                           // rows start on 16 bytes: two 16-byte reads a fragment
#pragma unroll
    for (int f = 0; f < QF; ++f) {
      float x[8];
      const int dim0 = 32 * f + 8 * kb;
      if (wide && valid && f < qf && dim0 + 8 <= d) {
        const float4 a = *reinterpret_cast<const float4*>(qrow + dim0), b = *reinterpret_cast<const float4*>(qrow + dim0 + 4);
        x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w, x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] = (valid && f < qf && dim0 + e < d) ? qrow[dim0 + e] : 0.f;
      }
      qb[f] = __builtin_bit_cast(bf16x8, make_uint4(pack_bf16(x[0], x[1]), pack_bf16(x[2], x[3]), pack_bf16(x[4], x[5]),
                                                    pack_bf16(x[6], x[7])));
    }
  }
  float m = -INFINITY, l = 0.f;
  if (parts == 1 && sink && valid) {                       // the sink: maximum s_h, sum 1 (held once a column), result 0
    m = sink[head];
    l = kb == 0 ? 1.f : 0.f;
  }
  f32x4 o[VTW];
#pragma unroll
  for (int t = 0; t < VTW; ++t) o[t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // Staging: a unit is two neighbouring keys by eight dims; a thread owns one pair of keys (jp) and the chunks
  // c0, c0 + 16, ... of their rows, and fetches its units of the next step into registers while this step's products
  // run.  The keys' places in the cache (a table entry, a division) are found once a step and a step further ahead
  // than the rows themselves, so that a row's read never waits for its table entry.  The transposed copy takes a word
  // per dim: the two keys' elements side by side, so that a wave's writes spread over the banks (a 2-byte write per
  // key put 32 lanes on one bank).
  constexpr int CSTEP = LM_THREADS / (LM_KEYS / 2);
  constexpr int NU = (QF * 4 + CSTEP - 1) / CSTEP;
  const int chunks = dp / 8, jp = tid % (LM_KEYS / 2), c0 = tid / (LM_KEYS / 2);
  uint4 ahead[NU][2];
  int place[2];                                             // the cache slots of keys 2 jp, 2 jp + 1 of a step; -1: none
  auto lookup = [&](int j0) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int key = j0 + 2 * jp + e;
      place[e] = key < end ? table[key / page_size] * page_size + key % page_size : -1;
    }
  };
  auto fetch = [&]() {
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      const int chunk = c0 + CSTEP * u, dim = chunk * 8;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (chunk < chunks && place[e] >= 0 && dim < d)
          v = dim < rank ? *reinterpret_cast<const uint4*>(latent + (size_t)place[e] * rank + dim)
                         : *reinterpret_cast<const uint4*>(rope + (size_t)place[e] * rot + (dim - rank));
        ahead[u][e] = v;
      }
    }
  };
  lookup(begin);
  fetch();
  lookup(begin + LM_KEYS);
  for (int j0 = begin; j0 < end; j0 += LM_KEYS) {
    __syncthreads();                                        // the last step's reads are done
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      const int chunk = c0 + CSTEP * u, dim = chunk * 8;
      if (chunk < chunks) {
        const uint4 a = ahead[u][0], b = ahead[u][1];
        *reinterpret_cast<uint4*>(ks + (2 * jp) * krow + dim) = a;
        *reinterpret_cast<uint4*>(ks + (2 * jp + 1) * krow + dim) = b;
        if (dim < rank) {
          const uint32_t wa[4] = {a.x, a.y, a.z, a.w}, wb[4] = {b.x, b.y, b.z, b.w};
          uint32_t* column = reinterpret_cast<uint32_t*>(vts) + jp;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            column[(dim + 2 * e) * (LM_VROW / 2)] = (wa[e] & 0xffffu) | (wb[e] << 16);
            column[(dim + 2 * e + 1) * (LM_VROW / 2)] = (wa[e] >> 16) | (wb[e] & 0xffff0000u);
          }
        }
      }
    }
    __syncthreads();
    if (j0 + LM_KEYS < end) {
      fetch();
      lookup(j0 + 2 * LM_KEYS);
    }
    if (!working) continue;
    // ---- scores: the two sub-tiles' sums side by side; eight fragments of the staged keys are on their way from LDS
    // before the first product, one more is asked for with every product
    f32x4 sc[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    {
      const bf16_t* krow_p = ks + (8 * (r >> 2) + (r & 3)) * krow + 8 * kb;     // sub-tile 0; sub-tile 1 is four keys on
#pragma unroll
      for (int f = 0; f < QF; ++f)
        if (EXACT || f < qf) {
          sc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(krow_p + 32 * f), qb[f], sc[0], 0, 0, 0);
          sc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(krow_p + 4 * krow + 32 * f), qb[f],
                                                          sc[1], 0, 0, 0);
        }
      if constexpr (EXACT && !SPLIT) {
        __builtin_amdgcn_sched_group_barrier(0x100, LM_AHEAD, 0);
#pragma unroll
        for (int i = 0; i < 2 * QF - LM_AHEAD; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, LM_AHEAD, 0);
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int jt = 0; jt < 2; ++jt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = j0 + 8 * kb + 4 * jt + i;
        const float v = (key <= pos && key >= low && key < end) ? sc[jt][i] * scale : -INFINITY;
        sc[jt][i] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, QIL_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, QIL_WAVE));
    // The exponentials' reference m is a column's maximum as of some earlier step: it is raised, and the sums
    // rescaled, only when a score passes it by more than LM_SLACK (so p <= exp(LM_SLACK), which float32 sums and
    // bfloat16 probabilities hold as well as p <= 1).  In most steps no column of the wave rescales, and the
    // accumulators stay where the matrix cores keep them.
    const float m_new = (mx > m + LM_SLACK) ? mx : m;
    if (__builtin_amdgcn_ballot_w64(m_new != m) != 0) {     // wave-uniform
      asm volatile("" ::: "memory");                        // keeps this a branch: the multiplications are not speculated
      const float alpha = (m_new == m) ? 1.f : __builtin_amdgcn_exp2f((m - m_new) * LOG2E);
      l *= alpha;
#pragma unroll
      for (int t = 0; t < VTW; ++t)
        if (EXACT || t0 + t < vt) {
#pragma unroll
          for (int i = 0; i < 4; ++i) o[t][i] *= alpha;
        }
      m = m_new;
    }
    float psum = 0.f;
#pragma unroll
    for (int jt = 0; jt < 2; ++jt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = (sc[jt][i] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((sc[jt][i] - m) * LOG2E);
        sc[jt][i] = p;
        psum += p;
      }
    l += psum;
    // ---- U^T += C^T P^T
    const bf16x8 pb = __builtin_bit_cast(bf16x8, make_uint4(pack_bf16(sc[0][0], sc[0][1]), pack_bf16(sc[0][2], sc[0][3]),
                                                            pack_bf16(sc[1][0], sc[1][1]), pack_bf16(sc[1][2], sc[1][3])));
#pragma unroll
    for (int t = 0; t < VTW; ++t)
      if (EXACT || t0 + t < vt)
        o[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(vts + (16 * (t0 + t) + r) * LM_VROW + 8 * kb),
                                                       pb, o[t], 0, 0, 0);
    if constexpr (EXACT && !SPLIT) {                                  // fragments ahead of the products, as for the scores
      __builtin_amdgcn_sched_group_barrier(0x100, LM_AHEAD, 0);
#pragma unroll
      for (int i = 0; i < VTW - LM_AHEAD; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, LM_AHEAD, 0);
    }
  }
  if (!working) return;
  l += __shfl_xor(l, 16, QIL_WAVE);
  l += __shfl_xor(l, 32, QIL_WAVE);
  if (!valid) return;
  if (parts == 1) {
    const float inv = (gate ? gate[gcol] : 1.f) / l;
    float* dst = out + gcol * rank + 16 * t0 + 4 * kb;
#pragma unroll
    for (int t = 0; t < VTW; ++t)
      if (EXACT || t0 + t < vt)
        *reinterpret_cast<float4*>(dst + 16 * t) = make_float4(o[t][0] * inv, o[t][1] * inv, o[t][2] * inv, o[t][3] * inv);
    return;
  }
  const size_t cell = gcol * parts + part;
  if (kb == 0 && (!SPLIT || wave == 0)) {
    part_m[cell] = m;
    part_l[cell] = l;
  }
  float* dst = part_acc + cell * rank + 16 * t0 + 4 * kb;
#pragma unroll
  for (int t = 0; t < VTW; ++t)
    if (EXACT || t0 + t < vt) *reinterpret_cast<float4*>(dst + 16 * t) = make_float4(o[t][0], o[t][1], o[t][2], o[t][3]);
}

// out[column] = sum_p w_p acc_p / (sum_p w_p l_p + exp(sink - M)), w_p = exp(m_p - M), M the largest of the parts'
// references and the sink, over the parts that the row's position reaches.  One block per (row, head); the parts'
// weights are made once, side by side, and kept in LDS (`parts` floats of dynamic LDS), so that the sums below wait
// for no value that another read has to bring first.
__global__ void latent_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_m,
                                    const float* __restrict__ part_l, const int* __restrict__ positions,
                                    const float* __restrict__ sink, const float* __restrict__ gate,
                                    float* __restrict__ out, int heads, int rank, int P, int parts, int window) {
  extern __shared__ float weight[];
  __shared__ float scratch[16];
  const int n = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, nt = blockDim.x;
  const size_t column = (size_t)n * heads + h;
  const int reached = min(parts, positions[n] / P + 1);
  const int from = window > 0 ? max(0, positions[n] - window + 1) / P : 0;     // the part of the row's oldest visible key
  const float floor_ = sink ? sink[h] : -INFINITY;
  float top = floor_;
  for (int p = from + tid; p < reached; p += nt) {
    const float mp = part_m[column * parts + p];
    weight[p] = mp;
    top = fmaxf(top, mp);
  }
  top = block_max(top, scratch);
  float below = (sink && tid == 0) ? expf(floor_ - top) : 0.f;
  for (int p = from + tid; p < reached; p += nt) {          // a thread rereads only what it wrote
    const float mp = weight[p], w = mp > -INFINITY ? expf(mp - top) : 0.f;
    weight[p] = w;
    below += w * part_l[column * parts + p];
  }
  below = block_sum(below, scratch);                        // its barriers also publish the weights
  const float inv = (gate ? gate[column] : 1.f) / below;
  const float* acc_p = part_acc + column * parts * rank;
  for (int c = tid; c < rank; c += nt) {
    float acc = 0.f;
#pragma unroll 4
    for (int p = from; p < reached; ++p) acc += weight[p] * acc_p[(size_t)p * rank + c];
    out[column * rank + c] = acc * inv;
  }
}

static int lm_lds_bytes(int rank, int rot) {
  const int dp = (rank + rot + 31) / 32 * 32;
  return (LM_KEYS * (dp + 8) + rank * LM_VROW) * (int)sizeof(bf16_t);
}

template <int QF, int VT, bool EXACT, bool SPLIT>
static int lm_launch(dim3 grid, size_t lds, hipStream_t s, const float* q, const bf16_t* latent, const bf16_t* rope,
                     const int* tables, int table_stride, const int* cu_seqlens, const int* seq_starts, int n_seqs,
                     int single, const float* sink, const float* gate, float* out, float* part_acc, float* part_m,
                     float* part_l, int heads, int rank, int rot, int page_size, float scale, int rt, int hb, int P, int parts,
                     int window) {
  auto kernel = latent_mfma_kernel<QF, VT, EXACT, SPLIT>;
  static bool raised = false;                                // per instantiation
  if (lds > 64 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return (int)e;
    raised = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(LM_THREADS), lds, s, q, latent, rope, tables, table_stride, cu_seqlens, seq_starts,
                     n_seqs, single, sink, gate, out, part_acc, part_m, part_l, heads, rank, rot, page_size, scale, rt, hb,
                     P, parts, window);
  return 0;
}

extern "C" {

int qil_latent_mfma_takes(int heads, int rank, int rot) {
  return heads >= 1 && rank >= 16 && rank % 16 == 0 && rot >= 0 && rot % 8 == 0 && rank + rot <= 640 && rank <= 512 &&
         lm_lds_bytes(rank, rot) <= 160 * 1024;
}

// (rows a block, heads a block, keys a part, parts) for a step: blocks of up to 64 columns (16 where every sequence
// has one row: the split form); the keys in parts of at least 64 while the blocks are fewer than two a compute unit.
// With a window a block walks at most the window and its own rows, so that span is what the parts divide; parts
// still count from key 0 (those outside every row's window do nothing).
void qil_latent_mfma_plan(int n_rows, int n_seqs, int single, int heads, int max_context, int window, int* rt, int* hb,
                          int* P, int* parts) {
  const int most = single ? 16 : 64;                          // single rows: one wave's columns a block
  *hb = heads < most ? heads : most;
  *rt = single ? 1 : (64 / *hb > 0 ? 64 / *hb : 1);
  const int tiles = single ? n_seqs : (n_rows + *rt - 1) / *rt + n_seqs;
  const long blocks = (long)tiles * ((heads + *hb - 1) / *hb);
  int want = (int)((2 * QIL_CUS + blocks - 1) / blocks);
  if (want < 1) want = 1;
  int span = max_context;                                     // what a block walks when it walks everything its rows see
  if (want > 1 && window > 0 && window + *rt - 1 < span) span = window + *rt - 1;
  int part = ((span + want - 1) / want + 31) / 32 * 32;      // (enough blocks: one part, and a block begins at its window)
  if (part < 64) part = 64;                                   // two steps a block: shorter parts cost more in the merge than they save
  *P = part;
  *parts = (max_context + part - 1) / part;
  if (*parts < 1) *parts = 1;
}

size_t qil_latent_mfma_workspace(int n_rows, int heads, int rank, int parts) {
  return parts > 1 ? (size_t)n_rows * heads * parts * (rank + 2) * sizeof(float) : 0;
}

// q float32 [n_rows, heads, rank + rot]; out float32 [n_rows, heads, rank]; workspace as qil_latent_mfma_workspace says.
// single: every sequence has one row (n_seqs == n_rows).  rt, hb, P, parts: as qil_latent_mfma_plan gave them.
int qil_latent_mfma(const float* q, const void* latent, const void* rope, const int* tables, int table_stride,
                    const int* cu_seqlens, const int* seq_starts, const int* positions, const float* sink,
                    const float* gate, float* out, float* workspace, int n_rows, int n_seqs, int single, int heads, int rank,
                    int rot, int page_size, float scale, int window, int rt, int hb, int P, int parts, hipStream_t s) {
  if (n_rows == 0) return 0;
  if (!qil_latent_mfma_takes(heads, rank, rot) || page_size < 1 || rt < 1 || hb < 1 || rt * hb > (single ? 16 : 64) || P < 32 || P % 32 ||
      parts < 1 || parts > 8192 || (single && n_seqs != n_rows) || (parts > 1 && !workspace))
    return -1;
  const int tiles = single ? n_seqs : (n_rows + rt - 1) / rt + n_seqs;
  dim3 grid(tiles, (heads + hb - 1) / hb, parts);
  const size_t lds = (size_t)lm_lds_bytes(rank, rot);
  float* part_acc = workspace;
  float* part_m = parts > 1 ? workspace + (size_t)n_rows * heads * parts * rank : nullptr;
  float* part_l = parts > 1 ? part_m + (size_t)n_rows * heads * parts : nullptr;
  const int qf = (rank + rot + 31) / 32, vt = rank / 16;
  int status;
#define QIL_LM_ARGS                                                                                                  \
  grid, lds, s, q, (const bf16_t*)latent, (const bf16_t*)rope, tables, table_stride, cu_seqlens, seq_starts, n_seqs, \
      single, parts == 1 ? sink : nullptr, parts == 1 ? gate : nullptr, out, part_acc, part_m, part_l, heads, rank, rot,     \
      page_size, scale, rt, hb, P, parts, window
#define QIL_LM(QF, VT, EXACT) \
  status = single ? lm_launch<QF, VT, EXACT, true>(QIL_LM_ARGS) : lm_launch<QF, VT, EXACT, false>(QIL_LM_ARGS)
  if (qf == 18 && vt == 32) QIL_LM(18, 32, true);
  else if (qf <= 8 && vt <= 8) QIL_LM(8, 8, false);
  else if (qf <= 12 && vt <= 16) QIL_LM(12, 16, false);
  else QIL_LM(20, 32, false);
#undef QIL_LM
#undef QIL_LM_ARGS
  if (status) return status;
  if (parts > 1)
    hipLaunchKernelGGL(latent_merge_kernel, dim3(n_rows, heads), dim3(rank >= 256 ? 256 : 64), parts * sizeof(float), s, part_acc, part_m,
                       part_l, positions, sink, gate, out, heads, rank, P, parts, window);
  QIL_RETURN_LAUNCH_STATUS();
}

}  // extern "C"
