// Paged attention on the vector units, for every size: any page size, head_dim in steps of 16 up
// to 256, any number of heads and groups, portions of prompts beside single decoded tokens.
// All arithmetic is 32-bit whatever the storage type, so this is the attention of the true 32-bit
// path and the fallback of the bf16 path for shapes that the matrix-core kernels refuse.
//
// One workgroup takes BM consecutive queries of one request (one "tile") and one query head, and
// walks that request's keys in tiles of BN through its block table with an online softmax
// (running maximum m, running sum l, accumulator rescaled by exp(m_old - m_new)).
//
// A query at absolute position p sees key j iff j <= p and (window <= 0 or j > p - window).
// Scores are scaled by `scale` (1/sqrt(head_dim) in the reference: src/dli/model/llama.py:165-177,
// src/dli/model/paged_attention.py:150,274).
//
//
// Optional changes to the scores, each a parameter (all off: plain causal softmax attention):
//   chunk > 0     a query also sees only keys of its own chunk, floor(j / chunk) == floor(p / chunk),
//                 chunks counted from position 0 of the request;
//   r1, r2        per query head, r1[h] * log(1 + r2[h] * (p - j)) is taken off the scaled score;
//   sink != 0     the softmax's denominator has one more term, exp(0): a key of score 0 without a
//                 value, so a row's weights may add up to less than one;
//   value_dim     the size of a value where it differs from a key's;
//   gate          float32 [tokens][gate_stride]: the result is multiplied by sigmoid(gate) element
//                 by element (same layout as the output);
//   keep_first    with a window: keys at positions below keep_first stay visible however far back they lie;
//   v_heads       the value pages hold v_heads heads, a divisor of kv_heads, and kv head g reads the values of
//                 head g % v_heads (several score maps over one set of values);
//   out32         float32 [tokens][out_stride]: the result goes there unrounded instead of to `out`.
// tile_entry == nullptr: every entry is a single row (steps of single tokens, whose launches read
// nothing that the host made from the step's lengths); a kernel of its own takes these, below.
//
// Page layout: K [pages][kv_heads][page_size][head_dim], V [pages][kv_heads][value_dim][page_size].
#include "common.h"

struct ScoreChanges {
  int chunk;
  int sink;
  const float* r1;
  const float* r2;
  int value_dim;
  const float* gate;
  int64_t gate_stride;
  int keep_first;
  int v_heads;
  float* out32;
};

template <typename T, int RM, int RN, int DC>
__global__ __launch_bounds__(256) void attention_generic_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, T* __restrict__ out, int64_t out_stride,
    const int* __restrict__ q_start, const int* __restrict__ kv_len,
    const int* __restrict__ block_tables, int table_stride, const int* __restrict__ tile_entry,
    const int* __restrict__ tile_q0, int q_heads, int kv_heads, int head_dim, int page_size,
    float scale, int window, ScoreChanges sc) {
  constexpr int BM = 16 * RM, BN = 16 * RN, DMAX = 16 * DC;
  __shared__ float qs[BM][DMAX + 1];
  __shared__ float ks[BN][DMAX + 1];
  __shared__ float vs[BN][DMAX + 1];
  __shared__ float ps[BM][BN + 1];

  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const int entry = tile_entry != nullptr ? tile_entry[blockIdx.x] : blockIdx.x;
  const int q0 = tile_entry != nullptr ? tile_q0[blockIdx.x] : 0;
  const int head = blockIdx.y;
  const int value_dim = sc.value_dim;
  const float r1 = sc.r1 != nullptr ? sc.r1[head] : 0.f, r2 = sc.r1 != nullptr ? sc.r2[head] : 0.f;
  const int kvh = head / (q_heads / kv_heads);
  const int vh = kvh % sc.v_heads;
  const int tok0 = q_start[entry];
  const int q_len = q_start[entry + 1] - tok0;
  const int n_keys = kv_len[entry];
  const int first_pos = n_keys - q_len;  // absolute position of this request's first query here
  const int rows = min(BM, q_len - q0);
  const int* table = block_tables + (int64_t)entry * table_stride;

  for (int idx = tid; idx < BM * head_dim; idx += 256) {
    const int r = idx / head_dim, c = idx - r * head_dim;
    qs[r][c] = r < rows ? to_f32(q[(int64_t)(tok0 + q0 + r) * q_stride + (int64_t)head * head_dim + c]) * scale : 0.f;
  }

  float m_run[RM], l_run[RM], acc[RM][DC];
#pragma unroll
  for (int i = 0; i < RM; ++i) {
    m_run[i] = sc.sink ? 0.f : -INFINITY;  // the sink: a key of score 0 that brings no value
    l_run[i] = sc.sink ? 1.f : 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c) acc[i][c] = 0.f;
  }

  const int pos_lo = first_pos + q0, pos_hi = first_pos + q0 + rows - 1;
  int j_lo = sc.chunk > 0 ? pos_lo / sc.chunk * sc.chunk : 0;   // nothing before it is seen
  int j_begin = j_lo;
  if (window > 0) j_begin = max(j_lo, pos_lo - window + 1);
  j_begin = j_begin / BN * BN;
  j_lo = j_lo / BN * BN;
  const int keep = window > 0 ? sc.keep_first : 0;              // keys below it are seen from any distance
  const int j_end = rows > 0 ? pos_hi + 1 : 0;

  for (int j0 = keep > j_lo ? j_lo : j_begin; j0 < j_end; j0 += BN) {
    if (j0 >= keep && j0 < j_begin) j0 = j_begin;               // between the kept keys and the window: nothing
    __syncthreads();  // previous tile's reads of ks/vs/ps are done (and qs is written)
    for (int idx = tid; idx < BN * head_dim; idx += 256) {
      const int r = idx / head_dim, c = idx - r * head_dim;
      const int j = j0 + r;
      float kv = 0.f;
      if (j < j_end) {
        const int64_t page = max(table[j / page_size], 0);   // (a page that a window has passed: any page, its keys are not seen)
        kv = to_f32(k_pages[((page * kv_heads + kvh) * page_size + j % page_size) * head_dim + c]);
      }
      ks[r][c] = kv;
    }
    for (int idx = tid; idx < BN * value_dim; idx += 256) {
      const int c = idx / BN, r = idx - c * BN;  // key index fastest: contiguous in a V page
      const int j = j0 + r;
      float vv = 0.f;
      if (j < j_end) {
        const int64_t page = max(table[j / page_size], 0);   // (a page that a window has passed: any page, its keys are not seen)
        vv = to_f32(v_pages[((page * sc.v_heads + vh) * value_dim + c) * page_size + j % page_size]);
      }
      vs[r][c] = vv;
    }
    __syncthreads();

    float s[RM][RN];
#pragma unroll
    for (int i = 0; i < RM; ++i)
#pragma unroll
      for (int jj = 0; jj < RN; ++jj) s[i][jj] = 0.f;
    for (int c = 0; c < head_dim; ++c) {
      float qa[RM], kb[RN];
#pragma unroll
      for (int i = 0; i < RM; ++i) qa[i] = qs[ty * RM + i][c];
#pragma unroll
      for (int jj = 0; jj < RN; ++jj) kb[jj] = ks[tx + 16 * jj][c];
#pragma unroll
      for (int i = 0; i < RM; ++i)
#pragma unroll
        for (int jj = 0; jj < RN; ++jj) s[i][jj] = fmaf(qa[i], kb[jj], s[i][jj]);
    }

#pragma unroll
    for (int i = 0; i < RM; ++i) {
      const int r = ty * RM + i;
      const int pos = first_pos + q0 + r;
      float tile_max = -INFINITY;
#pragma unroll
      for (int jj = 0; jj < RN; ++jj) {
        const int j = j0 + tx + 16 * jj;
        const bool visible = r < rows && j <= pos && (window <= 0 || j > pos - window || j < sc.keep_first) &&
                             (sc.chunk <= 0 || j / sc.chunk == pos / sc.chunk);
        if (sc.r1 != nullptr && visible) s[i][jj] -= r1 * log1pf(r2 * (float)(pos - j));
        s[i][jj] = visible ? s[i][jj] : -INFINITY;
        tile_max = fmaxf(tile_max, s[i][jj]);
      }
#pragma unroll
      for (int msk = 8; msk > 0; msk >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, msk, DLI_WAVE));
      const float m_new = fmaxf(m_run[i], tile_max);
      float alpha = 1.f, tile_sum = 0.f;
      if (m_new > -INFINITY) {
        alpha = expf(m_run[i] - m_new);  // exp(-inf) = 0 on the first visible tile
#pragma unroll
        for (int jj = 0; jj < RN; ++jj) {
          const float p = expf(s[i][jj] - m_new);
          ps[r][tx + 16 * jj] = p;
          tile_sum += p;
        }
      } else {
#pragma unroll
        for (int jj = 0; jj < RN; ++jj) ps[r][tx + 16 * jj] = 0.f;
      }
#pragma unroll
      for (int msk = 8; msk > 0; msk >>= 1) tile_sum += __shfl_xor(tile_sum, msk, DLI_WAVE);
      l_run[i] = l_run[i] * alpha + tile_sum;
      m_run[i] = m_new;
#pragma unroll
      for (int c = 0; c < DC; ++c) acc[i][c] *= alpha;
    }
    __syncthreads();

    for (int jj = 0; jj < BN; ++jj) {
      float pv[RM];
#pragma unroll
      for (int i = 0; i < RM; ++i) pv[i] = ps[ty * RM + i][jj];
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        if (c * 16 < value_dim) {
          const float vv = vs[jj][tx + 16 * c];
#pragma unroll
          for (int i = 0; i < RM; ++i) acc[i][c] = fmaf(pv[i], vv, acc[i][c]);
        }
      }
    }
  }

#pragma unroll
  for (int i = 0; i < RM; ++i) {
    const int r = ty * RM + i;
    if (r >= rows) continue;
    const float inv = l_run[i] > 0.f ? 1.f / l_run[i] : 0.f;
    T* o = out + (int64_t)(tok0 + q0 + r) * out_stride + (int64_t)head * value_dim;
    const float* g = sc.gate != nullptr ? sc.gate + (int64_t)(tok0 + q0 + r) * sc.gate_stride + (int64_t)head * value_dim
                                        : nullptr;
#pragma unroll
    for (int c = 0; c < DC; ++c)
      if (tx + 16 * c < value_dim) {
        float y = acc[i][c] * inv;
        if (g != nullptr) y *= 1.f / (1.f + expf(-g[tx + 16 * c]));
        if (sc.out32 != nullptr) sc.out32[(int64_t)(tok0 + q0 + r) * out_stride + (int64_t)head * value_dim + tx + 16 * c] = y;
        else o[tx + 16 * c] = from_f32<T>(y);
      }
  }
}

template <typename T, int RM, int RN, int DC>
static int launch_generic(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                          void* out, int64_t out_stride, const int* q_start, const int* kv_len,
                          const int* block_tables, int table_stride, const int* tile_entry,
                          const int* tile_q0, int tiles, int q_heads, int kv_heads, int head_dim,
                          int page_size, float scale, int window, ScoreChanges sc, hipStream_t stream) {
  attention_generic_kernel<T, RM, RN, DC><<<dim3(tiles, q_heads), 256, 0, stream>>>(
      (const T*)q, q_stride, (const T*)k_pages, (const T*)v_pages, (T*)out, out_stride, q_start,
      kv_len, block_tables, table_stride, tile_entry, tile_q0, q_heads, kv_heads, head_dim,
      page_size, scale, window, sc);
  return dli_launch_status();
}

// ---------------------------------------------------------------------------------------------
// Steps of single tokens: one workgroup takes one (entry, kv head, group of up to GQ query heads
// that share it) and its waves (eight, or four) take the blocks of 64 visible keys in turn. In a block, lane j
// owns key j: it reads the key's row (16 bytes at a time) and makes its GQ scores against the
// queries in LDS, the changes to the scores are applied, and each head's reference point moves to
// the block's maximum (one wave reduction a head); the weights then go through LDS and the lanes
// change roles: lane c owns value column c (+ 64, ...) and adds up the block's 64 keys, whose
// values lie side by side in a page's row. The waves' states are merged through LDS at the
// end. The same arithmetic as the tile kernel, in another order: 32-bit throughout.
template <typename T> struct Pack16;   // what 16 bytes hold
template <> struct Pack16<bf16_t> { static constexpr int N = 8; typedef __bf16 type __attribute__((ext_vector_type(8))); };
template <> struct Pack16<float> { static constexpr int N = 4; typedef float type __attribute__((ext_vector_type(4))); };

template <typename T, int GQ, int VC>
__global__ __launch_bounds__(512) void attention_scored_decode_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    T* __restrict__ out, int64_t out_stride, const int* __restrict__ kv_len, const int* __restrict__ block_tables,
    int table_stride, int q_heads, int kv_heads, int head_dim, int page_size, float scale, int window,
    ScoreChanges sc, float* __restrict__ parts, int splits) {
  constexpr int PN = Pack16<T>::N;
  typedef typename Pack16<T>::type P16;
  extern __shared__ float lds[];
  const int value_dim = sc.value_dim;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, waves = blockDim.x / 64, threads = blockDim.x;
  float* qs = lds;                               // [GQ][head_dim]
  float* ps = qs + GQ * head_dim;                // [waves][GQ][64]
  float* ms = ps + waves * GQ * 64;              // [waves][GQ] reference points, then [waves][GQ] sums
  float* accs = ms + 2 * waves * GQ;             // [waves][GQ][VC * 64]
  const int entry = blockIdx.x / splits, split = blockIdx.x % splits, kvh = blockIdx.y;
  const int vh = kvh % sc.v_heads;
  const int group = q_heads / kv_heads;
  const int h0 = kvh * group + blockIdx.z * GQ;                  // first query head of this workgroup
  const int nh = min(GQ, kvh * group + group - h0);              // heads that exist
  const int n_keys = kv_len[entry];
  const int pos = n_keys - 1;
  const int* table = block_tables + (int64_t)entry * table_stride;

  for (int idx = tid; idx < GQ * head_dim; idx += threads) {
    const int h = idx / head_dim, c = idx - h * head_dim;
    qs[idx] = h < nh ? to_f32(q[(int64_t)entry * q_stride + (int64_t)(h0 + h) * head_dim + c]) * scale : 0.f;
  }
  float r1[GQ], r2[GQ], m_run[GQ], l_run[GQ], acc[GQ][VC];
#pragma unroll
  for (int h = 0; h < GQ; ++h) {
    r1[h] = sc.r1 != nullptr && h < nh ? sc.r1[h0 + h] : 0.f;
    r2[h] = sc.r1 != nullptr && h < nh ? sc.r2[h0 + h] : 0.f;
    m_run[h] = sc.sink && wave == 0 && split == 0 ? 0.f : -INFINITY;           // the sink is counted once, by wave 0
    l_run[h] = sc.sink && wave == 0 && split == 0 && lane == 0 ? 1.f : 0.f;    // (sums are kept lane by lane until the end)
#pragma unroll
    for (int c = 0; c < VC; ++c) acc[h][c] = 0.f;
  }
  const int j_lo = sc.chunk > 0 ? pos / sc.chunk * sc.chunk : 0;   // nothing before it is seen
  int j_begin = j_lo;
  if (window > 0) j_begin = max(j_lo, pos - window + 1);
  const int keep = window > 0 ? sc.keep_first : 0;                 // keys below it are seen from any distance
  // the blocks of 64 keys that hold something visible: those of the kept keys that lie before the window's, then the window's
  const int b_win = j_begin / 64;
  const int nb_keep = keep > j_lo ? max(min((keep + 63) / 64, b_win) - j_lo / 64, 0) : 0;
  const int nb_all = nb_keep + pos / 64 - b_win + 1;
  __syncthreads();

  const bool k_packs = head_dim % PN == 0, v_packs = page_size % PN == 0;
  // blocks of 64 keys go round the waves of the `splits` workgroups that share this (entry, heads)
  for (int b = split * waves + wave; b < nb_all; b += waves * splits) {
    const int j0 = (b < nb_keep ? j_lo / 64 + b : b_win + b - nb_keep) * 64;
    const int j = j0 + lane;
    const bool seen = j <= pos && j >= j_lo && (j >= j_begin || j < keep);
    // the page of this lane's key, for its own row of K and, handed round, for the rows of V (a key
    // past the request's last page reads the table's last entry: its weight is zero)
    const int my_page = max(table[min(j / page_size, table_stride - 1)], 0);
    float s[GQ];
#pragma unroll
    for (int h = 0; h < GQ; ++h) s[h] = 0.f;
    if (seen) {
      const int64_t page = my_page;
      const T* kr = k_pages + ((page * kv_heads + kvh) * page_size + j % page_size) * head_dim;
      if (k_packs) {
        for (int d = 0; d < head_dim; d += PN) {
          const P16 kk = *reinterpret_cast<const P16*>(kr + d);
#pragma unroll
          for (int e = 0; e < PN; ++e) {
            const float kf = to_f32((T)kk[e]);
#pragma unroll
            for (int h = 0; h < GQ; ++h) s[h] = fmaf(qs[h * head_dim + d + e], kf, s[h]);
          }
        }
      } else {
        for (int d = 0; d < head_dim; ++d) {
          const float kf = to_f32(kr[d]);
#pragma unroll
          for (int h = 0; h < GQ; ++h) s[h] = fmaf(qs[h * head_dim + d], kf, s[h]);
        }
      }
    }
    const float dist = (float)(pos - j);
#pragma unroll
    for (int h = 0; h < GQ; ++h) {
      float sh = seen ? s[h] - (sc.r1 != nullptr ? r1[h] * log1pf(r2[h] * dist) : 0.f) : -INFINITY;
      const float m_new = fmaxf(m_run[h], wave_max(sh));
      float p = 0.f, alpha = 1.f;
      if (m_new > -INFINITY) {
        alpha = expf(m_run[h] - m_new);
        p = expf(sh - m_new);
      }
      l_run[h] = l_run[h] * alpha + p;
      m_run[h] = m_new;
#pragma unroll
      for (int c = 0; c < VC; ++c) acc[h][c] *= alpha;
      ps[(wave * GQ + h) * 64 + lane] = p;
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    // lanes are value columns now
    const int last = min(63, pos - j0);
    const int first = keep > 0 ? 0 : max(0, j_begin - j0);   // (keys that are not seen weigh nothing)
    if (v_packs) {
      // every pack of the block's 64 keys is asked for before the first is used; keys that are not
      // seen have weight zero and lie in pages that exist (or in the table's last entry's page)
      constexpr int PACKS = 64 / PN;
#pragma unroll
      for (int c = 0; c < VC; ++c) {
        const int col = min(lane + 64 * c, value_dim - 1);
        P16 vv[PACKS];
#pragma unroll
        for (int k = 0; k < PACKS; ++k) {
          const int64_t page = __shfl(my_page, k * PN, DLI_WAVE);
          vv[k] = *reinterpret_cast<const P16*>(v_pages + ((page * sc.v_heads + vh) * value_dim + col) * page_size +
                                                (j0 + k * PN) % page_size);
        }
#pragma unroll
        for (int k = 0; k < PACKS; ++k)
#pragma unroll
          for (int e = 0; e < PN; ++e) {
            const float vf = to_f32((T)vv[k][e]);
#pragma unroll
            for (int h = 0; h < GQ; ++h) acc[h][c] = fmaf(ps[(wave * GQ + h) * 64 + k * PN + e], vf, acc[h][c]);
          }
      }
      __builtin_amdgcn_wave_barrier();
      continue;
    }
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      const int col = lane + 64 * c;
      if (col < value_dim) {
        int jj = first;
        while (jj <= last) {
          const int jk = j0 + jj;
          const int64_t page = max(table[jk / page_size], 0);
          const int off = jk % page_size;
          const T* vr = v_pages + ((page * sc.v_heads + vh) * value_dim + col) * page_size + off;
          if (v_packs && off % PN == 0 && jj + PN - 1 <= last) {
            const P16 vv = *reinterpret_cast<const P16*>(vr);
#pragma unroll
            for (int e = 0; e < PN; ++e) {
              const float vf = to_f32((T)vv[e]);
#pragma unroll
              for (int h = 0; h < GQ; ++h) acc[h][c] = fmaf(ps[(wave * GQ + h) * 64 + jj + e], vf, acc[h][c]);
            }
            jj += PN;
          } else {
            const float vf = to_f32(vr[0]);
#pragma unroll
            for (int h = 0; h < GQ; ++h) acc[h][c] = fmaf(ps[(wave * GQ + h) * 64 + jj], vf, acc[h][c]);
            jj += 1;
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // the four waves' states meet: reference points and sums first, then the accumulators
#pragma unroll
  for (int h = 0; h < GQ; ++h) {
    const float l = wave_sum(l_run[h]);
    if (lane == 0) {
      ms[wave * GQ + h] = m_run[h];
      ms[waves * GQ + wave * GQ + h] = l;
    }
#pragma unroll
    for (int c = 0; c < VC; ++c) accs[((wave * GQ + h) * VC + c) * 64 + lane] = acc[h][c];
  }
  __syncthreads();
  for (int idx = tid; idx < nh * value_dim; idx += threads) {
    const int h = idx / value_dim, col = idx - h * value_dim;
    float m = -INFINITY;
    for (int w = 0; w < waves; ++w) m = fmaxf(m, ms[w * GQ + h]);
    float l = 0.f, o = 0.f;
    for (int w = 0; w < waves; ++w) {
      const float mw = ms[w * GQ + h];
      if (mw > -INFINITY) {
        const float f = expf(mw - m);
        l += ms[waves * GQ + w * GQ + h] * f;
        o += accs[((w * GQ + h) * VC + col / 64) * 64 + col % 64] * f;
      }
    }
    if (splits > 1) {
      // this workgroup's share: the sum as it is, with its reference point and denominator behind it
      float* part = parts + (((int64_t)entry * q_heads + h0 + h) * splits + split) * (value_dim + 2);
      part[col] = o;
      if (col == 0) {
        part[value_dim] = m;
        part[value_dim + 1] = l;
      }
      continue;
    }
    float y = l > 0.f ? o / l : 0.f;
    const int64_t at = (int64_t)(h0 + h) * value_dim + col;
    if (sc.gate != nullptr) y *= 1.f / (1.f + expf(-sc.gate[(int64_t)entry * sc.gate_stride + at]));
    if (sc.out32 != nullptr) sc.out32[(int64_t)entry * out_stride + at] = y;
    else out[(int64_t)entry * out_stride + at] = from_f32<T>(y);
  }
}

// The shares of the workgroups that split an entry's keys meet: parts [entries][q_heads][splits][value_dim + 2].
// One workgroup an (entry, head), a thread a value column; sums in the order of the splits.
template <typename T>
__global__ void attention_scored_merge_kernel(const float* __restrict__ parts, int splits, int q_heads, int value_dim,
                                              const float* __restrict__ gate, int64_t gate_stride, T* __restrict__ out,
                                              int64_t out_stride, float* __restrict__ out32) {
  const int entry = blockIdx.x, head = blockIdx.y;
  const float* base = parts + ((int64_t)entry * q_heads + head) * splits * (value_dim + 2);
  float m = -INFINITY;
  for (int s = 0; s < splits; ++s) m = fmaxf(m, base[s * (value_dim + 2) + value_dim]);
  for (int col = threadIdx.x; col < value_dim; col += blockDim.x) {
    float l = 0.f, o = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float ms = base[s * (value_dim + 2) + value_dim];
      if (ms > -INFINITY) {
        const float f = expf(ms - m);
        l += base[s * (value_dim + 2) + value_dim + 1] * f;
        o += base[s * (value_dim + 2) + col] * f;
      }
    }
    float y = l > 0.f ? o / l : 0.f;
    const int64_t at = (int64_t)head * value_dim + col;
    if (gate != nullptr) y *= 1.f / (1.f + expf(-gate[(int64_t)entry * gate_stride + at]));
    if (out32 != nullptr) out32[(int64_t)entry * out_stride + at] = y;
    else out[(int64_t)entry * out_stride + at] = from_f32<T>(y);
  }
}

template <typename T, int GQ>
static int launch_scored_decode(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages, void* out,
                                int64_t out_stride, const int* kv_len, const int* block_tables, int table_stride,
                                int entries, int q_heads, int kv_heads, int head_dim, int page_size, float scale,
                                int window, ScoreChanges sc, float* parts, int splits, hipStream_t stream) {
  const int group = q_heads / kv_heads, vc = (sc.value_dim + 63) / 64;
  if (parts == nullptr || splits < 1) splits = 1;
  if ((int64_t)entries * splits > 0x7fffffff) return DLI_ERR_ARGUMENT;
  const dim3 grid(entries * splits, kv_heads, (group + GQ - 1) / GQ);
  // eight waves where their states fit 64 KB of LDS, else four: the chain of a wave's
  // blocks (table entry, key rows, value rows, each a trip to memory) is as long as its blocks
#define DECODE_LAUNCH(VC)                                                                                   \
  {                                                                                                         \
    int waves = 8;                                                                                          \
    size_t bytes = 0;                                                                                       \
    for (;; waves /= 2) {                                                                                   \
      bytes = sizeof(float) * ((size_t)GQ * head_dim + waves * GQ * 64 + 2 * waves * GQ + waves * GQ * VC * 64); \
      if (bytes <= 65536 || waves == 4) break;                                                              \
    }                                                                                                       \
    attention_scored_decode_kernel<T, GQ, VC><<<grid, 64 * waves, bytes, stream>>>(                         \
        (const T*)q, q_stride, (const T*)k_pages, (const T*)v_pages, (T*)out, out_stride, kv_len,           \
        block_tables, table_stride, q_heads, kv_heads, head_dim, page_size, scale, window, sc, parts, splits); \
  }
  if (vc <= 1) DECODE_LAUNCH(1) else if (vc == 2) DECODE_LAUNCH(2) else DECODE_LAUNCH(4)
#undef DECODE_LAUNCH
  if (splits > 1) {
    const int status = dli_launch_status();
    if (status != DLI_OK) return status;
    attention_scored_merge_kernel<T><<<dim3(entries, q_heads), sc.value_dim <= 64 ? 64 : sc.value_dim <= 128 ? 128 : 256, 0,
                                       stream>>>(parts, splits, q_heads, sc.value_dim, sc.gate, sc.gate_stride, (T*)out,
                                                 out_stride, sc.out32);
  }
  return dli_launch_status();
}

// Queries per tile for a head_dim (the larger of the key's and the value's size): the host builds
// its tile list with this.
extern "C" int dli_attention_generic_tile_rows(int head_dim) {
  if (head_dim <= 0 || head_dim > 256) return DLI_ERR_ARGUMENT;
  return head_dim <= 128 ? 32 : 16;
}

// The attention with every change to the scores as a parameter (see the head of this file).
// chunk 0, sink 0, r1 = r2 = gate = nullptr and value_dim == head_dim: the plain attention.
static int attention_scored(const void* q, int64_t q_stride, const void* k_pages,
                            const void* v_pages, void* out, int64_t out_stride,
                            const int* q_start, const int* kv_len, const int* block_tables,
                            int table_stride, const int* tile_entry, const int* tile_q0,
                            int tiles, int q_heads, int kv_heads, int head_dim, int value_dim,
                            int page_size, float scale, int window, int chunk, int sink,
                            const float* r1, const float* r2, const float* gate,
                            int64_t gate_stride, int keep_first, int v_heads, float* out32, float* parts, int splits,
                            int is_bf16, hipStream_t stream) {
  if (tiles <= 0) return DLI_OK;
  if (v_heads <= 0) v_heads = kv_heads;
  if (keep_first < 0 || kv_heads <= 0 || kv_heads % v_heads != 0) return DLI_ERR_ARGUMENT;
  const int dmax = head_dim > value_dim ? head_dim : value_dim;
  if (head_dim <= 0 || value_dim <= 0 || dmax > 256 || q_heads <= 0 || kv_heads <= 0 ||
      q_heads % kv_heads != 0 || q_heads > 65535 || page_size <= 0 || table_stride <= 0 ||
      window < 0 || chunk < 0 || (r1 == nullptr) != (r2 == nullptr) ||
      (tile_entry == nullptr) != (tile_q0 == nullptr))
    return DLI_ERR_ARGUMENT;
  const ScoreChanges sc = {chunk, sink, r1, r2, value_dim, gate, gate_stride, keep_first, v_heads, out32};
  if (tile_entry == nullptr) {
    // every entry is one row: the kernel whose lanes own keys, then value columns
    const int group = q_heads / kv_heads;
#define DECODE_ARGS                                                                                      \
  q, q_stride, k_pages, v_pages, out, out_stride, kv_len, block_tables, table_stride, tiles, q_heads,   \
      kv_heads, head_dim, page_size, scale, window, sc, parts, splits, stream
    if (is_bf16) {
      if (group == 1) return launch_scored_decode<bf16_t, 1>(DECODE_ARGS);
      if (group <= 4) return launch_scored_decode<bf16_t, 4>(DECODE_ARGS);
      return launch_scored_decode<bf16_t, 8>(DECODE_ARGS);
    }
    if (group == 1) return launch_scored_decode<float, 1>(DECODE_ARGS);
    if (group <= 4) return launch_scored_decode<float, 4>(DECODE_ARGS);
    return launch_scored_decode<float, 8>(DECODE_ARGS);
#undef DECODE_ARGS
  }
#define GENERIC_ARGS                                                                              \
  q, q_stride, k_pages, v_pages, out, out_stride, q_start, kv_len, block_tables, table_stride,   \
      tile_entry, tile_q0, tiles, q_heads, kv_heads, head_dim, page_size, scale, window, sc, stream
  if (is_bf16) {
    if (dmax <= 64) return launch_generic<bf16_t, 2, 2, 4>(GENERIC_ARGS);
    if (dmax <= 128) return launch_generic<bf16_t, 2, 2, 8>(GENERIC_ARGS);
    return launch_generic<bf16_t, 1, 1, 16>(GENERIC_ARGS);
  }
  if (dmax <= 64) return launch_generic<float, 2, 2, 4>(GENERIC_ARGS);
  if (dmax <= 128) return launch_generic<float, 2, 2, 8>(GENERIC_ARGS);
  return launch_generic<float, 1, 1, 16>(GENERIC_ARGS);
#undef GENERIC_ARGS
}

extern "C" int dli_attention_scored(const void* q, int64_t q_stride, const void* k_pages,
                                    const void* v_pages, void* out, int64_t out_stride,
                                    const int* q_start, const int* kv_len, const int* block_tables,
                                    int table_stride, const int* tile_entry, const int* tile_q0,
                                    int tiles, int q_heads, int kv_heads, int head_dim, int value_dim,
                                    int page_size, float scale, int window, int chunk, int sink,
                                    const float* r1, const float* r2, const float* gate,
                                    int64_t gate_stride, int keep_first, int v_heads, float* out32, int is_bf16,
                                    hipStream_t stream) {
  return attention_scored(q, q_stride, k_pages, v_pages, out, out_stride, q_start, kv_len, block_tables, table_stride,
                          tile_entry, tile_q0, tiles, q_heads, kv_heads, head_dim, value_dim, page_size, scale, window,
                          chunk, sink, r1, r2, gate, gate_stride, keep_first, v_heads, out32, nullptr, 1, is_bf16, stream);
}

// How many workgroups share the keys of an (entry, group of query heads) in a step of single tokens: as
// many as bring the launch to about two workgroups a compute unit, sixteen at most. It depends on the
// heads and the number of entries, never on their lengths. A step of many entries fills the chip by
// itself and is not cut (cutting it costs more than it gains).
extern "C" int dli_attention_scored_splits(int q_heads, int kv_heads, int entries) {
  if (q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads != 0 || entries <= 0) return 1;
  const int group = q_heads / kv_heads, gq = group == 1 ? 1 : group <= 4 ? 4 : 8;
  const int64_t workgroups = (int64_t)entries * kv_heads * ((group + gq - 1) / gq);
  const int64_t splits = 512 / workgroups;
  return splits < 1 ? 1 : splits > 16 ? 16 : (int)splits;
}

// A step of single tokens (every entry one row) with each entry's keys cut over `splits` workgroups:
// parts is float [entries * q_heads * splits * (value_dim + 2)] of scratch.
extern "C" int dli_attention_scored_single(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                           void* out, int64_t out_stride, const int* kv_len, const int* block_tables,
                                           int table_stride, int entries, int q_heads, int kv_heads, int head_dim,
                                           int value_dim, int page_size, float scale, int window, int chunk, int sink,
                                           const float* r1, const float* r2, const float* gate, int64_t gate_stride,
                                           int keep_first, int v_heads, float* out32, float* parts, int splits,
                                           int is_bf16, hipStream_t stream) {
  if (splits < 1 || splits > 64 || (splits > 1 && parts == nullptr)) return DLI_ERR_ARGUMENT;
  return attention_scored(q, q_stride, k_pages, v_pages, out, out_stride, nullptr, kv_len, block_tables, table_stride,
                          nullptr, nullptr, entries, q_heads, kv_heads, head_dim, value_dim, page_size, scale, window,
                          chunk, sink, r1, r2, gate, gate_stride, keep_first, v_heads, out32, parts, splits, is_bf16, stream);
}

extern "C" int dli_attention_generic(const void* q, int64_t q_stride, const void* k_pages,
                                     const void* v_pages, void* out, int64_t out_stride,
                                     const int* q_start, const int* kv_len, const int* block_tables,
                                     int table_stride, const int* tile_entry, const int* tile_q0,
                                     int tiles, int q_heads, int kv_heads, int head_dim, int page_size,
                                     float scale, int window, int is_bf16, hipStream_t stream) {
  if (head_dim % 16 != 0 || tile_entry == nullptr) return tiles <= 0 ? DLI_OK : DLI_ERR_ARGUMENT;
  return attention_scored(q, q_stride, k_pages, v_pages, out, out_stride, q_start, kv_len,
                          block_tables, table_stride, tile_entry, tile_q0, tiles, q_heads,
                          kv_heads, head_dim, head_dim, page_size, scale, window, 0, 0, nullptr,
                          nullptr, nullptr, 0, 0, kv_heads, nullptr, nullptr, 1, is_bf16, stream);
}
