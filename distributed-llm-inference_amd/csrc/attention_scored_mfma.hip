// Attention with changed scores for the portions of a bfloat16 step, on the matrix cores.
//
// The same scores as csrc/attention_generic.hip (chunked mask, window, per-head logarithmic distance
// penalty, sink, values of another size than keys, sigmoid gate, kept first keys, value heads shared by
// several key heads, an unrounded result), computed with
// v_mfma_f32_16x16x16_bf16 in transposed form, S^T = K Q^T and O^T = V^T P^T: a lane then holds four
// consecutive keys' scores of ONE query (query = lane % 16), so the running maximum, the sum and the
// rescaling of a query stay in its four lanes, and the result of the first product is, lane by lane,
// already the operand of the second. A wave owns 16 queries of one head and walks their visible
// keys 64 at a time; every operand comes straight from memory in the order the pages keep it (a key's
// dims side by side, a value row's keys side by side), eight bytes a lane and product, and waves
// neither share nor wait: four waves of a workgroup take neighbouring query rows, so their keys meet
// in the cache. Exponentials are exp2 with log2(e) folded into the scale; the penalty is
// r1 log2(1 + r2 d) in that domain (one v_log_f32). P is rounded to bfloat16 for the second product
// while the running sum keeps the unrounded values, as in the other matrix-core attention.
//
// Needs head_dim and value_dim of 16 to 96 in steps of 16, or 128 (or, where values are as long as keys,
// as when a cached latent is both, any multiple of 16 up to 256), and page_size % 4 == 0; other shapes,
// and the 32-bit runtime, take the vector-unit kernel.
#include "common.h"

typedef short short4s __attribute__((ext_vector_type(4)));
typedef float float4s __attribute__((ext_vector_type(4)));

struct ScoredArgs {
  const bf16_t* q; int64_t q_stride;
  const bf16_t* k_pages; const bf16_t* v_pages;
  bf16_t* out; int64_t out_stride;
  const int* q_start; const int* kv_len; const int* block_tables; int table_stride;
  const int* tile_entry; const int* tile_q0;
  int q_heads, kv_heads, page_size;
  float scale; int window, chunk, sink;
  const float* r1; const float* r2;
  const float* gate; int64_t gate_stride;
  int keep_first, v_heads;
  float* out32;
};

template <int DT, int VT>   // head_dim = 16 DT, value_dim = 16 VT
__global__ __launch_bounds__(256) void attention_scored_mfma_kernel(ScoredArgs a) {
  constexpr int D = 16 * DT, V = 16 * VT;
  constexpr float LOG2E = 1.4426950408889634f;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int col = lane & 15, grp = lane >> 4;
  const int entry = a.tile_entry[blockIdx.x], head = blockIdx.y;
  const int kvh = head / (a.q_heads / a.kv_heads);
  const int tok0 = a.q_start[entry], q_len = a.q_start[entry + 1] - tok0;
  const int n_keys = a.kv_len[entry], first_pos = n_keys - q_len;
  const int qrow0 = a.tile_q0[blockIdx.x] + wave * 16;   // this wave's first query within the entry
  if (qrow0 >= q_len) return;                            // (waves do not wait for each other)
  const bool q_live = qrow0 + col < q_len;
  const int my_q = min(qrow0 + col, q_len - 1);
  const int pos = first_pos + my_q;
  const int ps = a.page_size, G = a.kv_heads, GV = a.v_heads, vh = kvh % a.v_heads;
  const int* table = a.block_tables + (int64_t)entry * a.table_stride;

  short4s qb[DT];   // Q^T: dims 16 d + 4 grp .. + 3 of this lane's query
  {
    const bf16_t* qr = a.q + (int64_t)(tok0 + my_q) * a.q_stride + (int64_t)head * D + 4 * grp;
#pragma unroll
    for (int d = 0; d < DT; ++d) qb[d] = *reinterpret_cast<const short4s*>(qr + 16 * d);
  }
  const float r1 = a.r1 != nullptr ? a.r1[head] : 0.f, r2 = a.r1 != nullptr ? a.r2[head] : 0.f;
  const float scale2 = a.scale * LOG2E;
  const int p_lo = first_pos + qrow0, p_hi = first_pos + min(qrow0 + 15, q_len - 1);
  int j_lo = a.chunk > 0 ? p_lo / a.chunk * a.chunk : 0;        // nothing before it is seen
  int j_begin = j_lo;
  if (a.window > 0) j_begin = max(j_lo, p_lo - a.window + 1);
  j_begin = j_begin / 64 * 64;
  j_lo = j_lo / 64 * 64;
  const int keep = a.window > 0 ? a.keep_first : 0;             // keys below it are seen from any distance
  const int my_chunk = a.chunk > 0 ? pos / a.chunk : 0;

  float4s acc[VT];
#pragma unroll
  for (int t = 0; t < VT; ++t) acc[t] = float4s{0.f, 0.f, 0.f, 0.f};
  float m_run = a.sink ? 0.f : -INFINITY;              // the sink: a key of score 0 without a value,
  float l_run = a.sink && grp == 0 ? 1.f : 0.f;        // counted once a query (sums are per lane until the end)

  for (int j0 = keep > j_lo ? j_lo : j_begin; j0 <= p_hi; j0 += 64) {
    if (j0 >= keep && j0 < j_begin) j0 = j_begin;               // between the kept keys and the window: nothing
    float4s s[4];
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {
      const int key = j0 + 16 * sub + col;              // the key whose row this lane reads
      const int64_t page = max(table[min(key / ps, a.table_stride - 1)], 0);   // (a page that a window has passed: any page will do)
      const bf16_t* kr = a.k_pages + ((page * G + kvh) * ps + key % ps) * D + 4 * grp;
      float4s c = float4s{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int d = 0; d < DT; ++d)
        c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const short4s*>(kr + 16 * d), qb[d], c, 0, 0, 0);
      s[sub] = c;                                       // c[i]: key j0 + 16 sub + 4 grp + i against query `col`
    }
    float mx = -INFINITY;
#pragma unroll
    for (int sub = 0; sub < 4; ++sub)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int j = j0 + 16 * sub + 4 * grp + i;
        const bool seen = q_live && j <= pos && (a.window <= 0 || j > pos - a.window || j < a.keep_first) &&
                          (a.chunk <= 0 || j / a.chunk == my_chunk);
        float x = s[sub][i] * scale2;
        if (a.r1 != nullptr) x -= r1 * __builtin_amdgcn_logf(1.f + r2 * (float)max(pos - j, 0));
        x = seen ? x : -INFINITY;
        s[sub][i] = x;
        mx = fmaxf(mx, x);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, DLI_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, DLI_WAVE));
    const float m_new = fmaxf(m_run, mx);
    const bool any = m_new > -INFINITY;
    const float alpha = any ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.f;
    float sum = 0.f;
    short4s pb[4];
#pragma unroll
    for (int sub = 0; sub < 4; ++sub)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = any ? __builtin_amdgcn_exp2f(s[sub][i] - m_new) : 0.f;   // exp2(-inf) = 0 for what is not seen
        sum += p;
        const bf16_t pr = (bf16_t)p;
        pb[sub][i] = *reinterpret_cast<const short*>(&pr);
      }
    l_run = l_run * alpha + sum;
    m_run = m_new;
#pragma unroll
    for (int t = 0; t < VT; ++t) acc[t] *= alpha;
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {
      const int key = j0 + 16 * sub + 4 * grp;          // the four keys whose values this lane reads, one value row a product
      const int64_t page = max(table[min(key / ps, a.table_stride - 1)], 0);   // (a page that a window has passed: any page will do)
      const bf16_t* vr = a.v_pages + ((page * GV + vh) * V + col) * ps + key % ps;
#pragma unroll
      for (int t = 0; t < VT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const short4s*>(vr + (int64_t)16 * t * ps),
                                                          pb[sub], acc[t], 0, 0, 0);
    }
  }
  float l = l_run + __shfl_xor(l_run, 16, DLI_WAVE);
  l += __shfl_xor(l, 32, DLI_WAVE);
  if (!q_live) return;
  const float inv = l > 0.f ? 1.f / l : 0.f;
  // acc[t][i] is value 16 t + 4 grp + i of query `col`: four neighbours in the output row
  const int64_t row = tok0 + my_q;
#pragma unroll
  for (int t = 0; t < VT; ++t) {
    const int64_t at = (int64_t)head * V + 16 * t + 4 * grp;
    short4s o;
    float4s of;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float y = acc[t][i] * inv;
      if (a.gate != nullptr) y *= 1.f / (1.f + __expf(-a.gate[row * a.gate_stride + at + i]));
      of[i] = y;
      const bf16_t yb = (bf16_t)y;
      o[i] = *reinterpret_cast<const short*>(&yb);
    }
    if (a.out32 != nullptr) *reinterpret_cast<float4s*>(a.out32 + row * a.out_stride + at) = of;
    else *reinterpret_cast<short4s*>(a.out + row * a.out_stride + at) = o;
  }
}

// Whether the matrix-core kernel takes these sizes (tiles of 64 queries).
extern "C" int dli_attention_scored_mfma_supports(int head_dim, int value_dim, int page_size) {
  const int dt = head_dim / 16, vt = value_dim / 16;
  return head_dim > 0 && value_dim > 0 && head_dim % 16 == 0 && value_dim % 16 == 0 &&
         (((dt <= 6 || dt == 8) && (vt <= 6 || vt == 8)) || (dt == vt && dt <= 16)) && page_size > 0 && page_size % 4 == 0;
}

template <int DT>
static int launch_scored_mfma(const ScoredArgs& a, int tiles, int value_dim, hipStream_t stream) {
  const dim3 grid(tiles, a.q_heads);
#define VCASE(VT) case VT: attention_scored_mfma_kernel<DT, VT><<<grid, 256, 0, stream>>>(a); break;
  switch (value_dim / 16) {
    VCASE(1) VCASE(2) VCASE(3) VCASE(4) VCASE(5) VCASE(6) VCASE(8)
    default: return DLI_ERR_ARGUMENT;
  }
#undef VCASE
  return dli_launch_status();
}

// Values as long as keys, of the sizes that the cases above leave out.
template <int DT>
static int launch_scored_mfma_square(const ScoredArgs& a, int tiles, hipStream_t stream) {
  attention_scored_mfma_kernel<DT, DT><<<dim3(tiles, a.q_heads), 256, 0, stream>>>(a);
  return dli_launch_status();
}

extern "C" int dli_attention_scored_mfma(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                                         void* out, int64_t out_stride, const int* q_start, const int* kv_len,
                                         const int* block_tables, int table_stride, const int* tile_entry,
                                         const int* tile_q0, int tiles, int q_heads, int kv_heads, int head_dim,
                                         int value_dim, int page_size, float scale, int window, int chunk, int sink,
                                         const float* r1, const float* r2, const float* gate, int64_t gate_stride,
                                         int keep_first, int v_heads, float* out32, hipStream_t stream) {
  if (tiles <= 0) return DLI_OK;
  if (v_heads <= 0) v_heads = kv_heads;
  if (keep_first < 0 || kv_heads <= 0 || kv_heads % v_heads != 0) return DLI_ERR_ARGUMENT;
  if (!dli_attention_scored_mfma_supports(head_dim, value_dim, page_size) || q_heads <= 0 || kv_heads <= 0 ||
      q_heads % kv_heads != 0 || q_heads > 65535 || table_stride <= 0 || window < 0 || chunk < 0 ||
      (r1 == nullptr) != (r2 == nullptr) || tile_entry == nullptr || tile_q0 == nullptr || q_stride % 4 != 0 ||
      out_stride % 4 != 0)
    return DLI_ERR_ARGUMENT;
  ScoredArgs a;
  a.q = (const bf16_t*)q; a.q_stride = q_stride; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
  a.out = (bf16_t*)out; a.out_stride = out_stride; a.q_start = q_start; a.kv_len = kv_len;
  a.block_tables = block_tables; a.table_stride = table_stride; a.tile_entry = tile_entry; a.tile_q0 = tile_q0;
  a.q_heads = q_heads; a.kv_heads = kv_heads; a.page_size = page_size; a.scale = scale; a.window = window;
  a.chunk = chunk; a.sink = sink; a.r1 = r1; a.r2 = r2; a.gate = gate; a.gate_stride = gate_stride;
  a.keep_first = keep_first; a.v_heads = v_heads; a.out32 = out32;
  switch (head_dim / 16) {
    case 1: return launch_scored_mfma<1>(a, tiles, value_dim, stream);
    case 2: return launch_scored_mfma<2>(a, tiles, value_dim, stream);
    case 3: return launch_scored_mfma<3>(a, tiles, value_dim, stream);
    case 4: return launch_scored_mfma<4>(a, tiles, value_dim, stream);
    case 5: return launch_scored_mfma<5>(a, tiles, value_dim, stream);
    case 6: return launch_scored_mfma<6>(a, tiles, value_dim, stream);
    case 8: return launch_scored_mfma<8>(a, tiles, value_dim, stream);
    case 7: return launch_scored_mfma_square<7>(a, tiles, stream);
    case 9: return launch_scored_mfma_square<9>(a, tiles, stream);
    case 10: return launch_scored_mfma_square<10>(a, tiles, stream);
    case 11: return launch_scored_mfma_square<11>(a, tiles, stream);
    case 12: return launch_scored_mfma_square<12>(a, tiles, stream);
    case 13: return launch_scored_mfma_square<13>(a, tiles, stream);
    case 14: return launch_scored_mfma_square<14>(a, tiles, stream);
    case 15: return launch_scored_mfma_square<15>(a, tiles, stream);
    case 16: return launch_scored_mfma_square<16>(a, tiles, stream);
    default: return DLI_ERR_ARGUMENT;
  }
}
