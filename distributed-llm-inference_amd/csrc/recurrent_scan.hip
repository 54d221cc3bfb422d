// Linear recurrences with a matrix state per head, S [key channel][value channel] in 32-bit,
// carried from token to token of a request in its state slot. Two rules, one kernel:
//
//   RULE_DELTA   u = k / sqrt(sum k^2 + 1e-6);
//                S <- diag(w) S - (a * u) (u^T S) + k v^T   (both terms read the old S);   o = S^T r
//   RULE_BONUS   o = (S + diag(bonus) k v^T)^T r;   S <- diag(w) S + k v^T
//
// with the decay w and the removal rate a per key channel given ready made (32-bit; the kernel of
// the low-rank projection's second half makes them: every wave of a head would otherwise repeat
// their exponentials),
//
// followed, per token and head, by o / sqrt(mean(o^2) + eps) * norm_w * gate, with gate =
// sigmoid(g_pre) (RULE_DELTA) or silu(g_pre) (RULE_BONUS); the result is written in the type of
// the product that reads it. Everything here is 32-bit arithmetic on 32-bit inputs.
//
// One wave takes one (entry, head, slice of 4 value columns) and walks the entry's tokens in
// order; waves never wait for each other. Lane (v, part) keeps the D / 16 state values
// S[part's keys][v] in registers: a column of S never leaves its sixteen neighbouring lanes (a DPP
// row), whose partial dot products meet in four DPP swaps (heads whose size is no multiple of 16:
// eight lanes a column, eight columns a wave). A wave alone on its SIMD issues an instruction
// every four to five cycles, so the chain over a request's tokens is as long as a token's
// instructions: many lanes a column keep that to some fifty. The per-token vectors of 16
// tokens (8 for heads above 64; one in a step of single tokens) are staged in LDS at once: the
// loads of the next batch are in flight while the chain over this batch's tokens runs, and the
// chain itself reads LDS and registers only. o goes out in 32-bit; a second kernel normalises
// each head's o and applies the gate (it needs all of a head's columns, which lie in several
// waves). The sums of a token do not depend on where a step cut the request: the state is the
// only thing carried, and it is carried exactly.
//
// State slot layout: [heads][D (value)][D (key)] floats at `state + slot * state_stride`.
// A request whose first row of the step has position 0 starts from a zero state.
#include "common.h"

#define RULE_DELTA 0
#define RULE_BONUS 1
#define GATE_NONE 2   // head_norm_gate alone: the per-head norm without a gate

struct ScanArgs {
  const float* r; const float* k; const float* v;   // [rows][heads * D], each with its row stride
  const float* w_pre;                                // the decay w
  const float* a_pre; const float* a_bias;           // RULE_DELTA: the removal rate a (a_bias: unused, kept for the layout)
  const float* g_pre;                                // gate before its activation
  int64_t r_stride, k_stride, v_stride, w_stride, a_stride, g_stride;
  const float* bonus;                                // RULE_BONUS: [heads][D]
  const float* norm_w;                               // [heads * D]
  float eps;
  float* state; int64_t state_stride;
  const int* q_start; const int* positions; const int* state_slots;
  float* o_raw; int64_t o_stride;                    // the recurrence's own output, before norm and gate
  void* out; int64_t out_stride;
  int heads;
};

// Sum over the eight lanes of an octet (every lane gets it): two DPP quad permutes, then the
// mirror of a half row, which swaps an octet's two quads (whose lanes already agree).
__device__ __forceinline__ float octet_sum(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, false));
  return x;
}

// Sum over the sixteen lanes of a row: the octet's sum, then the mirror of the row, which swaps its octets.
__device__ __forceinline__ float row_sum(float x) {
  x = octet_sum(x);
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, false));
  return x;
}
template <int PARTS> __device__ __forceinline__ float parts_sum(float x) { return PARTS == 16 ? row_sum(x) : octet_sum(x); }

// PARTS lanes share a value column (16 where the head's size allows, else 8); a wave holds 64 / PARTS columns.
template <int NK, int PARTS, int RULE, int TB>
__global__ __launch_bounds__(64) void recurrent_scan_kernel(ScanArgs p) {
  constexpr int D = NK * PARTS, COLS = 64 / PARTS, PER = (TB * D + 63) / 64;  // PER: what a lane stages per vector and batch
  __shared__ float sk[PER * 64], sw[PER * 64], sa[RULE == RULE_DELTA ? PER * 64 : 1], sr[PER * 64];
  const int lane = threadIdx.x, vloc = lane / PARTS, part = lane % PARTS;
  const int entry = blockIdx.x, head = blockIdx.y, col = blockIdx.z * COLS + vloc;
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int64_t col0 = (int64_t)head * D;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + ((int64_t)head * D + col) * D + part * NK;
  float s[NK], bon[NK];
  const bool fresh = p.positions[row0] == 0;
#pragma unroll
  for (int i = 0; i < NK; ++i) {
    s[i] = fresh ? 0.f : st[i];
    bon[i] = RULE == RULE_BONUS ? p.bonus[col0 + part * NK + i] : 0.f;
  }

  constexpr int PV = (TB * COLS + 63) / 64;
  __shared__ float sv[PV * 64], skn[TB];
  float pk[PER], pw[PER], pa[PER], pr[PER], pv[PV];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int m = 0; m < PER; ++m) {
      const int e = min(lane + 64 * m, TB * D - 1), t = e / D, c = e - t * D;
      const int64_t row = row0 + min(t0 + t, n_rows - 1);
      pk[m] = p.k[row * p.k_stride + col0 + c];
      pr[m] = p.r[row * p.r_stride + col0 + c];
      pw[m] = p.w_pre[row * p.w_stride + col0 + c];
      if (RULE == RULE_DELTA) pa[m] = p.a_pre[row * p.a_stride + col0 + c];
    }
#pragma unroll
    for (int m = 0; m < PV; ++m) {
      const int e = min(lane + 64 * m, TB * COLS - 1);
      pv[m] = p.v[(int64_t)(row0 + min(t0 + e / COLS, n_rows - 1)) * p.v_stride + col0 + blockIdx.z * COLS + e % COLS];
    }
  };
  // One token of the chain, from LDS and registers only. Nothing but s hangs on the token before:
  // the reads of the next tokens can be issued while this one's sums are made.
  auto step = [&](int t, int64_t row) {
    const float* kt = sk + t * D + part * NK;
    const float* wt = sw + t * D + part * NK;
    const float* rt = sr + t * D + part * NK;
    const float v = sv[t * COLS + vloc];
    float o0 = 0.f, o1 = 0.f;
    if (RULE == RULE_DELTA) {
      const float* at = sa + t * D + part * NK;     // a * u, made when the batch was staged
      const float kn = skn[t];
      float ks0 = 0.f, ks1 = 0.f;
#pragma unroll
      for (int i = 0; i < NK; ++i) {
        if (i & 1) ks1 = fmaf(kt[i], s[i], ks1); else ks0 = fmaf(kt[i], s[i], ks0);
      }
      const float us = parts_sum<PARTS>(ks0 + ks1) * kn;       // u^T S for this column, u = k * kn
#pragma unroll
      for (int i = 0; i < NK; ++i) {
        s[i] = wt[i] * s[i] - at[i] * us + kt[i] * v;
        if (i & 1) o1 = fmaf(s[i], rt[i], o1); else o0 = fmaf(s[i], rt[i], o0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NK; ++i) {
        const float kv = kt[i] * v;
        if (i & 1) o1 = fmaf(s[i] + bon[i] * kv, rt[i], o1); else o0 = fmaf(s[i] + bon[i] * kv, rt[i], o0);
        s[i] = wt[i] * s[i] + kv;
      }
    }
    const float o = parts_sum<PARTS>(o0 + o1);
    if (part == 0) p.o_raw[row * p.o_stride + col0 + col] = o;
  };
  fetch(0);
  for (int t0 = 0; t0 < n_rows; t0 += TB) {
#pragma unroll
    for (int m = 0; m < PER; ++m) {
      const int e = lane + 64 * m;
      sk[e] = pk[m];
      sr[e] = pr[m];
      sw[e] = pw[m];
      if (RULE == RULE_DELTA) sa[e] = pa[m];
    }
#pragma unroll
    for (int m = 0; m < PV; ++m) sv[lane + 64 * m] = pv[m];
    if (TB > 1 && t0 + TB < n_rows) fetch(t0 + TB);  // on their way while the chain below runs
    __syncthreads();                                 // (one wave: orders its LDS writes before its reads)
    if (RULE == RULE_DELTA) {
      // each token's 1 / sqrt(sum k^2 + 1e-6): four lanes a token add up a quarter of its keys each
      for (int t = lane >> 2; t < TB; t += 16) {
        float kk = 0.f;
        for (int c = (lane & 3) * (D / 4); c < ((lane & 3) + 1) * (D / 4); ++c) kk = fmaf(sk[t * D + c], sk[t * D + c], kk);
        kk += __shfl_xor(kk, 1, DLI_WAVE);
        kk += __shfl_xor(kk, 2, DLI_WAVE);
        if ((lane & 3) == 0) skn[t] = 1.f / sqrtf(kk + 1e-6f);
      }
      __syncthreads();
      // the removal rate times the unit key, a * u = a * k / |k|, off the chain as well
#pragma unroll
      for (int m = 0; m < PER; ++m) {
        const int e = lane + 64 * m;
        sa[e] *= sk[e] * skn[min(e / D, TB - 1)];
      }
      __syncthreads();
    }
    const int nb = min(TB, n_rows - t0);
    if (nb == TB) {
#pragma unroll
      for (int t = 0; t < TB; ++t) step(t, row0 + t0 + t);
    } else {
      for (int t = 0; t < nb; ++t) step(t, row0 + t0 + t);
    }
    __syncthreads();  // the chain has read this batch before the next one is written
  }
#pragma unroll
  for (int i = 0; i < NK; ++i) st[i] = s[i];
}

// Heads of any other size (1 to 1024): a thread a value column, the column's state read and written in
// the request's slot token by token, the token's vectors in LDS. Slow, and only there so that no
// size is refused; the same sums in the same order per column as above are not promised, the same
// result to rounding is.
template <int RULE>
__global__ void recurrent_scan_any_kernel(ScanArgs p, int D) {
  extern __shared__ float sh[];
  float *sk = sh, *sw = sh + D, *sa = sh + 2 * D, *sr = sh + 3 * D, *scratch = sh + 4 * D;
  const int v = threadIdx.x;
  const bool live = v < D;
  const int entry = blockIdx.x, head = blockIdx.y;
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int64_t col0 = (int64_t)head * D;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + ((int64_t)head * D + (live ? v : 0)) * D;
  if (live && p.positions[row0] == 0)
    for (int c = 0; c < D; ++c) st[c] = 0.f;
  for (int t = 0; t < n_rows; ++t) {
    const int64_t row = row0 + t;
    __syncthreads();
    if (live) {
      sk[v] = p.k[row * p.k_stride + col0 + v];
      sw[v] = p.w_pre[row * p.w_stride + col0 + v];
      sr[v] = p.r[row * p.r_stride + col0 + v];
      sa[v] = RULE == RULE_DELTA ? p.a_pre[row * p.a_stride + col0 + v] : p.bonus[col0 + v];
    }
    const float kk = block_sum(live ? sk[v] * sk[v] : 0.f, scratch);   // (its barriers also publish the vectors)
    if (!live) continue;
    const float kn = 1.f / sqrtf(kk + 1e-6f);
    const float vv = p.v[row * p.v_stride + col0 + v];
    float o = 0.f;
    if (RULE == RULE_DELTA) {
      float us = 0.f;
      for (int c = 0; c < D; ++c) us = fmaf(sk[c] * kn, st[c], us);
      for (int c = 0; c < D; ++c) {
        const float s = sw[c] * st[c] - (sa[c] * (sk[c] * kn)) * us + sk[c] * vv;
        st[c] = s;
        o = fmaf(s, sr[c], o);
      }
    } else {
      for (int c = 0; c < D; ++c) {
        const float kv = sk[c] * vv;
        o = fmaf(st[c] + sa[c] * kv, sr[c], o);
        st[c] = sw[c] * st[c] + kv;
      }
    }
    p.o_raw[row * p.o_stride + col0 + v] = o;
  }
}

// out = o / sqrt(mean_head(o^2) + eps) * norm_w * gate(g_pre), head by head: a wave a (row, head).
// den (may be nullptr) float32 [rows][heads]: o is divided by it first, head by head.
template <typename T, int RULE>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, int64_t o_stride,
                                                             const float* __restrict__ g_pre, int64_t g_stride,
                                                             const float* __restrict__ norm_w, float eps,
                                                             T* __restrict__ out, int64_t out_stride, int heads, int dim,
                                                             const float* __restrict__ den) {
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE;
  const int h = blockIdx.y * 4 + wave;
  if (h < heads) {
    const float* oh = o + row * o_stride + (int64_t)h * dim;
    const float dn = den != nullptr ? 1.f / den[row * heads + h] : 1.f;
    float ss = 0.f;
    for (int c = lane; c < dim; c += DLI_WAVE) ss += (oh[c] * dn) * (oh[c] * dn);
    const float r = dn / sqrtf(wave_sum(ss) / (float)dim + eps);
    for (int c = lane; c < dim; c += DLI_WAVE) {
      float gate = 1.f;                                   // RULE 2: no gate (g_pre is not read)
      if (RULE != GATE_NONE) {
        const float g = g_pre[row * g_stride + (int64_t)h * dim + c];
        gate = RULE == RULE_DELTA ? 1.f / (1.f + expf(-g)) : g / (1.f + expf(-g));
      }
      out[row * out_stride + (int64_t)h * dim + c] = from_f32<T>(oh[c] * r * norm_w[(int64_t)h * dim + c] * gate);
    }
  }
}

// The same for one head that spans a long row: a workgroup a row.
template <typename T, int RULE>
__global__ __launch_bounds__(256) void row_norm_gate_kernel(const float* __restrict__ o, int64_t o_stride,
                                                            const float* __restrict__ g_pre, int64_t g_stride,
                                                            const float* __restrict__ norm_w, float eps, T* __restrict__ out,
                                                            int64_t out_stride, int dim, const float* __restrict__ den) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const float* oh = o + row * o_stride;
  const float dn = den != nullptr ? 1.f / den[row] : 1.f;
  float ss = 0.f;
  for (int c = threadIdx.x; c < dim; c += blockDim.x) ss += (oh[c] * dn) * (oh[c] * dn);
  const float r = dn / sqrtf(block_sum(ss, scratch) / (float)dim + eps);
  for (int c = threadIdx.x; c < dim; c += blockDim.x) {
    float gate = 1.f;
    if (RULE != GATE_NONE) {
      const float g = g_pre[row * g_stride + c];
      gate = RULE == RULE_DELTA ? 1.f / (1.f + expf(-g)) : g / (1.f + expf(-g));
    }
    out[row * out_stride + c] = from_f32<T>(oh[c] * r * norm_w[c] * gate);
  }
}

template <int RULE>
static int launch_scan(const ScanArgs& p, int entries, int rows, int dim, int out_is_bf16, hipStream_t stream) {
  // sixteen lanes a column (four columns a wave) where the head's size is a multiple of 16, else eight
  const int parts = dim % 16 == 0 ? 16 : 8;
  const dim3 grid(entries, p.heads, dim / (64 / parts));
  // a step of single tokens stages one token a wave; any other stages 16 (8 for heads above 64)
  const bool single = rows == entries;
#define SCAN_CASE(DIM, PARTS, TBM)                                                                          \
  case DIM:                                                                                                 \
    if (single) recurrent_scan_kernel<DIM / PARTS, PARTS, RULE, 1><<<grid, 64, 0, stream>>>(p);             \
    else recurrent_scan_kernel<DIM / PARTS, PARTS, RULE, TBM><<<grid, 64, 0, stream>>>(p);                  \
    break;
  switch (dim) {
    SCAN_CASE(16, 16, 16) SCAN_CASE(24, 8, 16) SCAN_CASE(32, 16, 16) SCAN_CASE(40, 8, 16) SCAN_CASE(48, 16, 16)
    SCAN_CASE(56, 8, 16) SCAN_CASE(64, 16, 16) SCAN_CASE(80, 16, 8) SCAN_CASE(96, 16, 8) SCAN_CASE(112, 16, 8)
    SCAN_CASE(128, 16, 8)
    default: {
      const int threads = (dim + 63) / 64 * 64;
      recurrent_scan_any_kernel<RULE><<<dim3(entries, p.heads), threads, (4 * dim + 16) * sizeof(float), stream>>>(p, dim);
    }
  }
#undef SCAN_CASE
  if (dli_launch_status() != DLI_OK) return DLI_ERR_LAUNCH;
  if (out_is_bf16)
    head_norm_gate_kernel<bf16_t, RULE><<<dim3(rows, (p.heads + 3) / 4), 256, 0, stream>>>(p.o_raw, p.o_stride, p.g_pre, p.g_stride, p.norm_w, p.eps,
                                                                  (bf16_t*)p.out, p.out_stride, p.heads, dim, nullptr);
  else
    head_norm_gate_kernel<float, RULE><<<dim3(rows, (p.heads + 3) / 4), 256, 0, stream>>>(p.o_raw, p.o_stride, p.g_pre, p.g_stride, p.norm_w, p.eps,
                                                                 (float*)p.out, p.out_stride, p.heads, dim, nullptr);
  return dli_launch_status();
}

// Head sizes that are taken: 16 to 64 in steps of 8 and 80 to 128 in steps of 16 by the kernel
// above, any other from 1 to 1024 by the slow one.
extern "C" int dli_recurrent_scan_supports(int dim) { return dim >= 1 && dim <= 1024; }

extern "C" int dli_recurrent_scan(const float* r, int64_t r_stride, const float* k, int64_t k_stride, const float* v,
                                  int64_t v_stride, const float* w_pre, int64_t w_stride, const float* a_pre,
                                  int64_t a_stride, const float* a_bias, const float* g_pre, int64_t g_stride,
                                  const float* bonus, const float* norm_w, float eps, float* state,
                                  int64_t state_stride, const int* q_start, const int* positions,
                                  const int* state_slots, float* o_raw, int64_t o_stride, void* out,
                                  int64_t out_stride, int entries, int rows, int heads, int dim, int rule,
                                  int out_is_bf16, hipStream_t stream) {
  if (entries <= 0 || rows <= 0) return DLI_OK;
  if (rows < entries || !dli_recurrent_scan_supports(dim) || heads <= 0 || heads > 65535 || (rule != RULE_DELTA && rule != RULE_BONUS) ||
      state_stride < (int64_t)heads * dim * dim || (rule == RULE_DELTA && a_pre == nullptr) ||
      (rule == RULE_BONUS && bonus == nullptr))
    return DLI_ERR_ARGUMENT;
  ScanArgs p;
  p.r = r; p.k = k; p.v = v; p.w_pre = w_pre; p.a_pre = a_pre; p.a_bias = a_bias; p.g_pre = g_pre;
  p.r_stride = r_stride; p.k_stride = k_stride; p.v_stride = v_stride; p.w_stride = w_stride;
  p.a_stride = a_stride; p.g_stride = g_stride;
  p.bonus = bonus; p.norm_w = norm_w; p.eps = eps; p.state = state; p.state_stride = state_stride;
  p.q_start = q_start; p.positions = positions; p.state_slots = state_slots; p.out = out; p.out_stride = out_stride;
  p.o_raw = o_raw; p.o_stride = o_stride;
  p.heads = heads;
  if (o_raw == nullptr || o_stride < (int64_t)heads * dim) return DLI_ERR_ARGUMENT;
  return rule == RULE_DELTA ? launch_scan<RULE_DELTA>(p, entries, rows, dim, out_is_bf16, stream)
                            : launch_scan<RULE_BONUS>(p, entries, rows, dim, out_is_bf16, stream);
}

// The per-head norm and gate alone, for a recurrence whose own kernel leaves o in 32-bit:
// out = o / sqrt(mean_head(o^2) + eps) * norm_w * gate(g_pre), gate_silu: silu, else sigmoid.
// norm_w holds heads * dim values (a weight that the heads share is repeated by the caller).
extern "C" int dli_head_norm_gate(const float* o, int64_t o_stride, const float* g_pre, int64_t g_stride,
                                  const float* norm_w, float eps, void* out, int64_t out_stride, int rows, int heads,
                                  int dim, int gate, const float* den, int out_is_bf16, hipStream_t stream) {
  // gate: 0 sigmoid(g_pre), 1 silu(g_pre), 2 none
  if (rows <= 0) return DLI_OK;
  const int64_t width = (int64_t)heads * dim;
  if (heads <= 0 || dim <= 0 || o_stride < width || out_stride < width || gate < 0 || gate > 2 ||
      (gate != GATE_NONE && (g_pre == nullptr || g_stride < width)))
    return DLI_ERR_ARGUMENT;
  const dim3 grid(rows, (heads + 3) / 4);
  if (grid.y > 65535) return DLI_ERR_ARGUMENT;
#define HNG(T, RULE)                                                                                                     \
  do {                                                                                                                   \
    if (heads == 1 && dim > 256)                                                                                         \
      row_norm_gate_kernel<T, RULE><<<rows, 256, 0, stream>>>(o, o_stride, g_pre, g_stride, norm_w, eps, (T*)out, out_stride, dim, den); \
    else                                                                                                                 \
      head_norm_gate_kernel<T, RULE><<<grid, 256, 0, stream>>>(o, o_stride, g_pre, g_stride, norm_w, eps, (T*)out, out_stride, heads, dim, den); \
  } while (0)
  if (out_is_bf16) { if (gate == GATE_NONE) HNG(bf16_t, GATE_NONE); else if (gate) HNG(bf16_t, RULE_BONUS); else HNG(bf16_t, RULE_DELTA); }
  else { if (gate == GATE_NONE) HNG(float, GATE_NONE); else if (gate) HNG(float, RULE_BONUS); else HNG(float, RULE_DELTA); }
#undef HNG
  return dli_launch_status();
}
