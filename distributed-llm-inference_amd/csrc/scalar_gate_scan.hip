// Linear recurrences with a matrix state per head under scalar gates: with a keep factor a_t and a write
// factor b_t per token and head, a query q and a key k (D values a head) and a value v (V values a head),
//
//   S_t = a_t S_(t-1) + b_t k_t v_t^T,   o_t = S_t^T q_t      (o is made from the state that already holds the token)
//
// Two uses: a constant decay per head (a = decay[head], b = 1: linear attention with a decay), and a matrix
// memory with exponential input and forget gates, whose factors come from log gates i_t, f_t under a running
// reference point m (m_0 = 0):
//
//   m_t = max(f_t + m_(t-1), i_t),  a_t = exp(f_t + m_(t-1) - m_t),  b_t = exp(i_t - m_t)
//
// and whose result is divided by max(|n_t . q_t|, exp(-m_t)) + 1e-6 with n_t = a_t n_(t-1) + b_t k_t. n is the
// state's column for a value that is always one, so the scan carries V + 1 columns and leaves the
// denominators in an array of their own (`den`), for the kernel that normalises the heads.
//
// S is float32 [heads][V (+ 1)][D] in the request's state slot (then m [heads] for the matrix memory) and
// starts from zeros where the entry's first row has position 0; an entry's rows are walked in order from
// what the step before left. Everything is 32-bit.
//
//   exp_gates          from the gates' 32-bit pre-activations: i = cap tanh((x_i + b_i) / cap),
//                      f = logsigmoid(cap tanh((x_f + b_f) / cap)), then m, a, b and exp(-m) per token and head.
//                      A wave an (entry, head); 64 tokens at a time: with F the running sum of f inside the
//                      block, m_t = F_t + max(m_in, max_(s <= t)(i_s - F_s)), two scans over the lanes
//   scalar_gate_scan   the recurrence
//   silu_columns       silu in place on some columns of a float32 matrix (a step with portions applies it to q, k and v
//                      beforehand, all threads at once; inside the scan it would sit on the one wave that walks the tokens)
//
// The scan: one wave takes one (entry, head, slice of 4 columns). Sixteen lanes (a DPP row) share a column: lane
// (col, part) keeps S[part's D/16 keys][col] in registers, and a token's sum over the keys meets in four DPP
// swaps. The vectors of TB tokens are staged in LDS (with silu and the query's scale applied on the way, off the
// chain) while the next TB are in flight. Heads whose D is no multiple of 16 (or above 256) take a
// thread-per-column kernel with the state in memory.
#include "common.h"

struct SgArgs {
  const float* q; int64_t q_stride;      // [rows][>= heads * D], already at the first column
  const float* k; int64_t k_stride;
  const float* v; int64_t v_stride;      // [rows][>= heads * V]
  const float* keep; const float* write; int64_t gate_stride;   // [rows][heads]; keep == nullptr: decay[head] and 1
  const float* decay;                    // [heads]
  const float* floor;                    // [rows][heads] exp(-m_t): with it the last column is n, and den is written
  float* den;                            // [rows][heads]
  float* state; int64_t state_stride;
  const int* q_start; const int* positions; const int* state_slots;
  float* o; int64_t o_stride;            // [rows][heads * V]
  int heads, vdim;
  float q_scale; int silu;
};

__device__ __forceinline__ float sg_row_sum(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, false));
  return x;
}

__device__ __forceinline__ float sg_act(float x, int silu) { return silu ? x / (1.f + expf(-x)) : x; }

// NK keys a lane, D = 16 NK; TB tokens staged at once (1 in a step of single tokens). GATED: keep and write factors
// per token (else the head's constant decay and one), and with them the column of n and the denominators; SILU:
// q, k and v pass through silu on their way into LDS. No load hangs on a condition (what is not wanted is read
// from a clamped place and dropped), so that a batch's loads stay in flight while the chain of the one before runs.
template <int NK, int TB, bool GATED, bool SILU>
__global__ __launch_bounds__(64) void scalar_gate_scan_kernel(SgArgs p) {
  constexpr int D = NK * 16, COLS = 4, PER = (TB * D + 63) / 64;
  __shared__ float sk[PER * 64], sq[PER * 64], sv[TB * COLS], sa[TB], sb[TB], sfl[TB];
  const int lane = threadIdx.x, vloc = lane / 16, part = lane % 16;
  const int entry = blockIdx.x, head = blockIdx.y;
  const int V = p.vdim, VX = V + (GATED ? 1 : 0);
  const int my_col = (int)blockIdx.z * COLS + vloc;
  const int col = min(my_col, VX - 1);          // lanes past the last column repeat it and store nothing
  const bool live = my_col < VX, is_n = GATED && col == V;
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int64_t qk_col = (int64_t)head * D, v_col = (int64_t)head * V;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + ((int64_t)head * VX + col) * D + part * NK;
  float s[NK];
  const bool fresh = p.positions[row0] == 0;
#pragma unroll
  for (int i = 0; i < NK; ++i) {
    const float old = st[i];
    s[i] = fresh ? 0.f : old;
  }
  const float decay = GATED ? 1.f : p.decay[head];
  float pk[PER], pq[PER], pv = 0.f, pa = 1.f, pb = 1.f, pf = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int m = 0; m < PER; ++m) {
      const int e = min(lane + 64 * m, TB * D - 1), t = e / D, c = e - t * D;
      const int64_t row = row0 + min(t0 + t, n_rows - 1);
      pk[m] = p.k[row * p.k_stride + qk_col + c];
      pq[m] = p.q[row * p.q_stride + qk_col + c];
    }
    {
      const int64_t row = row0 + min(t0 + min(lane / COLS, TB - 1), n_rows - 1);
      const int c = (int)blockIdx.z * COLS + lane % COLS;
      pv = p.v[row * p.v_stride + v_col + min(c, V - 1)];
    }
    if (GATED) {
      const int64_t row = row0 + min(t0 + min(lane, TB - 1), n_rows - 1);
      pa = p.keep[row * p.gate_stride + head];
      pb = p.write[row * p.gate_stride + head];
      pf = p.floor[row * p.gate_stride + head];
    }
  };
  auto step = [&](int t, int64_t row) {
    const float* kt = sk + t * D + part * NK;
    const float* qt = sq + t * D + part * NK;
    const float a = sa[t], bv = sb[t] * sv[t * COLS + vloc];
    float o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      s[i] = fmaf(a, s[i], bv * kt[i]);
      if (i & 1) o1 = fmaf(qt[i], s[i], o1); else o0 = fmaf(qt[i], s[i], o0);
    }
    const float o = sg_row_sum(o0 + o1);
    if (part == 0 && live) {
      if (is_n) p.den[row * p.heads + head] = fmaxf(fabsf(o), sfl[t]) + 1e-6f;
      else p.o[row * p.o_stride + v_col + col] = o;
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < n_rows; t0 += TB) {
#pragma unroll
    for (int m = 0; m < PER; ++m) {
      sk[lane + 64 * m] = sg_act(pk[m], SILU);
      sq[lane + 64 * m] = sg_act(pq[m], SILU) * p.q_scale;
    }
    if (lane < TB * COLS) {
      const int c = (int)blockIdx.z * COLS + lane % COLS;
      sv[lane] = GATED && c >= V ? 1.f : sg_act(pv, SILU);   // the column of n reads a value of one
    }
    if (lane < TB) {
      sa[lane] = GATED ? pa : decay;
      sb[lane] = pb;
      sfl[lane] = pf;
    }
    if (TB > 1) fetch(t0 + TB);  // on their way while the chain below runs (past the last row: the last row again, dropped)
    __syncthreads();
    const int nb = min(TB, n_rows - t0);
    if (nb == TB) {
#pragma unroll
      for (int t = 0; t < TB; ++t) step(t, row0 + t0 + t);
    } else {
      for (int t = 0; t < nb; ++t) step(t, row0 + t0 + t);
    }
    __syncthreads();  // the chain has read this batch before the next one is written
  }
  if (live)
#pragma unroll
    for (int i = 0; i < NK; ++i) st[i] = s[i];
}

// Any D and V: a thread a column, the column's state in the request's slot.
__global__ void scalar_gate_any_kernel(SgArgs p, int D) {
  extern __shared__ float sh[];
  float *sk = sh, *sq = sh + D;
  const int V = p.vdim, VX = V + (p.floor != nullptr ? 1 : 0);
  const int c = blockIdx.z * blockDim.x + threadIdx.x;
  const bool live = c < VX, is_n = p.floor != nullptr && c == V;
  const int entry = blockIdx.x, head = blockIdx.y;
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int64_t qk_col = (int64_t)head * D, v_col = (int64_t)head * V;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + ((int64_t)head * VX + (live ? c : 0)) * D;
  if (live && p.positions[row0] == 0)
    for (int i = 0; i < D; ++i) st[i] = 0.f;
  for (int t = 0; t < n_rows; ++t) {
    const int64_t row = row0 + t;
    __syncthreads();
    for (int i = threadIdx.x; i < D; i += blockDim.x) {
      sk[i] = sg_act(p.k[row * p.k_stride + qk_col + i], p.silu);
      sq[i] = sg_act(p.q[row * p.q_stride + qk_col + i], p.silu) * p.q_scale;
    }
    __syncthreads();
    if (!live) continue;
    const float a = p.keep != nullptr ? p.keep[row * p.gate_stride + head] : p.decay[head];
    const float b = p.keep != nullptr ? p.write[row * p.gate_stride + head] : 1.f;
    const float bv = b * (is_n ? 1.f : sg_act(p.v[row * p.v_stride + v_col + c], p.silu));
    float o = 0.f;
    for (int i = 0; i < D; ++i) {
      const float s = fmaf(a, st[i], bv * sk[i]);
      st[i] = s;
      o = fmaf(sq[i], s, o);
    }
    if (is_n) p.den[row * p.heads + head] = fmaxf(fabsf(o), p.floor[row * p.gate_stride + head]) + 1e-6f;
    else p.o[row * p.o_stride + v_col + c] = o;
  }
}

// Steps with portions, heads of 16 to 64 keys in steps of 16: the same recurrence 64 tokens at a time on the matrix
// cores, all in 32-bit (v_mfma_f32_16x16x4_f32). With A_t the running sum of log a inside the chunk (never above zero,
// so every factor below is at most one), w_s = exp(A_last - A_s) b_s and S the state before the chunk:
//
//   P[t][s] = (q_t . k_s) exp(A_t - A_s) b_s  for s <= t,   o_t = sum_s P[t][s] v_s + exp(A_t) S^T q_t,
//   S <- exp(A_last) S + sum_s w_s k_s v_s^T,
//
// and for the matrix memory n_t . q_t = sum_s P[t][s] + exp(A_t) (n . q_t), n <- exp(A_last) n + sum_s w_s k_s.
// A workgroup of four waves takes one (entry, head, slice of 16 value columns) and walks the entry's chunks in
// order, the next chunk's rows on their way into registers while this one is multiplied. Q, K and P lie in LDS row by
// row, V and the state's slice column by column (as the state is kept), every row padded by four floats: a lane
// then reads the four k of four consecutive matrix instructions as one 16-byte access (the instructions' k may be
// dealt to the lanes in any order as long as both operands agree: lane group g takes k = 16 step + 4 g .. + 3),
// and sixteen rows fall into all 64 banks. Wave w makes the rows 16 w .. 16 w + 15 of P and of the chunk's
// results, and sixteen keys' rows of the new state. Rows past the entry's last count as a = 1, b = 0 and
// q = k = v = 0. The slice that holds column 0 also carries n and writes the denominators.
typedef float sg_f4 __attribute__((ext_vector_type(4)));

template <int D, bool GATED>
__global__ __launch_bounds__(256) void scalar_gate_chunk_kernel(SgArgs p, const float* __restrict__ log_keep) {
  constexpr int C = 64, VS = 16, DS = D + 4, PS = C + 4, QK_PER = C * D / 256, V_PER = C * VS / 256;
  __shared__ __attribute__((aligned(16))) float sQ[C * DS], sK[C * DS], sP[C * PS], sVt[VS * PS], sSt[VS * DS], sW[C];
  __shared__ float sN[D], sB[C], sFl[C];
  __shared__ double sA[C];   // the running sums of log a: their differences are taken before rounding (a chunk's sum may
                             // reach the hundreds, where a float's last bit is 1e-5 of the factor it stands for)
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int li = lane % 16, lk = lane / 16;                 // a matrix operand's row (or column) and its group of k; a result's column and group of four rows
  const int entry = blockIdx.x, head = blockIdx.y, v0 = (int)blockIdx.z * VS;
  const int V = p.vdim, VX = V + (GATED ? 1 : 0);
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const bool fresh = p.positions[row0] == 0, with_n = GATED && blockIdx.z == 0;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + (int64_t)head * VX * D;
  const int64_t qk_col = (int64_t)head * D, v_col = (int64_t)head * V;
  for (int idx = tid; idx < D * VS; idx += 256) {
    const int j = idx / D, d = idx - j * D;                 // the state keeps a column's keys side by side
    const float old = v0 + j < V ? st[(int64_t)(v0 + j) * D + d] : 0.f;
    sSt[j * DS + d] = fresh ? 0.f : old;
  }
  if (tid < D) {
    const float old = with_n ? st[(int64_t)V * D + tid] : 0.f;
    sN[tid] = fresh ? 0.f : old;
  }
  const float log_decay = GATED ? 0.f : fmaxf(logf(p.decay[head]), -1e30f);
  float rq[QK_PER], rk[QK_PER], rv[V_PER], rla = 0.f, rb = 0.f, rfl = 0.f;
  auto fetch = [&](int t0) {                                // rows past the last: the last row again, dropped when staged
#pragma unroll
    for (int m = 0; m < QK_PER; ++m) {
      const int idx = tid + 256 * m, t = idx / D, d = idx - t * D;
      const int64_t row = row0 + min(t0 + t, n_rows - 1);
      rk[m] = p.k[row * p.k_stride + qk_col + d];
      rq[m] = p.q[row * p.q_stride + qk_col + d];
    }
#pragma unroll
    for (int m = 0; m < V_PER; ++m) {
      const int idx = tid + 256 * m, t = idx / VS, j = idx - t * VS;
      const int64_t row = row0 + min(t0 + t, n_rows - 1);
      rv[m] = p.v[row * p.v_stride + v_col + min(v0 + j, V - 1)];
    }
    if (GATED) {
      const int64_t at = (int64_t)(row0 + min(t0 + lane, n_rows - 1)) * p.gate_stride + head;
      rla = log_keep[at];
      rb = p.write[at];
      rfl = p.floor[at];
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < n_rows; t0 += C) {
    const int nb = min(C, n_rows - t0);
    __syncthreads();                                        // the chunk before has been read, the state's slice is whole
#pragma unroll
    for (int m = 0; m < QK_PER; ++m) {
      const int idx = tid + 256 * m, t = idx / D, d = idx - t * D;
      sK[t * DS + d] = t < nb ? rk[m] : 0.f;
      sQ[t * DS + d] = t < nb ? rq[m] * p.q_scale : 0.f;
    }
#pragma unroll
    for (int m = 0; m < V_PER; ++m) {
      const int idx = tid + 256 * m, t = idx / VS, j = idx - t * VS;
      sVt[j * PS + t] = t < nb && v0 + j < V ? rv[m] : 0.f;
    }
    if (wave == 0) {
      double la = GATED ? rla : log_decay;
      float b = GATED ? rb : 1.f;
      if (lane >= nb) { la = 0.0; b = 0.f; }
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const double up = __shfl_up(la, d, DLI_WAVE);
        if (lane >= d) la += up;
      }
      const double last = __shfl(la, 63, DLI_WAVE);
      sA[lane] = la;
      sB[lane] = b;
      sW[lane] = expf((float)(last - la)) * b;
      sFl[lane] = rfl;
    }
    fetch(t0 + C);                                          // the next chunk's rows, on their way while this one is multiplied
    __syncthreads();
    const float a_last = (float)sA[C - 1];
    // P: this wave's sixteen rows against the key blocks up to its own
#pragma unroll
    for (int cb = 0; cb < 4; ++cb) {
      if (cb > wave) break;
      sg_f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int g = 0; g < D / 16; ++g) {
        const sg_f4 a4 = *reinterpret_cast<const sg_f4*>(sQ + (16 * wave + li) * DS + 16 * g + 4 * lk);
        const sg_f4 b4 = *reinterpret_cast<const sg_f4*>(sK + (16 * cb + li) * DS + 16 * g + 4 * lk);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[j], b4[j], acc, 0, 0, 0);
      }
      const int s_ = 16 * cb + li;
      const double as = sA[s_];
      const float bs = sB[s_];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = 16 * wave + 4 * lk + r;
        sP[t * PS + s_] = s_ <= t ? acc[r] * expf((float)(sA[t] - as)) * bs : 0.f;
      }
    }
    __syncthreads();
    {
      sg_f4 acc = {0.f, 0.f, 0.f, 0.f}, far = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        if (g > wave) break;
        const sg_f4 a4 = *reinterpret_cast<const sg_f4*>(sP + (16 * wave + li) * PS + 16 * g + 4 * lk);
        const sg_f4 b4 = *reinterpret_cast<const sg_f4*>(sVt + li * PS + 16 * g + 4 * lk);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[j], b4[j], acc, 0, 0, 0);
      }
#pragma unroll
      for (int g = 0; g < D / 16; ++g) {
        const sg_f4 a4 = *reinterpret_cast<const sg_f4*>(sQ + (16 * wave + li) * DS + 16 * g + 4 * lk);
        const sg_f4 b4 = *reinterpret_cast<const sg_f4*>(sSt + li * DS + 16 * g + 4 * lk);
#pragma unroll
        for (int j = 0; j < 4; ++j) far = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[j], b4[j], far, 0, 0, 0);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = 16 * wave + 4 * lk + r;
        if (t < nb && v0 + li < V)
          p.o[(int64_t)(row0 + t0 + t) * p.o_stride + v_col + v0 + li] = fmaf(expf((float)sA[t]), far[r], acc[r]);
      }
      if (with_n) {                                         // row t = 16 wave + li, a quarter of its sums a lane
        const int t = 16 * wave + li;
        float sum = 0.f, qn = 0.f;
        for (int s_ = 16 * lk; s_ < 16 * lk + 16; ++s_) sum += s_ <= t ? sP[t * PS + s_] : 0.f;
        for (int d = lk * (D / 4); d < (lk + 1) * (D / 4); ++d) qn = fmaf(sQ[t * DS + d], sN[d], qn);
        sum += __shfl_xor(sum, 16, DLI_WAVE);
        sum += __shfl_xor(sum, 32, DLI_WAVE);
        qn += __shfl_xor(qn, 16, DLI_WAVE);
        qn += __shfl_xor(qn, 32, DLI_WAVE);
        if (lk == 0 && t < nb)
          p.den[(int64_t)(row0 + t0 + t) * p.heads + head] = fmaxf(fabsf(fmaf(expf((float)sA[t]), qn, sum)), sFl[t]) + 1e-6f;
      }
    }
    __syncthreads();                                        // the old state has been read by all
    if (wave < D / 16) {
      // the new state's keys 16 wave .. + 15 for the slice's sixteen columns: (w V)^T K, a result's row a column of the slice
      sg_f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const sg_f4 v4 = *reinterpret_cast<const sg_f4*>(sVt + li * PS + 16 * g + 4 * lk);
        const sg_f4 w4 = *reinterpret_cast<const sg_f4*>(sW + 16 * g + 4 * lk);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc = __builtin_amdgcn_mfma_f32_16x16x4f32(v4[j] * w4[j], sK[(16 * g + 4 * lk + j) * DS + 16 * wave + li], acc, 0, 0, 0);
      }
      const float keep_all = expf(a_last);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float* at = sSt + (4 * lk + r) * DS + 16 * wave + li;
        *at = fmaf(keep_all, *at, acc[r]);
      }
    }
    if (with_n && tid >= 192 && tid - 192 < D) {            // (the last wave has no rows of the state to make for heads under 64)
      const int d = tid - 192;
      float sum = 0.f;
#pragma unroll 8
      for (int s_ = 0; s_ < C; ++s_) sum = fmaf(sW[s_], sK[s_ * DS + d], sum);
      sN[d] = fmaf(expf(a_last), sN[d], sum);
    }
  }
  __syncthreads();
  for (int idx = tid; idx < D * VS; idx += 256) {
    const int j = idx / D, d = idx - j * D;
    if (v0 + j < V) st[(int64_t)(v0 + j) * D + d] = sSt[j * DS + d];
  }
  if (with_n && tid < D) st[(int64_t)V * D + tid] = sN[tid];
}

// pre [rows][stride]: the input gate's pre-activation of head h at column i_off + h, the forget gate's at
// f_off + h; m of head h at state[slot][m_off + h]. keep, write, floor: [rows][heads].
__global__ __launch_bounds__(64) void exp_gates_kernel(const float* __restrict__ pre, int64_t stride, int i_off, int f_off,
                                                       const float* __restrict__ i_bias, const float* __restrict__ f_bias,
                                                       float cap, float* __restrict__ state, int64_t state_stride,
                                                       int64_t m_off, const int* __restrict__ q_start,
                                                       const int* __restrict__ positions, const int* __restrict__ state_slots,
                                                       float* __restrict__ keep, float* __restrict__ write,
                                                       float* __restrict__ floor, float* __restrict__ log_keep, int heads) {
  const int lane = threadIdx.x, entry = blockIdx.x, head = blockIdx.y;
  const int row0 = q_start[entry], n_rows = q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  float* ms = state + (int64_t)state_slots[entry] * state_stride + m_off + head;
  const float m_old = *ms;
  float m_in = positions[row0] == 0 ? 0.f : m_old;
  const float ib = i_bias != nullptr ? i_bias[head] : 0.f, fb = f_bias != nullptr ? f_bias[head] : 0.f;
  for (int t0 = 0; t0 < n_rows; t0 += 64) {
    const int nb = min(64, n_rows - t0);
    const bool have = lane < nb;
    const int64_t row = row0 + t0 + min(lane, nb - 1);
    float gi = pre[row * stride + i_off + head] + ib, gf = pre[row * stride + f_off + head] + fb;
    if (cap > 0.f) {
      gi = cap * tanhf(gi / cap);
      gf = cap * tanhf(gf / cap);
    }
    gf = fminf(gf, 0.f) - log1pf(expf(-fabsf(gf)));          // log sigmoid
    if (!have) { gi = -INFINITY; gf = 0.f; }
    float F = gf;                                             // running sum of f inside the block
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float up = __shfl_up(F, d, DLI_WAVE);
      if (lane >= d) F += up;
    }
    float G = gi - F;                                         // running maximum of i_s - F_s
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float up = __shfl_up(G, d, DLI_WAVE);
      if (lane >= d) G = fmaxf(G, up);
    }
    const float m = F + fmaxf(m_in, G);
    float m_prev = __shfl_up(m, 1, DLI_WAVE);
    if (lane == 0) m_prev = m_in;
    if (have) {
      const int64_t at = (row0 + t0 + lane) * (int64_t)heads + head;
      keep[at] = expf(gf + m_prev - m);
      log_keep[at] = fminf(gf + m_prev - m, 0.f);
      write[at] = expf(gi - m);
      floor[at] = expf(-m);
    }
    m_in = __shfl(m, nb - 1, DLI_WAVE);
  }
  if (lane == 0) *ms = m_in;
}

// x [rows][stride] float32: the first `width` columns become silu of themselves. A thread an element.
__global__ void silu_columns_kernel(float* __restrict__ x, int64_t stride, int width) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= width) return;
  const float v = x[row * stride + i];
  x[row * stride + i] = v / (1.f + expf(-v));
}

extern "C" {

int dli_silu_columns(float* x, int64_t stride, int rows, int width, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0 || stride < width) return DLI_ERR_ARGUMENT;
  const dim3 grid(rows, (width + 255) / 256);
  if (grid.y > 65535) return DLI_ERR_ARGUMENT;
  silu_columns_kernel<<<grid, 256, 0, stream>>>(x, stride, width);
  return dli_launch_status();
}

int dli_exp_gates(const float* pre, int64_t stride, int i_off, int f_off, const float* i_bias, const float* f_bias, float cap,
                  float* state, int64_t state_stride, int64_t m_off, const int* q_start, const int* positions,
                  const int* state_slots, float* keep, float* write, float* floor, float* log_keep, int entries, int rows,
                  int heads, hipStream_t stream) {
  if (rows <= 0 || entries <= 0) return DLI_OK;
  if (rows < entries || heads <= 0 || heads > 65535 || i_off < 0 || f_off < 0 || i_off + heads > stride ||
      f_off + heads > stride || m_off < 0 || m_off + heads > state_stride || cap < 0.f)
    return DLI_ERR_ARGUMENT;
  exp_gates_kernel<<<dim3(entries, heads), 64, 0, stream>>>(pre, stride, i_off, f_off, i_bias, f_bias, cap, state,
                                                            state_stride, m_off, q_start, positions, state_slots, keep, write,
                                                            floor, log_keep, heads);
  return dli_launch_status();
}

// keep, write: [rows][heads] or both nullptr (then decay [heads] and a write factor of one); floor and den
// [rows][heads] come together, and with them the state has a column more a head.
int dli_scalar_gate_scan(const float* q, int64_t q_stride, const float* k, int64_t k_stride, const float* v, int64_t v_stride,
                         const float* keep, const float* write, const float* log_keep, int64_t gate_stride, const float* decay,
                         const float* floor, float* den, float* state, int64_t state_stride, const int* q_start, const int* positions,
                         const int* state_slots, float* o, int64_t o_stride, int entries, int rows, int heads, int dim,
                         int vdim, float q_scale, int silu, int chunked, hipStream_t stream) {
  if (rows <= 0 || entries <= 0) return DLI_OK;
  const int vx = vdim + (floor != nullptr ? 1 : 0);
  if (rows < entries || heads <= 0 || heads > 65535 || dim <= 0 || dim > 4096 || vdim <= 0 ||
      state_stride < (int64_t)heads * vx * dim || o_stride < (int64_t)heads * vdim || q_stride < (int64_t)heads * dim ||
      k_stride < (int64_t)heads * dim || v_stride < (int64_t)heads * vdim || (keep == nullptr) != (write == nullptr) ||
      (keep == nullptr && decay == nullptr) || (keep != nullptr && gate_stride < heads) || (floor == nullptr) != (den == nullptr) ||
      (floor != nullptr && keep == nullptr))
    return DLI_ERR_ARGUMENT;
  SgArgs p;
  p.q = q; p.q_stride = q_stride; p.k = k; p.k_stride = k_stride; p.v = v; p.v_stride = v_stride; p.keep = keep;
  p.write = write; p.gate_stride = gate_stride; p.decay = decay; p.floor = floor; p.den = den; p.state = state;
  p.state_stride = state_stride; p.q_start = q_start; p.positions = positions; p.state_slots = state_slots; p.o = o;
  p.o_stride = o_stride; p.heads = heads; p.vdim = vdim; p.q_scale = q_scale; p.silu = silu;
  const bool single = rows == entries;
  const dim3 grid(entries, heads, (vx + 3) / 4);
  if (grid.z > 65535) return DLI_ERR_ARGUMENT;
  const bool gated = keep != nullptr;
  if (gated && floor == nullptr) return DLI_ERR_ARGUMENT;   // (gates without a normaliser: no model asks for them yet)
  if (!single && !silu && dim % 16 == 0 && dim <= 64 && (!gated || log_keep != nullptr) && chunked) {
    // a step with portions: chunks of 64 tokens on the matrix cores
    const dim3 cgrid(entries, heads, (vdim + 15) / 16);
    if (cgrid.z > 65535) return DLI_ERR_ARGUMENT;
#define SG_CHUNK(DIM)                                                                                   \
  case DIM:                                                                                             \
    if (gated) scalar_gate_chunk_kernel<DIM, true><<<cgrid, 256, 0, stream>>>(p, log_keep);             \
    else scalar_gate_chunk_kernel<DIM, false><<<cgrid, 256, 0, stream>>>(p, log_keep);                  \
    break;
    switch (dim) { SG_CHUNK(16) SG_CHUNK(32) SG_CHUNK(48) SG_CHUNK(64) }
#undef SG_CHUNK
    return dli_launch_status();
  }
#define SG_LAUNCH(NK, TBV)                                                                                  \
  {                                                                                                         \
    if (gated) scalar_gate_scan_kernel<NK, TBV, true, false><<<grid, 64, 0, stream>>>(p);                  \
    else if (silu) scalar_gate_scan_kernel<NK, TBV, false, true><<<grid, 64, 0, stream>>>(p);              \
    else scalar_gate_scan_kernel<NK, TBV, false, false><<<grid, 64, 0, stream>>>(p);                       \
  }
#define SG_CASE(NK, TBM)                                                                     \
  case NK * 16:                                                                              \
    if (single) SG_LAUNCH(NK, 1) else SG_LAUNCH(NK, TBM)                                     \
    break;
  switch (gated && silu ? -1 : dim) {   // (silu under gates: the slow kernel takes every combination)
    SG_CASE(1, 16) SG_CASE(2, 16) SG_CASE(3, 16) SG_CASE(4, 16) SG_CASE(5, 8) SG_CASE(6, 8) SG_CASE(7, 8) SG_CASE(8, 8)
    SG_CASE(12, 4) SG_CASE(16, 4)
    default: {
      const int threads = vx >= 256 ? 256 : (vx + 63) / 64 * 64;
      scalar_gate_any_kernel<<<dim3(entries, heads, (vx + threads - 1) / threads), threads, 2 * dim * sizeof(float), stream>>>(
          p, dim);
    }
  }
#undef SG_CASE
#undef SG_LAUNCH
  return dli_launch_status();
}

}  // extern "C"
