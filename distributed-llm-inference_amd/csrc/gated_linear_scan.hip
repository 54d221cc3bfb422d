// A linear recurrence with a matrix state per head whose forget gate also decides what is written:
// with f in (0, 1) per key channel, a query q (D values a head) and a value v (V values a head),
//
//   S <- diag(f) S + (1 - f) v^T,   o = S^T q      (o is made from the state that already holds the token)
//
// S is float32 [heads][V][D] in the request's state slot and starts from zeros where the entry's first
// row has position 0; an entry's rows are walked in order from what the step before left. Everything is
// 32-bit.
//
//   bounded_gates       from a step's 32-bit projections: q = silu(q_pre) and
//                       f = lower + (1 - lower) sigmoid(f_pre + bias), in place
//   gated_linear_scan   the recurrence
//
// One wave takes one (entry, head, slice of 4 value columns). Sixteen lanes (a DPP row) share a column:
// lane (col, part) keeps S[part's D/16 keys][col] in registers, and a token's sum over the keys meets in
// four DPP swaps. The vectors of TB tokens are staged in LDS while the next TB are in flight. Heads
// whose D is no multiple of 16 (or above 256) take a thread-per-column kernel with the state in memory.
#include "common.h"

// proj [rows][stride]: q_pre at column q_off, f_pre at column f_off, `width` values each. A thread an element.
__global__ void bounded_gates_kernel(float* __restrict__ proj, int64_t stride, int q_off, int f_off,
                                     const float* __restrict__ f_bias, const float* __restrict__ lower, int width) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= width) return;
  float* pr = proj + row * stride;
  const float q = pr[q_off + i];
  pr[q_off + i] = q / (1.f + expf(-q));
  const float l = lower != nullptr ? lower[i] : 0.f;
  const float g = 1.f / (1.f + expf(-(pr[f_off + i] + (f_bias != nullptr ? f_bias[i] : 0.f))));
  pr[f_off + i] = l + (1.f - l) * g;
}

struct GlArgs {
  const float* proj; int64_t stride;   // [rows][stride]: q, f (heads x D each) and v (heads x V) at their columns
  int q_off, f_off, v_off;
  float* state; int64_t state_stride;
  const int* q_start; const int* positions; const int* state_slots;
  float* o; int64_t o_stride;          // [rows][heads * V]
  int heads, vdim;
};

__device__ __forceinline__ float gl_row_sum(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, false));
  return x;
}

// NK keys a lane, D = 16 NK; TB tokens staged at once (1 in a step of single tokens).
template <int NK, int TB>
__global__ __launch_bounds__(64) void gated_linear_scan_kernel(GlArgs p) {
  constexpr int D = NK * 16, COLS = 4, PER = (TB * D + 63) / 64;
  __shared__ float sf[PER * 64], sq[PER * 64], sv[TB * COLS];
  const int lane = threadIdx.x, vloc = lane / 16, part = lane % 16;
  const int entry = blockIdx.x, head = blockIdx.y;
  const int V = p.vdim;
  const int col = min((int)blockIdx.z * COLS + vloc, V - 1);   // lanes past the last column repeat it and store nothing
  const bool live = (int)blockIdx.z * COLS + vloc < V;
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int64_t q_col = p.q_off + (int64_t)head * D, f_col = p.f_off + (int64_t)head * D, v_col = p.v_off + (int64_t)head * V;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + ((int64_t)head * V + col) * D + part * NK;
  float s[NK];
  const bool fresh = p.positions[row0] == 0;
#pragma unroll
  for (int i = 0; i < NK; ++i) {
    const float old = st[i];
    s[i] = fresh ? 0.f : old;
  }
  float pf[PER], pq[PER], pv = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int m = 0; m < PER; ++m) {
      const int e = min(lane + 64 * m, TB * D - 1), t = e / D, c = e - t * D;
      const int64_t row = row0 + min(t0 + t, n_rows - 1);
      pf[m] = p.proj[row * p.stride + f_col + c];
      pq[m] = p.proj[row * p.stride + q_col + c];
    }
    if (lane < TB * COLS) {
      const int64_t row = row0 + min(t0 + lane / COLS, n_rows - 1);
      pv = p.proj[row * p.stride + v_col + min((int)blockIdx.z * COLS + lane % COLS, V - 1)];
    }
  };
  auto step = [&](int t, int64_t row) {
    const float* ft = sf + t * D + part * NK;
    const float* qt = sq + t * D + part * NK;
    const float v = sv[t * COLS + vloc];
    float o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      const float f = ft[i];
      s[i] = fmaf(f, s[i], (1.f - f) * v);
      if (i & 1) o1 = fmaf(qt[i], s[i], o1); else o0 = fmaf(qt[i], s[i], o0);
    }
    const float o = gl_row_sum(o0 + o1);
    if (part == 0 && live) p.o[row * p.o_stride + (int64_t)head * V + col] = o;
  };
  fetch(0);
  for (int t0 = 0; t0 < n_rows; t0 += TB) {
#pragma unroll
    for (int m = 0; m < PER; ++m) {
      sf[lane + 64 * m] = pf[m];
      sq[lane + 64 * m] = pq[m];
    }
    if (lane < TB * COLS) sv[lane] = pv;
    if (TB > 1 && t0 + TB < n_rows) fetch(t0 + TB);  // on their way while the chain below runs
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

// Any D and V: a thread a value column, the column's state in the request's slot.
__global__ void gated_linear_any_kernel(GlArgs p, int D) {
  extern __shared__ float sh[];
  float *sf = sh, *sq = sh + D;
  const int v = blockIdx.z * blockDim.x + threadIdx.x, V = p.vdim;
  const bool live = v < V;
  const int entry = blockIdx.x, head = blockIdx.y;
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int64_t q_col = p.q_off + (int64_t)head * D, f_col = p.f_off + (int64_t)head * D, v_col = p.v_off + (int64_t)head * V;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + ((int64_t)head * V + (live ? v : 0)) * D;
  if (live && p.positions[row0] == 0)
    for (int c = 0; c < D; ++c) st[c] = 0.f;
  for (int t = 0; t < n_rows; ++t) {
    const int64_t row = row0 + t;
    __syncthreads();
    for (int c = threadIdx.x; c < D; c += blockDim.x) {
      sf[c] = p.proj[row * p.stride + f_col + c];
      sq[c] = p.proj[row * p.stride + q_col + c];
    }
    __syncthreads();
    if (!live) continue;
    const float vv = p.proj[row * p.stride + v_col + v];
    float o = 0.f;
    for (int c = 0; c < D; ++c) {
      const float s = fmaf(sf[c], st[c], (1.f - sf[c]) * vv);
      st[c] = s;
      o = fmaf(sq[c], s, o);
    }
    p.o[row * p.o_stride + (int64_t)head * V + v] = o;
  }
}

extern "C" {

int dli_bounded_gates(float* proj, int64_t stride, int q_off, int f_off, const float* f_bias, const float* lower, int rows,
                      int width, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0 || q_off < 0 || f_off < 0 || q_off + width > stride || f_off + width > stride ||
      (q_off < f_off + width && f_off < q_off + width))
    return DLI_ERR_ARGUMENT;
  const dim3 grid(rows, (width + 255) / 256);
  if (grid.y > 65535) return DLI_ERR_ARGUMENT;
  bounded_gates_kernel<<<grid, 256, 0, stream>>>(proj, stride, q_off, f_off, f_bias, lower, width);
  return dli_launch_status();
}

int dli_gated_linear_scan(const float* proj, int64_t stride, int q_off, int f_off, int v_off, float* state,
                          int64_t state_stride, const int* q_start, const int* positions, const int* state_slots, float* o,
                          int64_t o_stride, int entries, int rows, int heads, int dim, int vdim, hipStream_t stream) {
  if (rows <= 0 || entries <= 0) return DLI_OK;
  if (rows < entries || heads <= 0 || heads > 65535 || dim <= 0 || dim > 4096 || vdim <= 0 ||
      state_stride < (int64_t)heads * vdim * dim || o_stride < (int64_t)heads * vdim || q_off < 0 || f_off < 0 ||
      v_off < 0 || q_off + (int64_t)heads * dim > stride || f_off + (int64_t)heads * dim > stride ||
      v_off + (int64_t)heads * vdim > stride)
    return DLI_ERR_ARGUMENT;
  GlArgs p;
  p.proj = proj; p.stride = stride; p.q_off = q_off; p.f_off = f_off; p.v_off = v_off; p.state = state;
  p.state_stride = state_stride; p.q_start = q_start; p.positions = positions; p.state_slots = state_slots; p.o = o;
  p.o_stride = o_stride; p.heads = heads; p.vdim = vdim;
  const bool single = rows == entries;
  const dim3 grid(entries, heads, (vdim + 3) / 4);
  if (grid.z > 65535) return DLI_ERR_ARGUMENT;
#define GL_CASE(NK, TBM)                                                                      \
  case NK * 16:                                                                               \
    if (single) gated_linear_scan_kernel<NK, 1><<<grid, 64, 0, stream>>>(p);                  \
    else gated_linear_scan_kernel<NK, TBM><<<grid, 64, 0, stream>>>(p);                       \
    break;
  switch (dim) {
    GL_CASE(1, 16) GL_CASE(2, 16) GL_CASE(3, 16) GL_CASE(4, 16) GL_CASE(5, 8) GL_CASE(6, 8) GL_CASE(7, 8) GL_CASE(8, 8)
    GL_CASE(12, 4) GL_CASE(16, 4)
    default: {
      const int threads = vdim >= 256 ? 256 : (vdim + 63) / 64 * 64;
      gated_linear_any_kernel<<<dim3(entries, heads, (vdim + threads - 1) / threads), threads, 2 * dim * sizeof(float),
                                stream>>>(p, dim);
    }
  }
#undef GL_CASE
  return dli_launch_status();
}

}  // extern "C"
