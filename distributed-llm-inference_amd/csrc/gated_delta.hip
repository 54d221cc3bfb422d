// The gated delta rule: a matrix state S [key][value] per head in 32-bit, carried from token to token
// of a request in its state slot, with one decay g and one write strength beta per head and token:
//
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q      (in this order: o is made from the state that already holds the token)
//
// Keys and values may differ in size (D keys, V values a head), and several value heads may share
// the q and k of one of `kv_heads` heads. Around it, in the same 32-bit arithmetic:
//
//   conv_prepare       from the 32-bit projections of a step's rows: a short causal convolution over
//                      time per channel of q, k and v (the last taps-1 inputs of the step before come
//                      from the request's state; zeros before position 0), silu, q and k made unit
//                      vectors per head (q also times D^-1/2), beta = sigmoid(b),
//                      g = exp(-exp(A_log) softplus(a + dt_bias))
//   conv_keep          the step's last taps-1 inputs into the request's state
//   causal_conv        the short causal convolution alone, for any mixer: per channel, with an optional bias and
//                      silu, from the same kind of kept inputs; the result in 32-bit and, if wanted, once more
//                      in the type of the product that reads it next
//   gated_delta_scan   the recurrence; o in 32-bit
//
// With old state S, ks = S^T k and qs = S^T q (both from the old S, so their sums run side by side):
// u = beta (v - g ks), S_new = g S + k u^T, o = g qs + u (k . q).
//
// One wave takes one (entry, head, slice of 4 value columns) and walks the entry's tokens in order.
// Sixteen lanes (a DPP row) share a column: lane (col, part) keeps S[part's D/16 keys][col] in
// registers, and the two dot products of a token meet in four DPP swaps each. The vectors of 16
// tokens are staged in LDS while the next 16 are in flight, so the chain reads LDS and registers
// only. Heads whose D is no multiple of 16 (or above 256) take a thread-per-column kernel that keeps
// the state in memory: slow, there so that no size is refused.
//
// State slot: [heads][V][D] floats, then [taps-1][channels] floats of kept inputs (the last row is
// the newest). A request whose first row of the step has position 0 starts from zeros; nothing
// needs clearing when a slot changes hands.
#include "common.h"

// The entry that holds `row`: the last e with q_start[e] <= row.
__device__ __forceinline__ int gd_entry_of_row(const int* __restrict__ q_start, int entries, int row) {
  int lo = 0, hi = entries - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= row) lo = mid; else hi = mid - 1;
  }
  return lo;
}

struct PrepArgs {
  const float* proj; int64_t stride;       // [rows][stride]: q | k | v channels from column 0, then what follows
  int b_off, a_off;                        // columns of beta's and the decay's pre-activations (heads each)
  const float* conv_w;                     // [channels][taps], the last column the current token's
  const float* a_log; const float* dt_bias;  // [heads]
  const float* kept; int64_t state_stride; // the requests' kept inputs: state + offset, [taps-1][channels] a slot
  const int* q_start; const int* positions; const int* state_slots;
  float* out; int64_t out_stride;          // [rows][channels + 2 heads]: q | k | v | beta | g
  int entries, heads, kv_heads, dim, vdim, taps;
};

// One input of the convolution of channel c, `back` places before `row` (which lies at position pos of
// its request, whose step starts at row `first`): from the step's rows, from the kept inputs, or zero.
__device__ __forceinline__ float conv_input(const PrepArgs& p, const float* kept, int channels, int row, int first, int pos,
                                            int back, int c) {
  if (pos - back < 0) return 0.f;                               // before the sequence
  const int src = row - back;
  return src >= first ? p.proj[(int64_t)src * p.stride + c] : kept[(int64_t)(p.taps - 1 - (first - src)) * channels + c];
}

__device__ __forceinline__ float conv_silu(const PrepArgs& p, const float* kept, int channels, int row, int first, int pos, int c) {
  float acc = 0.f;
  for (int j = p.taps - 1; j >= 0; --j)                         // oldest input first
    acc = fmaf(p.conv_w[(int64_t)c * p.taps + (p.taps - 1 - j)], conv_input(p, kept, channels, row, first, pos, j, c), acc);
  return acc / (1.f + expf(-acc));
}

// A wave a (row, unit). Units: the 2 kv_heads heads of q and k (convolution, silu, unit length), then the
// channels of v in runs of 64 (convolution, silu), then one for beta and g of all heads.
__global__ __launch_bounds__(64) void conv_prepare_kernel(PrepArgs p) {
  const int row = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  const int qk = p.kv_heads * p.dim, hv = p.heads * p.vdim, channels = 2 * qk + hv;
  const int v_units = (hv + 63) / 64;
  float* out = p.out + (int64_t)row * p.out_stride;
  if (unit == 2 * p.kv_heads + v_units) {
    for (int h = lane; h < p.heads; h += DLI_WAVE) {
      const float b = p.proj[(int64_t)row * p.stride + p.b_off + h];
      const float a = p.proj[(int64_t)row * p.stride + p.a_off + h] + p.dt_bias[h];
      const float softplus = a > 20.f ? a : log1pf(expf(a));
      out[channels + h] = 1.f / (1.f + expf(-b));
      out[channels + p.heads + h] = expf(-expf(p.a_log[h]) * softplus);
    }
    return;
  }
  const int e = gd_entry_of_row(p.q_start, p.entries, row);
  const int first = p.q_start[e], pos = p.positions[row];
  const float* kept = p.kept + (int64_t)p.state_slots[e] * p.state_stride;
  if (unit >= 2 * p.kv_heads) {
    const int c = 2 * qk + (unit - 2 * p.kv_heads) * 64 + lane;
    if (c < channels) out[c] = conv_silu(p, kept, channels, row, first, pos, c);
    return;
  }
  const int c0 = unit * p.dim;                                  // q heads, then k heads
  float ss = 0.f;
  for (int c = lane; c < p.dim; c += DLI_WAVE) {
    const float y = conv_silu(p, kept, channels, row, first, pos, c0 + c);
    out[c0 + c] = y;
    ss += y * y;
  }
  const float r = (1.f / sqrtf(wave_sum(ss) + 1e-6f)) * (unit < p.kv_heads ? 1.f / sqrtf((float)p.dim) : 1.f);
  for (int c = lane; c < p.dim; c += DLI_WAVE) out[c0 + c] *= r;   // (each lane scales what it wrote itself)
}

// A thread a channel: it reads what it needs of the old kept inputs before it writes the new ones,
// and no other thread touches its channel. (Runs after conv_prepare of the same step.)
#define GD_MAX_TAPS 16
__global__ void conv_keep_kernel(const float* __restrict__ proj, int64_t stride, float* kept_base, int64_t state_stride,
                                 const int* __restrict__ q_start, const int* __restrict__ positions,
                                 const int* __restrict__ state_slots, int channels, int taps) {
  const int e = blockIdx.x;
  const int first = q_start[e], end = q_start[e + 1];
  if (end <= first) return;
  const int pos0 = positions[first];
  float* kept = kept_base + (int64_t)state_slots[e] * state_stride;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  float fresh[GD_MAX_TAPS];
  for (int i = 0; i < taps - 1; ++i) {            // new kept row i holds the input `taps-1-i` places before `end`
    const int src = end - (taps - 1 - i);
    float x;
    if (src >= first) x = proj[(int64_t)src * stride + c];
    else if (pos0 - (first - src) < 0) x = 0.f;
    else x = kept[(int64_t)(taps - 1 - (first - src)) * channels + c];
    fresh[i] = x;
  }
  for (int i = 0; i < taps - 1; ++i) kept[(int64_t)i * channels + c] = fresh[i];
}

// A thread a (row, channel). x [rows][stride] holds the inputs of `channels` channels from column 0.
template <typename T>
__global__ void causal_conv_kernel(const float* __restrict__ x, int64_t stride, const float* __restrict__ conv_w,
                                   const float* __restrict__ bias, const float* kept_base, int64_t state_stride,
                                   const int* __restrict__ q_start, int entries, const int* __restrict__ positions,
                                   const int* __restrict__ state_slots, float* __restrict__ out, int64_t out_stride,
                                   T* __restrict__ rounded, int64_t rounded_stride, int channels, int taps, int act) {
  const int row = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int e = gd_entry_of_row(q_start, entries, row);
  const int first = q_start[e], pos = positions[row];
  const float* kept = kept_base + (int64_t)state_slots[e] * state_stride;
  float acc = bias != nullptr ? bias[c] : 0.f;
  for (int j = taps - 1; j >= 0; --j) {                          // oldest input first
    float in = 0.f;
    if (pos - j >= 0) {
      const int src = row - j;
      in = src >= first ? x[(int64_t)src * stride + c] : kept[(int64_t)(taps - 1 - (first - src)) * channels + c];
    }
    acc = fmaf(conv_w[(int64_t)c * taps + (taps - 1 - j)], in, acc);
  }
  if (act == 1) acc = acc / (1.f + expf(-acc));
  out[(int64_t)row * out_stride + c] = acc;
  if (rounded != nullptr) rounded[(int64_t)row * rounded_stride + c] = from_f32<T>(acc);
}

struct GdArgs {
  const float* prep; int64_t stride;   // [rows][stride]: q | k | v | beta | g as conv_prepare leaves them
  float* state; int64_t state_stride;
  const int* q_start; const int* positions; const int* state_slots;
  float* o; int64_t o_stride;          // [rows][heads * V]
  int heads, kv_heads, vdim;
};

__device__ __forceinline__ float gd_row_sum(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, false));
  return x;
}

// NK keys a lane, D = 16 NK; TB tokens staged at once (1 in a step of single tokens).
template <int NK, int TB>
__global__ __launch_bounds__(64) void gated_delta_scan_kernel(GdArgs p) {
  constexpr int D = NK * 16, COLS = 4, PER = (TB * D + 63) / 64;
  __shared__ float sk[PER * 64], sq[PER * 64], sv[TB * COLS], sbg[TB * 2], skq[TB];
  const int lane = threadIdx.x, vloc = lane / 16, part = lane % 16;
  const int entry = blockIdx.x, head = blockIdx.y;
  const int V = p.vdim;
  const int col = min((int)blockIdx.z * COLS + vloc, V - 1);   // lanes past the last column repeat it and store nothing
  const bool live = (int)blockIdx.z * COLS + vloc < V;
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int kvh = head / (p.heads / p.kv_heads);
  const int qk = p.kv_heads * D;
  const int64_t q_col = (int64_t)kvh * D, k_col = qk + (int64_t)kvh * D, v_col = 2 * (int64_t)qk + (int64_t)head * V;
  const int64_t b_col = 2 * (int64_t)qk + (int64_t)p.heads * V + head, g_col = b_col + p.heads;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + ((int64_t)head * V + col) * D + part * NK;
  float s[NK];
  const bool fresh = p.positions[row0] == 0;
#pragma unroll
  for (int i = 0; i < NK; ++i) s[i] = fresh ? 0.f : st[i];

  float pk[PER], pq[PER], pv = 0.f, pbg = 0.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int m = 0; m < PER; ++m) {
      const int e = min(lane + 64 * m, TB * D - 1), t = e / D, c = e - t * D;
      const int64_t row = row0 + min(t0 + t, n_rows - 1);
      pk[m] = p.prep[row * p.stride + k_col + c];
      pq[m] = p.prep[row * p.stride + q_col + c];
    }
    if (lane < TB * COLS) {
      const int64_t row = row0 + min(t0 + lane / COLS, n_rows - 1);
      pv = p.prep[row * p.stride + v_col + min((int)blockIdx.z * COLS + lane % COLS, V - 1)];
    }
    if (lane < TB * 2) {
      const int64_t row = row0 + min(t0 + lane / 2, n_rows - 1);
      pbg = p.prep[row * p.stride + ((lane & 1) ? g_col : b_col)];
    }
  };
  auto step = [&](int t, int64_t row) {
    const float* kt = sk + t * D + part * NK;
    const float* qt = sq + t * D + part * NK;
    const float v = sv[t * COLS + vloc], beta = sbg[2 * t], g = sbg[2 * t + 1], kq = skq[t];
    float ks0 = 0.f, ks1 = 0.f, qs0 = 0.f, qs1 = 0.f;
#pragma unroll
    for (int i = 0; i < NK; ++i) {
      if (i & 1) { ks1 = fmaf(kt[i], s[i], ks1); qs1 = fmaf(qt[i], s[i], qs1); }
      else { ks0 = fmaf(kt[i], s[i], ks0); qs0 = fmaf(qt[i], s[i], qs0); }
    }
    const float ks = gd_row_sum(ks0 + ks1), qs = gd_row_sum(qs0 + qs1);
    const float u = beta * (v - g * ks);
#pragma unroll
    for (int i = 0; i < NK; ++i) s[i] = fmaf(kt[i], u, g * s[i]);
    if (part == 0 && live) p.o[row * p.o_stride + (int64_t)head * V + col] = fmaf(u, kq, g * qs);
  };
  fetch(0);
  for (int t0 = 0; t0 < n_rows; t0 += TB) {
#pragma unroll
    for (int m = 0; m < PER; ++m) {
      sk[lane + 64 * m] = pk[m];
      sq[lane + 64 * m] = pq[m];
    }
    if (lane < TB * COLS) sv[lane] = pv;
    if (lane < TB * 2) sbg[lane] = pbg;
    if (TB > 1 && t0 + TB < n_rows) fetch(t0 + TB);  // on their way while the chain below runs
    __syncthreads();
    // each token's k . q: four lanes a token add up a quarter of the keys each
    for (int t = lane >> 2; t < TB; t += 16) {
      float kq = 0.f;
      for (int c = (lane & 3) * (D / 4); c < ((lane & 3) + 1) * (D / 4); ++c) kq = fmaf(sk[t * D + c], sq[t * D + c], kq);
      kq += __shfl_xor(kq, 1, DLI_WAVE);
      kq += __shfl_xor(kq, 2, DLI_WAVE);
      if ((lane & 3) == 0) skq[t] = kq;
    }
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
__global__ void gated_delta_any_kernel(GdArgs p, int D) {
  extern __shared__ float sh[];
  float *sk = sh, *sq = sh + D;
  const int v = blockIdx.z * blockDim.x + threadIdx.x, V = p.vdim;
  const bool live = v < V;
  const int entry = blockIdx.x, head = blockIdx.y;
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int kvh = head / (p.heads / p.kv_heads);
  const int qk = p.kv_heads * D;
  const int64_t q_col = (int64_t)kvh * D, k_col = qk + (int64_t)kvh * D, v_col = 2 * (int64_t)qk + (int64_t)head * V;
  const int64_t b_col = 2 * (int64_t)qk + (int64_t)p.heads * V + head, g_col = b_col + p.heads;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + ((int64_t)head * V + (live ? v : 0)) * D;
  if (live && p.positions[row0] == 0)
    for (int c = 0; c < D; ++c) st[c] = 0.f;
  for (int t = 0; t < n_rows; ++t) {
    const int64_t row = row0 + t;
    __syncthreads();
    for (int c = threadIdx.x; c < D; c += blockDim.x) {
      sk[c] = p.prep[row * p.stride + k_col + c];
      sq[c] = p.prep[row * p.stride + q_col + c];
    }
    __syncthreads();
    if (!live) continue;
    const float beta = p.prep[row * p.stride + b_col], g = p.prep[row * p.stride + g_col];
    const float vv = p.prep[row * p.stride + v_col + v];
    float ks = 0.f, qs = 0.f, kq = 0.f;
    for (int c = 0; c < D; ++c) {
      ks = fmaf(sk[c], st[c], ks);
      qs = fmaf(sq[c], st[c], qs);
      kq = fmaf(sk[c], sq[c], kq);
    }
    const float u = beta * (vv - g * ks);
    for (int c = 0; c < D; ++c) st[c] = fmaf(sk[c], u, g * st[c]);
    p.o[row * p.o_stride + (int64_t)head * V + v] = fmaf(u, kq, g * qs);
  }
}

extern "C" {

int dli_gated_delta_max_taps() { return GD_MAX_TAPS; }

int dli_conv_prepare(const float* proj, int64_t stride, int b_off, int a_off, const float* conv_w, const float* a_log,
                     const float* dt_bias, float* state, int64_t state_stride, int64_t kept_offset, const int* q_start,
                     const int* positions, const int* state_slots, float* out, int64_t out_stride, int entries, int rows,
                     int heads, int kv_heads, int dim, int vdim, int taps, hipStream_t stream) {
  if (rows <= 0 || entries <= 0) return DLI_OK;
  const int64_t channels = 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || vdim <= 0 || taps < 1 || taps > GD_MAX_TAPS ||
      stride < channels || out_stride < channels + 2 * heads || b_off < channels || a_off < channels ||
      b_off + heads > stride || a_off + heads > stride || state_stride < kept_offset + (taps - 1) * channels)
    return DLI_ERR_ARGUMENT;
  PrepArgs p;
  p.proj = proj; p.stride = stride; p.b_off = b_off; p.a_off = a_off; p.conv_w = conv_w; p.a_log = a_log;
  p.dt_bias = dt_bias; p.kept = state + kept_offset; p.state_stride = state_stride; p.q_start = q_start;
  p.positions = positions; p.state_slots = state_slots; p.out = out; p.out_stride = out_stride; p.entries = entries;
  p.heads = heads; p.kv_heads = kv_heads; p.dim = dim; p.vdim = vdim; p.taps = taps;
  const int units = 2 * kv_heads + (int)(((int64_t)heads * vdim + 63) / 64) + 1;
  if (units > 65535) return DLI_ERR_ARGUMENT;
  conv_prepare_kernel<<<dim3(rows, units), 64, 0, stream>>>(p);
  if (dli_launch_status() != DLI_OK) return DLI_ERR_LAUNCH;
  if (taps > 1) {
    const dim3 grid(entries, (unsigned)((channels + 255) / 256));
    conv_keep_kernel<<<grid, 256, 0, stream>>>(proj, stride, state + kept_offset, state_stride, q_start, positions,
                                               state_slots, (int)channels, taps);
  }
  return dli_launch_status();
}

// act: 0 none, 1 silu. rounded (may be nullptr): the result once more, bf16 if rounded_is_bf16 else float.
int dli_causal_conv(const float* x, int64_t stride, const float* conv_w, const float* bias, float* state,
                    int64_t state_stride, int64_t kept_offset, const int* q_start, const int* positions,
                    const int* state_slots, float* out, int64_t out_stride, void* rounded, int64_t rounded_stride,
                    int rounded_is_bf16, int entries, int rows, int channels, int taps, int act, hipStream_t stream) {
  if (rows <= 0 || entries <= 0) return DLI_OK;
  if (channels <= 0 || taps < 1 || taps > GD_MAX_TAPS || stride < channels || out_stride < channels ||
      (rounded != nullptr && rounded_stride < channels) || act < 0 || act > 1 ||
      state_stride < kept_offset + (int64_t)(taps - 1) * channels)
    return DLI_ERR_ARGUMENT;
  const dim3 grid(rows, (channels + 255) / 256);
  if (grid.y > 65535) return DLI_ERR_ARGUMENT;
  if (rounded_is_bf16)
    causal_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, stride, conv_w, bias, state + kept_offset, state_stride, q_start,
                                                         entries, positions, state_slots, out, out_stride, (bf16_t*)rounded,
                                                         rounded_stride, channels, taps, act);
  else
    causal_conv_kernel<float><<<grid, 256, 0, stream>>>(x, stride, conv_w, bias, state + kept_offset, state_stride, q_start,
                                                        entries, positions, state_slots, out, out_stride, (float*)rounded,
                                                        rounded_stride, channels, taps, act);
  if (dli_launch_status() != DLI_OK) return DLI_ERR_LAUNCH;
  if (taps > 1) {
    const dim3 keep(entries, (channels + 255) / 256);
    conv_keep_kernel<<<keep, 256, 0, stream>>>(x, stride, state + kept_offset, state_stride, q_start, positions,
                                               state_slots, channels, taps);
  }
  return dli_launch_status();
}

int dli_gated_delta_scan(const float* prep, int64_t stride, float* state, int64_t state_stride, const int* q_start,
                         const int* positions, const int* state_slots, float* o, int64_t o_stride, int entries, int rows,
                         int heads, int kv_heads, int dim, int vdim, hipStream_t stream) {
  if (rows <= 0 || entries <= 0) return DLI_OK;
  if (rows < entries || heads <= 0 || heads > 65535 || kv_heads <= 0 || heads % kv_heads || dim <= 0 || dim > 4096 ||
      vdim <= 0 || state_stride < (int64_t)heads * vdim * dim || o_stride < (int64_t)heads * vdim ||
      stride < 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim + 2 * heads)
    return DLI_ERR_ARGUMENT;
  GdArgs p;
  p.prep = prep; p.stride = stride; p.state = state; p.state_stride = state_stride; p.q_start = q_start;
  p.positions = positions; p.state_slots = state_slots; p.o = o; p.o_stride = o_stride; p.heads = heads;
  p.kv_heads = kv_heads; p.vdim = vdim;
  const bool single = rows == entries;
  const dim3 grid(entries, heads, (vdim + 3) / 4);
#define GD_CASE(NK, TBM)                                                                     \
  case NK * 16:                                                                              \
    if (single) gated_delta_scan_kernel<NK, 1><<<grid, 64, 0, stream>>>(p);                  \
    else gated_delta_scan_kernel<NK, TBM><<<grid, 64, 0, stream>>>(p);                       \
    break;
  switch (dim) {
    GD_CASE(1, 16) GD_CASE(2, 16) GD_CASE(3, 16) GD_CASE(4, 16) GD_CASE(5, 8) GD_CASE(6, 8) GD_CASE(7, 8) GD_CASE(8, 8)
    GD_CASE(12, 4) GD_CASE(16, 4)
    default: {
      const int threads = vdim >= 256 ? 256 : (vdim + 63) / 64 * 64;
      gated_delta_any_kernel<<<dim3(entries, heads, (vdim + threads - 1) / threads), threads, 2 * dim * sizeof(float),
                               stream>>>(p, dim);
    }
  }
#undef GD_CASE
  return dli_launch_status();
}

}  // extern "C"
