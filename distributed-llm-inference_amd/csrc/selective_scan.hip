// The selective scan: a diagonal linear recurrence per channel whose decay and input depend on the
// token. For channel c with N states, step size dt_c (already positive), input x_c, and the token's
// vectors B and C (N values each, shared by all channels):
//
//   S[c][n] <- exp(dt_c A[c][n]) S[c][n] + dt_c x_c B[n],   A = -exp(A_log)
//   y_c = sum_n S[c][n] C[n] + D_c x_c,   out_c = y_c * silu(z_c)   (z == nullptr: no gate)
//
// S is float32 [channels][N] in the request's state slot and starts from zeros where the entry's
// first row has position 0; an entry's rows are walked in order from what the step before left.
// Everything here is 32-bit; `out` has the type T of what the next product reads.
//
// Sixteen lanes (a DPP row) share a channel: lane `part` keeps the states n = part + 16 j, j < NPER, in
// registers (so the 16 lanes read B and C as one run), and a token's sum over n meets in four DPP
// swaps. A wave takes four channels, a workgroup sixteen. N up to 256. A few tokens' operands are held in
// registers while the next few are in flight.
#include "common.h"

struct SsmArgs {
  const float* x; int64_t x_stride;          // [rows][channels]: the convolution's output after its activation
  const float* dt; int64_t dt_stride;        // [rows][channels]: step sizes
  const float* bc; int64_t bc_stride;        // [rows][>=]: B at column b_off, C at column c_off, N values each
  int b_off, c_off;
  const float* z; int64_t z_stride;          // [rows][channels]: the gate's pre-activation, or nullptr
  const float* a_log;                        // [channels][N]
  const float* d;                            // [channels], or nullptr
  float* state; int64_t state_stride;
  const int* q_start; const int* positions; const int* state_slots;
  void* out; int64_t out_stride;             // [rows][channels]
  int channels, n;
};

__device__ __forceinline__ float ssm_row_sum(float x) {
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, false));
  x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, false));
  return x;
}

// SINGLE: every entry is one row (a step of single tokens): blocks of one token.
template <typename T, int NPER, bool SINGLE>
__global__ __launch_bounds__(256) void selective_scan_kernel(SsmArgs p) {
  const int entry = blockIdx.x;
  const int ch = blockIdx.y * 16 + threadIdx.x / 16, part = threadIdx.x % 16;
  const bool live = ch < p.channels;
  const int c = live ? ch : p.channels - 1;          // lanes past the last channel repeat it and store nothing
  const int row0 = p.q_start[entry], n_rows = p.q_start[entry + 1] - row0;
  if (n_rows <= 0) return;
  const int N = p.n;
  const float* __restrict__ x = p.x;
  const float* __restrict__ dt = p.dt;
  const float* __restrict__ bc = p.bc;
  const float* __restrict__ z = p.z;
  T* __restrict__ out = (T*)p.out;
  float* st = p.state + (int64_t)p.state_slots[entry] * p.state_stride + (int64_t)c * N;
  const bool fresh = p.positions[row0] == 0;
  float a[NPER], s[NPER];
  int at[NPER];
  bool valid[NPER];
#pragma unroll
  for (int j = 0; j < NPER; ++j) {
    valid[j] = part + 16 * j < N;
    at[j] = valid[j] ? part + 16 * j : N - 1;
    a[j] = valid[j] ? -expf(p.a_log[(int64_t)c * N + at[j]]) : 0.f;
    const float old = st[at[j]];
    s[j] = (fresh || !valid[j]) ? 0.f : old;
  }
  const float dc = p.d != nullptr ? p.d[c] : 0.f;
  // Tokens go in blocks of TB whose operands are asked for two blocks ahead: the chain over tokens is
  // one multiply-add a state, and nothing on it waits for memory. The decay is exp2 of a product with
  // log2(e) folded into A.
  constexpr int TB = SINGLE ? 1 : NPER <= 2 ? 8 : NPER <= 4 ? 4 : NPER <= 8 ? 2 : 1;
  constexpr float LOG2E = 1.4426950408889634f;
#pragma unroll
  for (int j = 0; j < NPER; ++j) a[j] *= LOG2E;
  struct Block { float dt[TB], x[TB], z[TB], b[TB][NPER], c[TB][NPER]; };
  auto fetch = [&](Block& k, int t0) {        // rows past the step's last repeat it
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      const int64_t row = row0 + min(t0 + i, n_rows - 1);
      k.dt[i] = dt[row * p.dt_stride + c];
      k.x[i] = x[row * p.x_stride + c];
      k.z[i] = z != nullptr ? z[row * p.z_stride + c] : 0.f;
#pragma unroll
      for (int j = 0; j < NPER; ++j) {
        k.b[i][j] = bc[row * p.bc_stride + p.b_off + at[j]];
        k.c[i][j] = bc[row * p.bc_stride + p.c_off + at[j]];
      }
    }
  };
  auto compute = [&](const Block& k, int t0) {
    // everything of a token that is not on the chain over tokens is made for all TB at once: decays,
    // inputs and the gate's factor; then the chain, then the sums over the sixteen lanes
    float decay[TB][NPER], gate[TB], y[TB];
#pragma unroll
    for (int i = 0; i < TB; ++i) {
#pragma unroll
      for (int j = 0; j < NPER; ++j) decay[i][j] = __builtin_amdgcn_exp2f(k.dt[i] * a[j]);
      const float g = k.z[i];
      gate[i] = z != nullptr ? g * __builtin_amdgcn_rcpf(1.f + __expf(-g)) : 1.f;
    }
    const int full = min(TB, n_rows - t0);       // (the same for every lane of the workgroup)
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      const float dx = k.dt[i] * k.x[i];
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < NPER; ++j) {
        // rows past the step's last change nothing
        const float next = valid[j] ? fmaf(decay[i][j], s[j], dx * k.b[i][j]) : 0.f;
        s[j] = i < full ? next : s[j];
        acc = fmaf(next, k.c[i][j], acc);
      }
      y[i] = acc;
    }
#pragma unroll
    for (int i = 0; i < TB; ++i) {
      const float v = fmaf(dc, k.x[i], ssm_row_sum(y[i])) * gate[i];
      if (part == 0 && live && i < full) out[(row0 + t0 + i) * p.out_stride + c] = from_f32<T>(v);
    }
  };
  // three blocks of registers go round: while one is computed the next two are in flight, so a block's
  // trip to memory has two blocks' arithmetic to hide behind
  Block k0, k1, k2;
  fetch(k0, 0);
  fetch(k1, TB);
  for (int t0 = 0; t0 < n_rows; t0 += 3 * TB) {
    fetch(k2, t0 + 2 * TB);
    compute(k0, t0);
    if (t0 + TB >= n_rows) break;
    fetch(k0, t0 + 3 * TB);
    compute(k1, t0 + TB);
    if (t0 + 2 * TB >= n_rows) break;
    fetch(k1, t0 + 4 * TB);
    compute(k2, t0 + 2 * TB);
  }
  if (live)
#pragma unroll
    for (int j = 0; j < NPER; ++j)
      if (valid[j]) st[at[j]] = s[j];
}

extern "C" {

int dli_selective_scan_max_states() { return 256; }

int dli_selective_scan(const float* x, int64_t x_stride, const float* dt, int64_t dt_stride, const float* bc,
                       int64_t bc_stride, int b_off, int c_off, const float* z, int64_t z_stride, const float* a_log,
                       const float* d, float* state, int64_t state_stride, const int* q_start, const int* positions,
                       const int* state_slots, void* out, int64_t out_stride, int entries, int rows, int channels, int n,
                       int out_is_bf16, hipStream_t stream) {
  if (rows <= 0 || entries <= 0) return DLI_OK;
  if (rows < entries || channels <= 0 || n <= 0 || n > 256 || x_stride < channels || dt_stride < channels ||
      out_stride < channels || (z != nullptr && z_stride < channels) || b_off < 0 || c_off < 0 ||
      b_off + n > bc_stride || c_off + n > bc_stride || state_stride < (int64_t)channels * n)
    return DLI_ERR_ARGUMENT;
  SsmArgs p;
  p.x = x; p.x_stride = x_stride; p.dt = dt; p.dt_stride = dt_stride; p.bc = bc; p.bc_stride = bc_stride;
  p.b_off = b_off; p.c_off = c_off; p.z = z; p.z_stride = z_stride; p.a_log = a_log; p.d = d; p.state = state;
  p.state_stride = state_stride; p.q_start = q_start; p.positions = positions; p.state_slots = state_slots;
  p.out = out; p.out_stride = out_stride; p.channels = channels; p.n = n;
  const dim3 grid(entries, (channels + 15) / 16);
  if (grid.y > 65535) return DLI_ERR_ARGUMENT;
  const int per = (n + 15) / 16;
#define SSM_LAUNCH(NPER)                                                                \
  {                                                                                     \
    if (rows == entries) {                                                              \
      if (out_is_bf16) selective_scan_kernel<bf16_t, NPER, true><<<grid, 256, 0, stream>>>(p);   \
      else selective_scan_kernel<float, NPER, true><<<grid, 256, 0, stream>>>(p);       \
    } else if (out_is_bf16) selective_scan_kernel<bf16_t, NPER, false><<<grid, 256, 0, stream>>>(p); \
    else selective_scan_kernel<float, NPER, false><<<grid, 256, 0, stream>>>(p);        \
  }
  if (per <= 1) SSM_LAUNCH(1) else if (per <= 2) SSM_LAUNCH(2) else if (per <= 4) SSM_LAUNCH(4)
  else if (per <= 8) SSM_LAUNCH(8) else SSM_LAUNCH(16)
#undef SSM_LAUNCH
  return dli_launch_status();
}

}  // extern "C"
