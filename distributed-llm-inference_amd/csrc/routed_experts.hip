// Feed-forward layers beyond the gated product: a polynomial activation with norms, and a mixture of
// small experts with a router. T is the type of what the matrix products read and write (float on the
// 32-bit path, bf16 when serving); statistics, the router and every sum are 32-bit.
//
//   poly_norm        out(T) = a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N(x) = x / sqrt(mean(x^2) + eps)
//                    over the row; z is the 32-bit result of the product before it
//   clamped_glu      y = g sigmoid(alpha g) (u + shift), g = min(gate, limit), u = clamp(up, -limit, limit); an infinite
//                    limit, alpha 1 and shift 0 give the plain silu(gate) * up
//   router_choose    softmax over all router outputs; choice = score + correction; only the `keep` groups of
//                    neighbours with the largest best choice stay; the `top` largest choices; weights = the chosen
//                    scores (without correction) / (their sum + 1e-20) * scale
//   expert_sort      the (token, choice) slots of real experts in runs by expert, and the list of row tiles
//   expert_up/down   the experts' products over those tiles (on the matrix cores for bfloat16 and sizes that are
//                    multiples of 32, else on the vector units, any size), the clamped activation between
//                    them; the down product leaves each slot's 32-bit result in the slot's own row
//   expert_combine   out = sum_j w_j (expert j's result, or the input itself for an identity expert)
//                    + sigmoid(shared gate) * shared expert's result
//
// A row's result never depends on its place in a tile or on the other rows: every output sums its k in
// ascending order.
#include "common.h"

__global__ void poly_norm_kernel_f32in(const float* __restrict__ z, int64_t z_stride, const float* __restrict__ coef,
                                       void* __restrict__ out_, int64_t out_stride, int ff, float eps, int out_is_bf16) {
  __shared__ float scratch[3][16];
  const int64_t row = blockIdx.x;
  const float* zr = z + row * z_stride;
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE, waves = blockDim.x / DLI_WAVE;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < ff; i += blockDim.x) {
    const float x = zr[i], x2 = x * x, x3 = x2 * x;
    s2 += x2;
    s4 += x2 * x2;
    s6 += x3 * x3;
  }
  // the three sums meet in one exchange through LDS
  s2 = wave_sum(s2); s4 = wave_sum(s4); s6 = wave_sum(s6);
  if (lane == 0) { scratch[0][wave] = s2; scratch[1][wave] = s4; scratch[2][wave] = s6; }
  __syncthreads();
  float t2 = 0.f, t4 = 0.f, t6 = 0.f;
  for (int w = 0; w < waves; ++w) { t2 += scratch[0][w]; t4 += scratch[1][w]; t6 += scratch[2][w]; }   // same order in every thread
  const float r1 = 1.f / sqrtf(t2 / (float)ff + eps), r2 = 1.f / sqrtf(t4 / (float)ff + eps), r3 = 1.f / sqrtf(t6 / (float)ff + eps);
  const float a = coef[0], b = coef[1], c = coef[2], e = coef[3];
  for (int i = threadIdx.x; i < ff; i += blockDim.x) {
    const float x = zr[i], x2 = x * x;
    const float y = a * (x * r1) + b * (x2 * r2) + c * ((x2 * x) * r3) + e;
    if (out_is_bf16) ((bf16_t*)out_)[row * out_stride + i] = (bf16_t)y;
    else ((float*)out_)[row * out_stride + i] = y;
  }
}

__device__ __forceinline__ float clamped_glu(float gate, float up, float limit, float alpha, float up_shift) {
  const float g = fminf(gate, limit), u = fminf(fmaxf(up, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + up_shift);
}

template <typename T>
__global__ void clamped_glu_kernel(const T* __restrict__ gate_up, int64_t stride, T* __restrict__ out, int ff, float limit,
                                   float alpha, float up_shift) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i < ff)
    out[row * ff + i] = from_f32<T>(clamped_glu(to_f32(gate_up[row * stride + i]), to_f32(gate_up[row * stride + ff + i]), limit, alpha, up_shift));
}

// The better of two (value, index) pairs: the larger value, the lower index on a tie.
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
  for (int m = DLI_WAVE / 2; m > 0; m >>= 1) {
    const float v2 = __shfl_xor(v, m, DLI_WAVE);
    const int i2 = __shfl_xor(i, m, DLI_WAVE);
    if (v2 > v || (v2 == v && i2 < i)) { v = v2; i = i2; }
  }
}

// A wave a token. logits [rows][stride]: the first `total` columns are the router's outputs.
__global__ __launch_bounds__(64) void router_choose_kernel(const float* __restrict__ logits, int64_t stride,
                                                           const float* __restrict__ bias,
                                                           const float* __restrict__ correction, int total, int count,
                                                           int keep, int top, float scale, int* __restrict__ ids,
                                                           float* __restrict__ weights) {
  extern __shared__ float sh[];
  float *s = sh, *choice = sh + total, *gbest = sh + 2 * total;
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x;
  const float* z = logits + row * stride;
  float m = -INFINITY;
  for (int i = lane; i < total; i += DLI_WAVE) m = fmaxf(m, z[i] + (bias != nullptr ? bias[i] : 0.f));
  m = wave_max(m);
  float sum = 0.f;
  for (int i = lane; i < total; i += DLI_WAVE) {
    const float e = expf(z[i] + (bias != nullptr ? bias[i] : 0.f) - m);
    s[i] = e;
    sum += e;
  }
  sum = wave_sum(sum);
  for (int i = lane; i < total; i += DLI_WAVE) {
    const float p = s[i] / sum;
    s[i] = p;
    choice[i] = p + (correction != nullptr ? correction[i] : 0.f);
  }
  __syncthreads();
  if (count > 1) {
    const int per = total / count;
    for (int g = lane; g < count; g += DLI_WAVE) {
      float b = -INFINITY;
      for (int i = g * per; i < (g + 1) * per; ++i) b = fmaxf(b, choice[i]);
      gbest[g] = b;
    }
    __syncthreads();
    for (int round = 0; round < keep; ++round) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int g = lane; g < count; g += DLI_WAVE) {
        const float v = gbest[g];
        if (v == v && (v > bv || (v == bv && g < bi))) { bv = v; bi = g; }   // (NaN marks a group already kept)
      }
      wave_argmax(bv, bi);
      __syncthreads();
      if (lane == 0 && bi < count) gbest[bi] = __builtin_nanf("");
      __syncthreads();
    }
    for (int i = lane; i < total; i += DLI_WAVE) {
      const float g = gbest[i / per];
      if (g == g) choice[i] = -INFINITY;        // its group was not kept
    }
    __syncthreads();
  }
  float chosen_sum = 0.f, mine = 0.f;            // lane j keeps the j-th choice (top <= 64)
  int my_id = 0;
  for (int j = 0; j < top; ++j) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lane; i < total; i += DLI_WAVE) {
      const float v = choice[i];
      if (v == v && (v > bv || (v == bv && i < bi))) { bv = v; bi = i; }      // (NaN marks an expert already chosen)
    }
    wave_argmax(bv, bi);
    bi = min(bi, total - 1);
    __syncthreads();
    const float p = s[bi];
    chosen_sum += p;
    if (lane == j) { mine = p; my_id = bi; }
    if (lane == 0) choice[bi] = __builtin_nanf("");
    __syncthreads();
  }
  if (lane < top) {
    ids[row * top + lane] = my_id;
    weights[row * top + lane] = mine / (chosen_sum + 1e-20f) * scale;
  }
}

#define EX_BM 32
#define EX_BN 64
#define EX_BK 16

// One workgroup. ids [slots]: the chosen expert of every (token, choice) slot; ids at or above `experts`
// (identity experts) have no rows. Leaves offsets [experts + 1], order [rows of real experts] (the slot of
// every sorted row; inside an expert's run the rows come in whatever order the counter hands out, which
// no value depends on), the tiles (expert, first sorted row) of at most tile_rows rows, and their number.
__global__ __launch_bounds__(1024) void expert_sort_kernel(const int* __restrict__ ids, int slots, int experts,
                                                           int* __restrict__ offsets, int* __restrict__ order,
                                                           int* __restrict__ tile_expert, int* __restrict__ tile_row0,
                                                           int* __restrict__ tile_count, int max_tiles, int tile_rows) {
  extern __shared__ int shi[];
  int *counts = shi, *cursor = shi + experts;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < slots; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < experts) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0, tiles = 0;
    for (int e = 0; e < experts; ++e) {
      offsets[e] = at;
      cursor[e] = at;
      for (int r = 0; r < counts[e] && tiles < max_tiles; r += tile_rows) {
        tile_expert[tiles] = e;
        tile_row0[tiles] = at + r;
        ++tiles;
      }
      at += counts[e];
    }
    offsets[experts] = at;
    tile_count[0] = tiles;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < slots; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < experts) order[atomicAdd(&cursor[e], 1)] = i;
  }
}

struct ExpertArgs {
  const int* tile_expert; const int* tile_row0; const int* tile_count; const int* offsets; const int* order;
  int top, width, ff;
};

// y[sorted row][ff] = clamped_glu(h[token] . w_gate[e], h[token] . w_up[e]); w_gate, w_up [experts][ff][width].
template <typename T>
__global__ __launch_bounds__(256) void expert_up_kernel(ExpertArgs p, const T* __restrict__ h, int64_t h_stride,
                                                        const T* __restrict__ w_gate, const T* __restrict__ w_up,
                                                        T* __restrict__ y, float limit, float alpha, float up_shift) {
  const int tile = blockIdx.x;
  if (tile >= p.tile_count[0]) return;
  __shared__ float as[EX_BK][EX_BM + 1], gs[EX_BK][EX_BN + 4], us[EX_BK][EX_BN + 4];
  __shared__ int tok[EX_BM];
  const int e = p.tile_expert[tile], r0 = p.tile_row0[tile], rend = p.offsets[e + 1];
  const int n0 = blockIdx.y * EX_BN;
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  if (tid < EX_BM) tok[tid] = r0 + tid < rend ? p.order[r0 + tid] / p.top : -1;
  __syncthreads();
  const T* wg = w_gate + (int64_t)e * p.ff * p.width;
  const T* wu = w_up + (int64_t)e * p.ff * p.width;
  float accg[2][4] = {}, accu[2][4] = {};
  for (int k0 = 0; k0 < p.width; k0 += EX_BK) {
    for (int i = tid; i < EX_BM * EX_BK; i += 256) {
      const int r = i / EX_BK, k = i % EX_BK;
      as[k][r] = tok[r] >= 0 && k0 + k < p.width ? to_f32(h[(int64_t)tok[r] * h_stride + k0 + k]) : 0.f;
    }
    for (int i = tid; i < EX_BN * EX_BK; i += 256) {
      const int c = i / EX_BK, k = i % EX_BK;
      const bool ok = n0 + c < p.ff && k0 + k < p.width;
      gs[k][c] = ok ? to_f32(wg[(int64_t)(n0 + c) * p.width + k0 + k]) : 0.f;
      us[k][c] = ok ? to_f32(wu[(int64_t)(n0 + c) * p.width + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < EX_BK; ++k) {
      const float a0 = as[k][ty * 2], a1 = as[k][ty * 2 + 1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float g = gs[k][tx * 4 + j], u = us[k][tx * 4 + j];
        accg[0][j] = fmaf(a0, g, accg[0][j]);
        accg[1][j] = fmaf(a1, g, accg[1][j]);
        accu[0][j] = fmaf(a0, u, accu[0][j]);
        accu[1][j] = fmaf(a1, u, accu[1][j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = r0 + ty * 2 + i;
    if (r >= rend) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = n0 + tx * 4 + j;
      if (c < p.ff) y[(int64_t)r * p.ff + c] = from_f32<T>(clamped_glu(accg[i][j], accu[i][j], limit, alpha, up_shift));
    }
  }
}

// z[slot][width] = y[sorted row] . w_down[e]; w_down [experts][width][ff].
template <typename T>
__global__ __launch_bounds__(256) void expert_down_kernel(ExpertArgs p, const T* __restrict__ y, const T* __restrict__ w_down,
                                                          float* __restrict__ z) {
  const int tile = blockIdx.x;
  if (tile >= p.tile_count[0]) return;
  __shared__ float as[EX_BK][EX_BM + 1], ws[EX_BK][EX_BN + 4];
  const int e = p.tile_expert[tile], r0 = p.tile_row0[tile], rend = p.offsets[e + 1];
  const int n0 = blockIdx.y * EX_BN;
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const T* wd = w_down + (int64_t)e * p.width * p.ff;
  float acc[2][4] = {};
  for (int k0 = 0; k0 < p.ff; k0 += EX_BK) {
    for (int i = tid; i < EX_BM * EX_BK; i += 256) {
      const int r = i / EX_BK, k = i % EX_BK;
      as[k][r] = r0 + r < rend && k0 + k < p.ff ? to_f32(y[(int64_t)(r0 + r) * p.ff + k0 + k]) : 0.f;
    }
    for (int i = tid; i < EX_BN * EX_BK; i += 256) {
      const int c = i / EX_BK, k = i % EX_BK;
      ws[k][c] = n0 + c < p.width && k0 + k < p.ff ? to_f32(wd[(int64_t)(n0 + c) * p.ff + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < EX_BK; ++k) {
      const float a0 = as[k][ty * 2], a1 = as[k][ty * 2 + 1];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float w = ws[k][tx * 4 + j];
        acc[0][j] = fmaf(a0, w, acc[0][j]);
        acc[1][j] = fmaf(a1, w, acc[1][j]);
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = r0 + ty * 2 + i;
    if (r >= rend) continue;
    const int64_t slot = p.order[r];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = n0 + tx * 4 + j;
      if (c < p.width) z[slot * p.width + c] = acc[i][j];
    }
  }
}

// The same two products on the matrix cores (bfloat16; width and ff multiples of 32): tiles of EXM_BM
// sorted rows, a workgroup of four waves takes 128 features, each wave 32 of them (two blocks of 16) for
// all rows of the tile. v_mfma_f32_16x16x32_bf16 with the weights as the first operand: lane l supplies
// feature l % 16 of a block and row l % 16 of each block of 16 rows, and the eight k values
// 8 (l / 16) .. + 7 of a step of 32, read straight from memory (16 bytes a lane and operand; the rows of
// a tile are re-read by the four waves from the cache); the operands of the next step are asked for
// before this step's products are issued. A lane's results are four neighbouring features of one row.
// Every output sums its k in ascending steps of 32 whatever its tile, so a row's result depends on
// nothing beside the row.
#define EXM_BM 64
#define EXM_MB (EXM_BM / 16)
#define EXM_BN 128
typedef __bf16 exm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float exm_float4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ exm_bf16x8 exm_load(const bf16_t* p) { return *reinterpret_cast<const exm_bf16x8*>(p); }

__global__ __launch_bounds__(256) void expert_up_mfma_kernel(ExpertArgs p, const bf16_t* __restrict__ h, int64_t h_stride,
                                                             const bf16_t* __restrict__ w_gate,
                                                             const bf16_t* __restrict__ w_up, bf16_t* __restrict__ y,
                                                             float limit, float alpha, float up_shift) {
  const int tile = blockIdx.x;
  if (tile >= p.tile_count[0]) return;
  const int e = p.tile_expert[tile], r0 = p.tile_row0[tile], rend = p.offsets[e + 1];
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE;
  const int c = lane % 16, kq = (lane / 16) * 8;
  const int nw = blockIdx.y * EXM_BN + wave * 32;
  const bf16_t *wg[2], *wu[2], *xr[EXM_MB];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int n = min(nw + nb * 16 + c, p.ff - 1);                              // (a feature past the end repeats the last)
    wg[nb] = w_gate + ((int64_t)e * p.ff + n) * p.width + kq;
    wu[nb] = w_up + ((int64_t)e * p.ff + n) * p.width + kq;
  }
#pragma unroll
  for (int mb = 0; mb < EXM_MB; ++mb) {
    const int r = min(r0 + mb * 16 + c, rend - 1);                              // (a row past the end repeats the last)
    xr[mb] = h + (int64_t)(p.order[r] / p.top) * h_stride + kq;
  }
  exm_float4 accg[2][EXM_MB], accu[2][EXM_MB];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int mb = 0; mb < EXM_MB; ++mb) accg[nb][mb] = accu[nb][mb] = exm_float4{0.f, 0.f, 0.f, 0.f};
  const int blocks = (rend - r0 + 15) / 16;                                     // blocks of 16 rows that hold a row
  exm_bf16x8 a[2], b[2], x[EXM_MB];
  auto fetch = [&](int k) {
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) { a[nb] = exm_load(wg[nb] + k); b[nb] = exm_load(wu[nb] + k); }
#pragma unroll
    for (int mb = 0; mb < EXM_MB; ++mb) x[mb] = exm_load(xr[mb] + k);            // (unconditional: clamped rows are valid memory)
  };
  fetch(0);
  for (int k = 0; k < p.width; k += 32) {
    exm_bf16x8 a0[2], b0[2], x0[EXM_MB];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) { a0[nb] = a[nb]; b0[nb] = b[nb]; }
#pragma unroll
    for (int mb = 0; mb < EXM_MB; ++mb) x0[mb] = x[mb];
    fetch(min(k + 32, p.width - 32));                                           // the last turn asks for its own step again
#pragma unroll
    for (int mb = 0; mb < EXM_MB; ++mb) {
      if (mb < blocks) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          accg[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[nb], x0[mb], accg[nb][mb], 0, 0, 0);
          accu[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b0[nb], x0[mb], accu[nb][mb], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int mb = 0; mb < EXM_MB; ++mb) {
    const int r = r0 + mb * 16 + c;
    if (r >= rend) continue;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int n0 = nw + nb * 16 + (lane / 16) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n0 + i < p.ff) y[(int64_t)r * p.ff + n0 + i] = (bf16_t)clamped_glu(accg[nb][mb][i], accu[nb][mb][i], limit, alpha, up_shift);
    }
  }
}

__global__ __launch_bounds__(256) void expert_down_mfma_kernel(ExpertArgs p, const bf16_t* __restrict__ y,
                                                               const bf16_t* __restrict__ w_down, float* __restrict__ z) {
  const int tile = blockIdx.x;
  if (tile >= p.tile_count[0]) return;
  const int e = p.tile_expert[tile], r0 = p.tile_row0[tile], rend = p.offsets[e + 1];
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE;
  const int c = lane % 16, kq = (lane / 16) * 8;
  const int nw = blockIdx.y * EXM_BN + wave * 32;
  const bf16_t *wd[2], *yr[EXM_MB];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) wd[nb] = w_down + ((int64_t)e * p.width + min(nw + nb * 16 + c, p.width - 1)) * p.ff + kq;
#pragma unroll
  for (int mb = 0; mb < EXM_MB; ++mb) yr[mb] = y + (int64_t)min(r0 + mb * 16 + c, rend - 1) * p.ff + kq;
  exm_float4 acc[2][EXM_MB];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int mb = 0; mb < EXM_MB; ++mb) acc[nb][mb] = exm_float4{0.f, 0.f, 0.f, 0.f};
  const int blocks = (rend - r0 + 15) / 16;
  exm_bf16x8 a[2], x[EXM_MB];
  auto fetch = [&](int k) {
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) a[nb] = exm_load(wd[nb] + k);
#pragma unroll
    for (int mb = 0; mb < EXM_MB; ++mb) x[mb] = exm_load(yr[mb] + k);
  };
  fetch(0);
  for (int k = 0; k < p.ff; k += 32) {
    exm_bf16x8 a0[2], x0[EXM_MB];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) a0[nb] = a[nb];
#pragma unroll
    for (int mb = 0; mb < EXM_MB; ++mb) x0[mb] = x[mb];
    fetch(min(k + 32, p.ff - 32));
#pragma unroll
    for (int mb = 0; mb < EXM_MB; ++mb)
      if (mb < blocks)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0[nb], x0[mb], acc[nb][mb], 0, 0, 0);
  }
#pragma unroll
  for (int mb = 0; mb < EXM_MB; ++mb) {
    const int r = r0 + mb * 16 + c;
    if (r >= rend) continue;
    const int64_t slot = p.order[r];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
      const int n0 = nw + nb * 16 + (lane / 16) * 4;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n0 + i < p.width) z[slot * p.width + n0 + i] = acc[nb][mb][i];
    }
  }
}

// out[token] = sum_j weights[token][j] * (ids[token][j] < experts ? z[token * top + j] : h[token])
//            + sigmoid(shared_gate[token]) * shared[token]       (the shared expert, if there is one)
template <typename T>
__global__ void expert_combine_kernel(const int* __restrict__ ids, const float* __restrict__ weights,
                                      const float* __restrict__ z, const T* __restrict__ h, int64_t h_stride,
                                      const float* __restrict__ shared_gate, int64_t gate_stride,
                                      const float* __restrict__ shared, int64_t shared_stride, float* __restrict__ out,
                                      int top, int experts, int width) {
  const int64_t row = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= width) return;
  float sum = 0.f;
  for (int j = 0; j < top; ++j) {
    const int e = ids[row * top + j];
    const float v = e < experts ? z[(row * top + j) * width + c] : to_f32(h[row * h_stride + c]);
    sum = fmaf(weights[row * top + j], v, sum);
  }
  if (shared != nullptr) {
    const float g = shared_gate != nullptr ? 1.f / (1.f + expf(-shared_gate[row * gate_stride])) : 1.f;
    sum = fmaf(g, shared[row * shared_stride + c], sum);
  }
  out[row * width + c] = sum;
}

// A router that is a table: the experts of a token are the row of `table` [vocabulary][top] at its token id,
// each with the weight 1 / top. A thread a (token, choice).
__global__ void table_choose_kernel(const int* __restrict__ table, const int* __restrict__ token_ids, int n, int top,
                                    int vocab, int* __restrict__ ids, float* __restrict__ weights) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * top) return;
  const int t = i / top, j = i - t * top;
  const int tok = min(max(token_ids[t], 0), vocab - 1);
  ids[i] = table[(int64_t)tok * top + j];
  weights[i] = 1.f / (float)top;
}

extern "C" {

int dli_poly_norm(const float* z, int64_t z_stride, const float* coef, void* out, int64_t out_stride, int rows, int ff,
                  float eps, int out_is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (ff <= 0 || z_stride < ff || out_stride < ff) return DLI_ERR_ARGUMENT;
  poly_norm_kernel_f32in<<<rows, ff >= 4096 ? 512 : 256, 0, stream>>>(z, z_stride, coef, out, out_stride, ff, eps, out_is_bf16);
  return dli_launch_status();
}

int dli_clamped_glu(const void* gate_up, int64_t stride, void* out, int rows, int ff, float limit, float alpha, float up_shift, int is_bf16,
                    hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (ff <= 0 || stride < 2 * (int64_t)ff) return DLI_ERR_ARGUMENT;
  const dim3 grid(rows, (ff + 255) / 256);
  if (is_bf16) clamped_glu_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gate_up, stride, (bf16_t*)out, ff, limit, alpha, up_shift);
  else clamped_glu_kernel<float><<<grid, 256, 0, stream>>>((const float*)gate_up, stride, (float*)out, ff, limit, alpha, up_shift);
  return dli_launch_status();
}

int dli_router_choose(const float* logits, int64_t stride, const float* bias, const float* correction, int rows, int total, int count, int keep,
                      int top, float scale, int* ids, float* weights, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (total <= 0 || total > 4096 || stride < total || top < 1 || top > 64 || top > total || count < 1 || total % count ||
      keep < 1 || keep > count || (int64_t)keep * (total / count) < top)
    return DLI_ERR_ARGUMENT;
  router_choose_kernel<<<rows, 64, (2 * total + count) * sizeof(float), stream>>>(logits, stride, bias, correction, total, count, keep,
                                                                                  top, scale, ids, weights);
  return dli_launch_status();
}

// Whether the matrix-core kernels take these sizes, and the rows of a tile of the kernels that will run.
static bool expert_mfma(int width, int ff, int is_bf16) { return is_bf16 && width % 32 == 0 && ff % 32 == 0; }
int dli_expert_tile_rows(int width, int ff, int is_bf16) { return expert_mfma(width, ff, is_bf16) ? EXM_BM : EX_BM; }

// The experts' part of a mixture for `rows` tokens: sort, up product with activation, down product.
// ids [rows][top]; scratch: offsets [experts + 1], order [rows * top], tile_expert and tile_row0 [max_tiles],
// tile_count [1] (int32), y [rows * top][ff] (T), z [rows * top][width] (float32).
int dli_expert_products(const int* ids, const void* h, int64_t h_stride, const void* w_gate, const void* w_up,
                        const void* w_down, int* offsets, int* order, int* tile_expert, int* tile_row0, int* tile_count,
                        int max_tiles, void* y, float* z, int rows, int top, int experts, int width, int ff, float limit,
                        float alpha, float up_shift, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  const int64_t slots = (int64_t)rows * top;
  if (top < 1 || experts < 1 || experts > 4096 || width <= 0 || ff <= 0 || h_stride < width || slots > (1 << 30) ||
      max_tiles < 1 || max_tiles > 65535 * 16)
    return DLI_ERR_ARGUMENT;
  const bool mfma = expert_mfma(width, ff, is_bf16);
  if (mfma && ((h_stride % 8) || ((uintptr_t)h % 16) || ((uintptr_t)w_gate % 16) || ((uintptr_t)w_up % 16) ||
               ((uintptr_t)w_down % 16) || ((uintptr_t)y % 16)))
    return DLI_ERR_ARGUMENT;
  expert_sort_kernel<<<1, 1024, 2 * experts * sizeof(int), stream>>>(ids, (int)slots, experts, offsets, order, tile_expert,
                                                                     tile_row0, tile_count, max_tiles, mfma ? EXM_BM : EX_BM);
  if (dli_launch_status() != DLI_OK) return DLI_ERR_LAUNCH;
  ExpertArgs p;
  p.tile_expert = tile_expert; p.tile_row0 = tile_row0; p.tile_count = tile_count; p.offsets = offsets; p.order = order;
  p.top = top; p.width = width; p.ff = ff;
  const int bn = mfma ? EXM_BN : EX_BN;
  const dim3 up_grid(max_tiles, (ff + bn - 1) / bn), down_grid(max_tiles, (width + bn - 1) / bn);
  if (mfma) {
    expert_up_mfma_kernel<<<up_grid, 256, 0, stream>>>(p, (const bf16_t*)h, h_stride, (const bf16_t*)w_gate,
                                                       (const bf16_t*)w_up, (bf16_t*)y, limit, alpha, up_shift);
    expert_down_mfma_kernel<<<down_grid, 256, 0, stream>>>(p, (const bf16_t*)y, (const bf16_t*)w_down, z);
  } else if (is_bf16) {
    expert_up_kernel<bf16_t><<<up_grid, 256, 0, stream>>>(p, (const bf16_t*)h, h_stride, (const bf16_t*)w_gate,
                                                          (const bf16_t*)w_up, (bf16_t*)y, limit, alpha, up_shift);
    expert_down_kernel<bf16_t><<<down_grid, 256, 0, stream>>>(p, (const bf16_t*)y, (const bf16_t*)w_down, z);
  } else {
    expert_up_kernel<float><<<up_grid, 256, 0, stream>>>(p, (const float*)h, h_stride, (const float*)w_gate,
                                                         (const float*)w_up, (float*)y, limit, alpha, up_shift);
    expert_down_kernel<float><<<down_grid, 256, 0, stream>>>(p, (const float*)y, (const float*)w_down, z);
  }
  return dli_launch_status();
}

int dli_expert_combine(const int* ids, const float* weights, const float* z, const void* h, int64_t h_stride,
                       const float* shared_gate, int64_t gate_stride, const float* shared, int64_t shared_stride, float* out,
                       int rows, int top, int experts, int width, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (top < 1 || width <= 0 || h_stride < width || (shared != nullptr && shared_stride < width)) return DLI_ERR_ARGUMENT;
  const dim3 grid(rows, (width + 255) / 256);
  if (is_bf16)
    expert_combine_kernel<bf16_t><<<grid, 256, 0, stream>>>(ids, weights, z, (const bf16_t*)h, h_stride, shared_gate, gate_stride,
                                                            shared, shared_stride, out, top, experts, width);
  else
    expert_combine_kernel<float><<<grid, 256, 0, stream>>>(ids, weights, z, (const float*)h, h_stride, shared_gate, gate_stride,
                                                           shared, shared_stride, out, top, experts, width);
  return dli_launch_status();
}

int dli_table_choose(const int* table, const int* token_ids, int n, int top, int vocab, int* ids, float* weights,
                     hipStream_t stream) {
  if (n <= 0) return DLI_OK;
  if (top <= 0 || vocab <= 0 || (int64_t)n * top > 0x7fffffff) return DLI_ERR_ARGUMENT;
  table_choose_kernel<<<(n * top + 255) / 256, 256, 0, stream>>>(table, token_ids, n, top, vocab, ids, weights);
  return dli_launch_status();
}

}  // extern "C"
