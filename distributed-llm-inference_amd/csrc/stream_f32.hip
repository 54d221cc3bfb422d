// Kernels for models whose residual stream is kept in 32-bit whatever the type of the matrix
// products: the stream `x` is float32 [tokens][width]; T is the type of what the products read and
// write (float on the 32-bit path, bf16 when serving). Statistics, sums, angles and activations
// are 32-bit.
//
//   embed_sinusoid     x = table[id] + pe(position), pe[2i] = sin(p f_i), pe[2i+1] = cos(p f_i)
//   cast_from_f32      the stream rounded to T, as the operand of a product
//   norm_into_stream   x += w * y / sqrt(mean(y^2) + eps)   (a norm on a sublayer's output); like the embedding
//                      it can leave the new stream once more in bf16, for the product that reads it next
//   rms_norm_from_f32  out(T) = w * x / sqrt(mean(x^2) + eps)
//   post_norm_stream   x <- w * s / sqrt(mean(s^2) + eps) with s = alpha x + r y, r = sigmoid(g + b) element by element
//                      or 1 (a norm after the residual sum, the summand under a gate of its own)
//   softcap            y = cap * tanh(y / cap)
//   token_shift        S mixes of each row with the row before it, x + (prev - x) * mu_s; the row
//                      before a step's first row comes from the request's state, which then
//                      receives the step's last row
//   lowrank_out        y = bias + W2 act(t): the second half of a low-rank projection, 32-bit (W2 given transposed)
//   qk_unit_cache      per-head unit RMS of q and k, value mixing, cache write
//   rotary_cache       rotary rotation of q and k from 32-bit projections (pairs side by side or half a
//                      head apart, the first rot_dims components of a head), cache write
//   group_norm         out(T) = w * x / sqrt(mean_part(x^2) + eps), a row's equal consecutive parts each by
//                      its own root mean square; with delta: x += delta first, in place
//   branch_norm_mean   the mean of up to four branches' outputs, each first divided by its root mean
//                      square over the row and multiplied by its own weight
//   branch_weighted_sum  the sum of up to four branches' outputs, each times a constant of its own
//   diff_head_norm     two attention maps over the same values combined head by head: a1 - lambda a2, divided by
//                      its root mean square over the head, times a constant and a sigmoid gate per head
//   scale_f32          y *= c in place
//   rms_norm_pair      two norms of the same row (two weights) from one pass over its statistics
//   add_pair_into_stream  x += a + b
#include "common.h"

template <typename T>
__global__ void embed_sinusoid_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                      const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                      float* __restrict__ out, bf16_t* __restrict__ rounded, int width) {
  const int64_t row = blockIdx.x;
  const T* src = table + (int64_t)ids[row] * width;
  const float p = (float)positions[row];
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float sum = to_f32(src[i]);
    if (inv_freq != nullptr) {   // (nullptr: the token's row alone)
      const float angle = p * inv_freq[i >> 1];
      sum += (i & 1) ? cosf(angle) : sinf(angle);
    }
    out[row * width + i] = sum;
    if (rounded != nullptr) rounded[row * width + i] = (bf16_t)sum;
  }
}

template <typename T>
__global__ void cast_from_f32_kernel(const float* __restrict__ x, T* __restrict__ out, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<T>(x[i]);
}

// `rounded` (may be nullptr): the new stream once more in type R, for the product that reads it next.
template <typename T, typename R>
__global__ void norm_into_stream_kernel(const T* __restrict__ y, int64_t y_stride, const float* __restrict__ weight,
                                        float* __restrict__ x, R* __restrict__ rounded, int width, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * y_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float f = to_f32(yr[i]);
    ss += f * f;
  }
  const float r = 1.f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  float* xr = x + row * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float sum = xr[i] + weight[i] * (to_f32(yr[i]) * r);
    xr[i] = sum;
    if (rounded != nullptr) rounded[row * width + i] = from_f32<R>(sum);
  }
}

template <typename T>
__global__ void rms_norm_from_f32_kernel(const float* __restrict__ x, const float* __restrict__ weight,
                                         T* __restrict__ out, int width, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const float* xr = x + row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) ss += xr[i] * xr[i];
  const float r = 1.f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) out[row * width + i] = from_f32<T>(weight[i] * (xr[i] * r));
}

// A workgroup a row. Each thread reads back only what it wrote itself.
template <typename Y, typename R>
__global__ void post_norm_stream_kernel(const Y* __restrict__ y, int64_t y_stride, const float* __restrict__ g,
                                        int64_t g_stride, const float* __restrict__ g_bias,
                                        const float* __restrict__ weight, float* __restrict__ x, R* __restrict__ rounded,
                                        int width, float alpha, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  float* xr = x + row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float t = to_f32(y[row * y_stride + i]);
    if (g != nullptr) t *= 1.f / (1.f + expf(-(g[row * g_stride + i] + (g_bias != nullptr ? g_bias[i] : 0.f))));
    const float s = fmaf(alpha, xr[i], t);
    xr[i] = s;
    ss += s * s;
  }
  const float r = 1.f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = weight[i] * (xr[i] * r);
    xr[i] = v;
    if (rounded != nullptr) rounded[row * width + i] = from_f32<R>(v);
  }
}

__global__ void softcap_kernel(float* __restrict__ y, int64_t n, float cap) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = cap * tanhf(y[i] / cap);
}

// The entry that holds `row`: the last e with q_start[e] <= row.
__device__ __forceinline__ int entry_of_row(const int* __restrict__ q_start, int entries, int row) {
  int lo = 0, hi = entries - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= row) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// A thread an element (grid: rows x blocks of the width). The thread that reads a request's state
// for the entry's first row is also the one that writes the entry's last row there, after its
// read: no other thread touches that element in this launch.
template <typename T>
__global__ void token_shift_kernel(const float* __restrict__ x, const float* __restrict__ mu, int mixes,
                                   float* state, int64_t state_stride, const int* __restrict__ q_start, int entries,
                                   const int* __restrict__ positions, const int* __restrict__ state_slots,
                                   T* __restrict__ out, int rows, int width) {
  const int row = blockIdx.x;
  const int e = entry_of_row(q_start, entries, row);
  const int first = q_start[e], last = q_start[e + 1] - 1;
  const float* xr = x + (int64_t)row * width;
  float* st = state + (int64_t)state_slots[e] * state_stride;
  const bool from_state = row == first;
  const bool fresh = positions[row] == 0;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i < width) {
    const float cur = xr[i];
    float prev;
    if (from_state) {
      prev = fresh ? 0.f : st[i];
      st[i] = x[(int64_t)last * width + i];
    } else {
      prev = xr[i - width];
    }
    for (int s = 0; s < mixes; ++s)
      out[((int64_t)s * rows + row) * width + i] = from_f32<T>(cur + (prev - cur) * mu[(int64_t)s * width + i]);
  }
}

// act: 0 none, 1 tanh. t is [rows][t_stride] (rank values a row), w2t [rank][features] (the matrix
// transposed, so that neighbouring threads read neighbouring weights), out [rows][features].
// out_act: what becomes of y before it is stored: 0 y itself; 1 exp(-exp(-1/2) sigmoid(y)) and
// 2 exp(-exp(y)), the decays of the two recurrences; 3 softplus(y), a step size. rate (may be nullptr): [rows][rate_stride], with
// features values a row that become sigmoid(rate + rate_bias) in place (the delta rule's removal
// rate, made here because a thread a (row, feature) is what this launch already has).
__global__ void lowrank_out_kernel(const float* __restrict__ t, int64_t t_stride, const float* __restrict__ w2t,
                                   const float* __restrict__ bias, float* __restrict__ out, int features, int rank,
                                   int act, int out_act, float* __restrict__ rate, int64_t rate_stride,
                                   const float* __restrict__ rate_bias) {
  extern __shared__ float ts[];
  const int64_t row = blockIdx.x;
  for (int j = threadIdx.x; j < rank; j += blockDim.x) {
    const float v = t[row * t_stride + j];
    ts[j] = act == 1 ? tanhf(v) : v;
  }
  __syncthreads();
  const int c = blockIdx.y * blockDim.x + threadIdx.x;   // a feature a thread
  if (c >= features) return;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;          // four sums: the weights' loads do not wait for each other
  int j = 0;
  for (; j + 4 <= rank; j += 4) {
    const float a = w2t[(int64_t)j * features + c], b = w2t[(int64_t)(j + 1) * features + c];
    const float d = w2t[(int64_t)(j + 2) * features + c], e = w2t[(int64_t)(j + 3) * features + c];
    s0 = fmaf(ts[j], a, s0);
    s1 = fmaf(ts[j + 1], b, s1);
    s2 = fmaf(ts[j + 2], d, s2);
    s3 = fmaf(ts[j + 3], e, s3);
  }
  for (; j < rank; ++j) s0 = fmaf(ts[j], w2t[(int64_t)j * features + c], s0);
  float y = ((s0 + s1) + (s2 + s3)) + (bias != nullptr ? bias[c] : 0.f);
  if (out_act == 1) y = expf(-0.6065306597126334f / (1.f + expf(-y)));
  else if (out_act == 2) y = expf(-expf(y));
  else if (out_act == 3) y = y > 20.f ? y : log1pf(expf(y));
  out[row * features + c] = y;
  if (rate != nullptr) {
    float* r = rate + row * rate_stride + c;
    *r = 1.f / (1.f + expf(-(*r + (rate_bias != nullptr ? rate_bias[c] : 0.f))));
  }
}

// proj [tokens][stride] float32 holds q (q_heads x dim), k (kv_heads x dim) and v (kv_heads x vdim)
// at the given column offsets. q and k are divided by their root mean square over dim, head by
// head. v is mixed with the values that an earlier layer computed for the same token,
// v <- (1 - lambda) v + lambda v_first (lambda == nullptr: no mixing; v_first_out != nullptr: this
// layer's v is written there for the later ones). The unit k and the v that results go to the
// token's cache slot (negative: not cached).
template <typename T>
__global__ void qk_unit_cache_kernel(const float* __restrict__ proj, int64_t stride, int q_off, int k_off, int v_off,
                                     T* __restrict__ q_out, const float* __restrict__ lambda,
                                     const float* __restrict__ v_first_in, float* __restrict__ v_first_out,
                                     const int* __restrict__ slots, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                     int q_heads, int kv_heads, int dim, int vdim, int page_size, float eps) {
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE, waves = blockDim.x / DLI_WAVE;
  const float* pr = proj + row * stride;
  const int slot = slots[row];
  const int64_t page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  for (int h = wave; h < q_heads + kv_heads; h += waves) {
    const bool is_q = h < q_heads;
    const float* src = is_q ? pr + q_off + (int64_t)h * dim : pr + k_off + (int64_t)(h - q_heads) * dim;
    float ss = 0.f;
    for (int c = lane; c < dim; c += DLI_WAVE) ss += src[c] * src[c];
    const float r = 1.f / sqrtf(wave_sum(ss) / (float)dim + eps);
    if (is_q) {
      for (int c = lane; c < dim; c += DLI_WAVE) q_out[(row * q_heads + h) * dim + c] = from_f32<T>(src[c] * r);
    } else if (slot >= 0) {
      T* dst = k_pages + ((page * kv_heads + (h - q_heads)) * page_size + off) * dim;
      for (int c = lane; c < dim; c += DLI_WAVE) dst[c] = from_f32<T>(src[c] * r);
    }
  }
  const float lam = lambda != nullptr ? lambda[0] : 0.f;
  for (int i = threadIdx.x; i < kv_heads * vdim; i += blockDim.x) {
    float v = pr[v_off + i];
    if (lambda != nullptr) v = (1.f - lam) * v + lam * v_first_in[row * kv_heads * vdim + i];
    if (v_first_out != nullptr) v_first_out[row * kv_heads * vdim + i] = v;
    if (slot >= 0) {
      const int g = i / vdim, c = i - g * vdim;
      v_pages[((page * kv_heads + g) * vdim + c) * page_size + off] = from_f32<T>(v);
    }
  }
}

// cos and sin of position * freq with the product's rounding error taken back: the product's low
// half (one fused multiply-add) turns the functions by their own derivatives.
__device__ __forceinline__ void rotary_cos_sin(float position, float freq, float* c, float* s) {
  const float hi = position * freq;
  const float lo = fmaf(position, freq, -hi);
  float sh, ch;
  sincosf(hi, &sh, &ch);
  *c = fmaf(-lo, sh, ch);
  *s = fmaf(lo, ch, sh);
}

// proj [tokens][stride] float32 holds q (q_heads x dim), k (kv_heads x dim) and v (kv_heads x vdim) at
// the given column offsets. The first rot_dims components of every q and k head are rotated by
// position * inv_freq[i]: pair i is (2i, 2i+1) where `interleaved`, else (i, i + rot_dims/2); the
// other components pass. q goes out in T; the rotated k and v go to the token's cache slot
// (negative: not cached). A thread an element: it reads its partner from proj. `bias` (may be nullptr)
// holds a value for every column of proj and is added before anything else. The pages may hold fewer
// value heads than key heads (v_heads), and none at all where the mixer reads another's (kv_heads 0).
template <typename T>
__global__ void rotary_cache_kernel(const float* __restrict__ proj, int64_t stride, int q_off, int k_off, int v_off,
                                    const float* __restrict__ bias,
                                    const int* __restrict__ positions, const float* __restrict__ inv_freq, int rot_dims,
                                    int interleaved, T* __restrict__ q_out, const int* __restrict__ slots,
                                    T* __restrict__ k_pages, T* __restrict__ v_pages, int q_heads, int kv_heads, int v_heads,
                                    int dim, int vdim, int page_size) {
  const int64_t row = blockIdx.x;
  const float* pr = proj + row * stride;
  const float p = (float)positions[row];
  const int slot = slots != nullptr ? slots[row] : -1;
  const int64_t page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  const int half = rot_dims / 2;
  for (int i = threadIdx.x; i < (q_heads + kv_heads) * dim; i += blockDim.x) {
    const int h = i / dim, c = i - h * dim;
    const bool is_q = h < q_heads;
    const int64_t at = is_q ? q_off + (int64_t)h * dim : k_off + (int64_t)(h - q_heads) * dim;
    const float* src = pr + at;
    const float* bs = bias != nullptr ? bias + at : nullptr;
    float y = src[c] + (bs != nullptr ? bs[c] : 0.f);
    if (c < rot_dims) {
      int pair, partner;
      bool first;
      if (interleaved) { pair = c >> 1; partner = c ^ 1; first = (c & 1) == 0; }
      else { first = c < half; pair = first ? c : c - half; partner = first ? c + half : c - half; }
      float cs, sn;
      rotary_cos_sin(p, inv_freq[pair], &cs, &sn);
      const float other = src[partner] + (bs != nullptr ? bs[partner] : 0.f);
      y = first ? y * cs - other * sn : y * cs + other * sn;
    }
    if (is_q) q_out[(row * q_heads + h) * dim + c] = from_f32<T>(y);
    else if (slot >= 0) k_pages[((page * kv_heads + (h - q_heads)) * page_size + off) * dim + c] = from_f32<T>(y);
  }
  if (slot >= 0)
    for (int i = threadIdx.x; i < v_heads * vdim; i += blockDim.x) {
      const int g = i / vdim, c = i - g * vdim;
      v_pages[((page * v_heads + g) * vdim + c) * page_size + off] =
          from_f32<T>(pr[v_off + i] + (bias != nullptr ? bias[v_off + i] : 0.f));
    }
}

// x [rows][width] float32 (with delta: x += delta first, stored); each of `groups` equal consecutive
// parts of the row is divided by its own root mean square; out(T) = w * that. A workgroup a (row, part).
template <typename T>
__global__ void group_norm_kernel(float* __restrict__ x, const float* __restrict__ delta, int64_t delta_stride,
                                  const float* __restrict__ weight, T* __restrict__ out, int width, int groups, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const int part = width / groups, first = blockIdx.y * part;
  float* xr = x + row * width;
  float ss = 0.f;
  for (int i = first + threadIdx.x; i < first + part; i += blockDim.x) {
    float f = xr[i];
    if (delta != nullptr) {
      f += delta[row * delta_stride + i];
      xr[i] = f;
    }
    ss += f * f;
  }
  const float r = 1.f / sqrtf(block_sum(ss, scratch) / (float)part + eps);
  // (each thread reads back what it wrote itself)
  for (int i = first + threadIdx.x; i < first + part; i += blockDim.x)
    out[row * width + i] = from_f32<T>(weight[i] * (xr[i] * r));
}

struct BranchArgs {
  const float* y[4]; int64_t stride[4]; const float* weight[4];
  int count;
};

// (the branches' sums of squares are made side by side and meet in one exchange through LDS; COUNT is a
// template parameter so that no load hangs on a condition)
template <int COUNT>
__global__ void branch_norm_mean_kernel(BranchArgs b, float* __restrict__ out, int width, float eps) {
  __shared__ float scratch[COUNT][16];
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE, waves = blockDim.x / DLI_WAVE;
  float ss[COUNT];
#pragma unroll
  for (int j = 0; j < COUNT; ++j) ss[j] = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x)
#pragma unroll
    for (int j = 0; j < COUNT; ++j) {
      const float f = b.y[j][row * b.stride[j] + i];
      ss[j] += f * f;
    }
#pragma unroll
  for (int j = 0; j < COUNT; ++j) {
    ss[j] = wave_sum(ss[j]);
    if (lane == 0) scratch[j][wave] = ss[j];
  }
  __syncthreads();
  float r[COUNT];
#pragma unroll
  for (int j = 0; j < COUNT; ++j) {
    float total = 0.f;
    for (int w = 0; w < waves; ++w) total += scratch[j][w];   // same order in every thread
    r[j] = 1.f / sqrtf(total / (float)width + eps);
  }
  const float share = 1.f / (float)COUNT;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < COUNT; ++j) sum += b.weight[j][i] * (b.y[j][row * b.stride[j] + i] * r[j]);
    out[row * width + i] = sum * share;
  }
}

// Two attention maps over the same values become one result, head by head: with a1 = a[row][h] and
// a2 = a[row][heads + h] (value_dim values each), d = a1 - lambda a2 is divided by its root mean square over the
// head (no weight), multiplied by `after` and by sigmoid(gate[row][h]) (one number a head; nullptr: no gate).
// A wave a (row, head).
template <typename T>
__global__ __launch_bounds__(256) void diff_head_norm_kernel(const float* __restrict__ a, int64_t a_stride, float lambda,
                                                             float after, float eps, const float* __restrict__ gate,
                                                             int64_t gate_stride, T* __restrict__ out, int64_t out_stride,
                                                             int heads, int vdim) {
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x % DLI_WAVE, h = blockIdx.y * 4 + threadIdx.x / DLI_WAVE;
  if (h >= heads) return;
  const float* a1 = a + row * a_stride + (int64_t)h * vdim;
  const float* a2 = a + row * a_stride + (int64_t)(heads + h) * vdim;
  float ss = 0.f;
  for (int c = lane; c < vdim; c += DLI_WAVE) {
    const float d = a1[c] - lambda * a2[c];
    ss += d * d;
  }
  float r = after / sqrtf(wave_sum(ss) / (float)vdim + eps);
  if (gate != nullptr) r *= 1.f / (1.f + expf(-gate[row * gate_stride + h]));
  for (int c = lane; c < vdim; c += DLI_WAVE)
    out[row * out_stride + (int64_t)h * vdim + c] = from_f32<T>((a1[c] - lambda * a2[c]) * r);
}

// out = sum_b scale_b y_b for up to four float32 matrices of equal shape. A thread an element.
struct WeightedBranches { const float* y[4]; int64_t stride[4]; float scale[4]; int count; };
__global__ void branch_weighted_sum_kernel(WeightedBranches b, float* __restrict__ out, int width) {
  const int64_t row = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= width) return;
  float sum = 0.f;
  for (int j = 0; j < b.count; ++j) sum = fmaf(b.scale[j], b.y[j][row * b.stride[j] + i], sum);
  out[row * width + i] = sum;
}

__global__ void scale_f32_kernel(float* __restrict__ y, int64_t n, float scale) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] *= scale;
}

// Two norms of the same float32 row with one pass over its statistics: out1 = w1 * x * r, out2 = w2 * x * r,
// r = 1 / sqrt(mean(x^2) + eps) (a mixer and a feed-forward that read the same stream behind norms of their own).
template <typename T>
__global__ void rms_norm_pair_kernel(const float* __restrict__ x, const float* __restrict__ w1, const float* __restrict__ w2,
                                     T* __restrict__ out1, T* __restrict__ out2, int width, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const float* xr = x + row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) ss += xr[i] * xr[i];
  const float r = 1.f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = xr[i] * r;
    out1[row * width + i] = from_f32<T>(w1[i] * v);
    out2[row * width + i] = from_f32<T>(w2[i] * v);
  }
}

// x += a + b: two sublayers' results are added to each other and then into the stream. A thread an element.
__global__ void add_pair_into_stream_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ b,
                                            int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] += a[i] + b[i];
}

extern "C" {

int dli_embed_sinusoid(const void* table, const int* ids, const int* positions, const float* inv_freq, float* out,
                       void* rounded_bf16, int rows, int width, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0) return DLI_ERR_ARGUMENT;
  const int threads = width >= 1024 ? 256 : 128;
  if (is_bf16)
    embed_sinusoid_kernel<bf16_t><<<rows, threads, 0, stream>>>((const bf16_t*)table, ids, positions, inv_freq, out,
                                                                (bf16_t*)rounded_bf16, width);
  else
    embed_sinusoid_kernel<float><<<rows, threads, 0, stream>>>((const float*)table, ids, positions, inv_freq, out,
                                                               (bf16_t*)rounded_bf16, width);
  return dli_launch_status();
}

int dli_cast_from_f32(const float* x, void* out, int64_t n, int is_bf16, hipStream_t stream) {
  if (n <= 0) return DLI_OK;
  const int64_t blocks = (n + 255) / 256;
  if (blocks > 2147483647LL) return DLI_ERR_ARGUMENT;
  if (is_bf16) cast_from_f32_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(x, (bf16_t*)out, n);
  else cast_from_f32_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(x, (float*)out, n);
  return dli_launch_status();
}

int dli_norm_into_stream(const void* y, int64_t y_stride, const float* weight, float* x, void* rounded_bf16, int rows,
                         int width, float eps, int y_is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0 || y_stride < width) return DLI_ERR_ARGUMENT;
  const int threads = width >= 2048 ? 512 : 256;
  if (y_is_bf16)
    norm_into_stream_kernel<bf16_t, bf16_t><<<rows, threads, 0, stream>>>((const bf16_t*)y, y_stride, weight, x,
                                                                          (bf16_t*)rounded_bf16, width, eps);
  else
    norm_into_stream_kernel<float, bf16_t><<<rows, threads, 0, stream>>>((const float*)y, y_stride, weight, x,
                                                                         (bf16_t*)rounded_bf16, width, eps);
  return dli_launch_status();
}

int dli_rms_norm_from_f32(const float* x, const float* weight, void* out, int rows, int width, float eps, int is_bf16,
                          hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0) return DLI_ERR_ARGUMENT;
  const int threads = width >= 2048 ? 512 : 256;
  if (is_bf16)
    rms_norm_from_f32_kernel<bf16_t><<<rows, threads, 0, stream>>>(x, weight, (bf16_t*)out, width, eps);
  else
    rms_norm_from_f32_kernel<float><<<rows, threads, 0, stream>>>(x, weight, (float*)out, width, eps);
  return dli_launch_status();
}

int dli_post_norm_stream(const void* y, int64_t y_stride, const float* g, int64_t g_stride, const float* g_bias,
                         const float* weight, float* x, void* rounded_bf16, int rows, int width, float alpha, float eps,
                         int y_is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0 || y_stride < width || (g != nullptr && g_stride < width)) return DLI_ERR_ARGUMENT;
  const int threads = width >= 2048 ? 512 : 256;
  if (y_is_bf16)
    post_norm_stream_kernel<bf16_t, bf16_t><<<rows, threads, 0, stream>>>((const bf16_t*)y, y_stride, g, g_stride, g_bias,
                                                                          weight, x, (bf16_t*)rounded_bf16, width, alpha, eps);
  else
    post_norm_stream_kernel<float, bf16_t><<<rows, threads, 0, stream>>>((const float*)y, y_stride, g, g_stride, g_bias,
                                                                         weight, x, (bf16_t*)rounded_bf16, width, alpha, eps);
  return dli_launch_status();
}

int dli_softcap(float* y, int64_t n, float cap, hipStream_t stream) {
  if (n <= 0) return DLI_OK;
  const int64_t blocks = (n + 255) / 256;
  if (!(cap > 0.f) || blocks > 2147483647LL) return DLI_ERR_ARGUMENT;
  softcap_kernel<<<(unsigned)blocks, 256, 0, stream>>>(y, n, cap);
  return dli_launch_status();
}

int dli_token_shift(const float* x, const float* mu, int mixes, float* state, int64_t state_stride, const int* q_start,
                    int entries, const int* positions, const int* state_slots, void* out, int rows, int width,
                    int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0 || mixes <= 0 || entries <= 0 || state_stride < width) return DLI_ERR_ARGUMENT;
  const dim3 grid(rows, (width + 255) / 256);
  if (is_bf16)
    token_shift_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, mu, mixes, state, state_stride, q_start, entries,
                                                         positions, state_slots, (bf16_t*)out, rows, width);
  else
    token_shift_kernel<float><<<grid, 256, 0, stream>>>(x, mu, mixes, state, state_stride, q_start, entries,
                                                        positions, state_slots, (float*)out, rows, width);
  return dli_launch_status();
}

int dli_lowrank_out(const float* t, int64_t t_stride, const float* w2t, const float* bias, float* out, int rows,
                    int features, int rank, int act, int out_act, float* rate, int64_t rate_stride,
                    const float* rate_bias, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (features <= 0 || rank <= 0 || rank > 8192 || t_stride < rank || act < 0 || act > 1 || out_act < 0 || out_act > 3 ||
      (rate != nullptr && rate_stride < features))
    return DLI_ERR_ARGUMENT;
  lowrank_out_kernel<<<dim3(rows, (features + 255) / 256), 256, rank * sizeof(float), stream>>>(t, t_stride, w2t, bias, out,
                                                                                                features, rank, act, out_act,
                                                                                                rate, rate_stride, rate_bias);
  return dli_launch_status();
}

int dli_qk_unit_cache(const float* proj, int64_t stride, int q_off, int k_off, int v_off, void* q_out,
                      const float* lambda, const float* v_first_in, float* v_first_out, const int* slots,
                      void* k_pages, void* v_pages, int rows, int q_heads, int kv_heads, int dim, int vdim,
                      int page_size, float eps, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (q_heads <= 0 || kv_heads <= 0 || dim <= 0 || vdim <= 0 || page_size <= 0 ||
      (lambda != nullptr && v_first_in == nullptr))
    return DLI_ERR_ARGUMENT;
  if (is_bf16)
    qk_unit_cache_kernel<bf16_t><<<rows, 256, 0, stream>>>(proj, stride, q_off, k_off, v_off, (bf16_t*)q_out, lambda,
                                                           v_first_in, v_first_out, slots, (bf16_t*)k_pages,
                                                           (bf16_t*)v_pages, q_heads, kv_heads, dim, vdim, page_size, eps);
  else
    qk_unit_cache_kernel<float><<<rows, 256, 0, stream>>>(proj, stride, q_off, k_off, v_off, (float*)q_out, lambda,
                                                          v_first_in, v_first_out, slots, (float*)k_pages,
                                                          (float*)v_pages, q_heads, kv_heads, dim, vdim, page_size, eps);
  return dli_launch_status();
}

int dli_rotary_cache(const float* proj, int64_t stride, int q_off, int k_off, int v_off, const float* bias,
                     const int* positions, const float* inv_freq, int rot_dims, int interleaved, void* q_out,
                     const int* slots, void* k_pages, void* v_pages, int rows, int q_heads, int kv_heads, int v_heads,
                     int dim, int vdim, int page_size, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (q_heads <= 0 || kv_heads < 0 || v_heads < 0 || dim <= 0 || vdim <= 0 || page_size <= 0 || rot_dims < 0 ||
      rot_dims > dim || rot_dims % 2 || (rot_dims > 0 && inv_freq == nullptr) ||
      (kv_heads > 0 && (k_pages == nullptr || slots == nullptr)) || (v_heads > 0 && (v_pages == nullptr || slots == nullptr)))
    return DLI_ERR_ARGUMENT;
  if (is_bf16)
    rotary_cache_kernel<bf16_t><<<rows, 256, 0, stream>>>(proj, stride, q_off, k_off, v_off, bias, positions, inv_freq,
                                                          rot_dims, interleaved, (bf16_t*)q_out, slots, (bf16_t*)k_pages,
                                                          (bf16_t*)v_pages, q_heads, kv_heads, v_heads, dim, vdim, page_size);
  else
    rotary_cache_kernel<float><<<rows, 256, 0, stream>>>(proj, stride, q_off, k_off, v_off, bias, positions, inv_freq,
                                                         rot_dims, interleaved, (float*)q_out, slots, (float*)k_pages,
                                                         (float*)v_pages, q_heads, kv_heads, v_heads, dim, vdim, page_size);
  return dli_launch_status();
}

int dli_group_norm(float* x, const float* delta, int64_t delta_stride, const float* weight, void* out, int rows, int width,
                   int groups, float eps, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0 || groups <= 0 || width % groups || (delta != nullptr && delta_stride < width)) return DLI_ERR_ARGUMENT;
  if (groups > 65535) return DLI_ERR_ARGUMENT;
  const int part = width / groups, threads = part >= 2048 ? 512 : part >= 512 ? 256 : part >= 128 ? 128 : 64;
  const dim3 grid(rows, groups);
  if (is_bf16)
    group_norm_kernel<bf16_t><<<grid, threads, 0, stream>>>(x, delta, delta_stride, weight, (bf16_t*)out, width, groups, eps);
  else
    group_norm_kernel<float><<<grid, threads, 0, stream>>>(x, delta, delta_stride, weight, (float*)out, width, groups, eps);
  return dli_launch_status();
}

int dli_branch_norm_mean(const float* const* y, const int64_t* strides, const float* const* weights, int count, float* out,
                         int rows, int width, float eps, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0 || count < 1 || count > 4) return DLI_ERR_ARGUMENT;
  BranchArgs b;
  b.count = count;
  for (int j = 0; j < 4; ++j) {
    const int s = j < count ? j : 0;
    if (y[s] == nullptr || weights[s] == nullptr || strides[s] < width) return DLI_ERR_ARGUMENT;
    b.y[j] = y[s]; b.stride[j] = strides[s]; b.weight[j] = weights[s];
  }
  switch (count) {
    case 1: branch_norm_mean_kernel<1><<<rows, 256, 0, stream>>>(b, out, width, eps); break;
    case 2: branch_norm_mean_kernel<2><<<rows, 256, 0, stream>>>(b, out, width, eps); break;
    case 3: branch_norm_mean_kernel<3><<<rows, 256, 0, stream>>>(b, out, width, eps); break;
    default: branch_norm_mean_kernel<4><<<rows, 256, 0, stream>>>(b, out, width, eps);
  }
  return dli_launch_status();
}

int dli_diff_head_norm(const float* a, int64_t a_stride, float lambda, float after, float eps, const float* gate,
                       int64_t gate_stride, void* out, int64_t out_stride, int rows, int heads, int vdim, int is_bf16,
                       hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (heads <= 0 || vdim <= 0 || a_stride < (int64_t)2 * heads * vdim || out_stride < (int64_t)heads * vdim ||
      (gate != nullptr && gate_stride < heads))
    return DLI_ERR_ARGUMENT;
  const dim3 grid(rows, (heads + 3) / 4);
  if (grid.y > 65535) return DLI_ERR_ARGUMENT;
  if (is_bf16)
    diff_head_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>(a, a_stride, lambda, after, eps, gate, gate_stride, (bf16_t*)out,
                                                           out_stride, heads, vdim);
  else
    diff_head_norm_kernel<float><<<grid, 256, 0, stream>>>(a, a_stride, lambda, after, eps, gate, gate_stride, (float*)out,
                                                          out_stride, heads, vdim);
  return dli_launch_status();
}

int dli_branch_weighted_sum(const float* const* y, const int64_t* strides, const float* scales, int count, float* out,
                            int rows, int width, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (count < 1 || count > 4 || width <= 0) return DLI_ERR_ARGUMENT;
  WeightedBranches b;
  b.count = count;
  for (int j = 0; j < 4; ++j) {
    b.y[j] = j < count ? y[j] : nullptr;
    b.stride[j] = j < count ? strides[j] : 0;
    b.scale[j] = j < count ? scales[j] : 0.f;
    if (j < count && (y[j] == nullptr || strides[j] < width)) return DLI_ERR_ARGUMENT;
  }
  const dim3 grid(rows, (width + 255) / 256);
  if (grid.y > 65535) return DLI_ERR_ARGUMENT;
  branch_weighted_sum_kernel<<<grid, 256, 0, stream>>>(b, out, width);
  return dli_launch_status();
}

int dli_scale_f32(float* y, int64_t n, float scale, hipStream_t stream) {
  if (n <= 0) return DLI_OK;
  const int64_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffff) return DLI_ERR_ARGUMENT;
  scale_f32_kernel<<<(unsigned)blocks, 256, 0, stream>>>(y, n, scale);
  return dli_launch_status();
}

int dli_rms_norm_pair(const float* x, const float* w1, const float* w2, void* out1, void* out2, int rows, int width, float eps,
                      int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0) return DLI_ERR_ARGUMENT;
  const int threads = width >= 2048 ? 512 : 256;
  if (is_bf16)
    rms_norm_pair_kernel<bf16_t><<<rows, threads, 0, stream>>>(x, w1, w2, (bf16_t*)out1, (bf16_t*)out2, width, eps);
  else
    rms_norm_pair_kernel<float><<<rows, threads, 0, stream>>>(x, w1, w2, (float*)out1, (float*)out2, width, eps);
  return dli_launch_status();
}

int dli_add_pair_into_stream(float* x, const float* a, const float* b, int64_t n, hipStream_t stream) {
  if (n <= 0) return DLI_OK;
  const int64_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffff) return DLI_ERR_ARGUMENT;
  add_pair_into_stream_kernel<<<(unsigned)blocks, 256, 0, stream>>>(x, a, b, n);
  return dli_launch_status();
}

}  // extern "C"
