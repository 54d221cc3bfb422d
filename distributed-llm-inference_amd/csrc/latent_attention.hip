// Attention through a latent: what is cached per token is one normalised vector c of `rank` values, from
// which every head's keys and values are linear maps, k_h = U_h c and v_h = W_h c. The scores of head h are
// then (U_h^T q_h) . c and its result W_h (sum_j p_j c_j): the attention itself runs over the cached
// vectors as one shared kv head whose values are its keys, between two small products per head.
//
//   latent_norm_cache  from a step's 32-bit projections: the query's latent and the kv latent each
//                      divided by their root mean square and multiplied by a weight; the first goes out
//                      in T (the operand of the queries' product), the second into the token's cache
//                      slot, as a key (page [slot][rank]) and as a value (page [rank][slot])
//   head_products      out[t][h] = M_h x[t][h] for every head, M [heads][m][k]; optionally multiplied by
//                      sigmoid(gate) element by element. Every output sums its k in ascending order.
#include "common.h"

template <typename T>
__global__ void latent_norm_cache_kernel(const float* __restrict__ proj, int64_t stride, int q_off, int q_rank, int c_off,
                                         int rank, const float* __restrict__ q_weight, const float* __restrict__ c_weight,
                                         float eps, T* __restrict__ q_out, const int* __restrict__ slots,
                                         T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const float* pr = proj + row * stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) ss += pr[q_off + i] * pr[q_off + i];
  const float rq = 1.f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
    q_out[row * q_rank + i] = from_f32<T>(q_weight[i] * (pr[q_off + i] * rq));
  ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) ss += pr[c_off + i] * pr[c_off + i];
  const float rc = 1.f / sqrtf(block_sum(ss, scratch) / (float)rank + eps);
  const int slot = slots[row];
  if (slot < 0) return;                                // a padding row: nothing is cached
  const int64_t page = slot / page_size;
  const int off = slot % page_size;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const T c = from_f32<T>(c_weight[i] * (pr[c_off + i] * rc));
    k_pages[(page * page_size + off) * rank + i] = c;
    v_pages[(page * rank + i) * page_size + off] = c;
  }
}

#define HP_BM 16
#define HP_BN 64
#define HP_BK 32

// A workgroup: 16 rows x 64 outputs of one head; a thread one row and four outputs (tx, tx+16, ...).
template <typename T>
__global__ __launch_bounds__(256) void head_products_kernel(const T* __restrict__ x, int64_t x_stride,
                                                            const T* __restrict__ w, T* __restrict__ out,
                                                            int64_t out_stride, const float* __restrict__ gate,
                                                            int64_t gate_stride, int rows, int m, int k) {
  __shared__ float xs[HP_BM][HP_BK + 1];
  __shared__ float ws[HP_BN][HP_BK + 1];
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const int r0 = blockIdx.x * HP_BM, head = blockIdx.y, n0 = blockIdx.z * HP_BN;
  const T* wh = w + (int64_t)head * m * k;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < k; k0 += HP_BK) {
    __syncthreads();
    for (int idx = tid; idx < HP_BM * HP_BK; idx += 256) {
      const int r = idx / HP_BK, c = idx - r * HP_BK;
      xs[r][c] = (r0 + r < rows && k0 + c < k) ? to_f32(x[(int64_t)(r0 + r) * x_stride + (int64_t)head * k + k0 + c]) : 0.f;
    }
    for (int idx = tid; idx < HP_BN * HP_BK; idx += 256) {
      const int r = idx / HP_BK, c = idx - r * HP_BK;
      ws[r][c] = (n0 + r < m && k0 + c < k) ? to_f32(wh[(int64_t)(n0 + r) * k + k0 + c]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < HP_BK; ++c) {
      const float a = xs[ty][c];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = fmaf(a, ws[tx + 16 * j][c], acc[j]);
    }
  }
  const int r = r0 + ty;
  if (r >= rows) return;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + tx + 16 * j;
    if (n >= m) continue;
    float y = acc[j];
    const int64_t at = (int64_t)head * m + n;
    if (gate != nullptr) y *= 1.f / (1.f + expf(-gate[(int64_t)r * gate_stride + at]));
    out[(int64_t)r * out_stride + at] = from_f32<T>(y);
  }
}

extern "C" {

int dli_latent_norm_cache(const float* proj, int64_t stride, int q_off, int q_rank, int c_off, int rank,
                          const float* q_weight, const float* c_weight, float eps, void* q_out, const int* slots,
                          void* k_pages, void* v_pages, int rows, int page_size, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (q_rank <= 0 || rank <= 0 || page_size <= 0 || q_off < 0 || c_off < 0 || q_off + q_rank > stride ||
      c_off + rank > stride)
    return DLI_ERR_ARGUMENT;
  const int widest = q_rank > rank ? q_rank : rank;
  const int threads = widest >= 1024 ? 256 : widest >= 256 ? 128 : 64;
  if (is_bf16)
    latent_norm_cache_kernel<bf16_t><<<rows, threads, 0, stream>>>(proj, stride, q_off, q_rank, c_off, rank, q_weight,
                                                                   c_weight, eps, (bf16_t*)q_out, slots, (bf16_t*)k_pages,
                                                                   (bf16_t*)v_pages, page_size);
  else
    latent_norm_cache_kernel<float><<<rows, threads, 0, stream>>>(proj, stride, q_off, q_rank, c_off, rank, q_weight,
                                                                  c_weight, eps, (float*)q_out, slots, (float*)k_pages,
                                                                  (float*)v_pages, page_size);
  return dli_launch_status();
}

int dli_head_products(const void* x, int64_t x_stride, const void* w, void* out, int64_t out_stride, const float* gate,
                      int64_t gate_stride, int rows, int heads, int m, int k, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (heads <= 0 || heads > 65535 || m <= 0 || k <= 0 || x_stride < (int64_t)heads * k || out_stride < (int64_t)heads * m ||
      (gate != nullptr && gate_stride < (int64_t)heads * m))
    return DLI_ERR_ARGUMENT;
  const dim3 grid((rows + HP_BM - 1) / HP_BM, heads, (m + HP_BN - 1) / HP_BN);
  if (grid.z > 65535) return DLI_ERR_ARGUMENT;
  if (is_bf16)
    head_products_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, (const bf16_t*)w, (bf16_t*)out,
                                                           out_stride, gate, gate_stride, rows, m, k);
  else
    head_products_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, (const float*)w, (float*)out,
                                                          out_stride, gate, gate_stride, rows, m, k);
  return dli_launch_status();
}

}  // extern "C"
