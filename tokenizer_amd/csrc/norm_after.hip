// Norms that stand behind a sub-layer: the sub-layer's output is brought to unit RMS, scaled by a weight and added
// to the float residual stream, and the sum is normalised for the next sub-layer, all in one kernel (a row a
// workgroup; sums of squares, the stream and both norms in float).
#include "common.h"

#define NA_THREADS 256
#define NA_PER 16          // floats of a row that a thread keeps (rows of up to NA_THREADS * NA_PER elements)

__device__ __forceinline__ void na_store(float* p, float v) { *p = v; }
__device__ __forceinline__ void na_store(bf16_t* p, float v) { p->bits = float_to_bf16_bits(v); }

// residual: float [*, hidden].  delta (TD [*, hidden], or null): what is added to the stream; with `post_weight`
// (float [hidden]) it is first divided by its root mean square (post_eps inside the root) and multiplied by it.
// rows (or null): the rows to work on (row i of `out` is row rows[i] of the others); store_residual: the sum goes
// back into the stream.  weight (float [hidden], or null): out = sum / rms(sum) * weight; null: out = the sum.
template <typename TD, typename TO>
__global__ void __launch_bounds__(NA_THREADS)
norm_add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta, const float* __restrict__ post_weight,
                        float post_eps, const float* __restrict__ weight, float eps, TO* __restrict__ out,
                        const int* __restrict__ rows, int hidden, int store_residual) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* res = residual + (size_t)r * hidden;
  const TD* del = delta ? delta + (size_t)r * hidden : nullptr;
  float x[NA_PER], d[NA_PER];
#pragma unroll
  for (int c = 0; c < NA_PER; ++c) {
    const int h = c * NA_THREADS + threadIdx.x;
    x[c] = h < hidden ? res[h] : 0.f;
    d[c] = (del && h < hidden) ? ld(del + h) : 0.f;
  }
  if (del) {
    if (post_weight) {
      float sq = 0.f;
#pragma unroll
      for (int c = 0; c < NA_PER; ++c) sq += d[c] * d[c];
      const float inv = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + post_eps);
#pragma unroll
      for (int c = 0; c < NA_PER; ++c) {
        const int h = c * NA_THREADS + threadIdx.x;
        if (h < hidden) d[c] = d[c] * inv * post_weight[h];
      }
    }
#pragma unroll
    for (int c = 0; c < NA_PER; ++c) {
      const int h = c * NA_THREADS + threadIdx.x;
      x[c] += d[c];
      if (store_residual && h < hidden) res[h] = x[c];
    }
  }
  float inv = 1.f;
  if (weight) {
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < NA_PER; ++c) sq += x[c] * x[c];
    inv = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps);
  }
  TO* dst = out + (size_t)i * hidden;
#pragma unroll
  for (int c = 0; c < NA_PER; ++c) {
    const int h = c * NA_THREADS + threadIdx.x;
    if (h < hidden) na_store(dst + h, weight ? x[c] * inv * weight[h] : x[c]);
  }
}

// Rows longer than a workgroup's registers hold: the same sums, with the row read again from memory for every pass.
template <typename TD, typename TO>
__global__ void __launch_bounds__(NA_THREADS)
norm_add_rmsnorm_long_kernel(float* __restrict__ residual, const TD* __restrict__ delta, const float* __restrict__ post_weight,
                             float post_eps, const float* __restrict__ weight, float eps, TO* __restrict__ out,
                             const int* __restrict__ rows, int hidden, int store_residual) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* res = residual + (size_t)r * hidden;
  const TD* del = delta ? delta + (size_t)r * hidden : nullptr;
  float inv_d = 1.f;
  if (del && post_weight) {
    float sq = 0.f;
    for (int h = threadIdx.x; h < hidden; h += NA_THREADS) { const float v = ld(del + h); sq += v * v; }
    inv_d = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + post_eps);
  }
  float sq = 0.f;
  for (int h = threadIdx.x; h < hidden; h += NA_THREADS) {
    float v = res[h];
    if (del) v += post_weight ? ld(del + h) * inv_d * post_weight[h] : ld(del + h);
    sq += v * v;
  }
  const float inv = weight ? 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps) : 1.f;
  TO* dst = out + (size_t)i * hidden;
  for (int h = threadIdx.x; h < hidden; h += NA_THREADS) {
    float v = res[h];
    if (del) {
      v += post_weight ? ld(del + h) * inv_d * post_weight[h] : ld(del + h);
      if (store_residual) res[h] = v;
    }
    na_store(dst + h, weight ? v * inv * weight[h] : v);
  }
}

// delta_dtype, out_dtype: DT_F32 or DT_BF16 (a bfloat16 delta with a float result serves whoever wants the
// normalised term by itself).
extern "C" int ta_norm_add_rmsnorm(void* residual, const void* delta, const void* post_weight, float post_eps,
                                   const void* weight, float eps, void* out, const void* rows, int n_rows, int hidden,
                                   int store_residual, int delta_dtype, int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (hidden <= 0) return -1;
  const bool fits = hidden <= NA_THREADS * NA_PER;
#define GO(TD, TO)                                                                                                     \
  do {                                                                                                                 \
    if (fits)                                                                                                          \
      norm_add_rmsnorm_kernel<TD, TO><<<n_rows, NA_THREADS, 0, stream>>>(                                              \
          (float*)residual, (const TD*)delta, (const float*)post_weight, post_eps, (const float*)weight, eps, (TO*)out, \
          (const int*)rows, hidden, store_residual);                                                                   \
    else                                                                                                               \
      norm_add_rmsnorm_long_kernel<TD, TO><<<n_rows, NA_THREADS, 0, stream>>>(                                         \
          (float*)residual, (const TD*)delta, (const float*)post_weight, post_eps, (const float*)weight, eps, (TO*)out, \
          (const int*)rows, hidden, store_residual);                                                                   \
  } while (0)
  if (delta_dtype == DT_F32 && out_dtype == DT_F32) GO(float, float);
  else if (delta_dtype == DT_BF16 && out_dtype == DT_BF16) GO(bf16_t, bf16_t);
  else if (delta_dtype == DT_BF16 && out_dtype == DT_F32) GO(bf16_t, float);
  else return -1;
#undef GO
  return LAUNCH_STATUS();
}
