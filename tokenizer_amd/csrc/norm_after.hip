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
  // Everything a thread needs of the rows and the two weights is asked for at the start: one trip to memory.
  float x[NA_PER], d[NA_PER], behind_w[NA_PER], next_w[NA_PER];
#pragma unroll
  for (int c = 0; c < NA_PER; ++c) {
    const int h = c * NA_THREADS + threadIdx.x;
    const bool in = h < hidden;
    x[c] = in ? res[h] : 0.f;
    d[c] = (del && in) ? ld(del + h) : 0.f;
    behind_w[c] = (del && post_weight && in) ? post_weight[h] : 1.f;
    next_w[c] = (weight && in) ? weight[h] : 1.f;
  }
  if (del) {
    if (post_weight) {
      float sq = 0.f;
#pragma unroll
      for (int c = 0; c < NA_PER; ++c) sq += d[c] * d[c];
      const float inv = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + post_eps);
#pragma unroll
      for (int c = 0; c < NA_PER; ++c) d[c] *= inv * behind_w[c];
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
    if (h < hidden) na_store(dst + h, x[c] * inv * next_w[c]);
  }
}

// Four consecutive elements of a row as floats, and back.
__device__ __forceinline__ float4 na_ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 na_ld4(const bf16_t* p) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  return make_float4(bf16_bits_to_float(raw.x & 0xffffu), bf16_bits_to_float(raw.x >> 16),
                     bf16_bits_to_float(raw.y & 0xffffu), bf16_bits_to_float(raw.y >> 16));
}
__device__ __forceinline__ void na_st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void na_st4(bf16_t* p, float4 v) {
  uint2 raw;
  raw.x = (uint32_t)float_to_bf16_bits(v.x) | ((uint32_t)float_to_bf16_bits(v.y) << 16);
  raw.y = (uint32_t)float_to_bf16_bits(v.z) | ((uint32_t)float_to_bf16_bits(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = raw;
}
__device__ __forceinline__ float na_sq4(float4 v) { return v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w; }

// The same for rows whose length is a multiple of 4, up to CHUNKS * 1,024 elements: a thread takes four consecutive
// elements of each run of 1,024, so the rows and weights move sixteen bytes a load (eight for bfloat16); a thread
// past the row's end asks for the row's last elements and does not use them, so that no load stands behind a condition.
template <typename TD, typename TO, int CHUNKS, bool DELTA, bool POST, bool NEXT>
__global__ void __launch_bounds__(NA_THREADS)
norm_add_rmsnorm_vec_kernel(float* __restrict__ residual, const TD* __restrict__ delta, const float* __restrict__ post_weight,
                            float post_eps, const float* __restrict__ weight, float eps, TO* __restrict__ out,
                            const int* __restrict__ rows, int hidden, int store_residual) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* res = residual + (size_t)r * hidden;
  const TD* del = delta + (size_t)r * hidden;
  float4 x[CHUNKS], d[CHUNKS], behind_w[CHUNKS], next_w[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = min((c * NA_THREADS + (int)threadIdx.x) * 4, hidden - 4);
    x[c] = na_ld4(res + h);
    if (DELTA) d[c] = na_ld4(del + h);
    if (DELTA && POST) behind_w[c] = na_ld4(post_weight + h);
    if (NEXT) next_w[c] = na_ld4(weight + h);
  }
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  if (DELTA) {
    float inv = 1.f;
    if (POST) {
      float sq = 0.f;
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c)
        if ((c * NA_THREADS + (int)threadIdx.x) * 4 < hidden) sq += na_sq4(d[c]);
      inv = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + post_eps);
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int h = (c * NA_THREADS + (int)threadIdx.x) * 4;
      if (POST) {
        x[c].x += d[c].x * inv * behind_w[c].x; x[c].y += d[c].y * inv * behind_w[c].y;
        x[c].z += d[c].z * inv * behind_w[c].z; x[c].w += d[c].w * inv * behind_w[c].w;
      } else {
        x[c].x += d[c].x; x[c].y += d[c].y; x[c].z += d[c].z; x[c].w += d[c].w;
      }
      if (store_residual && h < hidden) na_st4(res + h, x[c]);
    }
  }
  float inv = 1.f;
  if (NEXT) {
    float sq = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
      if ((c * NA_THREADS + (int)threadIdx.x) * 4 < hidden) sq += na_sq4(x[c]);
    inv = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps);
  }
  TO* dst = out + (size_t)i * hidden;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = (c * NA_THREADS + (int)threadIdx.x) * 4;
    if (h >= hidden) continue;
    if (NEXT) na_st4(dst + h, make_float4(x[c].x * inv * next_w[c].x, x[c].y * inv * next_w[c].y, x[c].z * inv * next_w[c].z,
                                          x[c].w * inv * next_w[c].w));
    else na_st4(dst + h, x[c]);
  }
  (void)zero;
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

#define NA_MAX_SIDE 64     // the widest per-layer token input the fused kernel takes

__device__ __forceinline__ float na_gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// The same with a token input between the two norms: with x the stream after the first add,
//   g[j] = gelu_tanh(gate[j, :] . x) * table[token, offset + j]  (j < dim),  y = proj g,
//   x += y / sqrt(mean(y^2) + side_eps) * side_norm,
// and then the norm before the next sub-layer.  gate [>= dim, hidden], proj [hidden, proj_stride] (its first dim
// columns count), table [vocab, table_width] and delta have the type T; the stream, the dot products and the norms are float.
template <typename T>
__global__ void __launch_bounds__(NA_THREADS)
norm_side_norm_kernel(float* __restrict__ residual, const T* __restrict__ delta, const float* __restrict__ post_weight,
                      float post_eps, const T* __restrict__ gate, const T* __restrict__ proj, int proj_stride,
                      const float* __restrict__ side_norm, float side_eps, const T* __restrict__ table, int table_width,
                      const int* __restrict__ token_ids, int offset, int dim, const float* __restrict__ weight, float eps,
                      T* __restrict__ out, const int* __restrict__ rows, int hidden, int store_residual) {
  __shared__ float scratch[16];
  __shared__ float part_s[NA_THREADS / WAVE][NA_MAX_SIDE];
  __shared__ float g_s[NA_MAX_SIDE];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  float* res = residual + (size_t)r * hidden;
  const T* del = delta ? delta + (size_t)r * hidden : nullptr;
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
    for (int c = 0; c < NA_PER; ++c) x[c] += d[c];
  }
  // The gate's dot products: every thread's share of each, summed over the wave, then over the waves through LDS.
  const int chunks = (hidden + NA_THREADS - 1) / NA_THREADS;
  for (int j = 0; j < dim; ++j) {
    const T* row = gate + (size_t)j * hidden;
    float part = 0.f;
#pragma unroll
    for (int c = 0; c < NA_PER; ++c) {
      const int h = c * NA_THREADS + threadIdx.x;
      if (c < chunks && h < hidden) part = fmaf(ld(row + h), x[c], part);
    }
    part = wave_sum(part);
    if (lane == 0) part_s[wave][j] = part;
  }
  __syncthreads();
  if (threadIdx.x < dim) {
    float z = 0.f;
#pragma unroll
    for (int w = 0; w < NA_THREADS / WAVE; ++w) z += part_s[w][threadIdx.x];
    g_s[threadIdx.x] = na_gelu_tanh(z) * ld(table + (size_t)token_ids[r] * table_width + offset + threadIdx.x);
  }
  __syncthreads();
  float y[NA_PER], sq = 0.f;
#pragma unroll
  for (int c = 0; c < NA_PER; ++c) {
    const int h = c * NA_THREADS + threadIdx.x;
    y[c] = 0.f;
    if (c < chunks && h < hidden) {
      const T* row = proj + (size_t)h * proj_stride;
      float sum = 0.f;
      for (int j = 0; j < dim; ++j) sum = fmaf(ld(row + j), g_s[j], sum);
      y[c] = sum;
    }
    sq += y[c] * y[c];
  }
  const float inv_y = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + side_eps);
  sq = 0.f;
#pragma unroll
  for (int c = 0; c < NA_PER; ++c) {
    const int h = c * NA_THREADS + threadIdx.x;
    if (h < hidden) {
      x[c] += y[c] * inv_y * side_norm[h];
      if (store_residual) res[h] = x[c];
    }
    sq += x[c] * x[c];
  }
  float inv = 1.f;
  if (weight) inv = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps);
  T* dst = out + (size_t)i * hidden;
#pragma unroll
  for (int c = 0; c < NA_PER; ++c) {
    const int h = c * NA_THREADS + threadIdx.x;
    if (h < hidden) st(dst + h, weight ? x[c] * inv * weight[h] : x[c]);
  }
}

// Sixteen bytes of a row as floats: eight bfloat16 or four float elements.
template <typename T> struct NaVec;
template <> struct NaVec<bf16_t> {
  static constexpr int N = 8;
  __device__ static __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const uint4 raw = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(w[i] << 16); v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
  }
};
template <> struct NaVec<float> {
  static constexpr int N = 4;
  __device__ static __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 raw = *reinterpret_cast<const float4*>(p);
    v[0] = raw.x; v[1] = raw.y; v[2] = raw.z; v[3] = raw.w;
  }
};

#define NA_SIDE_PER_WAVE (NA_MAX_SIDE / (NA_THREADS / WAVE))

// The same for rows, token inputs and projections in whole pieces of sixteen bytes (hidden, dim and proj_stride
// multiples of 8 for bfloat16, of 4 for float), rows of up to CHUNKS * 1,024 elements.  A thread takes four consecutive
// elements of each run of 1,024; the stream after the first add goes through LDS; wave w forms the gate's dot
// products j = w, w + 4, ..., sixteen bytes of each row a lane and step, all rows of a step asked for at once; the
// projection's rows are read the same way, all of a thread's rows a step.
template <typename T, int CHUNKS>
__global__ void __launch_bounds__(NA_THREADS)
norm_side_norm_vec_kernel(float* __restrict__ residual, const T* __restrict__ delta, const float* __restrict__ post_weight,
                          float post_eps, const T* __restrict__ gate, const T* __restrict__ proj, int proj_stride,
                          const float* __restrict__ side_norm, float side_eps, const T* __restrict__ table, int table_width,
                          const int* __restrict__ token_ids, int offset, int dim, const float* __restrict__ weight, float eps,
                          T* __restrict__ out, const int* __restrict__ rows, int hidden, int store_residual) {
  constexpr int N = NaVec<T>::N;
  __shared__ float scratch[16];
  __shared__ float x_s[CHUNKS * 1024];
  __shared__ float g_s[NA_MAX_SIDE];
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  float* res = residual + (size_t)r * hidden;
  const T* del = delta ? delta + (size_t)r * hidden : nullptr;
  // The token's slice of the table is asked for now; it is used behind the dot products.
  float e = 0.f;
  if (threadIdx.x < dim) e = ld(table + (size_t)token_ids[r] * table_width + offset + threadIdx.x);
  // Everything a thread needs of the rows and the three weights is asked for at the start.
  float4 x[CHUNKS], d[CHUNKS], behind_w[CHUNKS], tail_w[CHUNKS], next_w[CHUNKS];
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f), one = make_float4(1.f, 1.f, 1.f, 1.f);
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = min((c * NA_THREADS + (int)threadIdx.x) * 4, hidden - 4);
    x[c] = na_ld4(res + h);
    d[c] = del ? na_ld4(del + h) : zero;
    behind_w[c] = (del && post_weight) ? na_ld4(post_weight + h) : one;
    tail_w[c] = na_ld4(side_norm + h);
    next_w[c] = weight ? na_ld4(weight + h) : one;
  }
  if (del) {
    float inv = 1.f;
    if (post_weight) {
      float sq = 0.f;
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c)
        if ((c * NA_THREADS + (int)threadIdx.x) * 4 < hidden) sq += na_sq4(d[c]);
      inv = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + post_eps);
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      x[c].x += d[c].x * inv * behind_w[c].x; x[c].y += d[c].y * inv * behind_w[c].y;
      x[c].z += d[c].z * inv * behind_w[c].z; x[c].w += d[c].w * inv * behind_w[c].w;
    }
  }
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = (c * NA_THREADS + (int)threadIdx.x) * 4;
    if (h < hidden) *reinterpret_cast<float4*>(x_s + h) = x[c];
  }
  __syncthreads();
  float acc[NA_SIDE_PER_WAVE];
#pragma unroll
  for (int jj = 0; jj < NA_SIDE_PER_WAVE; ++jj) acc[jj] = 0.f;
  for (int at = lane * N; at < hidden; at += WAVE * N) {
    float xv[N];
#pragma unroll
    for (int k = 0; k < N; ++k) xv[k] = x_s[at + k];
#pragma unroll
    for (int jj = 0; jj < NA_SIDE_PER_WAVE; ++jj) {
      const int j = wave + (NA_THREADS / WAVE) * jj;
      if (j < dim) {
        float gv[N];
        NaVec<T>::load(gate + (size_t)j * hidden + at, gv);
#pragma unroll
        for (int k = 0; k < N; ++k) acc[jj] = fmaf(gv[k], xv[k], acc[jj]);
      }
    }
  }
#pragma unroll
  for (int jj = 0; jj < NA_SIDE_PER_WAVE; ++jj) {
    const int j = wave + (NA_THREADS / WAVE) * jj;
    const float z = wave_sum(acc[jj]);
    if (lane == 0 && j < dim) g_s[j] = z;
  }
  __syncthreads();
  if (threadIdx.x < dim) g_s[threadIdx.x] = na_gelu_tanh(g_s[threadIdx.x]) * e;
  __syncthreads();
  float y[CHUNKS][4];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
    for (int q = 0; q < 4; ++q) y[c][q] = 0.f;
  for (int at = 0; at < dim; at += N) {
    float gv[N];
#pragma unroll
    for (int k = 0; k < N; ++k) gv[k] = g_s[at + k];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      const int h = min((c * NA_THREADS + (int)threadIdx.x) * 4, hidden - 4);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float pv[N];
        NaVec<T>::load(proj + (size_t)(h + q) * proj_stride + at, pv);
#pragma unroll
        for (int k = 0; k < N; ++k) y[c][q] = fmaf(pv[k], gv[k], y[c][q]);
      }
    }
  }
  float sq = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c)
    if ((c * NA_THREADS + (int)threadIdx.x) * 4 < hidden)
      sq += y[c][0] * y[c][0] + y[c][1] * y[c][1] + y[c][2] * y[c][2] + y[c][3] * y[c][3];
  const float inv_y = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + side_eps);
  sq = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = (c * NA_THREADS + (int)threadIdx.x) * 4;
    x[c].x += y[c][0] * inv_y * tail_w[c].x; x[c].y += y[c][1] * inv_y * tail_w[c].y;
    x[c].z += y[c][2] * inv_y * tail_w[c].z; x[c].w += y[c][3] * inv_y * tail_w[c].w;
    if (h < hidden) {
      if (store_residual) na_st4(res + h, x[c]);
      sq += na_sq4(x[c]);
    }
  }
  float inv = 1.f;
  if (weight) inv = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps);
  T* dst = out + (size_t)i * hidden;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int h = (c * NA_THREADS + (int)threadIdx.x) * 4;
    if (h >= hidden) continue;
    na_st4(dst + h, make_float4(x[c].x * inv * next_w[c].x, x[c].y * inv * next_w[c].y, x[c].z * inv * next_w[c].z,
                                x[c].w * inv * next_w[c].w));
  }
}

// dtype: of delta, gate, proj, table and out.  Returns -2 for sizes the fused kernel does not take (rows longer than
// a workgroup holds, a wider token input): the caller then runs the steps one by one.
extern "C" int ta_norm_side_norm(void* residual, const void* delta, const void* post_weight, float post_eps, const void* gate,
                                 const void* proj, int proj_stride, const void* side_norm, float side_eps, const void* table,
                                 int table_width, const void* token_ids, int offset, int dim, const void* weight, float eps,
                                 void* out, const void* rows, int n_rows, int hidden, int store_residual, int dtype,
                                 hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (hidden <= 0 || hidden > NA_THREADS * NA_PER || dim <= 0 || dim > NA_MAX_SIDE) return -2;
  if (offset < 0 || offset + dim > table_width || proj_stride < dim) return -1;
  const int piece = dtype == DT_F32 ? 4 : 8;
  if (hidden % piece == 0 && dim % piece == 0 && proj_stride % piece == 0 &&
      (((uintptr_t)gate | (uintptr_t)proj | (uintptr_t)residual | (uintptr_t)delta | (uintptr_t)post_weight |
        (uintptr_t)side_norm | (uintptr_t)weight | (uintptr_t)out) & 15) == 0) {
#define SIDE(TT, CH)                                                                                                   \
    norm_side_norm_vec_kernel<TT, CH><<<n_rows, NA_THREADS, 0, stream>>>(                                               \
        (float*)residual, (const TT*)delta, (const float*)post_weight, post_eps, (const TT*)gate, (const TT*)proj,      \
        proj_stride, (const float*)side_norm, side_eps, (const TT*)table, table_width, (const int*)token_ids, offset,   \
        dim, (const float*)weight, eps, (TT*)out, (const int*)rows, hidden, store_residual)
    if (dtype == DT_F32) { if (hidden <= 1024) SIDE(float, 1); else if (hidden <= 2048) SIDE(float, 2); else SIDE(float, 4); }
    else { if (hidden <= 1024) SIDE(bf16_t, 1); else if (hidden <= 2048) SIDE(bf16_t, 2); else SIDE(bf16_t, 4); }
#undef SIDE
    return LAUNCH_STATUS();
  }
  if (dtype == DT_F32)
    norm_side_norm_kernel<float><<<n_rows, NA_THREADS, 0, stream>>>(
        (float*)residual, (const float*)delta, (const float*)post_weight, post_eps, (const float*)gate, (const float*)proj,
        proj_stride, (const float*)side_norm, side_eps, (const float*)table, table_width, (const int*)token_ids, offset, dim,
        (const float*)weight, eps, (float*)out, (const int*)rows, hidden, store_residual);
  else
    norm_side_norm_kernel<bf16_t><<<n_rows, NA_THREADS, 0, stream>>>(
        (float*)residual, (const bf16_t*)delta, (const float*)post_weight, post_eps, (const bf16_t*)gate, (const bf16_t*)proj,
        proj_stride, (const float*)side_norm, side_eps, (const bf16_t*)table, table_width, (const int*)token_ids, offset, dim,
        (const float*)weight, eps, (bf16_t*)out, (const int*)rows, hidden, store_residual);
  return LAUNCH_STATUS();
}

// delta_dtype, out_dtype: DT_F32 or DT_BF16 (a bfloat16 delta with a float result serves whoever wants the
// normalised term by itself).
extern "C" int ta_norm_add_rmsnorm(void* residual, const void* delta, const void* post_weight, float post_eps,
                                   const void* weight, float eps, void* out, const void* rows, int n_rows, int hidden,
                                   int store_residual, int delta_dtype, int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (hidden <= 0) return -1;
  const bool fits = hidden <= NA_THREADS * NA_PER;
  const bool aligned = (((uintptr_t)residual | (uintptr_t)delta | (uintptr_t)post_weight | (uintptr_t)weight | (uintptr_t)out) & 15) == 0;
  if (fits && hidden % 4 == 0 && hidden >= 4 && aligned) {
#define VEC3(TD, TO, CH, DD, PP, NN)                                                                                   \
    norm_add_rmsnorm_vec_kernel<TD, TO, CH, DD, PP, NN><<<n_rows, NA_THREADS, 0, stream>>>(                             \
        (float*)residual, (const TD*)delta, (const float*)post_weight, post_eps, (const float*)weight, eps, (TO*)out,   \
        (const int*)rows, hidden, store_residual)
#define VEC2(TD, TO, CH)                                                                                               \
    do {                                                                                                               \
      if (delta && post_weight) { if (weight) VEC3(TD, TO, CH, true, true, true); else VEC3(TD, TO, CH, true, true, false); } \
      else if (delta) { if (weight) VEC3(TD, TO, CH, true, false, true); else VEC3(TD, TO, CH, true, false, false); }   \
      else { if (weight) VEC3(TD, TO, CH, false, false, true); else VEC3(TD, TO, CH, false, false, false); }            \
    } while (0)
#define VEC1(TD, TO)                                                                                                   \
    do {                                                                                                               \
      if (hidden <= 1024) VEC2(TD, TO, 1); else if (hidden <= 2048) VEC2(TD, TO, 2); else VEC2(TD, TO, 4);              \
    } while (0)
    if (delta_dtype == DT_F32 && out_dtype == DT_F32) VEC1(float, float);
    else if (delta_dtype == DT_BF16 && out_dtype == DT_BF16) VEC1(bf16_t, bf16_t);
    else if (delta_dtype == DT_BF16 && out_dtype == DT_F32) VEC1(bf16_t, float);
    else return -1;
#undef VEC1
#undef VEC2
#undef VEC3
    return LAUNCH_STATUS();
  }
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
