// What stands between the joined q/k/v projection and the attention, for mixers whose rotation covers only the first
// coordinates of a head: bias, an RMS norm over all query rows at once and over all key rows at once, the rotation
// with angles formed in the kernel, and the write of keys and values into their pages.  A workgroup a token.
#include "common.h"

#define RP_THREADS 256
#define RP_MAX_HALF 128

// qkv: [n_tokens, row_stride]; a row holds n_q query heads and n_k key heads of d elements, then n_v value heads of dv
// elements (what lies behind them is not touched).  bias (float, or null) is added first.  q_norm / k_norm (float
// [n_q d] / [n_k d], or null): the query part (the key part) is divided by its root mean square over all its
// elements (eps inside the root) and multiplied by the weight.  rates (float [rot / 2]): coordinates i and
// i + rot / 2 of every query and key head turn by the angle position * rates[i], formed and taken sine and cosine of
// in float; coordinates from rot on pass.  slots (or null): page * page_size + offset of each token, negative =
// nothing is stored.  Key pages [n_pages, n_k, page_size, d]; value pages transposed inside a page,
// [n_pages, n_v, dv, page_size].
template <typename T>
__global__ void __launch_bounds__(RP_THREADS)
norm_rotate_store_kernel(T* __restrict__ qkv, int row_stride, const float* __restrict__ bias,
                         const int* __restrict__ positions, const float* __restrict__ rates, int rot,
                         const int* __restrict__ slots, T* __restrict__ k_pages, T* __restrict__ v_pages,
                         int n_q, int n_k, int n_v, int d, int dv, int page_size,
                         const float* __restrict__ q_norm, const float* __restrict__ k_norm, float eps) {
  __shared__ float scratch[16];
  __shared__ float cos_s[RP_MAX_HALF], sin_s[RP_MAX_HALF];
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * row_stride;
  const int q_size = n_q * d, k_size = n_k * d, half = rot / 2;
  const int slot = slots ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  if (half > 0) {
    const float position = (float)positions[t];
    for (int i = threadIdx.x; i < half; i += RP_THREADS) {
      float s, c;
      sincosf(position * rates[i], &s, &c);
      cos_s[i] = c;
      sin_s[i] = s;
    }
  }
  float inv_q = 1.f, inv_k = 1.f;
  if (q_norm) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < q_size; i += RP_THREADS) {
      const float v = ld(row + i) + (bias ? bias[i] : 0.f);
      sq += v * v;
    }
    inv_q = 1.0f / sqrtf(block_sum(sq, scratch) / (float)q_size + eps);
  }
  if (k_norm && k_size > 0) {
    float sq = 0.f;
    for (int i = threadIdx.x; i < k_size; i += RP_THREADS) {
      const float v = ld(row + q_size + i) + (bias ? bias[q_size + i] : 0.f);
      sq += v * v;
    }
    inv_k = 1.0f / sqrtf(block_sum(sq, scratch) / (float)k_size + eps);
  }
  __syncthreads();
  const bool changes = bias || q_norm || k_norm;
  // The pairs that turn.
  for (int idx = threadIdx.x; idx < (n_q + n_k) * half; idx += RP_THREADS) {
    const int head = idx / half, i = idx - head * half;
    const int at = head * d + i, with = at + half;
    float a = ld(row + at), b = ld(row + with);
    if (bias) { a += bias[at]; b += bias[with]; }
    const bool key = head >= n_q;
    if (!key && q_norm) { a *= inv_q * q_norm[at]; b *= inv_q * q_norm[with]; }
    if (key && k_norm) { a *= inv_k * k_norm[at - q_size]; b *= inv_k * k_norm[with - q_size]; }
    const float c = cos_s[i], s = sin_s[i];
    const float r1 = a * c - b * s, r2 = b * c + a * s;
    st(row + at, r1);
    st(row + with, r2);
    if (key && slot >= 0) {
      T* dst = k_pages + (((size_t)page * n_k + (head - n_q)) * page_size + off) * d;
      st(dst + i, r1);
      st(dst + half + i, r2);
    }
  }
  // The coordinates that pass.
  const int rest = d - rot;
  for (int idx = threadIdx.x; idx < (n_q + n_k) * rest; idx += RP_THREADS) {
    const int head = idx / rest, i = rot + (idx - head * rest);
    const int at = head * d + i;
    float a = ld(row + at);
    if (bias) a += bias[at];
    const bool key = head >= n_q;
    if (!key && q_norm) a *= inv_q * q_norm[at];
    if (key && k_norm) a *= inv_k * k_norm[at - q_size];
    if (changes) st(row + at, a);
    if (key && slot >= 0) {
      if (changes) a = ld(row + at);           // the page holds what the row holds, rounded the same way
      st(k_pages + (((size_t)page * n_k + (head - n_q)) * page_size + off) * d + i, a);
    }
  }
  // Values.
  const int v_at = q_size + k_size;
  for (int idx = threadIdx.x; idx < n_v * dv; idx += RP_THREADS) {
    float a = ld(row + v_at + idx);
    if (bias) { a += bias[v_at + idx]; st(row + v_at + idx, a); }
    if (slot >= 0) {
      const int head = idx / dv, i = idx - head * dv;
      st(v_pages + (((size_t)page * n_v + head) * dv + i) * page_size + off, a);
    }
  }
}

extern "C" int ta_norm_rotate_store(void* qkv, int row_stride, const void* bias, const void* positions, const void* rates,
                                    int rot, const void* slots, void* k_pages, void* v_pages, int n_tokens, int n_q,
                                    int n_k, int n_v, int d, int dv, int page_size, const void* q_norm,
                                    const void* k_norm, float eps, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (rot < 0 || rot % 2 || rot > d || rot / 2 > RP_MAX_HALF || d <= 0 || dv <= 0 || n_q < 0 || n_k < 0 || n_v < 0) return -1;
  if (rot > 0 && !rates) return -1;
  if (dtype == DT_F32)
    norm_rotate_store_kernel<float><<<n_tokens, RP_THREADS, 0, stream>>>(
        (float*)qkv, row_stride, (const float*)bias, (const int*)positions, (const float*)rates, rot, (const int*)slots,
        (float*)k_pages, (float*)v_pages, n_q, n_k, n_v, d, dv, page_size, (const float*)q_norm, (const float*)k_norm, eps);
  else
    norm_rotate_store_kernel<bf16_t><<<n_tokens, RP_THREADS, 0, stream>>>(
        (bf16_t*)qkv, row_stride, (const float*)bias, (const int*)positions, (const float*)rates, rot, (const int*)slots,
        (bf16_t*)k_pages, (bf16_t*)v_pages, n_q, n_k, n_v, d, dv, page_size, (const float*)q_norm, (const float*)k_norm, eps);
  return LAUNCH_STATUS();
}
