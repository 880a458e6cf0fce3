// What some mixers do with the attention's output before the output projection: the difference of two score maps'
// outputs brought to unit RMS per head, and a sigmoid gate per head.
#include "common.h"

#define AF_MAX_PER 4       // value heads of up to 256 elements: four a lane

// mixed: [n_tokens, n_heads * 2 * dv], laid out (kv head, map, head within the group, dv), `group` heads a kv head.
// out[t, h, :] = o / sqrt(mean(o^2) + eps) * out_scale with o = map 1 - lam[0] * map 2 of head h.  A wave a (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
differential_heads_kernel(const T* __restrict__ mixed, const float* __restrict__ lam, float eps, float out_scale,
                          int n_tokens, int n_heads, int group, int dv, T* __restrict__ out) {
  const int lane = threadIdx.x & (WAVE - 1);
  const long item = (long)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
  if (item >= (long)n_tokens * n_heads) return;
  const int t = (int)(item / n_heads), h = (int)(item % n_heads);
  const int g = h / group, j = h - g * group;
  const T* first = mixed + ((size_t)t * 2 * n_heads + (size_t)g * 2 * group + j) * dv;
  const T* second = first + (size_t)group * dv;
  const float factor = lam[0];
  float o[AF_MAX_PER], sq = 0.f;
#pragma unroll
  for (int r = 0; r < AF_MAX_PER; ++r) {
    const int i = lane + r * WAVE;
    o[r] = i < dv ? ld(first + i) - factor * ld(second + i) : 0.f;
    sq += o[r] * o[r];
  }
  const float inv = out_scale / sqrtf(wave_sum(sq) / (float)dv + eps);
  T* dst = out + ((size_t)t * n_heads + h) * dv;
#pragma unroll
  for (int r = 0; r < AF_MAX_PER; ++r) {
    const int i = lane + r * WAVE;
    if (i < dv) st(dst + i, o[r] * inv);
  }
}

// mixed[t, h, :] *= sigmoid(rows[t, offset + h]); rows has `row_stride` elements a token.
template <typename T>
__global__ void sigmoid_head_gate_kernel(T* __restrict__ mixed, const T* __restrict__ rows, int row_stride, int offset,
                                         int n_heads, int dv, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t th = idx / dv;
    const size_t t = th / n_heads;
    const int h = (int)(th - t * n_heads);
    const float z = ld(rows + t * row_stride + offset + h);
    st(mixed + idx, ld(mixed + idx) / (1.0f + expf(-z)));
  }
}

extern "C" int ta_differential_heads(const void* mixed, const void* lam, float eps, float out_scale, int n_tokens,
                                     int n_heads, int group, int dv, void* out, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (dv <= 0 || dv > AF_MAX_PER * WAVE || group <= 0 || n_heads % group) return -1;
  const long items = (long)n_tokens * n_heads;
  const int blocks = (int)((items + 3) / 4);
  if (dtype == DT_F32)
    differential_heads_kernel<float><<<blocks, 256, 0, stream>>>((const float*)mixed, (const float*)lam, eps, out_scale,
                                                                 n_tokens, n_heads, group, dv, (float*)out);
  else
    differential_heads_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)mixed, (const float*)lam, eps, out_scale,
                                                                  n_tokens, n_heads, group, dv, (bf16_t*)out);
  return LAUNCH_STATUS();
}

extern "C" int ta_sigmoid_head_gate(void* mixed, const void* rows, int row_stride, int offset, int n_tokens, int n_heads,
                                    int dv, int dtype, hipStream_t stream) {
  const size_t total = (size_t)n_tokens * n_heads * dv;
  if (total == 0) return 0;
  const int blocks = (int)((total + 255) / 256 < 65535 ? (total + 255) / 256 : 65535);
  if (dtype == DT_F32)
    sigmoid_head_gate_kernel<float><<<blocks, 256, 0, stream>>>((float*)mixed, (const float*)rows, row_stride, offset,
                                                                n_heads, dv, total);
  else
    sigmoid_head_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)mixed, (const bf16_t*)rows, row_stride, offset,
                                                                 n_heads, dv, total);
  return LAUNCH_STATUS();
}
