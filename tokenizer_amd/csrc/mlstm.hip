// Matrix-memory recurrence (mLSTM) over a batch of portions, with the state of every request in its slot, and the
// per-head norm with the output gate behind it.  Everything here is float: gates, decays, the running maximum, the
// state.  A state row is [heads * d * dv (C, per head [d, dv]) | heads * d (n) | heads (m)].
#include "common.h"

#define ML_MAX_D 256

__device__ __forceinline__ float capped(float z, float cap) { return cap * tanhf(z / cap); }
__device__ __forceinline__ float log_sigmoid(float z) { return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z)); }

// Pass 1, one wave per (portion, head): token by token the log gates i = cap(gi), f = logsigmoid(cap(gf)), the maximum
// m' = max(f + m, i), keep = exp(f + m - m'), take = exp(i - m'), n' = keep n + take k, and the divisor
// max(|n' . q|, exp(-m')) + 1e-6 with q scaled by 1/sqrt(d).  coef[t, h] = (keep, take, divisor); n and m go back into
// the state.  A portion that starts at position 0 starts from zeros, whatever the slot holds.
template <typename T>
__global__ void __launch_bounds__(WAVE)
mlstm_gates_kernel(const T* __restrict__ qkvg, int row_stride, const float* __restrict__ gates, int gate_stride,
                   float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_q,
                   const int* __restrict__ first_position, const int* __restrict__ state_slots,
                   float* __restrict__ coef, int heads, int d, int dv, float cap) {
  const int e = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int lo = cu_q[e], hi = cu_q[e + 1];
  if (hi <= lo) return;                                      // an entry that only fills the batch up
  float* row = state + (size_t)state_slots[e] * state_stride;
  float* n_state = row + (size_t)heads * d * dv + (size_t)h * d;
  float* m_state = row + (size_t)heads * d * dv + (size_t)heads * d + h;
  const bool fresh = first_position[e] == 0;
  float n[ML_MAX_D / WAVE];
#pragma unroll
  for (int r = 0; r < ML_MAX_D / WAVE; ++r) {
    const int j = lane + r * WAVE;
    n[r] = (!fresh && j < d) ? n_state[j] : 0.f;
  }
  float m = fresh ? 0.f : *m_state;
  const float q_scale = 1.0f / sqrtf((float)d);
  for (int t = lo; t < hi; ++t) {
    const T* x = qkvg + (size_t)t * row_stride;
    const float i = capped(gates[(size_t)t * gate_stride + h], cap);
    const float f = log_sigmoid(capped(gates[(size_t)t * gate_stride + heads + h], cap));
    const float m_new = fmaxf(f + m, i);
    const float keep = expf(f + m - m_new), take = expf(i - m_new);
    float dot = 0.f;
#pragma unroll
    for (int r = 0; r < ML_MAX_D / WAVE; ++r) {
      const int j = lane + r * WAVE;
      if (j < d) {
        const float q = ld(x + (size_t)h * d + j) * q_scale, k = ld(x + (size_t)(heads + h) * d + j);
        n[r] = fmaf(keep, n[r], take * k);
        dot = fmaf(n[r], q, dot);
      }
    }
    dot = wave_sum(dot);
    m = m_new;
    if (lane == 0) {
      float* c = coef + ((size_t)t * heads + h) * 3;
      c[0] = keep; c[1] = take; c[2] = fmaxf(fabsf(dot), expf(-m)) + 1e-6f;
    }
  }
#pragma unroll
  for (int r = 0; r < ML_MAX_D / WAVE; ++r) {
    const int j = lane + r * WAVE;
    if (j < d) n_state[j] = n[r];
  }
  if (lane == 0) *m_state = m;
}

// Pass 2, one workgroup of four waves per (portion, head, 64 columns of C): wave w keeps rows w, w + 4, ... of its
// columns in registers (PER rows a lane), C' = keep C + take k v^T, o = C'^T q / divisor, token by token; the four
// waves' parts of o are added through LDS.  Columns of C do not depend on each other, so workgroups share nothing.
// q and k of the next token are fetched while the current one is worked on.
template <typename T, int PER>
__global__ void __launch_bounds__(4 * WAVE)
mlstm_memory_kernel(const T* __restrict__ qkvg, int row_stride, const float* __restrict__ coef,
                    float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_q,
                    const int* __restrict__ first_position, const int* __restrict__ state_slots,
                    float* __restrict__ out, int heads, int d, int dv) {
  __shared__ float qk[2][2][ML_MAX_D];       // [token parity][q, k][d]
  __shared__ float part[2][4][WAVE];
  const int e = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int lo = cu_q[e], hi = cu_q[e + 1];
  if (hi <= lo) return;
  const int c = blockIdx.z * WAVE + lane;
  const bool live = c < dv;
  float* mem = state + (size_t)state_slots[e] * state_stride + (size_t)h * d * dv;
  const bool fresh = first_position[e] == 0;
  float C[PER];
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = wave + 4 * r;
    C[r] = (!fresh && live && j < d) ? mem[(size_t)j * dv + c] : 0.f;
  }
  const float q_scale = 1.0f / sqrtf((float)d);
  const int tid = threadIdx.x;
  // (Thread i brings q[i] and k[i]: d is at most 256, the workgroup's size.)
  float q_next = 0.f, k_next = 0.f;
  if (tid < d) {
    const T* x = qkvg + (size_t)lo * row_stride;
    q_next = ld(x + (size_t)h * d + tid) * q_scale;
    k_next = ld(x + (size_t)(heads + h) * d + tid);
  }
  qk[lo & 1][0][tid] = q_next;
  qk[lo & 1][1][tid] = k_next;
  __syncthreads();
  for (int t = lo; t < hi; ++t) {
    const int now = t & 1;
    if (t + 1 < hi && tid < d) {
      const T* x = qkvg + (size_t)(t + 1) * row_stride;
      q_next = ld(x + (size_t)h * d + tid) * q_scale;
      k_next = ld(x + (size_t)(heads + h) * d + tid);
    }
    const float* cf = coef + ((size_t)t * heads + h) * 3;
    const float keep = cf[0], take = cf[1], divisor = cf[2];
    const float v = live ? ld(qkvg + (size_t)t * row_stride + (size_t)2 * heads * d + (size_t)h * dv + c) : 0.f;
    const float tv = take * v;
    float acc = 0.f;
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int j = wave + 4 * r;
      if (j < d) {
        C[r] = fmaf(keep, C[r], qk[now][1][j] * tv);
        acc = fmaf(C[r], qk[now][0][j], acc);
      }
    }
    part[now][wave][lane] = acc;
    qk[now ^ 1][0][tid] = q_next;
    qk[now ^ 1][1][tid] = k_next;
    __syncthreads();
    if (wave == 0 && live) {
      const float sum = (part[now][0][lane] + part[now][1][lane]) + (part[now][2][lane] + part[now][3][lane]);
      out[(size_t)t * heads * dv + (size_t)h * dv + c] = sum / divisor;
    }
  }
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = wave + 4 * r;
    if (live && j < d) mem[(size_t)j * dv + c] = C[r];
  }
}

// out[t, h, :] = read[t, h, :] / sqrt(mean(read[t, h, :]^2) + eps) * weight[h, :] * sigmoid(gate[t, h, :]); `gate` lies
// in rows of `gate_stride` elements, from column `gate_offset` on.  One wave per (token, head).
template <typename T>
__global__ void __launch_bounds__(WAVE)
head_norm_gate_kernel(const float* __restrict__ read, const float* __restrict__ weight, const T* __restrict__ gate,
                      int gate_stride, int gate_offset, float eps, int heads, int dv, T* __restrict__ out) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* o = read + ((size_t)t * heads + h) * dv;
  float sq = 0.f;
  for (int j = lane; j < dv; j += WAVE) sq = fmaf(o[j], o[j], sq);
  const float inv = 1.0f / sqrtf(wave_sum(sq) / (float)dv + eps);
  const T* g = gate + (size_t)t * gate_stride + gate_offset + (size_t)h * dv;
  T* dst = out + ((size_t)t * heads + h) * dv;
  for (int j = lane; j < dv; j += WAVE) {
    const float z = ld(g + j);
    st(dst + j, o[j] * inv * weight[(size_t)h * dv + j] / (1.0f + expf(-z)));
  }
}

// qkvg: rows of `row_stride` elements, [heads d (q) | heads d (k) | heads dv (v) | ...]; gates float rows of `gate_stride`,
// [heads (input gate's pre-activation) | heads (forget gate's)]; coef: float scratch [n_tokens, heads, 3];
// out float [n_tokens, heads dv].
extern "C" int ta_mlstm_scan(const void* qkvg, int row_stride, const void* gates, int gate_stride, void* state,
                             long state_stride, const void* cu_q, const void* first_position, const void* state_slots,
                             void* coef, void* out, int n_entries, int heads, int d, int dv, float cap, int dtype,
                             hipStream_t stream) {
  if (n_entries <= 0) return 0;
  if (d < 1 || d > ML_MAX_D || dv < 1 || heads < 1 || state_stride < (long)heads * d * dv + (long)heads * d + heads) return -1;
  dim3 g1(n_entries, heads), g2(n_entries, heads, (dv + WAVE - 1) / WAVE);
  const int per = (d + 3) / 4;
#define PASS1(TT) mlstm_gates_kernel<TT><<<g1, WAVE, 0, stream>>>((const TT*)qkvg, row_stride, (const float*)gates, gate_stride, \
    (float*)state, (size_t)state_stride, (const int*)cu_q, (const int*)first_position, (const int*)state_slots, (float*)coef,   \
    heads, d, dv, cap)
#define PASS2(TT, PP) mlstm_memory_kernel<TT, PP><<<g2, 4 * WAVE, 0, stream>>>((const TT*)qkvg, row_stride, (const float*)coef, \
    (float*)state, (size_t)state_stride, (const int*)cu_q, (const int*)first_position, (const int*)state_slots, (float*)out,   \
    heads, d, dv)
#define BOTH(TT) PASS1(TT); if (per <= 8) PASS2(TT, 8); else if (per <= 16) PASS2(TT, 16); else if (per <= 32) PASS2(TT, 32); \
                 else PASS2(TT, 64)
  if (dtype == DT_F32) { BOTH(float); } else { BOTH(bf16_t); }
#undef BOTH
#undef PASS2
#undef PASS1
  return LAUNCH_STATUS();
}

extern "C" int ta_head_norm_gate(const void* read, const void* weight, const void* gate, int gate_stride,
                                 int gate_offset, float eps, int n_tokens, int heads, int dv, void* out, int dtype,
                                 hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  dim3 grid(n_tokens, heads);
  if (dtype == DT_F32)
    head_norm_gate_kernel<float><<<grid, WAVE, 0, stream>>>((const float*)read, (const float*)weight, (const float*)gate,
        gate_stride, gate_offset, eps, heads, dv, (float*)out);
  else
    head_norm_gate_kernel<bf16_t><<<grid, WAVE, 0, stream>>>((const float*)read, (const float*)weight, (const bf16_t*)gate,
        gate_stride, gate_offset, eps, heads, dv, (bf16_t*)out);
  return LAUNCH_STATUS();
}
