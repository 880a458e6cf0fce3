// Matrix-memory recurrence (mLSTM) over a batch of portions, with the state of every request in its slot, and the
// per-head norm with the output gate behind it.  Everything here is float: gates, decays, the running maximum, the
// state.  A state row is [heads * d * dv (C, per head [d, dv]) | heads * d (n) | heads (m)].
#include "common.h"

#define ML_MAX_D 256

__device__ __forceinline__ float capped(float z, float cap) { return cap * tanhf(z / cap); }
__device__ __forceinline__ float log_sigmoid(float z) { return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z)); }

#define ML_GROUP 16          // tokens whose q, k (and v) are brought into LDS in one trip

// Pass 1, one workgroup per (portion, head): token by token the log gates i = cap(gi), f = logsigmoid(cap(gf)), the
// maximum m' = max(f + m, i), keep = exp(f + m - m'), take = exp(i - m'), n' = keep n + take k, and the divisor
// max(|n' . q|, exp(-m')) + 1e-6 with q scaled by 1/sqrt(d).  coef[t, h] = (keep, take, divisor); n and m go back into
// the state.  A portion that starts at position 0 starts from zeros, whatever the slot holds.
// Tokens are taken sixteen at a time: all four waves bring their q and k rows into LDS in one trip (thread j brings
// column j; the next sixteen are asked for before the current ones are worked on), the gates are worked out side by
// side in sixteen lanes, and the first wave walks the recurrence itself token by token.
template <typename T>
__global__ void __launch_bounds__(4 * WAVE)
mlstm_gates_kernel(const T* __restrict__ qkvg, int row_stride, const float* __restrict__ gates, int gate_stride,
                   float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_q,
                   const int* __restrict__ first_position, const int* __restrict__ state_slots,
                   float* __restrict__ coef, int heads, int d, int dv, float cap) {
  __shared__ float q_s[ML_GROUP][ML_MAX_D], k_s[ML_GROUP][ML_MAX_D];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
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
    n[r] = (wave == 0 && !fresh && j < d) ? n_state[j] : 0.f;
  }
  float m = fresh ? 0.f : *m_state;
  const float q_scale = 1.0f / sqrtf((float)d);
  float q_next[ML_GROUP], k_next[ML_GROUP];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) {
      q_next[tok] = k_next[tok] = 0.f;
      if (tid < d && t0 + tok < hi) {
        const T* x = qkvg + (size_t)(t0 + tok) * row_stride;
        q_next[tok] = ld(x + (size_t)h * d + tid) * q_scale;
        k_next[tok] = ld(x + (size_t)(heads + h) * d + tid);
      }
    }
  };
  fetch(lo);
  for (int t0 = lo; t0 < hi; t0 += ML_GROUP) {
    __syncthreads();                                         // the group before has been worked off
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) { q_s[tok][tid] = q_next[tok]; k_s[tok][tid] = k_next[tok]; }
    // The gates of the group's tokens, one token a lane.
    float gi = 0.f, gf = 0.f;
    if (wave == 0 && lane < ML_GROUP && t0 + lane < hi) {
      gi = capped(gates[(size_t)(t0 + lane) * gate_stride + h], cap);
      gf = log_sigmoid(capped(gates[(size_t)(t0 + lane) * gate_stride + heads + h], cap));
    }
    if (t0 + ML_GROUP < hi) fetch(t0 + ML_GROUP);
    __syncthreads();
    if (wave != 0) continue;
    const int count = min(ML_GROUP, hi - t0);
    float keep_mine = 0.f, take_mine = 0.f, divisor_mine = 1.f;       // lane l keeps token l's three numbers
    for (int tok = 0; tok < count; ++tok) {
      const float i = __shfl(gi, tok, WAVE), f = __shfl(gf, tok, WAVE);
      const float m_new = fmaxf(f + m, i);
      const float keep = expf(f + m - m_new), take = expf(i - m_new);
      float dot = 0.f;
#pragma unroll
      for (int r = 0; r < ML_MAX_D / WAVE; ++r) {
        const int j = lane + r * WAVE;               // (columns past d hold zeros in LDS)
        n[r] = fmaf(keep, n[r], take * k_s[tok][j]);
        dot = fmaf(n[r], q_s[tok][j], dot);
      }
      dot = wave_sum(dot);
      m = m_new;
      if (lane == tok) { keep_mine = keep; take_mine = take; divisor_mine = fmaxf(fabsf(dot), expf(-m)) + 1e-6f; }
    }
    if (lane < count) {
      float* c = coef + ((size_t)(t0 + lane) * heads + h) * 3;
      c[0] = keep_mine; c[1] = take_mine; c[2] = divisor_mine;
    }
  }
  if (wave != 0) return;
#pragma unroll
  for (int r = 0; r < ML_MAX_D / WAVE; ++r) {
    const int j = lane + r * WAVE;
    if (j < d) n_state[j] = n[r];
  }
  if (lane == 0) *m_state = m;
}

// Pass 2, one workgroup of four waves per (portion, head, 16 columns of C).  A wave owns four columns; its lanes are
// (part p = lane / 4, column): lane (p, c) keeps rows p, p + 16, p + 32, ... of column c in registers (PER of them), so
// that C' = keep C + take k v^T and the sum over the rows for o = C'^T q / divisor need four exchanges between lanes per
// token and nothing else.  Columns of C do not depend on each other, so waves and workgroups share nothing but the rows
// of q, k and v, which come into LDS sixteen tokens at a time (thread j brings column j of q and of k; the next
// sixteen are asked for before the current ones are worked on).
template <typename T, int PER>
__global__ void __launch_bounds__(4 * WAVE)
mlstm_memory_kernel(const T* __restrict__ qkvg, int row_stride, const float* __restrict__ coef,
                    float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_q,
                    const int* __restrict__ first_position, const int* __restrict__ state_slots,
                    float* __restrict__ out, int heads, int d, int dv) {
  __shared__ float q_s[ML_GROUP][ML_MAX_D], k_s[ML_GROUP][ML_MAX_D], v_s[ML_GROUP][16], c_s[ML_GROUP][4];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int lo = cu_q[e], hi = cu_q[e + 1];
  if (hi <= lo) return;
  const int part = lane >> 2, local = wave * 4 + (lane & 3);
  const int c = blockIdx.z * 16 + local;
  const bool live = c < dv;
  float* mem = state + (size_t)state_slots[e] * state_stride + (size_t)h * d * dv;
  const bool fresh = first_position[e] == 0;
  float C[PER];
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = part + 16 * r;
    C[r] = (!fresh && live && j < d) ? mem[(size_t)j * dv + c] : 0.f;
  }
  const float q_scale = 1.0f / sqrtf((float)d);
  float q_next[ML_GROUP], k_next[ML_GROUP], v_next = 0.f, c_next = 1.f;
  auto fetch = [&](int t0) {
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) {
      q_next[tok] = k_next[tok] = 0.f;
      if (tid < d && t0 + tok < hi) {
        const T* x = qkvg + (size_t)(t0 + tok) * row_stride;
        q_next[tok] = ld(x + (size_t)h * d + tid) * q_scale;
        k_next[tok] = ld(x + (size_t)(heads + h) * d + tid);
      }
    }
    {
      const int tok = tid >> 4, col = blockIdx.z * 16 + (tid & 15);
      v_next = (col < dv && t0 + tok < hi)
          ? ld(qkvg + (size_t)(t0 + tok) * row_stride + (size_t)2 * heads * d + (size_t)h * dv + col) : 0.f;
    }
    if (tid < ML_GROUP * 3) {
      const int tok = tid / 3;
      c_next = t0 + tok < hi ? coef[((size_t)(t0 + tok) * heads + h) * 3 + (tid - tok * 3)] : 1.f;
    }
  };
  fetch(lo);
  for (int t0 = lo; t0 < hi; t0 += ML_GROUP) {
    __syncthreads();                                         // the group before has been worked off
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) { q_s[tok][tid] = q_next[tok]; k_s[tok][tid] = k_next[tok]; }
    v_s[tid >> 4][tid & 15] = v_next;
    if (tid < ML_GROUP * 3) c_s[tid / 3][tid % 3] = c_next;
    if (t0 + ML_GROUP < hi) fetch(t0 + ML_GROUP);
    __syncthreads();
    const int count = min(ML_GROUP, hi - t0);
    for (int tok = 0; tok < count; ++tok) {
      const float keep = c_s[tok][0], tv = c_s[tok][1] * v_s[tok][local];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < PER; ++r) {
        // (Rows past d hold zeros in q and k: they stay zero and add nothing.)
        C[r] = fmaf(keep, C[r], k_s[tok][part + 16 * r] * tv);
        acc = fmaf(C[r], q_s[tok][part + 16 * r], acc);
      }
      acc += __shfl_xor(acc, 4, WAVE);
      acc += __shfl_xor(acc, 8, WAVE);
      acc += __shfl_xor(acc, 16, WAVE);
      acc += __shfl_xor(acc, 32, WAVE);
      if (part == 0 && live) out[(size_t)(t0 + tok) * heads * dv + (size_t)h * dv + c] = acc / c_s[tok][2];
    }
  }
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = part + 16 * r;
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
  dim3 g1(n_entries, heads), g2(n_entries, heads, (dv + 15) / 16);
  const int per = (d + 15) / 16;
#define PASS1(TT) mlstm_gates_kernel<TT><<<g1, 4 * WAVE, 0, stream>>>((const TT*)qkvg, row_stride, (const float*)gates, gate_stride, \
    (float*)state, (size_t)state_stride, (const int*)cu_q, (const int*)first_position, (const int*)state_slots, (float*)coef,   \
    heads, d, dv, cap)
#define PASS2(TT, PP) mlstm_memory_kernel<TT, PP><<<g2, 4 * WAVE, 0, stream>>>((const TT*)qkvg, row_stride, (const float*)coef, \
    (float*)state, (size_t)state_stride, (const int*)cu_q, (const int*)first_position, (const int*)state_slots, (float*)out,   \
    heads, d, dv)
#define BOTH(TT) PASS1(TT); if (per <= 2) PASS2(TT, 2); else if (per <= 4) PASS2(TT, 4); else if (per <= 8) PASS2(TT, 8); \
                 else PASS2(TT, 16)
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
