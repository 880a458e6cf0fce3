// Several residual streams [tokens, S, width] (float): the embedding that fills them, the kernel that applies one
// sub-layer's write and makes the next sub-layer's normalised read, and the token shift with its per-request state.
#include "common.h"

#define MAX_STREAMS 16
#define KEPT_COLUMNS 16      // columns per thread whose read is kept in registers between the two passes

// out[t, s, :] = table[ids[t], :] (+ the position vector: entry 2i sin(p r_i), entry 2i+1 cos(p r_i)), for every s.
// Angles are float: position times rate, sine and cosine by the accurate routines.
template <typename T>
__global__ void __launch_bounds__(256)
embedding_streams_kernel(const int* __restrict__ ids, const T* __restrict__ table, const int* __restrict__ positions,
                         const float* __restrict__ rates, float* __restrict__ out, int width, int vocab, int n_streams) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0 || id >= vocab) id = 0;  // the host rejects such ids before the launch
  const float p = (float)positions[t];
  const T* row = table + (size_t)id * width;
  float* dst = out + (size_t)t * n_streams * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float v = ld(row + c);
    if (rates) {
      const float angle = p * rates[c >> 1];
      v += (c & 1) ? cosf(angle) : sinf(angle);
    }
    for (int s = 0; s < n_streams; ++s) dst[(size_t)s * width + c] = v;
  }
}

struct StreamCoefficients {
  float mix[MAX_STREAMS * MAX_STREAMS], out[MAX_STREAMS], read[MAX_STREAMS];
};

// One column of one token: the streams after the write (x' = M^T x + c * g * y), stored if asked, and the read r . x'.
// SMAX: a bound on S known when the kernel is compiled (4, 8 or 16), so that the loops over the streams unroll to the
// streams there are.
template <typename TY, int SMAX>
__device__ __forceinline__ float stream_column(float* __restrict__ x, const TY* __restrict__ y, const float* __restrict__ scale,
                                               const StreamCoefficients& k, int S, int width, int c, bool store) {
  float old[SMAX], u = 0.f;
#pragma unroll
  for (int s = 0; s < SMAX; ++s) old[s] = s < S ? x[(size_t)s * width + c] : 0.f;
  if (!y) {
#pragma unroll
    for (int s = 0; s < SMAX; ++s) if (s < S) u = fmaf(k.read[s], old[s], u);
    return u;
  }
  const float add = ld(y + c) * (scale ? scale[c] : 1.0f);
#pragma unroll
  for (int to = 0; to < SMAX; ++to) {
    if (to < S) {
      float v = 0.f;
#pragma unroll
      for (int s = 0; s < SMAX; ++s) if (s < S) v = fmaf(k.mix[s * MAX_STREAMS + to], old[s], v);
      v = fmaf(k.out[to], add, v);
      if (store) x[(size_t)to * width + c] = v;
      u = fmaf(k.read[to], v, u);
    }
  }
  return u;
}

// For output row i: r = rows ? rows[i] : i.  The write (y, mix [S, S] indexed [from, to], out [S], scale [width] or
// null; y null = no write) is applied to token r's streams (stored back unless `rows` picks a subset), then
// u = sum_s read[s] x_s, h = u / sqrt(mean(u^2) + eps) * gain[0].  With `mu` (one token per request): the row written is
// h + (before - h) * mu, `before` the state row of the token's request (zeros at position 0), and h becomes the state.
template <typename TY, typename TO, int SMAX>
__global__ void __launch_bounds__(1024)
streams_step_kernel(float* __restrict__ streams, const TY* __restrict__ y, const float* __restrict__ mix,
                    const float* __restrict__ out_coef, const float* __restrict__ scale, const float* __restrict__ read,
                    const float* __restrict__ gain, float eps, TO* __restrict__ out, const int* __restrict__ rows,
                    int width, int S, const float* __restrict__ mu, float* __restrict__ state,
                    const int* __restrict__ entry_of_token, const int* __restrict__ state_slots,
                    const int* __restrict__ positions) {
  __shared__ float scratch[16];
  __shared__ StreamCoefficients k;
  for (int i = threadIdx.x; i < MAX_STREAMS * MAX_STREAMS; i += blockDim.x) {
    const int s = i / MAX_STREAMS, to = i % MAX_STREAMS;
    k.mix[i] = (mix && s < S && to < S) ? mix[s * S + to] : 0.f;
    if (s == 0) {
      k.out[to] = (out_coef && to < S) ? out_coef[to] : 0.f;
      k.read[to] = to < S ? read[to] : 0.f;
    }
  }
  const int i = blockIdx.x;
  const int r = rows ? rows[i] : i;
  float* x = streams + (size_t)r * S * width;
  const TY* yr = y ? y + (size_t)r * width : nullptr;
  const bool store = y && !rows;
  if (width <= (int)blockDim.x) {
    // A thread per column (the launch of a step with few rows): everything the thread needs, the token's slot and
    // state row too, is asked for before anything is waited for, so the kernel is two trips to memory (the
    // coefficients and the rows; then the sum over the workgroup) where column after column it was five.
    const int c = threadIdx.x;
    const bool in = c < width;
    int slot = -1;
    bool first = false;
    if (mu) {
      const int e = entry_of_token[r];
      if (e >= 0) { slot = state_slots[e]; first = positions[r] == 0; }
    }
    float old[SMAX];
#pragma unroll
    for (int s = 0; s < SMAX; ++s) old[s] = (s < S && in) ? x[(size_t)s * width + c] : 0.f;
    const float add = (y && in) ? ld(yr + c) * (scale ? scale[c] : 1.0f) : 0.f;
    float before = 0.f, mu_c = 0.f;
    float* mine = nullptr;
    if (mu && slot >= 0 && in) {
      mine = state + (size_t)slot * width + c;
      before = first ? 0.f : *mine;
      mu_c = mu[c];
    }
    __syncthreads();
    float u = 0.f;
    if (!y) {
#pragma unroll
      for (int s = 0; s < SMAX; ++s) if (s < S) u = fmaf(k.read[s], old[s], u);
    } else {
#pragma unroll
      for (int to = 0; to < SMAX; ++to) {
        if (to < S) {
          float v = 0.f;
#pragma unroll
          for (int s = 0; s < SMAX; ++s) if (s < S) v = fmaf(k.mix[s * MAX_STREAMS + to], old[s], v);
          v = fmaf(k.out[to], add, v);
          if (store && in) x[(size_t)to * width + c] = v;
          u = fmaf(k.read[to], v, u);
        }
      }
    }
    const float total = block_sum(u * u, scratch);
    float h = u * (1.0f / sqrtf(total / (float)width + eps) * gain[0]);
    if (mine) {
      *mine = h;
      h = fmaf(before - h, mu_c, h);
    }
    if (in) st(out + (size_t)i * width + c, h);
    return;
  }
  __syncthreads();
  float kept[KEPT_COLUMNS], sq = 0.f;
  int n = 0;
  for (int c = threadIdx.x; c < width; c += blockDim.x, ++n) {
    const float u = stream_column<TY, SMAX>(x, yr, scale, k, S, width, c, store);
    if (n < KEPT_COLUMNS) kept[n] = u;
    sq = fmaf(u, u, sq);
  }
  const float total = block_sum(sq, scratch);
  const float inv = 1.0f / sqrtf(total / (float)width + eps) * gain[0];
  int slot = -1;
  bool first = false;
  if (mu) {
    const int e = entry_of_token[r];
    if (e >= 0) { slot = state_slots[e]; first = positions[r] == 0; }
  }
  TO* dst = out + (size_t)i * width;
  n = 0;
  for (int c = threadIdx.x; c < width; c += blockDim.x, ++n) {
    // (Past the kept columns the read is made again: from the streams as they are now if they were stored, which
    // adds the same numbers in the same order, else from the old ones.)
    const float u = n < KEPT_COLUMNS ? kept[n] : stream_column<TY, SMAX>(x, store ? (const TY*)nullptr : yr, scale, k, S, width, c, false);
    float h = u * inv;
    if (mu && slot >= 0) {
      float* mine = state + (size_t)slot * width + c;
      const float before = first ? 0.f : *mine;
      *mine = h;
      h = fmaf(before - h, mu[c], h);
    }
    st(dst + c, h);
  }
}

// Token shift over a batch of portions: out[t] = h[t] + (before - h[t]) * mu, `before` = h[t - 1] inside a portion, the
// request's state row for a portion's first token (zeros at position 0).  The block of a portion's first token also
// leaves the portion's last row in the state: it alone touches that row, after it has read it.
template <typename TO>
__global__ void __launch_bounds__(256)
token_shift_kernel(const float* __restrict__ h, const float* __restrict__ mu, float* __restrict__ state,
                   const int* __restrict__ cu_q, const int* __restrict__ first_position,
                   const int* __restrict__ state_slots, const int* __restrict__ entry_of_token, TO* __restrict__ out,
                   int width) {
  const int t = blockIdx.x;
  const int e = entry_of_token[t];
  const float* mine = h + (size_t)t * width;
  TO* dst = out + (size_t)t * width;
  if (e < 0) {                                               // a token that only fills the batch up
    for (int c = threadIdx.x; c < width; c += blockDim.x) st(dst + c, mine[c]);
    return;
  }
  const int first = cu_q[e], last = cu_q[e + 1] - 1;
  if (t != first) {
    const float* before = mine - width;
    for (int c = threadIdx.x; c < width; c += blockDim.x) st(dst + c, fmaf(before[c] - mine[c], mu[c], mine[c]));
    return;
  }
  float* kept = state + (size_t)state_slots[e] * width;
  const bool fresh = first_position[e] == 0;
  const float* tail = h + (size_t)last * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float before = fresh ? 0.f : kept[c];
    kept[c] = tail[c];
    st(dst + c, fmaf(before - mine[c], mu[c], mine[c]));
  }
}

extern "C" int ta_embedding_streams(const void* ids, const void* table, const void* positions, const void* rates,
                                    void* out, int n_tokens, int width, int vocab, int n_streams, int dtype,
                                    hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (n_streams < 1 || width < 1) return -1;
  if (dtype == DT_F32)
    embedding_streams_kernel<float><<<n_tokens, 256, 0, stream>>>((const int*)ids, (const float*)table, (const int*)positions,
        (const float*)rates, (float*)out, width, vocab, n_streams);
  else
    embedding_streams_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const int*)ids, (const bf16_t*)table, (const int*)positions,
        (const float*)rates, (float*)out, width, vocab, n_streams);
  return LAUNCH_STATUS();
}

// y_dtype: of `y`; out_dtype: of `out` (float32 rows for a token shift that follows, else the compute dtype).
extern "C" int ta_streams_step(void* streams, const void* y, const void* mix, const void* out_coef, const void* scale,
                               const void* read, const void* gain, float eps, void* out, const void* rows, int n_rows,
                               int width, int n_streams, int y_dtype, int out_dtype, const void* mu, void* state,
                               const void* entry_of_token, const void* state_slots, const void* positions,
                               hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (n_streams < 1 || n_streams > MAX_STREAMS || width < 1 || !read || !gain || !out) return -1;
  if (y && (!mix || !out_coef)) return -1;
  if (mu && (!state || !entry_of_token || !state_slots || !positions || rows)) return -1;
  // Few rows (a decode step): a thread per column, so that a row's loads are one trip to memory instead of one per
  // 256 columns; many rows fill the device with workgroups of 256.
  int threads = 256;
  if (n_rows <= 2 * compute_units()) threads = width >= 1024 ? 1024 : (width + WAVE - 1) / WAVE * WAVE;
#define GO(TY, TO) if (n_streams <= 4) GO_S(TY, TO, 4); else if (n_streams <= 8) GO_S(TY, TO, 8); else GO_S(TY, TO, 16)
#define GO_S(TY, TO, SS) streams_step_kernel<TY, TO, SS><<<n_rows, threads, 0, stream>>>((float*)streams, (const TY*)y, (const float*)mix, \
    (const float*)out_coef, (const float*)scale, (const float*)read, (const float*)gain, eps, (TO*)out, (const int*)rows,   \
    width, n_streams, (const float*)mu, (float*)state, (const int*)entry_of_token, (const int*)state_slots,                 \
    (const int*)positions)
  if (y_dtype == DT_F32) { if (out_dtype == DT_F32) { GO(float, float); } else return -1; }
  else { if (out_dtype == DT_F32) { GO(bf16_t, float); } else { GO(bf16_t, bf16_t); } }
#undef GO_S
#undef GO
  return LAUNCH_STATUS();
}

extern "C" int ta_token_shift(const void* h, const void* mu, void* state, const void* cu_q, const void* first_position,
                              const void* state_slots, const void* entry_of_token, void* out, int n_tokens, int width,
                              int out_dtype, hipStream_t stream) {
  if (n_tokens <= 0) return 0;
  if (out_dtype == DT_F32)
    token_shift_kernel<float><<<n_tokens, 256, 0, stream>>>((const float*)h, (const float*)mu, (float*)state, (const int*)cu_q,
        (const int*)first_position, (const int*)state_slots, (const int*)entry_of_token, (float*)out, width);
  else
    token_shift_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>((const float*)h, (const float*)mu, (float*)state, (const int*)cu_q,
        (const int*)first_position, (const int*)state_slots, (const int*)entry_of_token, (bf16_t*)out, width);
  return LAUNCH_STATUS();
}
