// Matrix-memory recurrence (mLSTM) over a batch of portions, with the state of every request in its slot, and the
// per-head norm with the output gate behind it.  Everything here is float: gates, decays, the running maximum, the
// state.  A state row is [heads * d * dv (C, per head [d, dv]) | heads * d (n) | heads (m)].
#include "common.h"

#define ML_MAX_D 256

__device__ __forceinline__ float capped(float z, float cap) { return cap * tanhf(z / cap); }
__device__ __forceinline__ float log_sigmoid(float z) { return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z)); }

#define ML_GROUP 16          // tokens whose q, k (and v) are brought into LDS in one trip

// Lane `from`'s value of v, the same for every lane (`from` is known when the kernel is compiled).
__device__ __forceinline__ float lane_value(float v, int from) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), from));
}

// x summed over the sixteen lanes of a row (lanes 16 i .. 16 i + 15), in every lane of the row: four rotations within the
// row, which cost no trip through LDS.
__device__ __forceinline__ float row_sum16(float x) {
#define ML_ROR(n) __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x120 | (n), 0xF, 0xF, false))
  x += ML_ROR(8);
  x += ML_ROR(4);
  x += ML_ROR(2);
  x += ML_ROR(1);
#undef ML_ROR
  return x;
}

// Pass 1, one workgroup per (portion, head): token by token the log gates i = cap(gi), f = logsigmoid(cap(gf)), the
// maximum m' = max(f + m, i), keep = exp(f + m - m'), take = exp(i - m'), n' = keep n + take k, and the divisor
// max(|n' . q|, exp(-m')) + 1e-6 with q scaled by 1/sqrt(d).  coef[t, h] = (keep, take, divisor); n and m go back into
// the state.  A portion that starts at position 0 starts from zeros, whatever the slot holds.
// Thread j owns column j of n (d is at most the workgroup's 256 threads).  Tokens are taken sixteen at a time: thread j
// brings column j of their q and k rows (the next sixteen are asked for before the current ones are worked on); every
// wave works out the sixteen tokens' gates side by side in sixteen lanes and walks the maximum's chain; the sums
// n' . q over the columns are made for all sixteen tokens together (within rows of sixteen lanes by rotations, the
// sixteen rows' sums through LDS).
template <typename T>
__global__ void __launch_bounds__(4 * WAVE)
mlstm_gates_kernel(const T* __restrict__ qkvg, int row_stride, const float* __restrict__ gates, int gate_stride,
                   float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_q,
                   const int* __restrict__ first_position, const int* __restrict__ state_slots,
                   float* __restrict__ coef, int heads, int d, int dv, float cap) {
  __shared__ float rows_s[ML_GROUP][16];                    // a token's sixteen row sums
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int lo = cu_q[e], hi = cu_q[e + 1];
  if (hi <= lo) return;                                      // an entry that only fills the batch up
  float* row = state + (size_t)state_slots[e] * state_stride;
  float* n_state = row + (size_t)heads * d * dv + (size_t)h * d;
  float* m_state = row + (size_t)heads * d * dv + (size_t)heads * d + h;
  const bool fresh = first_position[e] == 0;
  float n = (!fresh && tid < d) ? n_state[tid] : 0.f;
  float m = fresh ? 0.f : *m_state;
  const float q_scale = 1.0f / sqrtf((float)d);
  float q_now[ML_GROUP], k_now[ML_GROUP], q_next[ML_GROUP], k_next[ML_GROUP];
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
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) { q_now[tok] = q_next[tok]; k_now[tok] = k_next[tok]; }
    // The gates of the group's tokens, one token a lane.  A token past the portion's end changes nothing: its forget
    // gate is 0 (keep 1) and its input gate minus infinity (take 0).
    float gi = -INFINITY, gf = 0.f;
    if (lane < ML_GROUP && t0 + lane < hi) {
      gi = capped(gates[(size_t)(t0 + lane) * gate_stride + h], cap);
      gf = log_sigmoid(capped(gates[(size_t)(t0 + lane) * gate_stride + heads + h], cap));
    }
    if (t0 + ML_GROUP < hi) fetch(t0 + ML_GROUP);
    // The maximum's chain over the sixteen tokens (three operations a token); lane l keeps what token l needs of it.
    float m_before = 0.f, m_after = 0.f;
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) {
      const float i = lane_value(gi, tok), f = lane_value(gf, tok);
      const float m_new = fmaxf(f + m, i);
      if (lane == tok) { m_before = m; m_after = m_new; }
      m = m_new;
    }
    // Decays and the divisor's floor of all sixteen tokens side by side.
    const float keep_mine = expf(gf + m_before - m_after), take_mine = expf(gi - m_after), floor_mine = expf(-m_after);
    // n' = keep n + take k token by token, and this column's share of n' . q.
    float share[ML_GROUP];
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) {
      n = fmaf(lane_value(keep_mine, tok), n, lane_value(take_mine, tok) * k_now[tok]);
      share[tok] = n * q_now[tok];
    }
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) share[tok] = row_sum16(share[tok]);
    __syncthreads();                                         // the group before has been read
    if ((lane & 15) == 0) {
#pragma unroll
      for (int tok = 0; tok < ML_GROUP; ++tok) rows_s[tok][tid >> 4] = share[tok];
    }
    __syncthreads();
    if (wave == 0 && lane < ML_GROUP && t0 + lane < hi) {
      float dot = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) dot += rows_s[lane][r];
      float* c = coef + ((size_t)(t0 + lane) * heads + h) * 3;
      c[0] = keep_mine; c[1] = take_mine; c[2] = fmaxf(fabsf(dot), floor_mine) + 1e-6f;
    }
  }
  if (tid < d) n_state[tid] = n;
  if (tid == 0) *m_state = m;
}

// Pass 2, one workgroup of four waves per (portion, head, 16 columns of C).  A wave owns four columns; its lanes are
// (column, part p = lane % 16): lane (c, p) keeps rows p PER .. p PER + PER - 1 of column c in registers, so that
// C' = keep C + take k v^T needs nothing from other lanes and the sum over the rows for o = C'^T q / divisor is a sum
// within a row of sixteen lanes (four rotations, no trip through LDS).  Columns of C do not depend on each other, so
// waves and workgroups share nothing but the rows of q, k and v, which come into LDS sixteen tokens at a time (thread
// j brings column j of q and of k; the next sixteen are asked for before the current ones are worked on).
template <typename T, int PER>
__global__ void __launch_bounds__(4 * WAVE)
mlstm_memory_kernel(const T* __restrict__ qkvg, int row_stride, const float* __restrict__ coef,
                    float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_q,
                    const int* __restrict__ first_position, const int* __restrict__ state_slots,
                    float* __restrict__ out, int heads, int d, int dv) {
  __shared__ __attribute__((aligned(16))) float q_s[ML_GROUP][16 * PER], k_s[ML_GROUP][16 * PER];
  __shared__ float v_s[ML_GROUP][16], c_s[ML_GROUP][4];
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int lo = cu_q[e], hi = cu_q[e + 1];
  if (hi <= lo) return;
  const int part = lane & 15, local = wave * 4 + (lane >> 4);
  const int c = blockIdx.z * 16 + local;
  const bool live = c < dv;
  float* mem = state + (size_t)state_slots[e] * state_stride + (size_t)h * d * dv;
  const bool fresh = first_position[e] == 0;
  float C[PER];
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = part * PER + r;
    C[r] = (!fresh && live && j < d) ? mem[(size_t)j * dv + c] : 0.f;
  }
  const float q_scale = 1.0f / sqrtf((float)d);
  constexpr int PIECES = (16 * PER + 4 * WAVE - 1) / (4 * WAVE);      // columns of q (and of k) a thread brings: 1 here
  static_assert(PIECES == 1, "a thread brings one column");
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
    if (tid < 16 * PER) {
#pragma unroll
      for (int tok = 0; tok < ML_GROUP; ++tok) { q_s[tok][tid] = q_next[tok]; k_s[tok][tid] = k_next[tok]; }
    }
    v_s[tid >> 4][tid & 15] = v_next;
    if (tid < ML_GROUP * 3) c_s[tid / 3][tid % 3] = c_next;
    if (t0 + ML_GROUP < hi) fetch(t0 + ML_GROUP);
    __syncthreads();
    // Token by token C' = keep C + take k v^T and each lane's share of C'^T q; the sums over a column's sixteen lanes are
    // made afterwards for all sixteen tokens.  (A token past the portion's end has keep 1 and zeros for k and v: it
    // changes nothing.  Rows past d hold zeros in q and k: they stay zero and add nothing.)
    float share[ML_GROUP];
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) {
      const float keep = c_s[tok][0], tv = c_s[tok][1] * v_s[tok][local];
      float acc = 0.f;
      if constexpr (PER % 4 == 0) {
#pragma unroll
        for (int r = 0; r < PER; r += 4) {
          const float4 k4 = *reinterpret_cast<const float4*>(&k_s[tok][part * PER + r]);
          const float4 q4 = *reinterpret_cast<const float4*>(&q_s[tok][part * PER + r]);
          C[r] = fmaf(keep, C[r], k4.x * tv);         acc = fmaf(C[r], q4.x, acc);
          C[r + 1] = fmaf(keep, C[r + 1], k4.y * tv); acc = fmaf(C[r + 1], q4.y, acc);
          C[r + 2] = fmaf(keep, C[r + 2], k4.z * tv); acc = fmaf(C[r + 2], q4.z, acc);
          C[r + 3] = fmaf(keep, C[r + 3], k4.w * tv); acc = fmaf(C[r + 3], q4.w, acc);
        }
      } else {
#pragma unroll
        for (int r = 0; r < PER; ++r) {
          C[r] = fmaf(keep, C[r], k_s[tok][part * PER + r] * tv);
          acc = fmaf(C[r], q_s[tok][part * PER + r], acc);
        }
      }
      share[tok] = acc;
    }
#pragma unroll
    for (int tok = 0; tok < ML_GROUP; ++tok) share[tok] = row_sum16(share[tok]);
    if (part == 0 && live) {
#pragma unroll
      for (int tok = 0; tok < ML_GROUP; ++tok)
        if (t0 + tok < hi) out[(size_t)(t0 + tok) * heads * dv + (size_t)h * dv + c] = share[tok] / c_s[tok][2];
    }
  }
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int j = part * PER + r;
    if (live && j < d) mem[(size_t)j * dv + c] = C[r];
  }
}

// ---------------------------------------------------------------------------------------------------------------
// The same recurrence in chunks of 64 tokens, for portions of many tokens.  With b_t the sum of the forget gates from
// the chunk's first token to t, a_t = max over s <= t of (b_t - b_s + i_s) and m_0 the maximum before the chunk, the
// running maximum is m_t = max(b_t + m_0, a_t), and in terms of the state (C_0, n_0) before the chunk
//   C_t^T q_t = exp(b_t + m_0 - m_t) C_0^T q_t + sum over s <= t of exp(b_t - b_s + i_s - m_t) (q_t . k_s) v_s,
// likewise n_t . q_t; no exponent is above 0.  Three kernels: every chunk's own sums as if it started from nothing
// (all chunks side by side), the states before every chunk (one after the other, an element a thread), the reads (all
// chunks side by side; a workgroup per 64 columns of the values).  All of it in float; the sums b and the exponents' arguments in double, so that a difference
// of two long sums keeps its digits.  Products are 64 x 64 tiles through LDS, a 4 x 4 piece a thread.
#define MC_L 64            // tokens of a chunk, and the side of a tile
#define MC_LD 65           // floats from one row of a tile in LDS to the next

struct chunk_place { int entry, index, count, lo, n; };     // the entry, which of its `count` chunks, first row, rows

// Chunk g of the batch: entries in their order, each with as many chunks as its rows need.
__device__ __forceinline__ bool find_chunk(const int* __restrict__ cu_q, int n_entries, int g, chunk_place& p) {
  int base = 0;
  for (int e = 0; e < n_entries; ++e) {
    const int lo = cu_q[e], len = cu_q[e + 1] - lo;
    const int count = len > 0 ? (len + MC_L - 1) / MC_L : 0;
    if (g < base + count) {
      p.entry = e; p.index = g - base; p.count = count; p.lo = lo + p.index * MC_L;
      p.n = min(MC_L, lo + len - p.lo);
      return true;
    }
    base += count;
  }
  return false;
}

// The chunk's log input gates i_s, sums of forget gates b_s and maxima a_s as above (entries from n on repeat n - 1),
// by the first wave: sums and maxima along the lanes in six steps each, a_t = b_t + max over s <= t of (i_s - b_s).
__device__ __forceinline__ void chunk_gates(const float* __restrict__ gates, int gate_stride, int heads, int h, float cap,
                                            int lo, int n, float* i_s, double* b_s, float* a_s) {
  const int tid = threadIdx.x;
  if (tid < MC_L) {
    float gi = -INFINITY, gf = 0.f;
    if (tid < n) {
      gi = capped(gates[(size_t)(lo + tid) * gate_stride + h], cap);
      gf = log_sigmoid(capped(gates[(size_t)(lo + tid) * gate_stride + heads + h], cap));
    }
    double b = (double)gf;
#pragma unroll
    for (int off = 1; off < MC_L; off <<= 1) {
      const double other = __shfl_up(b, off);
      if (tid >= off) b += other;
    }
    double z = (double)gi - b;
#pragma unroll
    for (int off = 1; off < MC_L; off <<= 1) {
      const double other = __shfl_up(z, off);
      if (tid >= off) z = fmax(z, other);
    }
    i_s[tid] = gi; b_s[tid] = b; a_s[tid] = (float)(b + z);
  }
  __syncthreads();
}

// A tile of rows [row0, row0 + n) x columns [col0, col0 + 64) of `src` (rows of `stride` elements) into LDS, zeros
// outside n rows and `cols` columns; `scale` times every element.
template <typename T>
__device__ __forceinline__ void load_tile(float (*tile)[MC_LD], const T* __restrict__ src, size_t stride, int n, int cols,
                                          float scale) {
  constexpr int EACH = MC_L * MC_L / (4 * WAVE);             // all of a thread's elements are asked for before any is used
  const int c = threadIdx.x & 63, r0 = threadIdx.x >> 6;
  float got[EACH];
#pragma unroll
  for (int x = 0; x < EACH; ++x) {
    const int r = r0 + 4 * x;
    got[x] = (r < n && c < cols) ? ld(src + (size_t)r * stride + c) : 0.f;
  }
#pragma unroll
  for (int x = 0; x < EACH; ++x) tile[r0 + 4 * x][c] = got[x] * scale;
}

// Every chunk from nothing: local[g, h] = [sum_s w_s k_s v_s^T (d x dv) | sum_s w_s k_s (d)] with
// w_s = exp(b_last - b_s + i_s - a_last), and ends[g, h] = (b_last, a_last).
template <typename T>
__global__ void __launch_bounds__(4 * WAVE)
mlstm_chunk_local_kernel(const T* __restrict__ qkvg, int row_stride, const float* __restrict__ gates, int gate_stride,
                         const int* __restrict__ cu_q, int n_entries, float* __restrict__ local, float* __restrict__ ends,
                         int heads, int d, int dv, float cap) {
  __shared__ float k_s[MC_L][MC_LD], v_s[MC_L][MC_LD];
  __shared__ float i_s[MC_L], a_s[MC_L], w_s[MC_L];
  __shared__ double b_s[MC_L];
  const int g = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
  chunk_place p;
  if (!find_chunk(cu_q, n_entries, g, p)) return;
  const int n = p.n;
  chunk_gates(gates, gate_stride, heads, h, cap, p.lo, n, i_s, b_s, a_s);
  if (tid < MC_L)
    w_s[tid] = tid < n ? expf((float)((b_s[n - 1] - b_s[tid]) + (double)i_s[tid] - (double)a_s[n - 1])) : 0.f;
  if (tid == 0) {
    ends[((size_t)g * heads + h) * 2] = (float)b_s[n - 1];
    ends[((size_t)g * heads + h) * 2 + 1] = a_s[n - 1];
  }
  __syncthreads();
  const size_t total = (size_t)d * dv + d;
  float* dst = local + ((size_t)g * heads + h) * total;
  const T* rows = qkvg + (size_t)p.lo * row_stride;
  for (int j0 = 0; j0 < d; j0 += MC_L) {
    load_tile(k_s, rows + (size_t)(heads + h) * d + j0, (size_t)row_stride, n, d - j0, 1.f);
    for (int x = 0; x < MC_L * MC_L / (4 * WAVE); ++x) k_s[(tid >> 6) + 4 * x][tid & 63] *= w_s[(tid >> 6) + 4 * x];   // a thread's own
    __syncthreads();
    if (blockIdx.z == 0 && tid < MC_L && j0 + tid < d) {
      float sum = 0.f;
#pragma unroll 16
      for (int s = 0; s < MC_L; ++s) sum += k_s[s][tid];       // rows from n on hold zeros
      dst[(size_t)d * dv + j0 + tid] = sum;
    }
    {
      const int c0 = blockIdx.z * MC_L;                      // this workgroup's 64 columns of v
      load_tile(v_s, rows + (size_t)2 * heads * d + (size_t)h * dv + c0, (size_t)row_stride, n, dv - c0, 1.f);
      __syncthreads();
      float acc[4][4] = {};
#pragma unroll 8
      for (int s = 0; s < MC_L; ++s) {
        float kk[4], vv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) { kk[r] = k_s[s][ty * 4 + r]; vv[r] = v_s[s][tx + 16 * r]; }
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
          for (int c = 0; c < 4; ++c) acc[r][c] = fmaf(kk[r], vv[c], acc[r][c]);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const int j = j0 + ty * 4 + r, col = c0 + tx + 16 * c;
          if (j < d && col < dv) dst[(size_t)j * dv + col] = acc[r][c];
        }
      __syncthreads();                                       // the tiles are free again
    }
  }
}

// From chunk to chunk, an element of [C | n] a thread: local[g, h] becomes the state before chunk g, the state after
// the entry's last chunk goes into its slot, m_start[g, h] is the maximum before chunk g.  (The slot's m is written by
// the reads' kernel: every workgroup here reads it.)
__global__ void __launch_bounds__(4 * WAVE)
mlstm_chunk_carry_kernel(float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_q,
                         const int* __restrict__ first_position, const int* __restrict__ state_slots,
                         float* local, const float* __restrict__ ends, float* __restrict__ m_start,
                         int heads, int d, int dv) {
  const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int len = cu_q[e + 1] - cu_q[e];
  if (len <= 0) return;
  int base = 0;
  for (int x = 0; x < e; ++x) {
    const int l = cu_q[x + 1] - cu_q[x];
    base += l > 0 ? (l + MC_L - 1) / MC_L : 0;
  }
  const int count = (len + MC_L - 1) / MC_L;
  const size_t plane = (size_t)d * dv, total = plane + d, idx = (size_t)blockIdx.z * (4 * WAVE) + tid;
  const bool live = idx < total;
  float* row = state + (size_t)state_slots[e] * state_stride;
  float* mine = idx < plane ? row + (size_t)h * plane + idx : row + (size_t)heads * plane + (size_t)h * d + (idx - plane);
  const bool fresh = first_position[e] == 0;
  float x = (live && !fresh) ? *mine : 0.f;
  float m = fresh ? 0.f : row[(size_t)heads * plane + (size_t)heads * d + h];
  const size_t step = (size_t)heads * total;
  float* src = local + ((size_t)base * heads + h) * total + idx;
  float next = live ? src[0] : 0.f;
  for (int c = 0; c < count; ++c) {
    const float now = next;
    if (live) {
      src[(size_t)c * step] = x;
      if (c + 1 < count) next = src[(size_t)(c + 1) * step];
    }
    const float b_last = ends[((size_t)(base + c) * heads + h) * 2], a_last = ends[((size_t)(base + c) * heads + h) * 2 + 1];
    const float m_new = fmaxf(b_last + m, a_last);
    if (blockIdx.z == 0 && tid == 0) m_start[(size_t)(base + c) * heads + h] = m;
    x = fmaf(expf(b_last + m - m_new), x, expf(a_last - m_new) * now);
    m = m_new;
  }
  if (live) *mine = x;
}

// The reads of a chunk's tokens from the state before the chunk (`start`, what the carry left in `local`) and the
// chunk's own keys and values.
template <typename T>
__global__ void __launch_bounds__(4 * WAVE)
mlstm_chunk_read_kernel(const T* __restrict__ qkvg, int row_stride, const float* __restrict__ gates, int gate_stride,
                        float* __restrict__ state, size_t state_stride, const int* __restrict__ cu_q,
                        const int* __restrict__ state_slots, int n_entries, const float* __restrict__ local,
                        const float* __restrict__ ends, const float* __restrict__ m_start, float* __restrict__ out, int heads, int d, int dv, float cap) {
  __shared__ float q_s[MC_L][MC_LD], k_s[MC_L][MC_LD], p_s[MC_L][MC_LD];
  __shared__ float i_s[MC_L], a_s[MC_L], m_s[MC_L], w0_s[MC_L], div_s[MC_L], n0_s[MC_L];
  __shared__ double b_s[MC_L];
  const int g = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
  chunk_place p;
  if (!find_chunk(cu_q, n_entries, g, p)) return;
  const int n = p.n;
  chunk_gates(gates, gate_stride, heads, h, cap, p.lo, n, i_s, b_s, a_s);
  const float m0 = m_start[(size_t)g * heads + h];
  // After the entry's last chunk the slot's maximum is the one the carried state was scaled to, by the same operations.
  if (tid == 0 && p.index == p.count - 1)
    state[(size_t)state_slots[p.entry] * state_stride + (size_t)heads * d * dv + (size_t)heads * d + h] =
        fmaxf(ends[((size_t)g * heads + h) * 2] + m0, ends[((size_t)g * heads + h) * 2 + 1]);
  if (tid < MC_L) {
    const float m = fmaxf((float)(b_s[tid] + (double)m0), a_s[tid]);
    m_s[tid] = m;
    w0_s[tid] = expf((float)(b_s[tid] + (double)m0 - (double)m));
  }
  const size_t plane = (size_t)d * dv;
  const float* start = local + ((size_t)g * heads + h) * (plane + d);
  const T* rows = qkvg + (size_t)p.lo * row_stride;
  const float q_scale = 1.0f / sqrtf((float)d);
  // q_t . k_s over the whole of d, and n_0 . q_t (thread t).
  float acc[4][4] = {};
  float dn = 0.f;
  for (int j0 = 0; j0 < d; j0 += MC_L) {
    const int lim = min(MC_L, d - j0);
    __syncthreads();
    load_tile(q_s, rows + (size_t)h * d + j0, (size_t)row_stride, n, lim, q_scale);
    load_tile(k_s, rows + (size_t)(heads + h) * d + j0, (size_t)row_stride, n, lim, 1.f);
    if (tid < MC_L) n0_s[tid] = tid < lim ? start[plane + j0 + tid] : 0.f;
    __syncthreads();
#pragma unroll 8
    for (int jj = 0; jj < MC_L; ++jj) {                      // columns from lim on hold zeros
      float qq[4], kk[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) { qq[r] = q_s[ty * 4 + r][jj]; kk[r] = k_s[tx + 16 * r][jj]; }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = fmaf(qq[r], kk[c], acc[r][c]);
    }
    if (tid < MC_L) {
#pragma unroll 16
      for (int jj = 0; jj < MC_L; ++jj) dn = fmaf(q_s[tid][jj], n0_s[jj], dn);
    }
  }
  // Scores times their decays; nothing above the diagonal or past the chunk's rows.
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int t = ty * 4 + r, s = tx + 16 * c;
      float w = 0.f;
      if (s <= t && t < n) w = acc[r][c] * expf((float)((b_s[t] - b_s[s]) + (double)i_s[s] - (double)m_s[t]));
      p_s[t][s] = w;
    }
  __syncthreads();
  if (tid < MC_L) {
    float dot = w0_s[tid] * dn;
#pragma unroll 16
    for (int s = 0; s < MC_L; ++s) dot += p_s[tid][s];       // zeros above the diagonal
    div_s[tid] = fmaxf(fabsf(dot), expf(-m_s[tid])) + 1e-6f;
  }
  {
    const int c0 = blockIdx.z * MC_L;                        // this workgroup's 64 columns of the values
    float own[4][4] = {}, old[4][4] = {};
    __syncthreads();                                         // k_s is free, div_s is written
    load_tile(k_s, rows + (size_t)2 * heads * d + (size_t)h * dv + c0, (size_t)row_stride, n, dv - c0, 1.f);
    __syncthreads();
#pragma unroll 8
    for (int s = 0; s < MC_L; ++s) {
      float pp[4], vv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) { pp[r] = p_s[ty * 4 + r][s]; vv[r] = k_s[s][tx + 16 * r]; }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) own[r][c] = fmaf(pp[r], vv[c], own[r][c]);
    }
    for (int j0 = 0; j0 < d; j0 += MC_L) {
      const int lim = min(MC_L, d - j0);
      __syncthreads();
      load_tile(q_s, rows + (size_t)h * d + j0, (size_t)row_stride, n, lim, q_scale);
      load_tile(k_s, start + (size_t)j0 * dv + c0, (size_t)dv, lim, dv - c0, 1.f);
      __syncthreads();
#pragma unroll 8
      for (int jj = 0; jj < MC_L; ++jj) {
        float qq[4], cc[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) { qq[r] = q_s[ty * 4 + r][jj]; cc[r] = k_s[jj][tx + 16 * r]; }
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
          for (int c = 0; c < 4; ++c) old[r][c] = fmaf(qq[r], cc[c], old[r][c]);
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int t = ty * 4 + r, col = c0 + tx + 16 * c;
        if (t < n && col < dv)
          out[(size_t)(p.lo + t) * heads * dv + (size_t)h * dv + col] = fmaf(w0_s[t], old[r][c], own[r][c]) / div_s[t];
      }
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

// The chunked form of ta_mlstm_scan.  scratch: float [max_chunks * heads * (d dv + d + 3)], with max_chunks at least the
// number of 64-token chunks of all entries together (rows / 64 + entries is enough).
extern "C" int ta_mlstm_chunked(const void* qkvg, int row_stride, const void* gates, int gate_stride, void* state,
                                long state_stride, const void* cu_q, const void* first_position, const void* state_slots,
                                void* scratch, void* out, int n_entries, int max_chunks, int heads, int d, int dv, float cap,
                                int dtype, hipStream_t stream) {
  if (n_entries <= 0 || max_chunks <= 0) return 0;
  if (d < 1 || dv < 1 || heads < 1 || state_stride < (long)heads * d * dv + (long)heads * d + heads) return -1;
  const size_t total = (size_t)d * dv + d;
  float* local = (float*)scratch;
  float* ends = local + (size_t)max_chunks * heads * total;
  float* m_start = ends + (size_t)max_chunks * heads * 2;
  dim3 per_chunk(max_chunks, heads, (dv + MC_L - 1) / MC_L), per_entry(n_entries, heads, (unsigned)((total + 4 * WAVE - 1) / (4 * WAVE)));
#define CHUNKED(TT)                                                                                                        \
  mlstm_chunk_local_kernel<TT><<<per_chunk, 4 * WAVE, 0, stream>>>((const TT*)qkvg, row_stride, (const float*)gates,        \
      gate_stride, (const int*)cu_q, n_entries, local, ends, heads, d, dv, cap);                                           \
  mlstm_chunk_carry_kernel<<<per_entry, 4 * WAVE, 0, stream>>>((float*)state, (size_t)state_stride, (const int*)cu_q,       \
      (const int*)first_position, (const int*)state_slots, local, ends, m_start, heads, d, dv);                            \
  mlstm_chunk_read_kernel<TT><<<per_chunk, 4 * WAVE, 0, stream>>>((const TT*)qkvg, row_stride, (const float*)gates,         \
      gate_stride, (float*)state, (size_t)state_stride, (const int*)cu_q, (const int*)state_slots, n_entries, local,       \
      ends, m_start, (float*)out, heads, d, dv, cap)
  if (dtype == DT_F32) { CHUNKED(float); } else { CHUNKED(bf16_t); }
#undef CHUNKED
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
