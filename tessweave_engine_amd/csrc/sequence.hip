// Kernels over a step's flat ragged batch that look back along a sequence or carry per-request state:
// a learned position table added to the embedding, a short causal convolution over time with its last
// inputs kept per request (optionally behind an RMS norm), a gated linear recurrence, the per-layer token
// input, and the weighted sum over the results of all earlier layers.
//
// The batch is n_tokens rows grouped by sequence: sequence s owns rows q_start[s] .. q_start[s+1]-1 at
// positions kv_len[s] - q_len .. kv_len[s] - 1. State lives in float32 arrays indexed by the request's
// state slot. Everything here is float32 arithmetic; only inputs that come from a projection and outputs
// that feed one have the compute type.
#include "tw_common.h"

__device__ __forceinline__ float tw_gelu_tanh(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

__device__ __forceinline__ float tw_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }

// The sequence that owns token row `row` (q_start is ascending, q_start[n_seqs] = n_tokens).
__device__ __forceinline__ int tw_seq_of_row(const int* __restrict__ q_start, int n_seqs, int row) {
  int lo = 0, hi = n_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= row) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// ---- x[n] += table[ids[n]]; optionally keep a copy of the sum -------------------------------------------
template <typename T>
__global__ void add_table_rows_kernel(float* __restrict__ x, const T* __restrict__ table, const int* __restrict__ ids,
                                      int width, int rows, float* __restrict__ copy) {
  const int n = blockIdx.x;
  int id = ids[n];
  id = id < 0 ? 0 : (id >= rows ? rows - 1 : id);
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float v = x[(size_t)n * width + c] + tw_to_float(table[(size_t)id * width + c]);
    x[(size_t)n * width + c] = v;
    if (copy) copy[(size_t)n * width + c] = v;
  }
}

extern "C" int tw_add_table_rows(int dtype, float* x, const void* table, const int* ids, int n, int width, int rows,
                                 float* copy, hipStream_t stream) {
  TW_REQUIRE(x && table && ids && n >= 0 && width > 0 && rows > 0);
  if (n == 0) return 0;
  if (dtype == TW_DTYPE_BF16)
    add_table_rows_kernel<bf16_t><<<n, 256, 0, stream>>>(x, (const bf16_t*)table, ids, width, rows, copy);
  else if (dtype == TW_DTYPE_F32)
    add_table_rows_kernel<float><<<n, 256, 0, stream>>>(x, (const float*)table, ids, width, rows, copy);
  else
    return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- short causal convolution over time, with state ------------------------------------------------------
// v_t = NORM ? src_t * rsqrt(mean(src_t^2) + eps) * norm_w : src_t          (per channel c)
// out_t = identity * v_t + sum_j taps[c][j] * v_(t - K + 1 + j) + bias[c]
// Rows before this step's first token of the sequence come from the request's state, rows before the
// sequence's start are zeros. The state holds the last K - 1 values v in order (entry k is position
// len - (K - 1) + k) and exists twice: a step reads copy `phase` and the block of a sequence's last token
// writes copy `1 - phase`, so no block ever reads what another block of the same launch writes.
#define TW_CONV_MAX_TAPS 8

struct ConvArgs {
  const void* src; long ld_src;       // [n][ld_src], channel c at column c
  const float* norm_w;                // NORM only
  const float* row_rinv;              // NORM: rsqrt(mean square + eps) of every row of src, or null (the block sums the rows itself)
  const float* taps;                  // [C][K]
  const float* bias;                  // [C] or null
  float* state;                       // [requests][2][K - 1][C]
  const int* q_start; const int* kv_len; const int* state_slots; const int* phase;
  void* out; long ld_out;             // compute type, or null
  float* out32; long ld_out32;        // float32, or null
  int n_seqs, C, K;
  float eps, identity;
  int act;                            // 0: none; 1: SiLU of the result (after the bias), before the rounding
};

__device__ __forceinline__ float conv_act(float v, int act) { return act == 1 ? v / (1.f + expf(-v)) : v; }
__device__ __forceinline__ f32x4 conv_act(f32x4 v, int act) {
  if (act == 1) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = v[e] / (1.f + expf(-v[e]));
  }
  return v;
}

__device__ __forceinline__ f32x4 conv_load4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 conv_load4(const bf16_t* p) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
  return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
__device__ __forceinline__ void conv_store4(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
__device__ __forceinline__ void conv_store4(bf16_t* p, f32x4 v) {
  *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
}

// VEC: four consecutive channels a thread, 16-byte (8-byte for bfloat16) accesses; the launcher asks for it when
// the channel count, the row strides and the pointers allow.
template <typename SrcT, typename OutT, bool NORM, bool VEC>
__global__ __launch_bounds__(256) void causal_conv_kernel(ConvArgs a) {
  __shared__ float red[TW_CONV_MAX_TAPS][4];
  __shared__ float rinv[TW_CONV_MAX_TAPS];
  const int row = blockIdx.x;
  const int s = tw_seq_of_row(a.q_start, a.n_seqs, row);
  const int first = a.q_start[s], q_len = a.q_start[s + 1] - first;
  const int len = a.kv_len[s];
  const int start = len - q_len;                 // position of the step's first token of this sequence
  const int pos = start + (row - first);
  const int K = a.K, C = a.C;
  const int slot = a.state_slots[s], ph = a.phase[s] & 1;
  const float* old_state = a.state + ((size_t)slot * 2 + ph) * (size_t)(K - 1) * C;
  float* new_state = a.state + ((size_t)slot * 2 + (1 - ph)) * (size_t)(K - 1) * C;
  const bool last = pos == len - 1;
  const SrcT* src = (const SrcT*)a.src;
  // where each tap's row comes from: this step's rows, the state, or nothing (the same for the whole block)
  const SrcT* from_src[TW_CONV_MAX_TAPS];
  const float* from_state[TW_CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < TW_CONV_MAX_TAPS; ++j) {
    const int p = pos - (K - 1) + j;
    from_src[j] = (j < K && p >= start) ? src + (size_t)(first + p - start) * a.ld_src : nullptr;
    from_state[j] = (j < K && p < start && p >= 0) ? old_state + (size_t)(p - start + K - 1) * C : nullptr;
  }
  if (NORM && a.row_rinv) {
    if (threadIdx.x < TW_CONV_MAX_TAPS) {
      const int j = threadIdx.x, p = pos - (K - 1) + j;
      rinv[j] = (j < K && p >= start) ? a.row_rinv[first + p - start] : 0.f;
    }
    __syncthreads();
  } else if (NORM) {
    // every block sums whole rows, whatever share of the channels it then writes
    float sums[TW_CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < TW_CONV_MAX_TAPS; ++j) sums[j] = 0.f;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
#pragma unroll
      for (int j = 0; j < TW_CONV_MAX_TAPS; ++j)
        if (from_src[j]) {
          const float v = tw_to_float(from_src[j][c]);
          sums[j] += v * v;
        }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
    for (int j = 0; j < TW_CONV_MAX_TAPS; ++j) {
      if (j < K) {
        const float t = tw_wave_sum(sums[j]);
        if (lane == 0) red[j][wave] = t;
      }
    }
    __syncthreads();
    if (threadIdx.x < K) {
      const int j = threadIdx.x;
      rinv[j] = rsqrtf((red[j][0] + red[j][1] + red[j][2] + red[j][3]) / (float)C + a.eps);
    }
    __syncthreads();
  }
  const int share = ((C + gridDim.y - 1) / gridDim.y + 3) / 4 * 4;
  const int c_end = min(C, (int)(blockIdx.y + 1) * share);
  if constexpr (VEC) {
    for (int c = blockIdx.y * share + threadIdx.x * 4; c < c_end; c += blockDim.x * 4) {
      f32x4 v[TW_CONV_MAX_TAPS];
#pragma unroll
      for (int j = 0; j < TW_CONV_MAX_TAPS; ++j) {
        v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (from_src[j]) v[j] = conv_load4(from_src[j] + c);
        else if (from_state[j]) v[j] = conv_load4(from_state[j] + c);
      }
      f32x4 acc = a.bias ? conv_load4(a.bias + c) : f32x4{0.f, 0.f, 0.f, 0.f};
      const f32x4 nw = NORM ? conv_load4(a.norm_w + c) : f32x4{1.f, 1.f, 1.f, 1.f};
#pragma unroll
      for (int j = 0; j < TW_CONV_MAX_TAPS; ++j) {
        if (j < K) {
          if (NORM && from_src[j]) v[j] = v[j] * rinv[j] * nw;
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e] += a.taps[(size_t)(c + e) * K + j] * v[j][e];
          if (j == K - 1) acc += a.identity * v[j];
          if (last && j >= 1) conv_store4(new_state + (size_t)(j - 1) * C + c, v[j]);
        }
      }
      acc = conv_act(acc, a.act);
      if (a.out) conv_store4((OutT*)a.out + (size_t)row * a.ld_out + c, acc);
      if (a.out32) conv_store4(a.out32 + (size_t)row * a.ld_out32 + c, acc);
    }
    return;
  }
  for (int c = blockIdx.y * share + threadIdx.x; c < c_end; c += blockDim.x) {
    float v[TW_CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < TW_CONV_MAX_TAPS; ++j) {
      v[j] = 0.f;
      if (from_src[j]) v[j] = tw_to_float(from_src[j][c]);
      else if (from_state[j]) v[j] = from_state[j][c];
    }
    float acc = a.bias ? a.bias[c] : 0.f;
    const float nw = NORM ? a.norm_w[c] : 1.f;
#pragma unroll
    for (int j = 0; j < TW_CONV_MAX_TAPS; ++j) {
      if (j < K) {
        if (NORM && from_src[j]) v[j] = v[j] * rinv[j] * nw;
        acc += a.taps[(size_t)c * K + j] * v[j];
        if (j == K - 1) acc += a.identity * v[j];
        if (last && j >= 1) new_state[(size_t)(j - 1) * C + c] = v[j];
      }
    }
    acc = conv_act(acc, a.act);
    if (a.out) ((OutT*)a.out)[(size_t)row * a.ld_out + c] = tw_from_float<OutT>(acc);
    if (a.out32) a.out32[(size_t)row * a.ld_out32 + c] = acc;
  }
}

// The same convolution for steps of many rows: a block takes TW_CONV_TILE consecutive rows of the flat batch and
// walks them in order, four channels a thread, keeping the last K - 1 inputs in registers: a row is read once
// (plus K - 1 rows where a tile or a sequence's portion begins) instead of K times. With a norm the rows'
// statistics come from `row_rinv`. What a row reads and writes is exactly what `causal_conv_kernel` reads and
// writes for it.
#define TW_CONV_TILE 8
template <typename SrcT, typename OutT, bool NORM>
__global__ __launch_bounds__(256) void causal_conv_tile_kernel(ConvArgs a, int n_tokens) {
  __shared__ int info[TW_CONV_TILE][5];                   // per row of the tile: first row, start, length, slot, phase
  const int row0 = blockIdx.x * TW_CONV_TILE;
  const int rows = min(TW_CONV_TILE, n_tokens - row0);
  if (threadIdx.x < rows) {
    const int s = tw_seq_of_row(a.q_start, a.n_seqs, row0 + threadIdx.x);
    const int first = a.q_start[s], len = a.kv_len[s];
    info[threadIdx.x][0] = first;
    info[threadIdx.x][1] = len - (a.q_start[s + 1] - first);
    info[threadIdx.x][2] = len;
    info[threadIdx.x][3] = a.state_slots[s];
    info[threadIdx.x][4] = a.phase[s] & 1;
  }
  __syncthreads();
  const int K = a.K, C = a.C;
  const SrcT* src = (const SrcT*)a.src;
  for (int c = threadIdx.x * 4; c < C; c += blockDim.x * 4) {
    f32x4 w[TW_CONV_MAX_TAPS];                            // w[j][e]: tap j of channel c + e
#pragma unroll
    for (int j = 0; j < TW_CONV_MAX_TAPS; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) w[j][e] = j < K ? a.taps[(size_t)(c + e) * K + j] : 0.f;
    const f32x4 bias = a.bias ? conv_load4(a.bias + c) : f32x4{0.f, 0.f, 0.f, 0.f};
    const f32x4 nw = NORM ? conv_load4(a.norm_w + c) : f32x4{1.f, 1.f, 1.f, 1.f};
    f32x4 v[TW_CONV_MAX_TAPS];                            // v[j]: the input that meets tap j; v[K - 1] the current row's
    for (int i = 0; i < rows; ++i) {
      const int row = row0 + i;
      const int first = info[i][0], start = info[i][1], len = info[i][2];
      const int pos = start + (row - first);
      const float* old_state = a.state + ((size_t)info[i][3] * 2 + info[i][4]) * (size_t)(K - 1) * C;
      if (i == 0 || row == first) {
        // a tile or a portion begins: the earlier inputs come from this step's rows, the state, or nothing
#pragma unroll
        for (int j = 0; j < TW_CONV_MAX_TAPS - 1; ++j) {
          v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
          const int p = pos - (K - 1) + j;
          if (j < K - 1) {
            if (p >= start) {
              const int r = first + p - start;
              v[j] = conv_load4(src + (size_t)r * a.ld_src + c);
              if (NORM) v[j] = v[j] * a.row_rinv[r] * nw;
            } else if (p >= 0) {
              v[j] = conv_load4(old_state + (size_t)(p - start + K - 1) * C + c);
            }
          }
        }
      }
      f32x4 cur = conv_load4(src + (size_t)row * a.ld_src + c);
      if (NORM) cur = cur * a.row_rinv[row] * nw;
      f32x4 acc = bias + a.identity * cur;
#pragma unroll
      for (int j = 0; j < TW_CONV_MAX_TAPS - 1; ++j)
        if (j < K - 1) acc += w[j] * v[j];
      // (the current row meets the last tap, whose index is only known at run time)
#pragma unroll
      for (int j = 0; j < TW_CONV_MAX_TAPS; ++j)
        if (j == K - 1) acc += w[j] * cur;
      acc = conv_act(acc, a.act);
      if (a.out) conv_store4((OutT*)a.out + (size_t)row * a.ld_out + c, acc);
      if (a.out32) conv_store4(a.out32 + (size_t)row * a.ld_out32 + c, acc);
      // shift: what met tap j + 1 meets tap j for the next row
#pragma unroll
      for (int j = 0; j < TW_CONV_MAX_TAPS - 2; ++j)
        if (j < K - 2) v[j] = v[j + 1];
#pragma unroll
      for (int j = 0; j < TW_CONV_MAX_TAPS - 1; ++j)
        if (j == K - 2) v[j] = cur;
      if (pos == len - 1) {
        float* new_state = a.state + ((size_t)info[i][3] * 2 + (1 - info[i][4])) * (size_t)(K - 1) * C;
#pragma unroll
        for (int j = 0; j < TW_CONV_MAX_TAPS - 1; ++j)
          if (j < K - 1) conv_store4(new_state + (size_t)j * C + c, v[j]);
      }
    }
  }
}

// rinv[n] = rsqrt(mean(x[n]^2) + eps): one wave a row.
__global__ __launch_bounds__(256) void row_rinv_kernel(const float* __restrict__ x, long ld, float* __restrict__ rinv, int n, int C, float eps) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= n) return;
  const float* r = x + (size_t)row * ld;
  float sum = 0.f;
  if ((C & 3) == 0 && (ld & 3) == 0 && ((uintptr_t)x & 15) == 0) {
    for (int c = lane * 4; c < C; c += 256) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(r + c);
      sum += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
  } else {
    for (int c = lane; c < C; c += 64) sum += r[c] * r[c];
  }
  sum = tw_wave_sum(sum);
  if (lane == 0) rinv[row] = rsqrtf(sum / (float)C + eps);
}

// src_kind: 0 float32 rows, 1 rows of the compute type. norm_w non-null: RMS norm of the source rows first
// (float32 rows only).
extern "C" int tw_causal_conv(int dtype, int src_f32, const void* src, long ld_src, const float* norm_w, float eps,
                              const float* taps, const float* bias, float identity, float* state,
                              const int* q_start, const int* kv_len, const int* state_slots, const int* phase,
                              void* out, long ld_out, float* out32, long ld_out32, int n_tokens, int n_seqs,
                              int C, int K, float* row_scratch, int act, hipStream_t stream) {
  TW_REQUIRE(src && taps && state && q_start && kv_len && state_slots && phase && (out || out32));
  TW_REQUIRE(act == 0 || act == 1);
  TW_REQUIRE(n_tokens >= 0 && n_seqs >= 1 && C > 0 && K >= 1 && K <= TW_CONV_MAX_TAPS);
  TW_REQUIRE(ld_src >= C && (!out || ld_out >= C) && (!out32 || ld_out32 >= C));
  TW_REQUIRE(!norm_w || src_f32);
  if (n_tokens == 0) return 0;
  // many rows behind a norm: the rows' sums of squares are formed once, by a kernel of their own, instead of
  // `taps` times over by the blocks that need them (row_scratch: n_tokens floats)
  const float* row_rinv = nullptr;
  if (norm_w && row_scratch && n_tokens >= 512) {
    row_rinv_kernel<<<tw_div_up(n_tokens, 4), 256, 0, stream>>>((const float*)src, ld_src, row_scratch, n_tokens, C, eps);
    row_rinv = row_scratch;
  }
  ConvArgs a{src, ld_src, norm_w, row_rinv, taps, bias, state, q_start, kv_len, state_slots, phase,
             out, ld_out, out32, ld_out32, n_seqs, C, K, eps, identity, act};
  const bool bf = dtype == TW_DTYPE_BF16;
  TW_REQUIRE(bf || dtype == TW_DTYPE_F32);
  // few rows (decode steps): the channels are shared out over several blocks a row
  int shares = n_tokens >= 512 ? 1 : tw_div_up(C, 512);
  if (shares > 8) shares = 8;
  const dim3 n_blocks(n_tokens, shares);
  const int esize = bf ? 2 : 4, ssize = src_f32 ? 4 : esize;
  const bool vec = C % 4 == 0 && ld_src % 4 == 0 && (uintptr_t)src % (4 * ssize) == 0 &&
                   (!out || (ld_out % 4 == 0 && (uintptr_t)out % (4 * esize) == 0)) &&
                   (!out32 || (ld_out32 % 4 == 0 && (uintptr_t)out32 % 16 == 0)) && (uintptr_t)state % 16 == 0 &&
                   (!bias || (uintptr_t)bias % 16 == 0) && (!norm_w || (uintptr_t)norm_w % 16 == 0);
  const bool tiled = vec && n_tokens >= 512 && (!norm_w || row_rinv);
#define TW_CONV_LAUNCH(S, O, N)                                                                    \
  do {                                                                                             \
    if (tiled) causal_conv_tile_kernel<S, O, N><<<tw_div_up(n_tokens, TW_CONV_TILE), 256, 0, stream>>>(a, n_tokens); \
    else if (vec) causal_conv_kernel<S, O, N, true><<<n_blocks, 256, 0, stream>>>(a);              \
    else causal_conv_kernel<S, O, N, false><<<n_blocks, 256, 0, stream>>>(a);                      \
  } while (0)
  if (norm_w) {
    if (bf) TW_CONV_LAUNCH(float, bf16_t, true); else TW_CONV_LAUNCH(float, float, true);
  } else if (src_f32) {
    if (bf) TW_CONV_LAUNCH(float, bf16_t, false); else TW_CONV_LAUNCH(float, float, false);
  } else {
    if (bf) TW_CONV_LAUNCH(bf16_t, bf16_t, false); else TW_CONV_LAUNCH(float, float, false);
  }
#undef TW_CONV_LAUNCH
  return TW_LAUNCH_RESULT();
}

// ---- gated linear recurrence ---------------------------------------------------------------------------------
// Per sequence and channel, over the step's tokens in order:
//   r = sigmoid(gates[t][ga(c)]), i = sigmoid(gates[t][gi(c)])
//   a = exp(-decay * r * softplus(lam[c]))
//   S = a * S + sqrt(1 - a^2) * i * u[t][c]                 (S float32, kept per request)
//   out[t][c] = out_scale * S * gelu_tanh(branch[t][c])
// The gates of block b (bs = C / blocks channels) lie at columns [2 b bs, 2 b bs + bs) (recurrence gate)
// and [2 b bs + bs, 2 (b + 1) bs) (input gate): one packed product per block wrote them.
struct RecurrenceArgs {
  const float* gates; long ld_gates;
  const float* u; long ld_u;
  const void* branch; long ld_branch;
  const float* lam;
  float* state;                       // [requests][C]
  const int* q_start; const int* state_slots;
  void* out; long ld_out;
  int C, block_size;
  float decay, out_scale;
  int chunk;                          // tokens a thread walks; a sequence's portion is cut into chunks of this length
  int max_chunks;                     // chunks of the longest portion of the launch (1: no cutting, one kernel)
  float* part;                        // max_chunks > 1: [seq][max_chunks][3][C]: product of a, state from zero, (chunk 0) state before
  int out_pad;                        // columns [C, C + out_pad) of out are set to zero
};

// One step of the recurrence from the step's loaded inputs (recurrence gate, input gate, u); returns a_t and
// updates S.
__device__ __forceinline__ float recurrence_update(float gate_a, float gate_i, float u, float unit, float& S) {
  const float r = tw_sigmoid(gate_a);
  const float i = tw_sigmoid(gate_i);
  const float la = -unit * r;
  const float dec = expf(la);
  const float norm = sqrtf(fmaxf(0.f, -expm1f(2.f * la)));          // sqrt(1 - a^2) without cancellation
  S = dec * S + norm * i * u;
  return dec;
}

// One step of the recurrence for channel c at token t; returns a_t and adds into S.
__device__ __forceinline__ float recurrence_step(const RecurrenceArgs& a, int t, int c, int ga, int gi, float unit, float& S) {
  const float r = tw_sigmoid(a.gates[(size_t)t * a.ld_gates + ga]);
  const float i = tw_sigmoid(a.gates[(size_t)t * a.ld_gates + gi]);
  const float la = -unit * r;
  const float dec = expf(la);
  const float norm = sqrtf(fmaxf(0.f, -expm1f(2.f * la)));          // sqrt(1 - a^2) without cancellation
  S = dec * S + norm * i * a.u[(size_t)t * a.ld_u + c];
  return dec;
}

// FINAL false: a chunk's product of decays and its state from zero (and, chunk 0, the state before the step) go
// to `part`. FINAL true: the chunk's true start state is rebuilt from the chunks before it, the chunk is walked
// again and the outputs are written; the sequence's last chunk leaves the new state. A portion of one chunk
// (every decode step) needs the FINAL kernel only and reads the state itself.
template <typename T, bool FINAL>
__global__ __launch_bounds__(256) void gated_recurrence_kernel(RecurrenceArgs a) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int s = blockIdx.y, z = blockIdx.z;
  const int first = a.q_start[s], end = a.q_start[s + 1];
  const int n_chunks = (end - first + a.chunk - 1) / a.chunk;
  if (z >= n_chunks) return;
  const int t0 = first + z * a.chunk, t1 = min(end, t0 + a.chunk);
  T* out = (T*)a.out;
  if (FINAL && c >= a.C) {
    if (c < a.C + a.out_pad)
      for (int t = t0; t < t1; ++t) out[(size_t)t * a.ld_out + c] = tw_from_float<T>(0.f);
    return;
  }
  if (c >= a.C) return;
  float* st = a.state + (size_t)a.state_slots[s] * a.C + c;
  const float lam = a.lam[c];
  const float unit = a.decay * (lam > 20.f ? lam : log1pf(expf(lam)));
  const int b = c / a.block_size, k = c % a.block_size;
  const int ga = 2 * b * a.block_size + k, gi = ga + a.block_size;
  float* part = a.part ? a.part + ((size_t)s * a.max_chunks) * 3 * a.C + c : nullptr;
  if (!FINAL) {
    if (n_chunks == 1) return;
    float S = 0.f, P = 1.f;
    int t = t0;
    for (; t + 4 <= t1; t += 4) {                 // four steps' inputs requested together: the walk waits for memory once in four
      float xa[4], xi[4], xu[4];
#pragma unroll
      for (int k2 = 0; k2 < 4; ++k2) {
        xa[k2] = a.gates[(size_t)(t + k2) * a.ld_gates + ga];
        xi[k2] = a.gates[(size_t)(t + k2) * a.ld_gates + gi];
        xu[k2] = a.u[(size_t)(t + k2) * a.ld_u + c];
      }
#pragma unroll
      for (int k2 = 0; k2 < 4; ++k2) P *= recurrence_update(xa[k2], xi[k2], xu[k2], unit, S);
    }
    for (; t < t1; ++t) P *= recurrence_step(a, t, c, ga, gi, unit, S);
    part[((size_t)z * 3 + 0) * a.C] = P;
    part[((size_t)z * 3 + 1) * a.C] = S;
    if (z == 0) part[2 * (size_t)a.C] = *st;
    return;
  }
  float S;
  if (n_chunks == 1) {
    S = *st;
  } else {
    S = part[2 * (size_t)a.C];
    for (int j = 0; j < z; ++j) S = part[((size_t)j * 3 + 0) * a.C] * S + part[((size_t)j * 3 + 1) * a.C];
  }
  const T* branch = (const T*)a.branch;
  int t = t0;
  for (; t + 4 <= t1; t += 4) {
    float xa[4], xi[4], xu[4], xb[4];
#pragma unroll
    for (int k2 = 0; k2 < 4; ++k2) {
      xa[k2] = a.gates[(size_t)(t + k2) * a.ld_gates + ga];
      xi[k2] = a.gates[(size_t)(t + k2) * a.ld_gates + gi];
      xu[k2] = a.u[(size_t)(t + k2) * a.ld_u + c];
      xb[k2] = tw_to_float(branch[(size_t)(t + k2) * a.ld_branch + c]);
    }
#pragma unroll
    for (int k2 = 0; k2 < 4; ++k2) {
      recurrence_update(xa[k2], xi[k2], xu[k2], unit, S);
      out[(size_t)(t + k2) * a.ld_out + c] = tw_from_float<T>(a.out_scale * S * tw_gelu_tanh(xb[k2]));
    }
  }
  for (; t < t1; ++t) {
    recurrence_step(a, t, c, ga, gi, unit, S);
    const float y = tw_gelu_tanh(tw_to_float(branch[(size_t)t * a.ld_branch + c]));
    out[(size_t)t * a.ld_out + c] = tw_from_float<T>(a.out_scale * S * y);
  }
  if (z == n_chunks - 1) *st = S;
}

#define TW_RECURRENCE_CHUNK 32

extern "C" long tw_gated_recurrence_workspace_floats(int n_seqs, int max_q_len, int C) {
  const int chunks = tw_div_up(max_q_len, TW_RECURRENCE_CHUNK);
  return chunks > 1 ? (long)n_seqs * chunks * 3 * C : 0;
}

extern "C" int tw_gated_recurrence(int dtype, const float* gates, long ld_gates, const float* u, long ld_u,
                                   const void* branch, long ld_branch, const float* lam, float* state,
                                   const int* q_start, const int* state_slots, void* out, long ld_out, int n_seqs,
                                   int max_q_len, int C, int blocks, int out_pad, float decay, float out_scale,
                                   float* workspace, long workspace_floats, hipStream_t stream) {
  TW_REQUIRE(gates && u && branch && lam && state && q_start && state_slots && out);
  TW_REQUIRE(n_seqs >= 0 && max_q_len >= 1 && C > 0 && blocks > 0 && C % blocks == 0 && out_pad >= 0);
  TW_REQUIRE(ld_gates >= 2 * C && ld_u >= C && ld_branch >= C && ld_out >= C + out_pad);
  if (n_seqs == 0) return 0;
  const int chunks = tw_div_up(max_q_len, TW_RECURRENCE_CHUNK);
  TW_REQUIRE(chunks == 1 || (workspace && workspace_floats >= tw_gated_recurrence_workspace_floats(n_seqs, max_q_len, C)));
  RecurrenceArgs a{gates, ld_gates, u, ld_u, branch, ld_branch, lam, state, q_start, state_slots, out, ld_out,
                   C, C / blocks, decay, out_scale, TW_RECURRENCE_CHUNK, chunks, chunks > 1 ? workspace : nullptr, out_pad};
  TW_REQUIRE(dtype == TW_DTYPE_BF16 || dtype == TW_DTYPE_F32);
  const dim3 grid_part(tw_div_up(C, 256), n_seqs, chunks), grid(tw_div_up(C + out_pad, 256), n_seqs, chunks);
  if (chunks > 1) {
    if (dtype == TW_DTYPE_BF16) gated_recurrence_kernel<bf16_t, false><<<grid_part, 256, 0, stream>>>(a);
    else gated_recurrence_kernel<float, false><<<grid_part, 256, 0, stream>>>(a);
  }
  if (dtype == TW_DTYPE_BF16) gated_recurrence_kernel<bf16_t, true><<<grid, 256, 0, stream>>>(a);
  else gated_recurrence_kernel<float, true><<<grid, 256, 0, stream>>>(a);
  return TW_LAUNCH_RESULT();
}

// ---- block-diagonal product: out[n][b * No + o] = sum_i x[n][b * Ni + i] * w[b][o][i] + bias[b * No + o] ---------
// `blocks` square-ish matrices [No][Ni] side by side along the diagonal (the gates of a recurrence read only
// their own block of channels). One wave takes 16 rows and 64 output columns of one block: the weights are the
// A operand (so a lane ends with 4 consecutive output columns of one row), the rows the B operand, both read
// straight from memory in 16-byte fragments. Ni must be a multiple of 16 bytes, No of 16.
template <typename T>
__global__ __launch_bounds__(256) void block_diagonal_kernel(const T* __restrict__ x, long ldx, const T* __restrict__ w,
                                                             const float* __restrict__ bias, float* __restrict__ out,
                                                             long ldo, int n, int blocks, int Ni, int No, int col_groups) {
  typedef typename Elem<T>::Frag Frag;
  constexpr int EPF = Elem<T>::kPerFrag;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int unit = blockIdx.x * 4 + wave;                  // (block, group of 64 columns)
  const int b = unit / col_groups, cg = unit % col_groups;
  if (b >= blocks) return;
  const int row0 = blockIdx.y * 16;
  const int chunks = Ni / EPF, steps = (chunks + 3) / 4;
  const int row = row0 + r;
  const T* x_row = x + (size_t)(row < n ? row : 0) * ldx + (size_t)b * Ni;
  f32x4 acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int st = 0; st < steps; ++st) {
    const int chunk = st * 4 + g;
    const bool in = chunk < chunks;
    const Frag xf = (in && row < n) ? tw_load_frag(x_row + chunk * EPF) : Elem<T>::zero();
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int o = cg * 64 + t * 16 + r;
      const Frag wf = (in && o < No) ? tw_load_frag(w + ((size_t)b * No + o) * Ni + chunk * EPF) : Elem<T>::zero();
      tw_mma16(acc[t], wf, xf);                            // D[output 4g + e][row r]
    }
  }
  if (row >= n) return;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int o = cg * 64 + t * 16 + 4 * g;
    if (o < No) {
      f32x4 v = acc[t];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] += bias ? bias[(size_t)b * No + o + e] : 0.f;
      *reinterpret_cast<f32x4*>(out + (size_t)row * ldo + (size_t)b * No + o) = v;
    }
  }
}

extern "C" int tw_block_diagonal(int dtype, const void* x, long ldx, const void* w, const float* bias, float* out,
                                 long ldo, int n, int blocks, int Ni, int No, hipStream_t stream) {
  const int epf = dtype == TW_DTYPE_BF16 ? 8 : 4;
  TW_REQUIRE(x && w && out && n >= 0 && blocks > 0 && Ni > 0 && No > 0);
  TW_REQUIRE(dtype == TW_DTYPE_BF16 || dtype == TW_DTYPE_F32);
  TW_REQUIRE(Ni % epf == 0 && No % 16 == 0 && ldx % epf == 0 && ldx >= (long)blocks * Ni && ldo % 4 == 0 && ldo >= (long)blocks * No);
  TW_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)out % 16 == 0);
  if (n == 0) return 0;
  const int col_groups = tw_div_up(No, 64);
  const dim3 grid(tw_div_up((long)blocks * col_groups, 4), tw_div_up(n, 16));
  if (dtype == TW_DTYPE_BF16)
    block_diagonal_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, bias, out, ldo, n, blocks, Ni, No, col_groups);
  else
    block_diagonal_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, ldx, (const float*)w, bias, out, ldo, n, blocks, Ni, No, col_groups);
  return TW_LAUNCH_RESULT();
}

// ---- out = scale * act(gate) * up for [n][2F] rows holding gate | up -------------------------------------------
template <typename T>
__global__ void gelu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, long n, int inter, float scale) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n * inter) return;
  const long row = i / inter;
  const int col = (int)(i % inter);
  const float g = tw_to_float(gu[row * 2 * inter + col]), u = tw_to_float(gu[row * 2 * inter + inter + col]);
  out[i] = tw_from_float<T>(scale * tw_gelu_tanh(g) * u);
}

extern "C" int tw_gelu_mul(int dtype, const void* gu, void* out, int n, int inter, float scale, hipStream_t stream) {
  TW_REQUIRE(gu && out && n >= 0 && inter > 0);
  if (n == 0) return 0;
  const long total = (long)n * inter;
  const int blocks = tw_div_up(total, 256);
  if (dtype == TW_DTYPE_BF16) gelu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, n, inter, scale);
  else if (dtype == TW_DTYPE_F32) gelu_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)out, n, inter, scale);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- float32 rows rounded to the compute type ------------------------------------------------------------------
template <typename T>
__global__ void round_rows_kernel(const float* __restrict__ x, T* __restrict__ out, long total) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) out[i] = tw_from_float<T>(x[i]);
}

extern "C" int tw_round_rows(int dtype, const float* x, void* out, long total, hipStream_t stream) {
  TW_REQUIRE(x && out && total >= 0);
  if (total == 0) return 0;
  const int blocks = tw_div_up(total, 256);
  if (dtype == TW_DTYPE_BF16) round_rows_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, (bf16_t*)out, total);
  else if (dtype == TW_DTYPE_F32) round_rows_kernel<float><<<blocks, 256, 0, stream>>>(x, (float*)out, total);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- the per-layer token input's gate: out[n][k] = gelu_tanh(pre[n][k]) * table[token n][offset + k] ------------
template <typename T>
__global__ void token_gate_kernel(const float* __restrict__ pre, const T* __restrict__ table, long ld_table,
                                  const int* __restrict__ ids, const int* __restrict__ feed, int n_feed, int vocab,
                                  int offset, T* __restrict__ out, int n, int dim) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)n * dim) return;
  const int row = (int)(i / dim), k = (int)(i % dim);
  int id = ids[row];
  if (id < 0) id = (feed && -1 - id < n_feed) ? feed[-1 - id] : 0;
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  out[i] = tw_from_float<T>(tw_gelu_tanh(pre[i]) * tw_to_float(table[(size_t)id * ld_table + offset + k]));
}

extern "C" int tw_token_gate(int dtype, const float* pre, const void* table, long ld_table, const int* ids,
                             const int* feed, int n_feed, int vocab, int offset, void* out, int n, int dim,
                             hipStream_t stream) {
  TW_REQUIRE(pre && table && ids && out && n >= 0 && dim > 0 && offset >= 0 && offset + dim <= ld_table && vocab > 0);
  if (n == 0) return 0;
  const int blocks = tw_div_up((long)n * dim, 256);
  if (dtype == TW_DTYPE_BF16)
    token_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(pre, (const bf16_t*)table, ld_table, ids, feed, n_feed, vocab, offset, (bf16_t*)out, n, dim);
  else if (dtype == TW_DTYPE_F32)
    token_gate_kernel<float><<<blocks, 256, 0, stream>>>(pre, (const float*)table, ld_table, ids, feed, n_feed, vocab, offset, (float*)out, n, dim);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- end of a layer: add a unit-norm branch, keep the layer's result, mix the results so far --------------------
//   if y:  x[n] += mult * y[n] * rsqrt(mean(y[n]^2) + eps) * w
//   history[layer + 1][n] = x[n]
//   if mix: x[n] = sum_{j <= layer + 1} mix[j] * history[j][n]
// history[j] lies at history + j * history_stride.
__global__ __launch_bounds__(256) void layer_end_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                        const float* __restrict__ w, float eps, float mult,
                                                        float* __restrict__ history, long history_stride, int layer,
                                                        const float* __restrict__ mix, int width) {
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * width;
  float scale = 0.f;
  if (y) {
    float sum = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      const float v = y[row + c];
      sum += v * v;
    }
    sum = tw_block_sum(sum, red);
    scale = mult * rsqrtf(sum / (float)width + eps);
  }
  const int share = (width + gridDim.y - 1) / gridDim.y;
  const int c_end = min(width, (int)(blockIdx.y + 1) * share);
  for (int c = blockIdx.y * share + threadIdx.x; c < c_end; c += blockDim.x) {
    float v = x[row + c];
    if (y) v += scale * y[row + c] * w[c];
    if (history) history[(size_t)(layer + 1) * history_stride + row + c] = v;
    if (mix) {
      float acc = mix[layer + 1] * v;
      int j = 0;
      for (; j + 4 <= layer + 1; j += 4) {
        const float h0 = history[(size_t)j * history_stride + row + c], h1 = history[(size_t)(j + 1) * history_stride + row + c];
        const float h2 = history[(size_t)(j + 2) * history_stride + row + c], h3 = history[(size_t)(j + 3) * history_stride + row + c];
        acc += mix[j] * h0 + mix[j + 1] * h1 + mix[j + 2] * h2 + mix[j + 3] * h3;
      }
      for (; j <= layer; ++j) acc += mix[j] * history[(size_t)j * history_stride + row + c];
      v = acc;
    }
    x[row + c] = v;
  }
}

extern "C" int tw_layer_end(float* x, const float* y, const float* w, float eps, float mult, float* history,
                            long history_stride, int layer, const float* mix, int n, int width, hipStream_t stream) {
  TW_REQUIRE(x && n >= 0 && width > 0 && layer >= 0 && (!y || w) && (!mix || history));
  TW_REQUIRE(!history || history_stride >= (long)n * width);
  if (n == 0) return 0;
  int shares = n >= 512 ? 1 : tw_div_up(width, 512);
  if (shares > 8) shares = 8;
  layer_end_kernel<<<dim3(n, shares), 256, 0, stream>>>(x, y, w, eps, mult, history, history_stride, layer, mix, width);
  return TW_LAUNCH_RESULT();
}

// ---- token embedding plus a row of a hashed pair table, then an RMS norm -------------------------------------------
// x[n] = w * unit(scale * table[token n] + pairs[r(n)]),  r = (previous token * mul_prev + token * mul_cur) mod
// buckets, and r = buckets (the table's last row) for a sequence's first token. The token before a step's first
// token of a sequence is part of the request's state: int32 [requests][2], copy `phase` read, the other copy
// written by the block of the sequence's last token (so no block reads what another block of the launch writes).
// A token id -1 - k stands for feed[k]. The normed row goes to x (float32) and, rounded, to out.
template <typename T>
__global__ __launch_bounds__(256) void embed_hashed_kernel(
    const int* __restrict__ ids, const int* __restrict__ feed, int n_feed, const T* __restrict__ table,
    const T* __restrict__ pairs, const float* __restrict__ norm_w, const int* __restrict__ q_start,
    const int* __restrict__ kv_len, const int* __restrict__ state_slots, const int* __restrict__ phase,
    int* __restrict__ state, int n_seqs, int hidden, int vocab, long buckets, long mul_prev, long mul_cur, float scale,
    float eps, float* __restrict__ x, T* __restrict__ out) {
  __shared__ float lds[16];
  const int row = blockIdx.x;
  const int s = tw_seq_of_row(q_start, n_seqs, row);
  const int first = q_start[s], q_len = q_start[s + 1] - first;
  const int start = kv_len[s] - q_len;
  const int slot = state_slots[s], ph = phase[s] & 1;
  auto resolve = [&](int id) {
    if (id < 0) id = (feed && -1 - id < n_feed) ? feed[-1 - id] : 0;
    return id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  };
  const int token = resolve(ids[row]);
  long pair_row = buckets;
  if (row > first) {
    pair_row = ((long)resolve(ids[row - 1]) * mul_prev + (long)token * mul_cur) % buckets;
  } else if (start > 0) {
    pair_row = ((long)state[slot * 2 + ph] * mul_prev + (long)token * mul_cur) % buckets;
  }
  if (row == first + q_len - 1 && threadIdx.x == 0) state[slot * 2 + (1 - ph)] = token;
  const T* e = table + (size_t)token * hidden;
  const T* p = pairs + (size_t)pair_row * hidden;
  float* xr = x + (size_t)row * hidden;
  float ss = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float v = __fmaf_rn(scale, tw_to_float(e[c]), tw_to_float(p[c]));
    xr[c] = v;
    ss = __fmaf_rn(v, v, ss);
  }
  const float total = tw_block_sum(ss, lds);
  const float rinv = 1.f / sqrtf(total / (float)hidden + eps);
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float r = xr[c] * rinv * norm_w[c];
    xr[c] = r;
    if (out) out[(size_t)row * hidden + c] = tw_from_float<T>(r);
  }
}

extern "C" int tw_embed_hashed(int dtype, const int* ids, const int* feed, int n_feed, const void* table,
                               const void* pairs, const float* norm_w, const int* q_start, const int* kv_len,
                               const int* state_slots, const int* phase, int* state, int n, int n_seqs, int hidden,
                               int vocab, long buckets, long mul_prev, long mul_cur, float scale, float eps, float* x,
                               void* out, hipStream_t stream) {
  TW_REQUIRE(ids && table && pairs && norm_w && q_start && kv_len && state_slots && phase && state && x);
  TW_REQUIRE(n >= 0 && n_seqs > 0 && hidden > 0 && vocab > 0 && buckets > 0 && mul_prev >= 0 && mul_cur >= 0 && eps > 0.f);
  if (n == 0) return 0;
  if (dtype == TW_DTYPE_BF16)
    embed_hashed_kernel<bf16_t><<<n, 256, 0, stream>>>(ids, feed, n_feed, (const bf16_t*)table, (const bf16_t*)pairs, norm_w,
                                                       q_start, kv_len, state_slots, phase, state, n_seqs, hidden, vocab,
                                                       buckets, mul_prev, mul_cur, scale, eps, x, (bf16_t*)out);
  else if (dtype == TW_DTYPE_F32)
    embed_hashed_kernel<float><<<n, 256, 0, stream>>>(ids, feed, n_feed, (const float*)table, (const float*)pairs, norm_w,
                                                      q_start, kv_len, state_slots, phase, state, n_seqs, hidden, vocab,
                                                      buckets, mul_prev, mul_cur, scale, eps, x, (float*)out);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}
