// The matrix memory of the mLSTM: per head a state S [D][E], a normaliser n [D] and a running maximum m of the gates'
// logarithms, all float32 and all zero (m too) when a request opens. Per token, with the log input gate i and the log
// forget gate f (both capped: i = cap tanh(z_i / cap), f = logsigmoid(cap tanh(z_f / cap))):
//
//   m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k alone;
//   o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)
//
// q, k, v and the gates' raw values come as float32 rows of one packed product; everything here is float32.
// State layout: S [requests][H][Ep][Dp] (a value column's keys are contiguous; Dp, Ep: D and E rounded up to 16, the
// tails are zeros), n [requests][2][H][Dp] and m [requests][2][H] held twice: a step reads copy phase[s] and writes the
// other (several workgroups of a head read n and m while one of them writes).
//
// mlstm_walk: sequences of a few tokens, token by token. A workgroup owns 16 value columns of one (sequence, head);
// lane 16 c + s keeps the keys s, s + 16, .. of column c (and of n) in registers; a token's two products are a few
// multiply-adds and a sum over 16 neighbouring lanes.
//
// mlstm_chunk: longer portions, 16 tokens at once on the matrix unit (float32 products). With F_t the running sum of
// f inside the chunk, u_j = i_j - F_j, g_t = max(m0, max_{j <= t} u_j) and m_t = F_t + g_t:
//   o_t  = [ exp(m0 - g_t) S0^T q_t + sum_{j <= t} exp(u_j - g_t) (q_t . k_j) v_j ] / (max(|nq_t|, exp(-m_t)) + 1e-6)
//   nq_t =   exp(m0 - g_t) n0 . q_t + sum_{j <= t} exp(u_j - g_t) (q_t . k_j)
//   S    =   exp(m0 - g_last) S0 + sum_j exp(u_j - g_last) k_j v_j^T,   n likewise,   m = m_last
// (every exponent is at most 0). A workgroup owns up to 64 value columns of one (sequence, head), a wave 16 of them; a
// wave's part of S stays in registers in the layout that is both the accumulator of K'^T V and the B operand of Q S.
#include "tw_common.h"

struct MlstmArgs {
  const float* proj; long ld;        // a token's row: q at q_col + h D, k at k_col + h D, v at v_col + h E,
  int q_col, k_col, v_col;           // the gates' raw values at i_col + h and f_col + h
  int i_col, f_col;
  const float* i_bias; const float* f_bias;   // [H]
  float* S; float* n; float* m;
  const int* q_start; const int* state_slots; const int* phase;
  int seq0;
  float* out; long ld_out;           // [rows][H E]
  int H, D, E, Dp, Ep;
  float q_scale, cap;
  int gates_ready;                   // the rows hold i and f already (mlstm_gates_kernel ran), not the gates' raw values
};

// Inside a row of 16 lanes (DPP): the value of the lane N below (FILL where there is none), and the sum over the row.
template <int N>
__device__ __forceinline__ float ml_row_below(float v, float fill) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fill), __float_as_int(v), 0x110 + N, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ float ml_row_turned(float v) {
  return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float ml_row_sum(float v) {      // every lane of the row gets it
  v += ml_row_turned<0x128>(v);                             // the row rotated by 8 lanes, then by 4, 2, 1
  v += ml_row_turned<0x124>(v);
  v += ml_row_turned<0x122>(v);
  v += ml_row_turned<0x121>(v);
  return v;
}

__device__ __forceinline__ float ml_logsigmoid(float z) { return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z)); }

__device__ __forceinline__ void ml_gates(const MlstmArgs& a, const float* row, int head, float& i_log, float& f_log) {
  i_log = a.cap * tanhf((row[a.i_col + head] + a.i_bias[head]) / a.cap);
  f_log = ml_logsigmoid(a.cap * tanhf((row[a.f_col + head] + a.f_bias[head]) / a.cap));
}

// grid (Ep / 16, H, n_seqs), 256 threads
__global__ __launch_bounds__(256) void mlstm_walk_kernel(MlstmArgs a) {
  const int seq = a.seq0 + blockIdx.z, head = blockIdx.y;
  const int col = threadIdx.x >> 4, sl = threadIdx.x & 15;
  const int v = blockIdx.x * 16 + col;
  const int r0 = a.q_start[seq], r1 = a.q_start[seq + 1];
  if (r1 <= r0) return;
  const int slot = a.state_slots[seq], ph = a.phase[seq] & 1;
  const int J = a.Dp / 16;
  float* S = a.S + (((size_t)slot * a.H + head) * a.Ep + v) * a.Dp;
  const float* n_in = a.n + (((size_t)slot * 2 + ph) * a.H + head) * a.Dp;
  float* n_out = a.n + (((size_t)slot * 2 + (ph ^ 1)) * a.H + head) * a.Dp;
  float s[16], nn[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    s[j] = j < J ? S[sl + 16 * j] : 0.f;
    nn[j] = j < J ? n_in[sl + 16 * j] : 0.f;
  }
  float m = a.m[((size_t)slot * 2 + ph) * a.H + head];
  for (int row_i = r0; row_i < r1; ++row_i) {
    const float* row = a.proj + (size_t)row_i * a.ld;
    float i_log, f_log;
    ml_gates(a, row, head, i_log, f_log);
    const float m_new = fmaxf(f_log + m, i_log);
    const float keep = expf(f_log + m - m_new), take = expf(i_log - m_new);
    m = m_new;
    const float vv = v < a.E ? row[a.v_col + head * a.E + v] : 0.f;
    const float* q = row + a.q_col + head * a.D;
    const float* k = row + a.k_col + head * a.D;
    float po = 0.f, pn = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      if (j < J) {
        const int d = sl + 16 * j;
        const float kd = d < a.D ? k[d] : 0.f, qd = d < a.D ? q[d] * a.q_scale : 0.f;
        const float tk = take * kd;
        s[j] = __fmaf_rn(keep, s[j], tk * vv);
        nn[j] = __fmaf_rn(keep, nn[j], tk);
        po = __fmaf_rn(s[j], qd, po);
        pn = __fmaf_rn(nn[j], qd, pn);
      }
    }
    po = ml_row_sum(po);
    pn = ml_row_sum(pn);
    if (sl == 0 && v < a.E)
      a.out[(size_t)row_i * a.ld_out + head * a.E + v] = po / (fmaxf(fabsf(pn), expf(-m)) + 1e-6f);
  }
#pragma unroll
  for (int j = 0; j < 16; ++j)
    if (j < J) S[sl + 16 * j] = s[j];
  if (blockIdx.x == 0) {
    if (col == 0) {
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (j < J) n_out[sl + 16 * j] = nn[j];
    }
    if (threadIdx.x == 0) a.m[((size_t)slot * 2 + (ph ^ 1)) * a.H + head] = m;
  }
}

// grid (ceil(Ep / 64), H, n_seqs), 256 threads; dynamic LDS (ml_chunk_lds_floats).
// A chunk's rows are held twice in LDS and requested TWO chunks ahead: while chunk c is worked on, the rows of chunks
// c + 1 and c + 2 are in registers or on their way there from memory (a load takes longer than a chunk's arithmetic), and
// go to the other copy in LDS at the top of their iteration, so an iteration has two barriers and hardly waits for memory.
#define ML_L 16
static size_t ml_buffer_floats(int Dp) { return (size_t)2 * ML_L * (Dp + 4) + (size_t)ML_L * 68 + 6 * ML_L; }
static size_t ml_chunk_lds_floats(int Dp) { return 2 * ml_buffer_floats(Dp) + 4 * 64 * 4 + Dp + ML_L; }

template <int DT>      // key tiles of 16 a wave's part of S spans in registers (Dp <= 16 DT)
__global__ __launch_bounds__(256) void mlstm_chunk_kernel(MlstmArgs a) {
  extern __shared__ __attribute__((aligned(16))) float ml_lds[];
  const int seq = a.seq0 + blockIdx.z, head = blockIdx.y;
  const int r0 = a.q_start[seq], r1 = a.q_start[seq + 1];
  if (r1 <= r0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int Dp = a.Dp, QS = Dp + 4, tiles = Dp / 16;
  const size_t buffer = (size_t)2 * ML_L * QS + (size_t)ML_L * 68 + 6 * ML_L;
  f32x4* part = (f32x4*)(ml_lds + 2 * buffer);  // [4 waves][64 lanes]
  float* n_s = (float*)(part + 4 * 64);         // [Dp]
  float* nq_s = n_s + Dp;                       // [16] n0 . q_t
  const int slot = a.state_slots[seq], ph = a.phase[seq] & 1;
  const int v0 = blockIdx.x * 64 + wave * 16;   // this wave's value columns v0 .. v0 + 15
  const bool wave_on = v0 < a.Ep;
  float* S = a.S + (((size_t)slot * a.H + head) * a.Ep + v0 + r) * Dp;
  const float* n_in = a.n + (((size_t)slot * 2 + ph) * a.H + head) * Dp;
  float* n_out = a.n + (((size_t)slot * 2 + (ph ^ 1)) * a.H + head) * Dp;
  f32x4 acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    acc[dt] = (wave_on && dt < tiles) ? *reinterpret_cast<const f32x4*>(S + dt * 16 + 4 * g) : f32x4{0.f, 0.f, 0.f, 0.f};
  for (int d = threadIdx.x; d < Dp; d += 256) n_s[d] = n_in[d];
  float m0 = a.m[((size_t)slot * 2 + ph) * a.H + head];

  // ---- a chunk's rows on their way: groups of four elements, QK groups of q and of k a thread, one of v ------------
  constexpr int QK = DT / 4;                     // 16 rows x Dp / 4 groups over 256 threads
  const int groups = Dp / 4;                     // of a row of q or k
  const bool vec = a.D % 4 == 0 && a.E % 4 == 0 && a.ld % 4 == 0 && a.q_col % 4 == 0 && a.k_col % 4 == 0 && a.v_col % 4 == 0 &&
                   (uintptr_t)a.proj % 16 == 0;
  struct Rows {
    f32x4 q[QK], k[QK], v;
    float gate_i, gate_f;
  };
  Rows even, odd;                                // the rows of the chunks with even and with odd numbers
  auto four = [&](const float* p, int first, int size) -> f32x4 {      // elements first .. first + 3 of a head's `size`
    f32x4 x = {0.f, 0.f, 0.f, 0.f};
    if (vec) {
      if (first < size) x = *reinterpret_cast<const f32x4*>(p + first);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (first + e < size) x[e] = p[first + e];
    }
    return x;
  };
  auto request = [&](int c0, Rows& in) __attribute__((always_inline)) {
    const int valid = min(ML_L, r1 - c0);
#pragma unroll
    for (int i = 0; i < QK; ++i) {
      const int item = threadIdx.x + i * 256;
      const int t = item / groups, d = (item - t * groups) * 4;
      in.q[i] = in.k[i] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (t < valid && item < ML_L * groups) {
        const float* row = a.proj + (size_t)(c0 + t) * a.ld;
        in.q[i] = four(row + a.q_col + head * a.D, d, a.D);
        in.k[i] = four(row + a.k_col + head * a.D, d, a.D);
      }
    }
    {
      const int t = threadIdx.x >> 4, c = (threadIdx.x & 15) * 4;
      in.v = f32x4{0.f, 0.f, 0.f, 0.f};
      if (t < valid) in.v = four(a.proj + (size_t)(c0 + t) * a.ld + a.v_col + head * a.E, blockIdx.x * 64 + c, a.E);
    }
    in.gate_i = in.gate_f = 0.f;
    if (threadIdx.x < ML_L && threadIdx.x < valid) {
      const float* row = a.proj + (size_t)(c0 + threadIdx.x) * a.ld;
      in.gate_i = row[a.i_col + head];
      in.gate_f = row[a.f_col + head];
    }
  };
  request(r0, even);
  if (r0 + ML_L < r1) request(r0 + ML_L, odd);
  auto link = [&](int c0, int cur, Rows& in) __attribute__((always_inline)) {
    const int valid = min(ML_L, r1 - c0);
    float* Qs = ml_lds + cur * buffer;          // [16][Dp + 4], scaled queries
    float* Ks = Qs + ML_L * QS;                 // [16][Dp + 4]
    float* Vs = Ks + ML_L * QS;                 // [16][68]: this workgroup's 64 value columns
    float* u_s = Vs + ML_L * 68;                // [16] i_j - F_j (minus infinity behind the chunk's last token)
    float* g_s = u_s + ML_L;                    // [16] running maximum, m0 included
    float* F_s = g_s + ML_L;                    // [16]
    float* e_s = F_s + ML_L;                    // [16] exp(u_j - g_last): what key j adds to the state after the chunk
    float* c_s = e_s + ML_L;                    // [16] exp(m0 - g_t): what is left of the state before the chunk at token t
    float* f_s = c_s + ML_L;                    // [16] exp(-m_t): the floor of token t's denominator
    // ---- 1: the chunk's rows and gates into LDS -------------------------------------------------------------
#pragma unroll
    for (int i = 0; i < QK; ++i) {
      const int item = threadIdx.x + i * 256;
      const int t = item / groups, d = (item - t * groups) * 4;
      if (item < ML_L * groups) {
        *reinterpret_cast<f32x4*>(Qs + t * QS + d) = in.q[i] * a.q_scale;
        *reinterpret_cast<f32x4*>(Ks + t * QS + d) = in.k[i];
      }
    }
    *reinterpret_cast<f32x4*>(Vs + (threadIdx.x >> 4) * 68 + (threadIdx.x & 15) * 4) = in.v;
    if (threadIdx.x < ML_L) {
      const int t = threadIdx.x;
      float i_log = 0.f, f_log = 0.f;
      if (t < valid) {
        i_log = a.gates_ready ? in.gate_i : a.cap * tanhf((in.gate_i + a.i_bias[head]) / a.cap);
        f_log = a.gates_ready ? in.gate_f : ml_logsigmoid(a.cap * tanhf((in.gate_f + a.f_bias[head]) / a.cap));
      }
      float F = f_log;                            // inclusive running sum over the 16 lanes
      F += ml_row_below<1>(F, 0.f);
      F += ml_row_below<2>(F, 0.f);
      F += ml_row_below<4>(F, 0.f);
      F += ml_row_below<8>(F, 0.f);
      const float u = t < valid ? i_log - F : -INFINITY;
      float best = fmaxf(u, m0);                  // running maximum, m0 included
      best = fmaxf(best, ml_row_below<1>(best, -INFINITY));
      best = fmaxf(best, ml_row_below<2>(best, -INFINITY));
      best = fmaxf(best, ml_row_below<4>(best, -INFINITY));
      best = fmaxf(best, ml_row_below<8>(best, -INFINITY));
      u_s[t] = u;
      g_s[t] = best;
      F_s[t] = F;
      const float g_end = __shfl(best, valid - 1, TW_WAVE);
      e_s[t] = t < valid ? expf(u - g_end) : 0.f;
      c_s[t] = expf(m0 - best);
      f_s[t] = expf(-(F + best));
    }
    __syncthreads();
    if (c0 + 2 * ML_L < r1) request(c0 + 2 * ML_L, in);   // (its registers are free again: two chunks' rows travel at a time)
    // ---- 2: K Q^T over this wave's share of the key elements; n0 . q_t ------------------------------------
    {
      f32x4 p = {0.f, 0.f, 0.f, 0.f};
      for (int dt = wave; dt < tiles; dt += 4) {
        const f32x4 kf = *reinterpret_cast<const f32x4*>(Ks + r * QS + dt * 16 + 4 * g);
        const f32x4 qf = *reinterpret_cast<const f32x4*>(Qs + r * QS + dt * 16 + 4 * g);
        tw_mma16(p, kf, qf);                      // p[e]: k_(4 g + e) . q_r
      }
      part[wave * 64 + lane] = p;
      const int t = threadIdx.x >> 4, piece = threadIdx.x & 15;
      float sum = 0.f;
      for (int d = piece; d < Dp; d += 16) sum = __fmaf_rn(n_s[d], Qs[t * QS + d], sum);
      sum = ml_row_sum(sum);
      if (piece == 0) nq_s[t] = sum;
    }
    __syncthreads();
    // ---- 3: weights, outputs, the new state -------------------------------------------------------------------
    const int last = valid - 1;
    const float g_last = g_s[last];
    const float carry = c_s[last];                // what is left of the state before the chunk
    if (wave_on) {
      f32x4 w = part[lane] + part[64 + lane] + part[128 + lane] + part[192 + lane];
      const float g_t = g_s[r];
      float rows = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int j = 4 * g + e;
        w[e] = (j <= r && j < valid) ? expf(u_s[j] - g_t) * w[e] : 0.f;    // W[t = r][j]
        rows += w[e];
      }
      rows = tw_rows_sum(rows);
      const float nq = __fmaf_rn(c_s[r], nq_s[r], rows);
      const float den = fmaxf(fabsf(nq), f_s[r]) + 1e-6f;                  // of token r
      // values of keys 4 g .. 4 g + 3, column v0 + r
      f32x4 vf;
#pragma unroll
      for (int e = 0; e < 4; ++e) vf[e] = Vs[(4 * g + e) * 68 + wave * 16 + r];
      f32x4 o = {0.f, 0.f, 0.f, 0.f}, o2 = {0.f, 0.f, 0.f, 0.f};          // (two chains of products instead of one)
#pragma unroll
      for (int dt = 0; dt < DT; dt += 2) {
        if (dt < tiles) {
          const f32x4 qf = *reinterpret_cast<const f32x4*>(Qs + r * QS + dt * 16 + 4 * g);
          tw_mma16_k4(o, qf, acc[dt]);            // o[e]: token 4 g + e, column v0 + r
        }
        if (dt + 1 < tiles) {
          const f32x4 qf = *reinterpret_cast<const f32x4*>(Qs + r * QS + (dt + 1) * 16 + 4 * g);
          tw_mma16_k4(o2, qf, acc[dt + 1]);
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (o[e] + o2[e]) * c_s[4 * g + e];
      tw_mma16_k4(o, w, vf);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int t = 4 * g + e;
        const float den_t = __shfl(den, t, TW_WAVE);
        if (t < valid && v0 + r < a.E)
          a.out[(size_t)(c0 + t) * a.ld_out + head * a.E + v0 + r] = o[e] / den_t;
      }
      // S <- carry S + sum_j exp(u_j - g_last) k_j v_j^T
      float ej[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) ej[e] = e_s[4 * g + e];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        if (dt < tiles) {
          f32x4 kf;
#pragma unroll
          for (int e = 0; e < 4; ++e) kf[e] = Ks[(4 * g + e) * QS + dt * 16 + r] * ej[e];
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[dt][e] *= carry;
          tw_mma16_k4(acc[dt], kf, vf);
        }
      }
    }
    for (int d = threadIdx.x; d < Dp; d += 256) {
      float sum = carry * n_s[d];
      for (int j = 0; j < valid; ++j) sum = __fmaf_rn(e_s[j], Ks[j * QS + d], sum);
      n_s[d] = sum;
    }
    m0 = F_s[last] + g_last;
    // (no barrier here: the next iteration writes the other copy of the rows, and what it shares with this one, part, n_s
    // and nq_s, is written behind its first barrier, which every wave reaches only when it is done here)
  };
  for (int c0 = r0; c0 < r1; c0 += 2 * ML_L) {
    link(c0, 0, even);
    if (c0 + ML_L < r1) link(c0 + ML_L, 1, odd);
  }
  __syncthreads();
  if (wave_on) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      if (dt < tiles) *reinterpret_cast<f32x4*>(S + dt * 16 + 4 * g) = acc[dt];
  }
  if (blockIdx.x == 0) {
    for (int d = threadIdx.x; d < Dp; d += 256) n_out[d] = n_s[d];
    if (threadIdx.x == 0) a.m[((size_t)slot * 2 + (ph ^ 1)) * a.H + head] = m0;
  }
}

// The two gates of rows first_row .. n - 1, all heads, in place of their raw values: off the chunks' chain of dependent steps.
__global__ void mlstm_gates_kernel(float* proj, long ld, int i_col, int f_col, const float* __restrict__ i_bias,
                                   const float* __restrict__ f_bias, float cap, int first_row, int n, int H) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)(n - first_row) * H) return;
  const int head = (int)(i % H);
  float* row = proj + (size_t)(first_row + i / H) * ld;
  row[i_col + head] = cap * tanhf((row[i_col + head] + i_bias[head]) / cap);
  row[f_col + head] = ml_logsigmoid(cap * tanhf((row[f_col + head] + f_bias[head]) / cap));
}

// Sequences seq0 .. seq0 + n_seqs - 1. walk != 0: token by token (steps of a few tokens), else in chunks of 16.
extern "C" int tw_mlstm(float* proj, long ld, int q_col, int k_col, int v_col, int i_col, int f_col, const float* i_bias,
                        const float* f_bias, float* S, float* n, float* m, const int* q_start, const int* state_slots,
                        const int* phase, int seq0, int n_seqs, float* out, long ld_out, int H, int D, int E, float q_scale,
                        float cap, int walk, int first_row, int n_rows, hipStream_t stream) {
  TW_REQUIRE(proj && i_bias && f_bias && S && n && m && q_start && state_slots && phase && out);
  TW_REQUIRE(n_seqs >= 0 && seq0 >= 0 && H > 0 && D > 0 && D <= 256 && E > 0 && cap > 0.f);
  TW_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && i_col >= 0 && f_col >= 0);
  TW_REQUIRE(ld >= q_col + (long)H * D && ld >= k_col + (long)H * D && ld >= v_col + (long)H * E && ld >= i_col + (long)H &&
             ld >= f_col + (long)H && ld_out >= (long)H * E);
  if (n_seqs == 0) return 0;
  const int Dp = (D + 15) / 16 * 16, Ep = (E + 15) / 16 * 16;
  TW_REQUIRE((uintptr_t)S % 16 == 0);
  MlstmArgs a{proj, ld, q_col, k_col, v_col, i_col, f_col, i_bias, f_bias, S, n, m, q_start, state_slots, phase, seq0,
              out, ld_out, H, D, E, Dp, Ep, q_scale, cap, 0};
  if (walk) {
    mlstm_walk_kernel<<<dim3(Ep / 16, H, n_seqs), 256, 0, stream>>>(a);
    return TW_LAUNCH_RESULT();
  }
  // first_row >= 0: the launch's sequences own rows first_row .. n_rows - 1 of proj, whose gates are formed first, in place
  if (first_row >= 0 && n_rows > first_row) {
    const long items = (long)(n_rows - first_row) * H;
    mlstm_gates_kernel<<<tw_div_up(items, 256), 256, 0, stream>>>(proj, ld, i_col, f_col, i_bias, f_bias, cap, first_row, n_rows, H);
    a.gates_ready = 1;
  }
  const dim3 grid(tw_div_up(Ep, 64), H, n_seqs);
  const size_t lds = ml_chunk_lds_floats(Dp) * sizeof(float);
  if (Dp <= 64) {
    mlstm_chunk_kernel<4><<<grid, 256, lds, stream>>>(a);
  } else if (Dp <= 128) {
    mlstm_chunk_kernel<8><<<grid, 256, lds, stream>>>(a);
  } else {
    if (lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute((const void*)mlstm_chunk_kernel<16>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return (int)e;
    }
    mlstm_chunk_kernel<16><<<grid, 256, lds, stream>>>(a);
  }
  return TW_LAUNCH_RESULT();
}
