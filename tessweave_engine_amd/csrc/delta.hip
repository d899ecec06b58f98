// The gated delta rule: a recurrent mixer whose state is corrected towards each new value before it is read.
//
//   per value head h (its query/key head is h / (H / G)), S: [D][E] float32, carried from step to step:
//     q~ = q / sqrt(sum q^2 + 1e-6) * q_scale        k~ = k / sqrt(sum k^2 + 1e-6)
//     beta = sigmoid(b)      g = exp(-exp(A_log_h) * softplus(a + dt_bias_h))
//     S <- g S;   u = beta (v - S^T k~);   S <- S + k~ u^T;   o = S^T q~          (the read-out sees the token's write)
//
// q, k, v arrive in float32 (a short convolution's result), b and a are columns of a float32 projection; the unit
// norms, the gates, the state and every product with it are float32. A step's rows of one sequence are walked in
// order from the request's state, which the same lanes read at the start and write at the end: nothing depends on
// how a prompt was cut.
//
// A workgroup owns 256 / KS value columns of one (sequence, head). A wave holds 64 / KS of them: lane = KS * column +
// slice, and a lane keeps part `slice` of its column of S in registers (DPL elements), so both products of a token are
// DPL multiply-adds and a sum over KS neighbouring lanes (DPP: inside a quad, or rotations of a row of 16). What a token
// costs is the length of that dependent chain, so keys longer than 16 are cut into 16 slices: 8 multiply-adds a
// product at a key size of 128, and a head's columns spread over eight workgroups. The state lies in memory as
// [H][E][Dk] (a column of S is contiguous), Dk <= KS * DPL. Tokens are staged in LDS in chunks: the waves share a
// chunk's tokens out, norm q and k, form beta and g, then all walk the chunk.
#include "tw_common.h"

#define TW_DELTA_CHUNK 16
#define TW_DELTA_WALK_MOST 4          /* up to this many tokens a sequence, a step walks them one by one */

struct DeltaArgs {
  const float* qkv; long ld_qkv;      // q of key head j at q_col + j * D, k at k_col + j * D, v of head h at v_col + h * E
  int q_col, k_col, v_col;
  const float* ab; long ld_ab;        // b of head h at b_col + h, a at a_col + h
  int b_col, a_col;
  const float* A_log; const float* dt_bias;   // [H]
  float* state;                       // [requests][H][E][Dk]
  const int* q_start; const int* state_slots;
  float* out; long ld_out;            // float32 [n][>= H * E]: head h at h * E
  int H, G, D, E, Dk;
  float q_scale;
};

template <int CTRL>
__device__ __forceinline__ float delta_quad_swap(float v) {
  return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xf, 0xf, true));
}
// sum over KS neighbouring lanes (4: a quad; 16: a row); every lane gets it
template <int KS>
__device__ __forceinline__ float delta_group_sum(float v) {
  if constexpr (KS == 4) {
    v += delta_quad_swap<0xB1>(v);    // lanes 1 0 3 2
    v += delta_quad_swap<0x4E>(v);    // lanes 2 3 0 1
  } else {
    v += delta_quad_swap<0x128>(v);   // the row rotated by 8 lanes, then by 4, 2, 1
    v += delta_quad_swap<0x124>(v);
    v += delta_quad_swap<0x122>(v);
    v += delta_quad_swap<0x121>(v);
  }
  return v;
}

__device__ __forceinline__ float delta_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

template <int DPL, int KS>
__global__ __launch_bounds__(256) void delta_walk_kernel(DeltaArgs a, int seq0) {
  constexpr int SL = DPL + 4;                        // a slice's stride in LDS: the slices a read meets lie in different banks
  constexpr int ROW = KS * SL;
  constexpr int CW = 256 / KS, CV = 64 / KS;         // value columns a workgroup, a wave
  __shared__ __attribute__((aligned(16))) float q_s[TW_DELTA_CHUNK][ROW];
  __shared__ __attribute__((aligned(16))) float k_s[TW_DELTA_CHUNK][ROW];
  __shared__ float v_s[TW_DELTA_CHUNK][CW];
  __shared__ float gate_s[TW_DELTA_CHUNK][2];        // beta, g
  const int blocks_e = (a.E + CW - 1) / CW;
  const int eb = blockIdx.x % blocks_e, head = blockIdx.x / blocks_e;
  const int s = seq0 + blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slice = lane & (KS - 1);
  const int e = eb * CW + wave * CV + lane / KS;
  const bool live = e < a.E;
  const int kh = head / (a.H / a.G);
  const int first = a.q_start[s], last = a.q_start[s + 1];
  float* S_mem = a.state + (((size_t)a.state_slots[s] * a.H + head) * a.E + (live ? e : 0)) * a.Dk + slice * DPL;
  const bool held = live && slice * DPL < a.Dk;      // (Dk may be shorter than 4 * DPL: the last slices then hold nothing)
  float S[DPL];
#pragma unroll
  for (int i = 0; i < DPL; i += 4) {
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (held && slice * DPL + i < a.Dk) v = *reinterpret_cast<const f32x4*>(S_mem + i);
    S[i] = v[0]; S[i + 1] = v[1]; S[i + 2] = v[2]; S[i + 3] = v[3];
  }
  const float rate = -expf(a.A_log[head]);
  const float dt_bias = a.dt_bias[head];
  for (int t0 = first; t0 < last; t0 += TW_DELTA_CHUNK) {
    const int nt = min(TW_DELTA_CHUNK, last - t0);
    __syncthreads();                                 // the chunk before has been walked by every wave
    for (int i = wave; i < nt; i += 4) {
      const float* row = a.qkv + (size_t)(t0 + i) * a.ld_qkv;
      const float* qr = row + a.q_col + (size_t)kh * a.D;
      const float* kr = row + a.k_col + (size_t)kh * a.D;
      float qv[4], kv[4], qq = 0.f, kk = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = lane + 64 * j;
        qv[j] = d < a.D ? qr[d] : 0.f;
        kv[j] = d < a.D ? kr[d] : 0.f;
        qq = __fmaf_rn(qv[j], qv[j], qq);
        kk = __fmaf_rn(kv[j], kv[j], kk);
      }
      qq = tw_wave_sum(qq);
      kk = tw_wave_sum(kk);
      const float qn = a.q_scale / sqrtf(qq + 1e-6f), kn = 1.f / sqrtf(kk + 1e-6f);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = lane + 64 * j;
        if (d < KS * DPL) {
          q_s[i][(d / DPL) * SL + d % DPL] = qv[j] * qn;
          k_s[i][(d / DPL) * SL + d % DPL] = kv[j] * kn;
        }
      }
      const int ev = eb * CW + lane;
      if (lane < CW) v_s[i][lane] = ev < a.E ? row[a.v_col + (size_t)head * a.E + ev] : 0.f;
      if (lane == 0) {
        const float* ab = a.ab + (size_t)(t0 + i) * a.ld_ab;
        const float b = ab[a.b_col + head], x = ab[a.a_col + head];
        gate_s[i][0] = 1.f / (1.f + expf(-b));
        gate_s[i][1] = expf(rate * delta_softplus(x + dt_bias));
      }
    }
    __syncthreads();
    for (int i = 0; i < nt; ++i) {
      const float* kp = &k_s[i][slice * SL];
      const float* qp = &q_s[i][slice * SL];
      const float beta = gate_s[i][0], g = gate_s[i][1];
      float d0 = 0.f, d1 = 0.f, d2 = 0.f, d3 = 0.f;
#pragma unroll
      for (int j = 0; j < DPL; j += 4) {
        const f32x4 kq = *reinterpret_cast<const f32x4*>(kp + j);
        d0 = __fmaf_rn(S[j], kq[0], d0);
        d1 = __fmaf_rn(S[j + 1], kq[1], d1);
        d2 = __fmaf_rn(S[j + 2], kq[2], d2);
        d3 = __fmaf_rn(S[j + 3], kq[3], d3);
      }
      const float dot = delta_group_sum<KS>((d0 + d1) + (d2 + d3));
      const float u = beta * (v_s[i][wave * CV + lane / KS] - g * dot);
      float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
#pragma unroll
      for (int j = 0; j < DPL; j += 4) {
        const f32x4 kq = *reinterpret_cast<const f32x4*>(kp + j);
        const f32x4 qq = *reinterpret_cast<const f32x4*>(qp + j);
        S[j] = __fmaf_rn(kq[0], u, g * S[j]);
        S[j + 1] = __fmaf_rn(kq[1], u, g * S[j + 1]);
        S[j + 2] = __fmaf_rn(kq[2], u, g * S[j + 2]);
        S[j + 3] = __fmaf_rn(kq[3], u, g * S[j + 3]);
        o0 = __fmaf_rn(S[j], qq[0], o0);
        o1 = __fmaf_rn(S[j + 1], qq[1], o1);
        o2 = __fmaf_rn(S[j + 2], qq[2], o2);
        o3 = __fmaf_rn(S[j + 3], qq[3], o3);
      }
      const float o = delta_group_sum<KS>((o0 + o1) + (o2 + o3));
      if (live && slice == 0) a.out[(size_t)(t0 + i) * a.ld_out + (size_t)head * a.E + e] = o;
    }
  }
#pragma unroll
  for (int i = 0; i < DPL; i += 4)
    if (held && slice * DPL + i < a.Dk) *reinterpret_cast<f32x4*>(S_mem + i) = f32x4{S[i], S[i + 1], S[i + 2], S[i + 3]};
}

// The waves of a workgroup meet once each one's LDS traffic is done. (Unlike __syncthreads() this does not wait for loads
// from memory: the next chunk's rows stay on their way across it.)
__device__ __forceinline__ void delta_lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// ---- many tokens a sequence: chunks of 16 tokens, each solved at once ----------------------------------------------
// Inside a chunk with state S0 at its start, L_i = sum_{m <= i} log g_m (so that G_i = exp(L_i) and every quotient
// G_i / G_j, j <= i, is an exponential of a sum of logarithms that are at most 0):
//   u_i = beta_i (v_i - G_i S0^T k_i) - sum_{j < i} A_ij u_j,      A_ij = beta_i (G_i / G_j) (k_i . k_j)
//   o_i = G_i S0^T q_i + sum_{j <= i} (G_i / G_j) (q_i . k_j) u_j
//   S   = G_last S0 + sum_j (G_last / G_j) k_j u_j^T
// which is the token-by-token rule written out. All products are float32 on the matrix unit (16x16x4). A workgroup
// owns 16 value columns of one (sequence, head); its four waves own a quarter of the key elements each (NT tiles of 16),
// and a wave's part of S stays in registers in the layout that is both the B operand of K S and the accumulator of
// K^T W: lane (c, g) holds S[16 tile + 4 g + j][c]. Per chunk: the waves form their parts of K S0, Q S0, K K^T and
// Q K^T from the same fragments (the key rows of a chunk are the A operand of the first and both operands of the third),
// the parts meet in LDS and thread 16 i + j adds them up for the pair (i, j) and puts decay, beta and the unit norms on
// (q and k are multiplied as they come; their squared lengths are the diagonals of K K^T and of one more product, Q Q^T); every lane solves
// the triangular system of its column by substitution (after u_j is final every later row takes its term off: one
// multiply-add deep a token); one wave reads the chunk's outputs out (one more product), every wave updates its part
// of S. Tokens behind a sequence's end are staged as zeros with beta = 0 and g = 1: they change nothing. The next
// chunk's rows are on their way from memory while this one is worked on.
template <int NT>
__global__ __launch_bounds__(256) void delta_chunk_kernel(DeltaArgs a, int seq0) {
  constexpr int C = 16, DP = 64 * NT;                // key elements, rounded up: 16 NT a wave
  constexpr int ROW = DP + 4;                        // (+ 4: the four token rows a transposed read meets lie 16 banks apart)
  constexpr int PW = C + 4;
  __shared__ __attribute__((aligned(16))) float q_s[C][ROW];
  __shared__ __attribute__((aligned(16))) float k_s[C][ROW];
  __shared__ __attribute__((aligned(16))) float part_s[4][5][C][C];   // [wave][K S0, Q S0, K K^T, Q K^T, Q Q^T][row][column]
  __shared__ __attribute__((aligned(16))) float v_s[C][C];
  __shared__ __attribute__((aligned(16))) float pk_s[C][C];      // (S0^T k_i)[column]
  __shared__ __attribute__((aligned(16))) float pq_s[C][C];
  __shared__ __attribute__((aligned(16))) float at_s[C][PW];     // at_s[j][i] = A_ij (0 unless j < i)
  __shared__ __attribute__((aligned(16))) float qk_s[C][PW];     // qk_s[i][j] = (G_i / G_j) (q_i . k_j) (0 unless j <= i)
  __shared__ float beta_s[C], lg_s[C], g_s[C], tail_s[C];        // beta_i, log g_i, G_i, G_last / G_i * (1 / |k_i|)
  const int blocks_e = (a.E + 15) / 16;
  const int eb = blockIdx.x % blocks_e, head = blockIdx.x / blocks_e;
  const int s = seq0 + blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int e = eb * 16 + r;                         // this lane's value column
  const bool live = e < a.E;
  const int kh = head / (a.H / a.G);
  const int first = a.q_start[s], last = a.q_start[s + 1];
  if (first >= last) return;
  const int d_wave = 16 * NT * wave;                 // the wave's first key element
  float* S_mem = a.state + (((size_t)a.state_slots[s] * a.H + head) * a.E + (live ? e : 0)) * a.Dk;
  f32x4 S[NT];
#pragma unroll
  for (int mm = 0; mm < NT; ++mm) {
    const int d0 = d_wave + 16 * mm + 4 * g;
    S[mm] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (live && d0 < a.Dk) S[mm] = *reinterpret_cast<const f32x4*>(S_mem + d0);
  }
  const float rate = -expf(a.A_log[head]);
  const float dt_bias = a.dt_bias[head];

  // a wave stages tokens wave, wave + 4, wave + 8, wave + 12 of a chunk: their raw rows, in registers
  float rq[4][NT], rk[4][NT], rv[4], rb[4], ra[4];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) {
      const int t = t0 + wave + 4 * ii;
      const bool in = t < last;
      const float* row = a.qkv + (size_t)(in ? t : first) * a.ld_qkv;
      const float* qr = row + a.q_col + (size_t)kh * a.D;
      const float* kr = row + a.k_col + (size_t)kh * a.D;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const int d = lane + 64 * j;
        const bool ok = in && d < a.D;
        rq[ii][j] = ok ? qr[d] : 0.f;
        rk[ii][j] = ok ? kr[d] : 0.f;
      }
      const int ev = eb * 16 + r;
      rv[ii] = in && ev < a.E ? row[a.v_col + (size_t)head * a.E + ev] : 0.f;
      const float* ab = a.ab + (size_t)(in ? t : first) * a.ld_ab;
      rb[ii] = ab[a.b_col + head];
      ra[ii] = ab[a.a_col + head];
    }
  };
  auto stage = [&](int t0) {
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) {
      const int i = wave + 4 * ii;
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        q_s[i][lane + 64 * j] = rq[ii][j];           // (as they come: the unit norms are put on the products)
        k_s[i][lane + 64 * j] = rk[ii][j];
      }
      if (lane < 16) v_s[i][lane] = rv[ii];
    }
    // the gates of the wave's four tokens, one lane a token (every lane holds all four tokens' b and a)
    const int mine = lane & 3;
    const float b = mine == 0 ? rb[0] : mine == 1 ? rb[1] : mine == 2 ? rb[2] : rb[3];
    const float x = mine == 0 ? ra[0] : mine == 1 ? ra[1] : mine == 2 ? ra[2] : ra[3];
    if (lane < 4) {
      const int i = wave + 4 * mine;
      const bool in = t0 + i < last;
      beta_s[i] = in ? 1.f / (1.f + expf(-b)) : 0.f;
      lg_s[i] = in ? rate * delta_softplus(x + dt_bias) : 0.f;
    }
  };

  fetch(first);
  for (int t0 = first; t0 < last; t0 += C) {
    delta_lds_barrier();                             // the chunk before has been worked on by every wave
    stage(t0);
    if (t0 + C < last) fetch(t0 + C);
    delta_lds_barrier();

    // ---- this wave's parts of the four products -----------------------------------------------------------------------
    {
      f32x4 pk = {0.f, 0.f, 0.f, 0.f}, pq = pk, kk = pk, qk = pk, qq = pk;
#pragma unroll
      for (int mm = 0; mm < NT; ++mm) {
        const f32x4 kf = *reinterpret_cast<const f32x4*>(&k_s[r][d_wave + 16 * mm + 4 * g]);
        const f32x4 qf = *reinterpret_cast<const f32x4*>(&q_s[r][d_wave + 16 * mm + 4 * g]);
        tw_mma16(pk, kf, S[mm]);                     // [token][column]
        tw_mma16(pq, qf, S[mm]);
        tw_mma16(kk, kf, kf);                        // [token i][token j]
        tw_mma16(qk, qf, kf);
        tw_mma16(qq, qf, qf);                        // (its diagonal: the queries' squared lengths, as K K^T's are the keys')
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        part_s[wave][0][4 * g + j][r] = pk[j];
        part_s[wave][1][4 * g + j][r] = pq[j];
        part_s[wave][2][4 * g + j][r] = kk[j];
        part_s[wave][3][4 * g + j][r] = qk[j];
        part_s[wave][4][4 * g + j][r] = qq[j];
      }
    }
    delta_lds_barrier();

    // ---- thread 16 i + j adds the waves' parts up (in their order) and puts the decay between tokens i and j on -----
    {
      const int i = threadIdx.x >> 4, j = threadIdx.x & 15;
      auto whole = [&](int t, int row, int column) {
        return (part_s[0][t][row][column] + part_s[1][t][row][column]) + (part_s[2][t][row][column] + part_s[3][t][row][column]);
      };
      float sum[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) sum[t] = whole(t, i, j);
      // q and k were multiplied as they came: 1 / |k_i|, 1 / |k_j| and q_scale / |q_i| from the diagonals
      const float kn_i = 1.f / sqrtf(whole(2, i, i) + 1e-6f), kn_j = 1.f / sqrtf(whole(2, j, j) + 1e-6f);
      const float qn_i = a.q_scale / sqrtf(whole(4, i, i) + 1e-6f);
      float between = 0.f, upto = 0.f;               // log of G_i / G_j (j <= i), and L_i
#pragma unroll
      for (int m = 0; m < C; ++m) {
        const float lg = lg_s[m];
        if (m > j && m <= i) between += lg;
        if (m <= i) upto += lg;
      }
      const float decay = expf(between);
      pk_s[i][j] = kn_i * sum[0];
      pq_s[i][j] = qn_i * sum[1];
      at_s[j][i] = j < i ? beta_s[i] * decay * (kn_i * kn_j) * sum[2] : 0.f;
      qk_s[i][j] = j <= i ? decay * (qn_i * kn_j) * sum[3] : 0.f;
      if (j == 0) g_s[i] = expf(upto);
      if (i == C - 1) tail_s[j] = decay * kn_j;
    }
    delta_lds_barrier();

    // ---- the triangular system of this lane's column (the lanes of a column, in every wave, all solve it) -----------
    float u[C];
#pragma unroll
    for (int i = 0; i < C; ++i) u[i] = beta_s[i] * (v_s[i][r] - g_s[i] * pk_s[i][r]);
#pragma unroll
    for (int j = 0; j < C - 1; ++j) {
      float arow[C];
#pragma unroll
      for (int x = 0; x < C; x += 4) {
        const f32x4 v = *reinterpret_cast<const f32x4*>(&at_s[j][x]);
        arow[x] = v[0]; arow[x + 1] = v[1]; arow[x + 2] = v[2]; arow[x + 3] = v[3];
      }
#pragma unroll
      for (int i = j + 1; i < C; ++i) u[i] = __fmaf_rn(-arow[i], u[j], u[i]);
    }
    // u of tokens 4 g .. 4 g + 3: the B operand of the two products over tokens
    f32x4 ub;
#pragma unroll
    for (int j = 0; j < 4; ++j) ub[j] = g == 0 ? u[j] : g == 1 ? u[4 + j] : g == 2 ? u[8 + j] : u[12 + j];

    // ---- the read-out: o_i = G_i (S0^T q_i) + sum_j qk[i][j] u_j, by the chunk's wave in turn -------------------------
    if (wave == ((t0 - first) / C & 3)) {
      f32x4 o = {0.f, 0.f, 0.f, 0.f};
      const f32x4 w = *reinterpret_cast<const f32x4*>(&qk_s[r][4 * g]);
      tw_mma16(o, w, ub);                            // [token i][column]
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = 4 * g + j;
        const float out = __fmaf_rn(g_s[i], pq_s[i][r], o[j]);
        if (live && t0 + i < last) a.out[(size_t)(t0 + i) * a.ld_out + (size_t)head * a.E + e] = out;
      }
    }

    // ---- the state behind the chunk: S <- G_last S + K^T diag(G_last / G_j) U ----------------------------------------
    const float G_last = g_s[C - 1];
    f32x4 wb;
#pragma unroll
    for (int j = 0; j < 4; ++j) wb[j] = tail_s[4 * g + j] * ub[j];
#pragma unroll
    for (int mm = 0; mm < NT; ++mm) {
      f32x4 kt;                                      // A operand: row = key element 16 tile + r, reduction = token 4 g + j
#pragma unroll
      for (int j = 0; j < 4; ++j) kt[j] = k_s[4 * g + j][d_wave + 16 * mm + r];
#pragma unroll
      for (int j = 0; j < 4; ++j) S[mm][j] *= G_last;
      tw_mma16(S[mm], kt, wb);
    }
  }
#pragma unroll
  for (int mm = 0; mm < NT; ++mm) {
    const int d0 = d_wave + 16 * mm + 4 * g;
    if (live && d0 < a.Dk) *reinterpret_cast<f32x4*>(S_mem + d0) = S[mm];
  }
}

extern "C" int tw_delta_rule(const float* qkv, long ld_qkv, int q_col, int k_col, int v_col, const float* ab, long ld_ab,
                             int b_col, int a_col, const float* A_log, const float* dt_bias, float* state,
                             const int* q_start, const int* state_slots, float* out, long ld_out, int seq0, int n_seqs,
                             int max_q_len, int H, int G, int D, int E, int Dk, float q_scale, hipStream_t stream) {
  TW_REQUIRE(qkv && ab && A_log && dt_bias && state && q_start && state_slots && out);
  TW_REQUIRE(H > 0 && G > 0 && H % G == 0 && D > 0 && D <= 256 && E > 0 && Dk >= D && Dk % 4 == 0 && Dk <= 256);
  TW_REQUIRE(max_q_len >= 1);
  TW_REQUIRE(seq0 >= 0 && n_seqs >= 0 && ld_out >= (long)H * E && (uintptr_t)state % 16 == 0);
  TW_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && b_col >= 0 && a_col >= 0);
  TW_REQUIRE(ld_qkv >= (long)max(q_col, k_col) + (long)G * D && ld_qkv >= (long)v_col + (long)H * E);
  TW_REQUIRE(ld_ab >= (long)max(a_col, b_col) + H);
  if (n_seqs == 0) return 0;
  DeltaArgs a{qkv, ld_qkv, q_col, k_col, v_col, ab, ld_ab, b_col, a_col, A_log, dt_bias, state, q_start, state_slots,
              out, ld_out, H, G, D, E, Dk, q_scale};
  if (max_q_len > TW_DELTA_WALK_MOST) {
    // some sequence brings many tokens: every sequence of the step goes through the kernel that solves chunks at once
    const dim3 grid(H * tw_div_up(E, 16), n_seqs);
    if (Dk <= 64) delta_chunk_kernel<1><<<grid, 256, 0, stream>>>(a, seq0);
    else if (Dk <= 128) delta_chunk_kernel<2><<<grid, 256, 0, stream>>>(a, seq0);
    else delta_chunk_kernel<4><<<grid, 256, 0, stream>>>(a, seq0);
  } else if (Dk <= 16) {
    delta_walk_kernel<4, 4><<<dim3(H * tw_div_up(E, 64), n_seqs), 256, 0, stream>>>(a, seq0);
  } else {
    const dim3 grid(H * tw_div_up(E, 16), n_seqs);
    if (Dk <= 64) delta_walk_kernel<4, 16><<<grid, 256, 0, stream>>>(a, seq0);
    else if (Dk <= 128) delta_walk_kernel<8, 16><<<grid, 256, 0, stream>>>(a, seq0);
    else delta_walk_kernel<16, 16><<<grid, 256, 0, stream>>>(a, seq0);
  }
  return TW_LAUNCH_RESULT();
}

// out[n][h * E + e] = o[n][h * E + e] / sqrt(mean_e(o^2) + eps) * weight[e] * silu(gate[n][h * E + e]), rounded to the
// compute type: a unit norm per head with one weight vector shared by the heads, times a gate. One wave a (token, head).
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, long ld_o, const float* __restrict__ gate,
                                                             long ld_g, const float* __restrict__ weight, T* __restrict__ out,
                                                             long ld_out, int n, int H, int E, float eps, int weight_stride,
                                                             int gate_kind) {
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= n * H) return;
  const int lane = threadIdx.x & 63;
  const int row = unit / H, head = unit % H;
  const float* src = o + (size_t)row * ld_o + (size_t)head * E;
  float ss = 0.f;
  for (int e = lane; e < E; e += 64) ss = __fmaf_rn(src[e], src[e], ss);
  ss = tw_wave_sum(ss);
  const float rinv = 1.f / sqrtf(ss / (float)E + eps);
  const float* g = gate + (size_t)row * ld_g + (size_t)head * E;
  T* dst = out + (size_t)row * ld_out + (size_t)head * E;
  for (int e = lane; e < E; e += 64) {
    const float z = g[e];
    const float sig = 1.f / (1.f + expf(-z));
    // weight_stride: 0 for one weight vector for all heads, E for one a head; gate_kind 0: SiLU of the gate, 1: its sigmoid
    dst[e] = tw_from_float<T>(src[e] * rinv * weight[(size_t)head * weight_stride + e] * (gate_kind == 1 ? sig : z * sig));
  }
}

extern "C" int tw_head_norm_gate(int dtype, const float* o, long ld_o, const float* gate, long ld_g, const float* weight,
                                 void* out, long ld_out, int n, int H, int E, float eps, int weight_per_head, int gate_kind,
                                 hipStream_t stream) {
  TW_REQUIRE(o && gate && weight && out && n >= 0 && H > 0 && E > 0 && eps > 0.f && (gate_kind == 0 || gate_kind == 1));
  const int weight_stride = weight_per_head ? E : 0;
  TW_REQUIRE(ld_o >= (long)H * E && ld_g >= (long)H * E && ld_out >= (long)H * E);
  if (n == 0) return 0;
  const int blocks = tw_div_up((long)n * H, 4);
  if (dtype == TW_DTYPE_BF16)
    head_norm_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>(o, ld_o, gate, ld_g, weight, (bf16_t*)out, ld_out, n, H, E, eps, weight_stride, gate_kind);
  else if (dtype == TW_DTYPE_F32)
    head_norm_gate_kernel<float><<<blocks, 256, 0, stream>>>(o, ld_o, gate, ld_g, weight, (float*)out, ld_out, n, H, E, eps, weight_stride, gate_kind);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}
