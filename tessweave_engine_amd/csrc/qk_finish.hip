// What stands between the projections and the attention of a mixer whose queries and keys are normed as WHOLE rows and
// whose values are its keys: per token
//
//   q <- rotate(w_q * unit(q)),  k <- rotate(w_k * unit(k)),  v = k as it came (before norm and rotation)
//
// unit(.) over all heads of the row at once (H D elements of q, G D of k), rotation of the first `rot` elements of
// every head (pairing 0: element j with j + rot / 2; 1: element 2 j with 2 j + 1), by the angles of the token's
// position. q and k come as float32 rows (the results of short convolutions); statistics, weights and rotation are
// float32, and each result is rounded once to the compute type. The queries go to q_out with heads of Dp elements
// (tails of zeros), keys and values into the token's page slot:
//   keys [pages][G][P][Dp], values [pages][G][Dp][P] (transposed inside a page).
#include "tw_common.h"

struct QkFinishArgs {
  const float* src; long ld;
  int q_col, k_col;
  const float* wq; const float* wk;
  const float* cos_t; const float* sin_t;      // [n][rot / 2]
  void* q_out; long ld_q;
  void* keys; void* values; const int* slots;
  int H, G, D, Dp, rot, pairing, P;
  float eps;
};

__device__ __forceinline__ float qf_turned(const float* row, const float* w, float rinv, int base, int d, int rot, int pairing,
                                           const float* cs, const float* sn) {
  // element d of a head that starts at row[base]: normed, then turned if d < rot
  auto normed = [&](int e) { return row[base + e] * rinv * w[base + e]; };
  if (d >= rot) return normed(d);
  const int half = rot / 2;
  int pair, other;
  bool first;
  if (pairing == 1) {
    pair = d >> 1;
    first = (d & 1) == 0;
    other = first ? d + 1 : d - 1;
  } else {
    first = d < half;
    pair = first ? d : d - half;
    other = first ? d + half : d - half;
  }
  const float mine = normed(d), theirs = normed(other);
  const float c = cs[pair], s = sn[pair];
  // (u, v) -> (u c - v s, v c + u s)
  return first ? __fmaf_rn(mine, c, -__fmul_rn(theirs, s)) : __fmaf_rn(mine, c, __fmul_rn(theirs, s));
}

template <typename T>
__global__ __launch_bounds__(256) void qk_finish_kernel(QkFinishArgs a) {
  __shared__ float lds[16];
  const int n = blockIdx.x;
  const float* row = a.src + (size_t)n * a.ld;
  const int nq = a.H * a.D, nk = a.G * a.D;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < nq; i += blockDim.x) sq = __fmaf_rn(row[a.q_col + i], row[a.q_col + i], sq);
  for (int i = threadIdx.x; i < nk; i += blockDim.x) sk = __fmaf_rn(row[a.k_col + i], row[a.k_col + i], sk);
  const float tq = tw_block_sum(sq, lds);
  const float tk = tw_block_sum(sk, lds);
  const float rq = 1.f / sqrtf(tq / (float)nq + a.eps), rk = 1.f / sqrtf(tk / (float)nk + a.eps);
  const float* cs = a.cos_t + (size_t)n * (a.rot / 2);
  const float* sn = a.sin_t + (size_t)n * (a.rot / 2);
  T* q = (T*)a.q_out + (size_t)n * a.ld_q;
  for (int i = threadIdx.x; i < a.H * a.Dp; i += blockDim.x) {
    const int head = i / a.Dp, d = i % a.Dp;
    float v = 0.f;
    if (d < a.D) v = qf_turned(row + a.q_col, a.wq, rq, head * a.D, d, a.rot, a.pairing, cs, sn);
    q[i] = tw_from_float<T>(v);
  }
  const int slot = a.slots[n];
  if (slot < 0) return;
  const int page = slot / a.P, at = slot % a.P;
  for (int i = threadIdx.x; i < a.G * a.Dp; i += blockDim.x) {
    const int kvh = i / a.Dp, d = i % a.Dp;
    float k = 0.f, v = 0.f;
    if (d < a.D) {
      k = qf_turned(row + a.k_col, a.wk, rk, kvh * a.D, d, a.rot, a.pairing, cs, sn);
      v = row[a.k_col + kvh * a.D + d];
    }
    ((T*)a.keys)[(((size_t)page * a.G + kvh) * a.P + at) * a.Dp + d] = tw_from_float<T>(k);
    ((T*)a.values)[(((size_t)page * a.G + kvh) * a.Dp + d) * a.P + at] = tw_from_float<T>(v);
  }
}

extern "C" int tw_qk_finish(int dtype, const float* src, long ld, int q_col, int k_col, const float* wq, const float* wk,
                            const float* cos_t, const float* sin_t, void* q_out, long ld_q, void* keys, void* values,
                            const int* slots, int n, int H, int G, int D, int Dp, int rot, int pairing, int page_size,
                            float eps, hipStream_t stream) {
  TW_REQUIRE(src && wq && wk && q_out && keys && values && slots && n >= 0 && H > 0 && G > 0 && D > 0 && Dp >= D);
  TW_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D && (rot == 0 || (cos_t && sin_t)) && (pairing == 0 || pairing == 1));
  TW_REQUIRE(q_col >= 0 && k_col >= 0 && ld >= q_col + (long)H * D && ld >= k_col + (long)G * D && ld_q >= (long)H * Dp);
  TW_REQUIRE(page_size > 0 && eps > 0.f);
  if (n == 0) return 0;
  QkFinishArgs a{src, ld, q_col, k_col, wq, wk, cos_t, sin_t, q_out, ld_q, keys, values, slots, H, G, D, Dp, rot, pairing,
                 page_size, eps};
  if (dtype == TW_DTYPE_BF16) qk_finish_kernel<bf16_t><<<n, 256, 0, stream>>>(a);
  else if (dtype == TW_DTYPE_F32) qk_finish_kernel<float><<<n, 256, 0, stream>>>(a);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}
