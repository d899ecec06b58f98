// Attention over a cached LATENT: every token leaves one normed vector c (L elements) and one rotated key part
// kr (R elements) that all heads share; head a's key is [W_uk,a c | kr] and its value W_uv,a c. The products with
// W_uk and W_uv are moved to the query side and the output side:
//
//   score_a(i, j) = (W_uk,a^T q_plain,a(i)) . c_j + q_turned,a(i) . kr_j         out_a(i) = W_uv,a sum_j p_a(i, j) c_j
//
// so the attention itself runs over ONE key/value head whose key row is [c | kr] and whose value is c, and only
// c and kr are ever stored. Here: the kernel that finishes a token's projections (norm of c, rotation of kr and
// of the queries' rotated parts, cache write), and the per-head matrix product both sides use.
#include "tw_common.h"

// One rotated pair, products and sums spelled out (a*b - c*d left to the compiler becomes one fused form or the other).
__device__ __forceinline__ void lt_rotate_pair(float lo, float hi, float c, float s, float& out_lo, float& out_hi) {
  out_lo = __fmaf_rn(lo, c, -__fmul_rn(hi, s));
  out_hi = __fmaf_rn(hi, c, __fmul_rn(lo, s));
}

struct LatentFinishArgs {
  const void* proj; long ld;        // a token's projections: the heads' rotated query parts at q_col + a * Rp,
  int q_col, c_col, kr_col;         // the raw latent at c_col (L elements), the raw shared key part at kr_col
  const float* cos_t; const float* sin_t;    // [n][rot / 2]
  const float* norm_w;              // [L]
  void* q_out; long ld_q;           // [n][H][Lp + Rp]: this kernel fills columns Lp .. Lp + Rp of every head
  void* q_full; long ld_full;       // or null. [n][H][hd]: head a = [its D unrotated elements | its rotated part | zeros],
  int D, Dp, hd, full_from;         // for rows from full_from on (queries against keys expanded per head)
  void* keys; void* values;         // keys [pages][1][P][Lp + Rp], values [pages][1][Lp][P]; null: nothing is stored
  const int* slots;
  int H, L, Lp, Rp, rot, P;
  float eps;
};

template <typename T>
__global__ __launch_bounds__(256) void latent_finish_kernel(LatentFinishArgs a) {
  __shared__ float lds[16];
  const int n = blockIdx.x;
  const T* row = (const T*)a.proj + (size_t)n * a.ld;
  const int half = a.rot / 2;
  const float* cs = a.cos_t + (size_t)n * half;
  const float* sn = a.sin_t + (size_t)n * half;
  const int K = a.Lp + a.Rp;
  // the heads' rotated query parts
  T* q = (T*)a.q_out + (size_t)n * a.ld_q;
  for (int i = threadIdx.x; i < a.H * a.Rp; i += blockDim.x) {
    const int head = i / a.Rp, d = i % a.Rp;
    const T* src = row + a.q_col + head * a.Rp;
    float v;
    if (d < half) {
      float other;
      lt_rotate_pair(tw_to_float(src[d]), tw_to_float(src[d + half]), cs[d], sn[d], v, other);
    } else if (d < a.rot) {
      float other;
      lt_rotate_pair(tw_to_float(src[d - half]), tw_to_float(src[d]), cs[d - half], sn[d - half], other, v);
    } else {
      v = tw_to_float(src[d]);
    }
    q[(size_t)head * K + a.Lp + d] = tw_from_float<T>(v);
  }
  if (a.q_full && n >= a.full_from) {
    __syncthreads();                                                          // the rotated parts above, written by other threads
    T* qf = (T*)a.q_full + (size_t)n * a.ld_full;
    for (int i = threadIdx.x; i < a.H * a.hd; i += blockDim.x) {
      const int head = i / a.hd, d = i % a.hd;
      T v = tw_from_float<T>(0.f);
      if (d < a.D) v = row[head * a.Dp + d];                                   // (the unrotated parts lie first in the row)
      else if (d < a.D + a.Rp) v = q[(size_t)head * K + a.Lp + d - a.D];     // (turned or not; zeros behind the part's own size)
      qf[i] = v;
    }
  }
  if (!a.keys) return;
  const int slot = a.slots[n];
  // the latent's norm (every thread takes part in the sum, stored or not)
  float ss = 0.f;
  for (int i = threadIdx.x; i < a.L; i += blockDim.x) {
    const float v = tw_to_float(row[a.c_col + i]);
    ss = __fmaf_rn(v, v, ss);
  }
  const float total = tw_block_sum(ss, lds);
  if (slot < 0) return;
  const float rinv = 1.f / sqrtf(total / (float)a.L + a.eps);
  const int page = slot / a.P, at = slot % a.P;
  T* key = (T*)a.keys + ((size_t)page * a.P + at) * K;
  T* val = (T*)a.values + (size_t)page * a.Lp * a.P + at;
  for (int i = threadIdx.x; i < a.Lp; i += blockDim.x) {
    const T c = i < a.L ? tw_from_float<T>(tw_to_float(row[a.c_col + i]) * rinv * a.norm_w[i]) : tw_from_float<T>(0.f);
    key[i] = c;
    val[(size_t)i * a.P] = c;
  }
  for (int d = threadIdx.x; d < a.Rp; d += blockDim.x) {
    const T* src = row + a.kr_col;
    float v;
    if (d < half) {
      float other;
      lt_rotate_pair(tw_to_float(src[d]), tw_to_float(src[d + half]), cs[d], sn[d], v, other);
    } else if (d < a.rot) {
      float other;
      lt_rotate_pair(tw_to_float(src[d - half]), tw_to_float(src[d]), cs[d - half], sn[d - half], other, v);
    } else {
      v = tw_to_float(src[d]);                   // what the encoding does not turn passes (the padding behind it is zeros)
    }
    key[a.Lp + d] = tw_from_float<T>(v);
  }
}

extern "C" int tw_latent_finish(int dtype, const void* proj, long ld, int q_col, int c_col, int kr_col,
                                const float* cos_t, const float* sin_t, const float* norm_w, void* q_out, long ld_q,
                                void* q_full, long ld_full, int D, int Dp, int hd, int full_from,
                                void* keys, void* values, const int* slots, int n, int H, int L, int Lp, int Rp, int rot,
                                int page_size, float eps, hipStream_t stream) {
  TW_REQUIRE(proj && cos_t && sin_t && q_out && n >= 0 && H > 0 && Rp > 0 && rot > 0 && rot % 2 == 0 && rot <= Rp);
  if (q_full) TW_REQUIRE(D > 0 && Dp >= D && hd >= D + rot && ld_full >= (long)H * hd && full_from >= 0 && q_col >= H * Dp);
  TW_REQUIRE(q_col >= 0 && ld >= q_col + (long)H * Rp && ld_q >= (long)H * (Lp + Rp) && Lp >= 0);
  if (keys) {
    TW_REQUIRE(values && slots && norm_w && L > 0 && Lp >= L && page_size > 0 && eps > 0.f);
    TW_REQUIRE(c_col >= 0 && kr_col >= 0 && ld >= c_col + (long)L && ld >= kr_col + (long)Rp);
  }
  if (n == 0) return 0;
  LatentFinishArgs a{proj, ld, q_col, c_col, kr_col, cos_t, sin_t, norm_w, q_out, ld_q, q_full, ld_full, D, Dp, hd, full_from,
                     keys, values, slots, H, L, Lp, Rp, rot, page_size, eps};
  if (dtype == TW_DTYPE_BF16) latent_finish_kernel<bf16_t><<<n, 256, 0, stream>>>(a);
  else if (dtype == TW_DTYPE_F32) latent_finish_kernel<float><<<n, 256, 0, stream>>>(a);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- one small matrix per head: out[n][a * so + o] = sum_i x[n][a * sx + i] * w[a][o][i] ------------------------
// x and out hold the heads side by side, sx and so elements apart; w [heads][No][Ni] row-major. A wave takes 16
// rows and 64 output columns of one head; the weights are the A operand, so a lane ends with four consecutive
// output columns of one row. Sums are float32, rounded once to the compute type.
template <typename T>
__global__ __launch_bounds__(256) void head_linear_kernel(const T* __restrict__ x, long ldx, int sx, const T* __restrict__ w,
                                                          T* __restrict__ out, long ldo, int so, int n, int heads, int Ni,
                                                          int No, int col_groups) {
  typedef typename Elem<T>::Frag Frag;
  constexpr int EPF = Elem<T>::kPerFrag;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int unit = blockIdx.x * 4 + wave;
  const int head = unit / col_groups, cg = unit % col_groups;
  if (head >= heads) return;
  const int row = blockIdx.y * 16 + r;
  const int chunks = Ni / EPF, steps = (chunks + 3) / 4;
  const T* x_row = x + (size_t)(row < n ? row : 0) * ldx + (size_t)head * sx;
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
      const Frag wf = (in && o < No) ? tw_load_frag(w + ((size_t)head * No + o) * Ni + chunk * EPF) : Elem<T>::zero();
      tw_mma16(acc[t], wf, xf);                            // D[output 4g + e][row r]
    }
  }
  if (row >= n) return;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int o = cg * 64 + t * 16 + 4 * g;
    if (o < No) {
      T* dst = out + (size_t)row * ldo + (size_t)head * so + o;
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[e] = tw_from_float<T>(acc[t][e]);
    }
  }
}

extern "C" int tw_head_linear(int dtype, const void* x, long ldx, int sx, const void* w, void* out, long ldo, int so,
                              int n, int heads, int Ni, int No, hipStream_t stream) {
  const int epf = dtype == TW_DTYPE_BF16 ? 8 : 4;
  TW_REQUIRE(x && w && out && n >= 0 && heads > 0 && Ni > 0 && No > 0);
  TW_REQUIRE(dtype == TW_DTYPE_BF16 || dtype == TW_DTYPE_F32);
  TW_REQUIRE(Ni % epf == 0 && No % 4 == 0 && ldx % epf == 0 && sx % epf == 0 && sx >= 0 && so >= No);
  TW_REQUIRE(ldx >= (long)(heads - 1) * sx + Ni && ldo >= (long)(heads - 1) * so + No);
  TW_REQUIRE((uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0);
  if (n == 0) return 0;
  const int col_groups = tw_div_up(No, 64);
  const dim3 grid(tw_div_up((long)heads * col_groups, 4), tw_div_up(n, 16));
  if (dtype == TW_DTYPE_BF16)
    head_linear_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, ldx, sx, (const bf16_t*)w, (bf16_t*)out, ldo, so, n,
                                                         heads, Ni, No, col_groups);
  else
    head_linear_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, ldx, sx, (const float*)w, (float*)out, ldo, so, n,
                                                        heads, Ni, No, col_groups);
  return TW_LAUNCH_RESULT();
}

// ---- prompt portions: keys and values expanded per head for this step ------------------------------------------------
// Against many query rows it is cheaper to expand the cached latents once (k_a = W_uk,a c, v_a = W_uv,a c for every
// cached token of the sequences that bring a portion) and to run ordinary attention with one key/value head per
// query head than to carry the latent's size through every score. Two kernels around one matrix product:
//
//   latent_gather:        the key rows [c | kr] of sequences seq0 .. from their pages into rows of their own, sequence
//                         after sequence, each starting at a multiple of the page size (row = page of its own * P + place),
//                         and the block table of those pages
//   (product)             up[row] = [W_uk ; W_uv] c[row]
//   latent_expand_store:  keys [page][a][place][hd] = [up k-part of head a | kr | zeros], values [page][a][hd][place]
//                         = [up v-part | zeros]: the layout the attention kernels read
struct LatentGatherArgs {
  const void* keys;                  // [pages][1][P][K]
  const int* block_table; int table_stride;
  const int* kv_len; const int* kv_page_start;      // kv_page_start[s]: pages of their own before sequence s (all sequences of the step)
  void* rows;                        // [own pages * P][K]
  int* own_table; int own_stride;    // [>= seq0 + n_seqs][own_stride]
  int seq0, n_seqs, P, K;
};

template <typename T>
__global__ __launch_bounds__(256) void latent_gather_kernel(LatentGatherArgs a) {
  const int base = a.kv_page_start[a.seq0];
  const int pg = blockIdx.x;                                   // page of its own, counted from seq0's first
  int lo = a.seq0, hi = a.seq0 + a.n_seqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (a.kv_page_start[mid] - base <= pg) lo = mid; else hi = mid - 1;
  }
  const int s = lo, b = pg - (a.kv_page_start[s] - base);
  if (pg >= a.kv_page_start[a.seq0 + a.n_seqs] - base) return;
  if (threadIdx.x == 0) a.own_table[(size_t)s * a.own_stride + b] = pg;
  const int phys = a.block_table[(size_t)s * a.table_stride + b];
  const int live = min(a.P, a.kv_len[s] - b * a.P);
  const T* src = (const T*)a.keys + (size_t)(phys < 0 ? 0 : phys) * a.P * a.K;
  T* dst = (T*)a.rows + (size_t)pg * a.P * a.K;
  for (int i = threadIdx.x; i < a.P * a.K; i += blockDim.x)
    dst[i] = (phys >= 0 && i / a.K < live) ? src[i] : tw_from_float<T>(0.f);
}

extern "C" int tw_latent_gather(int dtype, const void* keys, const int* block_table, int table_stride, const int* kv_len,
                                const int* kv_page_start, void* rows, int* own_table, int own_stride, int seq0, int n_seqs,
                                int own_pages, int page_size, int K, hipStream_t stream) {
  TW_REQUIRE(keys && block_table && kv_len && kv_page_start && rows && own_table && seq0 >= 0 && n_seqs >= 0 && own_pages >= 0);
  TW_REQUIRE(page_size > 0 && K > 0 && own_stride > 0);
  if (n_seqs == 0 || own_pages == 0) return 0;
  LatentGatherArgs a{keys, block_table, table_stride, kv_len, kv_page_start, rows, own_table, own_stride, seq0, n_seqs, page_size, K};
  if (dtype == TW_DTYPE_BF16) latent_gather_kernel<bf16_t><<<own_pages, 256, 0, stream>>>(a);
  else if (dtype == TW_DTYPE_F32) latent_gather_kernel<float><<<own_pages, 256, 0, stream>>>(a);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// One workgroup a page: up [rows][H * D + H * E] (the heads' key parts, then their value parts), kr at rows[row][Lp ..].
// VEC (bfloat16, sizes and strides that are multiples of 8): 16 bytes a thread. A key row is copied in groups of 8
// elements; for the transposed values a thread gathers one element of 8 consecutive places (neighbouring threads
// read neighbouring elements of one row) and stores them as one group.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void latent_expand_store_kernel(const T* __restrict__ up, long ld_up, const T* __restrict__ rows,
                                                                  int K, int Lp, T* __restrict__ keys, T* __restrict__ values,
                                                                  int H, int D, int R, int E, int hd, int P) {
  const int pg = blockIdx.x;
  T* kp = keys + (size_t)pg * H * P * hd;
  T* vp = values + (size_t)pg * H * hd * P;
  if (VEC) {
    const int groups = hd / 8;
    for (int i = threadIdx.x; i < H * P * groups; i += blockDim.x) {
      const int d = (i % groups) * 8, t = (i / groups) % P, a = i / (groups * P);
      const size_t row = (size_t)pg * P + t;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (d < D) v = *reinterpret_cast<const u32x4*>(up + row * ld_up + a * D + d);
      else if (d < D + R) v = *reinterpret_cast<const u32x4*>(rows + row * K + Lp + d - D);
      *reinterpret_cast<u32x4*>(kp + ((size_t)a * P + t) * hd + d) = v;
    }
    const int tgs = P / 8;
    for (int i = threadIdx.x; i < H * tgs * hd; i += blockDim.x) {
      const int e = i % hd, tg = (i / hd) % tgs, a = i / (hd * tgs);
      bf16x8 v;
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const size_t row = (size_t)pg * P + tg * 8 + x;
        v[x] = e < E ? up[row * ld_up + (size_t)H * D + a * E + e] : (bf16_t)0.f;
      }
      *reinterpret_cast<bf16x8*>(vp + ((size_t)a * hd + e) * P + tg * 8) = v;
    }
    return;
  }
  for (int i = threadIdx.x; i < H * P * hd; i += blockDim.x) {
    const int d = i % hd, t = (i / hd) % P, a = i / (hd * P);
    const size_t row = (size_t)pg * P + t;
    T v = tw_from_float<T>(0.f);
    if (d < D) v = up[row * ld_up + a * D + d];
    else if (d < D + R) v = rows[row * K + Lp + d - D];
    kp[i] = v;
  }
  for (int i = threadIdx.x; i < H * hd * P; i += blockDim.x) {
    const int t = i % P, e = (i / P) % hd, a = i / (P * hd);
    const size_t row = (size_t)pg * P + t;
    vp[i] = e < E ? up[row * ld_up + (size_t)H * D + a * E + e] : tw_from_float<T>(0.f);
  }
}

extern "C" int tw_latent_expand_store(int dtype, const void* up, long ld_up, const void* rows, int K, int Lp, void* keys,
                                      void* values, int own_pages, int H, int D, int R, int E, int hd, int page_size,
                                      hipStream_t stream) {
  TW_REQUIRE(up && rows && keys && values && own_pages >= 0 && H > 0 && D > 0 && R >= 0 && E > 0 && page_size > 0);
  TW_REQUIRE(hd >= D + R && hd >= E && ld_up >= (long)H * (D + E) && K >= Lp + R);
  if (own_pages == 0) return 0;
  const bool vec = dtype == TW_DTYPE_BF16 && D % 8 == 0 && R % 8 == 0 && E % 8 == 0 && hd % 8 == 0 && page_size % 8 == 0 &&
                   ld_up % 8 == 0 && K % 8 == 0 && Lp % 8 == 0 && (uintptr_t)up % 16 == 0 && (uintptr_t)rows % 16 == 0 &&
                   (uintptr_t)keys % 16 == 0 && (uintptr_t)values % 16 == 0;
  if (vec)
    latent_expand_store_kernel<bf16_t, true><<<own_pages, 256, 0, stream>>>((const bf16_t*)up, ld_up, (const bf16_t*)rows, K, Lp,
                                                                            (bf16_t*)keys, (bf16_t*)values, H, D, R, E, hd, page_size);
  else if (dtype == TW_DTYPE_BF16)
    latent_expand_store_kernel<bf16_t, false><<<own_pages, 256, 0, stream>>>((const bf16_t*)up, ld_up, (const bf16_t*)rows, K, Lp,
                                                                             (bf16_t*)keys, (bf16_t*)values, H, D, R, E, hd, page_size);
  else if (dtype == TW_DTYPE_F32)
    latent_expand_store_kernel<float, false><<<own_pages, 256, 0, stream>>>((const float*)up, ld_up, (const float*)rows, K, Lp,
                                                                            (float*)keys, (float*)values, H, D, R, E, hd, page_size);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- one-token sequences: all heads of a sequence against the one cached head ------------------------------------------
// The query heads are the 16 columns of the matrix unit's tile (a launch has one workgroup row per 16 heads): per 16
// keys a wave forms S^T = K Q^T (keys down, heads across), so every head's probabilities leave the product in the
// layout the next one, O^T += V^T P^T, wants as its operand, and a key row is read once for 16 heads. Values are the
// first Lp elements of the key rows, kept a second time transposed inside a page ([Lp][P]) so that four consecutive
// keys of one element are one 8-byte load. A sequence's keys are cut into `splits` ranges for separate workgroups,
// whose waves take the range's tiles in turn; waves are combined through LDS, ranges by a second kernel in index order.
//
//   part [seq][head tile][split][16][Lp + 2]: output sums relative to the range's maximum, that maximum, the sum
struct LatentDecodeArgs {
  const void* q; long ldq;            // head a of sequence s at q + row(s) * ldq + a * K
  const void* keys; const void* values;
  const int* block_table; int table_stride;
  const int* q_start; const int* kv_len;
  void* out; long ldo;                // head a at out + row(s) * ldo + a * Lp
  float* part;
  float scale;
  int H, K, Lp, P, splits;
  const float* sink;                  // [H] or null: exp(sink_a) more in head a's denominator (no key, no value, not scaled)
};

template <typename T> __device__ __forceinline__ float lt_exp(float v);
template <> __device__ __forceinline__ float lt_exp<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ float lt_exp<bf16_t>(float v) { return __expf(v); }

template <typename T> struct LtQuad;
template <> struct LtQuad<float> { typedef f32x4 Type; };
template <> struct LtQuad<bf16_t> { typedef bf16x4 Type; };

template <typename T>
__global__ __launch_bounds__(256) void latent_decode_kernel(LatentDecodeArgs a) {
  typedef typename Elem<T>::Frag Frag;
  typedef typename LtQuad<T>::Type Quad;
  constexpr int EPF = Elem<T>::kPerFrag;
  constexpr int STEP = 4 * EPF;                 // key elements one product consumes
  constexpr int KC_MAX = 256 / STEP;
  constexpr int LT_MAX = 15;                    // Lp <= 240
  extern __shared__ float ld_lds[];
  const int s = blockIdx.x, split = blockIdx.y, ht = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int K = a.K, Lp = a.Lp, P = a.P;
  const int KC = (K + STEP - 1) / STEP, LT = Lp / 16;
  const int len = a.kv_len[s];
  const int row = a.q_start[s];
  const int head = ht * 16 + r;
  const int* table = a.block_table + (size_t)s * a.table_stride;
  const T* keys = (const T*)a.keys;
  const T* values = (const T*)a.values;
  // this lane's query fragments: head r, elements kc * STEP + g * EPF ..
  Frag qf[KC_MAX];
#pragma unroll
  for (int kc = 0; kc < KC_MAX; ++kc) {
    const int col = kc * STEP + g * EPF;
    qf[kc] = (kc < KC && col < K && head < a.H) ? tw_load_frag((const T*)a.q + (size_t)row * a.ldq + (size_t)head * K + col)
                                                 : Elem<T>::zero();
  }
  f32x4 O[LT_MAX];
#pragma unroll
  for (int lt = 0; lt < LT_MAX; ++lt) O[lt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, sum = 0.f;
  const int tiles = (len + 15) / 16;
  const int per = (tiles + a.splits - 1) / a.splits;
  const int t_begin = split * per, t_end = min(tiles, t_begin + per);
  for (int t = t_begin + wave; t < t_end; t += 4) {
    const bool edge = t * 16 + 16 > len;
    // S^T for 16 keys: this lane loads key t * 16 + r (a key past the end stands in for by the last one; masked below)
    const int pk = min(t * 16 + r, len - 1);
    const T* krow = keys + ((size_t)table[pk / P] * P + pk % P) * K;
    f32x4 S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kc = 0; kc < KC_MAX; ++kc) {
      if (kc < KC) {
        const int col = kc * STEP + g * EPF;
        const Frag kf = col < K ? tw_load_frag(krow + col) : Elem<T>::zero();
        tw_mma16(S, kf, qf[kc]);                  // S[j]: key t * 16 + 4 g + j against head r
      }
    }
    // values of keys t * 16 + 4 g .. + 3 (one page: pages hold a multiple of 4 keys)
    const int pv = min(t * 16 + 4 * g, (len - 1) / 4 * 4);
    const T* vbase = values + (size_t)table[pv / P] * Lp * P + pv % P;
    Quad vq[LT_MAX];
#pragma unroll
    for (int lt = 0; lt < LT_MAX; ++lt)
      if (lt < LT) vq[lt] = *reinterpret_cast<const Quad*>(vbase + (size_t)(lt * 16 + r) * P);
    float top = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      S[j] = (edge && t * 16 + 4 * g + j >= len) ? -INFINITY : S[j] * a.scale;
      top = fmaxf(top, S[j]);
    }
    top = tw_rows_max(top);                      // over the 16 keys, for head r
    const float m_new = fmaxf(m, top);
    const float alpha = m == -INFINITY ? 0.f : lt_exp<T>(m - m_new);
    f32x4 Pr;
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      Pr[j] = S[j] == -INFINITY ? 0.f : lt_exp<T>(S[j] - m_new);
      part += Pr[j];
    }
    sum = sum * alpha + tw_rows_sum(part);
    m = m_new;
#pragma unroll
    for (int lt = 0; lt < LT_MAX; ++lt) {
      if (lt < LT) {
        Quad v = vq[lt];
        if (edge) {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (t * 16 + 4 * g + j >= len) v[j] = tw_from_float<T>(0.f);     // whatever lies there must not reach a sum
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) O[lt][j] *= alpha;
        tw_mma16_k4(O[lt], v, Pr);               // O[lt][j]: element lt * 16 + 4 g + j of head r
      }
    }
  }
  // ---- the four waves' results through LDS: [wave][16 heads][Lp + 4] sums, then [wave][16] maxima and sums
  const int OS = Lp + 4;
  float* Ow = ld_lds;
  float* mw = Ow + (size_t)4 * 16 * OS;
  float* sw = mw + 64;
#pragma unroll
  for (int lt = 0; lt < LT_MAX; ++lt)
    if (lt < LT) *reinterpret_cast<f32x4*>(Ow + ((size_t)wave * 16 + r) * OS + lt * 16 + 4 * g) = O[lt];
  if (g == 0) {
    mw[wave * 16 + r] = m;
    sw[wave * 16 + r] = sum;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 16 * Lp; i += 256) {
    const int hh = i / Lp, l = i - hh * Lp;
    if (ht * 16 + hh >= a.H) continue;
    float top = fmaxf(fmaxf(mw[hh], mw[16 + hh]), fmaxf(mw[32 + hh], mw[48 + hh]));
    float o = 0.f, total = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = mw[w * 16 + hh] == -INFINITY ? 0.f : lt_exp<T>(mw[w * 16 + hh] - top);
      o += f * Ow[((size_t)w * 16 + hh) * OS + l];
      total += f * sw[w * 16 + hh];
    }
    if (a.splits == 1) {
      if (a.sink) {
        const float sk = a.sink[ht * 16 + hh];
        const float both = fmaxf(top, sk);
        const float f = top == -INFINITY ? 0.f : lt_exp<T>(top - both);
        o *= f;
        total = total * f + lt_exp<T>(sk - both);
      }
      ((T*)a.out)[(size_t)row * a.ldo + (size_t)(ht * 16 + hh) * Lp + l] = tw_from_float<T>(o / total);
    } else {
      float* dst = a.part + ((((size_t)s * gridDim.z + ht) * a.splits + split) * 16 + hh) * (Lp + 2);
      dst[l] = o;
      if (l == 0) {
        dst[Lp] = top;
        dst[Lp + 1] = total;
      }
    }
  }
}

// One workgroup a (sequence, head): the ranges' maxima and sums first (one thread a range), then a thread an element.
template <typename T>
__global__ __launch_bounds__(256) void latent_decode_merge_kernel(LatentDecodeArgs a) {
  __shared__ float weight[64];
  __shared__ float total_s;
  const int s = blockIdx.x, head = blockIdx.y;
  const int ht = head >> 4, hh = head & 15;
  const int Lp = a.Lp;
  const int row = a.q_start[s];
  const int head_tiles = (a.H + 15) / 16;
  const float* base = a.part + ((((size_t)s * head_tiles + ht) * a.splits) * 16 + hh) * (Lp + 2);
  const size_t stride = (size_t)16 * (Lp + 2);                  // from one range to the next
  if (threadIdx.x < 64) {
    const int sp = threadIdx.x;
    const float m = sp < a.splits ? base[sp * stride + Lp] : -INFINITY;
    float top = tw_wave_max(m);
    const float sk = a.sink ? a.sink[head] : -INFINITY;
    top = fmaxf(top, sk);
    const float f = m == -INFINITY ? 0.f : lt_exp<T>(m - top);
    weight[sp] = f;
    const float total = tw_wave_sum(sp < a.splits ? f * base[sp * stride + Lp + 1] : 0.f);
    if (sp == 0) total_s = total + (a.sink ? lt_exp<T>(sk - top) : 0.f);
  }
  __syncthreads();
  const float inv = 1.f / total_s;
  for (int l = threadIdx.x; l < Lp; l += 256) {
    float o = 0.f;
    for (int sp = 0; sp < a.splits; ++sp) o += weight[sp] * base[sp * stride + l];
    ((T*)a.out)[(size_t)row * a.ldo + (size_t)head * Lp + l] = tw_from_float<T>(o * inv);
  }
}

// Key ranges a sequence: enough workgroups for the chip, each range at least 8 tiles of 16 keys.
extern "C" int tw_latent_decode_splits(int n_seqs, int heads, int max_kv_len) {
  if (n_seqs <= 0) return 1;
  const int tiles = tw_div_up(max_kv_len, 16);
  int want = 512 / (n_seqs * tw_div_up(heads, 16));
  if (want > tiles / 8) want = tiles / 8;
  if (want > 64) want = 64;
  return want < 1 ? 1 : want;
}

extern "C" long tw_latent_decode_workspace_floats(int n_seqs, int heads, int Lp, int splits) {
  return splits > 1 ? (long)n_seqs * tw_div_up(heads, 16) * splits * 16 * (Lp + 2) : 0;
}

extern "C" int tw_latent_decode(int dtype, const void* q, long ldq, const void* keys, const void* values,
                                const int* block_table, int table_stride, const int* q_start, const int* kv_len,
                                int n_seqs, void* out, long ldo, float* workspace, long workspace_floats, int heads,
                                int K, int Lp, int page_size, float scale, int splits, const float* sink, hipStream_t stream) {
  TW_REQUIRE(q && keys && values && block_table && q_start && kv_len && out && n_seqs >= 0 && splits >= 1 && splits <= 64);
  TW_REQUIRE(heads >= 1 && K % 16 == 0 && K <= 256 && Lp % 16 == 0 && Lp >= 16 && Lp <= 240 && Lp <= K);
  TW_REQUIRE(page_size > 0 && page_size % 4 == 0);
  TW_REQUIRE(ldq >= (long)heads * K && ldo >= (long)heads * Lp);
  const int esize = dtype == TW_DTYPE_BF16 ? 2 : 4;
  TW_REQUIRE((uintptr_t)q % 16 == 0 && (uintptr_t)keys % 16 == 0 && (uintptr_t)values % 16 == 0 && (ldq * esize) % 16 == 0);
  if (splits > 1) TW_REQUIRE(workspace && workspace_floats >= tw_latent_decode_workspace_floats(n_seqs, heads, Lp, splits));
  if (n_seqs == 0) return 0;
  LatentDecodeArgs a{q, ldq, keys, values, block_table, table_stride, q_start, kv_len, out, ldo, workspace, scale,
                     heads, K, Lp, page_size, splits, sink};
  const int head_tiles = tw_div_up(heads, 16);
  const dim3 grid(n_seqs, splits, head_tiles);
  const size_t lds = ((size_t)4 * 16 * (Lp + 4) + 128) * sizeof(float);
  if (dtype == TW_DTYPE_BF16) {
    latent_decode_kernel<bf16_t><<<grid, 256, lds, stream>>>(a);
    if (splits > 1) latent_decode_merge_kernel<bf16_t><<<dim3(n_seqs, heads), 256, 0, stream>>>(a);
  } else if (dtype == TW_DTYPE_F32) {
    latent_decode_kernel<float><<<grid, 256, lds, stream>>>(a);
    if (splits > 1) latent_decode_merge_kernel<float><<<dim3(n_seqs, heads), 256, 0, stream>>>(a);
  } else {
    return TW_ERR_BAD_ARGUMENT;
  }
  return TW_LAUNCH_RESULT();
}
