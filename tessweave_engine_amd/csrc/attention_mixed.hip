// Attention whose scores are mixed across heads before the softmax, over the paged cache.
//
//   keys   [pages][kv_heads][page_size][D]
//   values [pages][kv_heads][E][page_size]     (transposed inside a page; E may differ from D)
//
// For query position i and key position j of one sequence (0 <= i - j < window, or every j <= i
// without a window; with a window, the first `keep` keys of the sequence stay visible to every later query, at
// their true positions):
//   raw_g(i, j)  = scale * q_ig . k_j,kv(g) - slope_g * (i - j)            (slopes optional)
//   s_h(i, j)    = sum_g talk[h][g] * raw_g(i, j)                          (talk optional: s = raw)
//   p_h(i, j)    = exp(s_h(i, j)) / (exp(sink_h) + sum_j' exp(s_h(i, j')))   (sink optional)
//   out_ih       = out_scale * sum_j p_h(i, j) v_j,kv(h)
// Scores, the mixing, the softmax and the output sums are float32.
//
// Because every head's score at (i, j) needs all heads' raw scores there, a workgroup takes 16
// query TOKENS with all their heads. Its waves share the heads out between them (HPW heads a
// wave). Per 16 keys a wave forms S^T = K Q^T for its heads on the matrix unit (accumulator
// element e of lane (r, g) is query row r against key 4g + e, the same place for every head),
// leaves the raw scores in LDS, and after one barrier reads all heads' raw scores of its own lane
// and mixes them for its heads: the mixing needs no exchange between lanes. The probabilities,
// still in accumulator layout, are the B operand of O^T += V^T P^T. The raw-score buffer exists
// twice, so one barrier per key tile is enough.
//
// A tile's keys can be cut into `splits` ranges for separate workgroups (one-token sequences, whose only tile
// would otherwise walk all keys alone; prompt portions with fewer tiles than the chip has CUs); a second kernel
// merges the partial results in index order.
#include "tw_common.h"

template <typename T> __device__ __forceinline__ float mx_exp(float v);
template <> __device__ __forceinline__ float mx_exp<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ float mx_exp<bf16_t>(float v) { return __expf(v); }

template <typename T> struct MxQuad;
template <> struct MxQuad<float> { typedef f32x4 Type; };
template <> struct MxQuad<bf16_t> { typedef bf16x4 Type; };

struct MixedAttnArgs {
  const void* q; long ldq;           // head h of token n at q + n * ldq + h * D
  const void* keys; const void* values;
  const int* block_table; int table_stride;
  const int* q_start; const int* kv_len;
  int seq0;
  void* out; long ldo;               // head h of token n at out + n * ldo + h * E
  const float* talk;                 // [H][H] or null
  const float* sink;                 // [H] or null
  const float* slopes;               // [H] or null
  float* part;                       // splits > 1: [seq - seq0][tile][split][H][rows_kept][E + 2] (output sums, max, sum)
  float scale, out_scale;
  int H, G, D, E, P, window, splits;
  int keep;                          // with a window: keys 0 .. keep - 1 are seen by every later query as well
  int page_shift;                    // log2(P) if P is a power of two, else -1
  int rows_kept;                     // rows of a tile whose partial results are kept: 1 for one-token sequences, else 16
  int q_in_lds;                      // 0: the tile's queries do not fit LDS beside the raw scores; fragments are read from memory
};

// Dynamic LDS: q tile [H][16][D + pad] of T (if it fits), raw scores [2][H][64] of f32x4, talk [H][H] floats.
template <typename T>
__host__ __device__ inline size_t mx_q_row(int D) { return (size_t)D + 16 / sizeof(T); }

template <typename T>
static size_t mx_lds_bytes(int H, int D, bool q_in_lds) {
  size_t q = q_in_lds ? (size_t)H * 16 * mx_q_row<T>(D) * sizeof(T) : 0;
  q = (q + 15) / 16 * 16;
  return q + (size_t)2 * H * 64 * 16 + (size_t)H * H * 4;
}

// HPW heads a wave, VT 16-column tiles of a head's values, WMAX the most waves a workgroup may have (it sets the
// registers a lane may use), AHEAD whether key fragments are requested a tile ahead (it costs registers), SHARE
// whether all heads of a wave read the same key/value head (its fragments are then loaded once for all of them,
// and everything a wave does once a key tile, page lookups, addresses, loads, is paid once for HPW heads).
// EXACT: the key size is exactly what four MFMA steps of fragments hold (128 in bfloat16, 64 in float32) and the
// value size is 16 VT: sizes and loop bounds are then compile-time constants.
template <typename T, int HPW, int VT, int WMAX, bool AHEAD, bool SHARE, bool EXACT>
__global__ __launch_bounds__(WMAX * 64) void attn_mixed_kernel(MixedAttnArgs a) {
  constexpr int KVN = SHARE ? 1 : HPW;                     // key/value heads a wave loads
  typedef typename Elem<T>::Frag Frag;
  typedef typename MxQuad<T>::Type Quad;
  constexpr int EPF = Elem<T>::kPerFrag;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int H = a.H, P = a.P;
  const int D = EXACT ? 16 * Elem<T>::kPerFrag : a.D, E = EXACT ? 16 * VT : a.E;
  const size_t qrow = mx_q_row<T>(D);
  T* lds_q = (T*)lds_raw;
  size_t q_bytes = a.q_in_lds ? (size_t)H * 16 * qrow * sizeof(T) : 0;
  q_bytes = (q_bytes + 15) / 16 * 16;
  f32x4* lds_s = (f32x4*)(lds_raw + q_bytes);
  float* lds_talk = (float*)(lds_raw + q_bytes + (size_t)2 * H * 64 * 16);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int seq = a.seq0 + blockIdx.y;
  const int q0 = a.q_start[seq], q_len = a.q_start[seq + 1] - q0;
  const int tile = blockIdx.x;
  if (tile * 16 >= q_len) return;
  const int kv_len = a.kv_len[seq];
  const int n_rows = min(16, q_len - tile * 16);
  const int pos0 = kv_len - q_len + tile * 16;              // position of the tile's first row
  const int t_row = r < n_rows ? pos0 + r : -1;
  const int* table = a.block_table + (size_t)seq * a.table_stride;
  const int heads_per_kv = H / a.G;
  const int chunks = EXACT ? 16 : D / EPF, steps = EXACT ? 4 : (chunks + 3) / 4, dts = EXACT ? VT : E / 16;

  // ---- stage the tile's queries and the mixing matrix ------------------------------------------------
  for (int i = threadIdx.x; i < (a.q_in_lds ? H * 16 * chunks : 0); i += blockDim.x) {
    const int chunk = i % chunks, row = (i / chunks) % 16, head = i / (chunks * 16);
    Frag f = Elem<T>::zero();
    if (row < n_rows)
      f = tw_load_frag((const T*)a.q + (size_t)(q0 + tile * 16 + row) * a.ldq + (size_t)head * D + chunk * EPF);
    *reinterpret_cast<Frag*>(lds_q + ((size_t)head * 16 + row) * qrow + chunk * EPF) = f;
  }
  for (int i = threadIdx.x; i < H * H; i += blockDim.x)
    lds_talk[i] = a.talk ? a.talk[i] : ((i / H == i % H) ? 1.f : 0.f);
  __syncthreads();

  // ---- the key tiles of this workgroup ---------------------------------------------------------------------
  const int lo = a.window > 0 ? max(0, pos0 - a.window + 1) : 0;       // first key any row of the tile sees
  const int hi = pos0 + n_rows - 1;                                     // last key (its own position)
  // The key tiles a workgroup walks are numbered without the gap between the kept first keys and the window: tiles
  // 0 .. kept - 1 hold the kept keys that lie before the window's first tile, the tiles behind them are the window's.
  const int keep = a.window > 0 ? a.keep : 0;
  const int win_lo = lo / 16;
  const int kept = min((keep + 15) / 16, win_lo);
  const int skip = win_lo - kept;                                        // key tile of walk index v >= kept: v + skip
  int tile_lo = 0, tile_hi = hi / 16 + 1 - skip;
  if (a.splits > 1) {
    const int per = (tile_hi - tile_lo + a.splits - 1) / a.splits;
    tile_lo = tile_lo + blockIdx.z * per;
    tile_hi = min(tile_hi, tile_lo + per);
  }
  auto key_tile = [&](int v) { return v < kept ? v : v + skip; };
  const bool with_sink = a.sink != nullptr && (a.splits == 1 || blockIdx.z == 0);

  float m[HPW], l[HPW];
  f32x4 acc[HPW][VT];
  float slope[HPW];
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    const int head = wave * HPW + i;
    m[i] = (with_sink && head < H) ? a.sink[head] : -INFINITY;     // the sink: a key of score sink_h and value zero
    l[i] = (with_sink && head < H) ? 1.f : 0.f;
    slope[i] = (a.slopes && head < H) ? a.slopes[head] : 0.f;
#pragma unroll
    for (int dt = 0; dt < VT; ++dt) acc[i][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const T* keys = (const T*)a.keys;
  const T* values = (const T*)a.values;
  const T* q_global = (const T*)a.q + (size_t)(q0 + tile * 16 + (r < n_rows ? r : 0)) * a.ldq;
  auto q_frag = [&](int head, int chunk) -> Frag {
    if (chunk >= chunks) return Elem<T>::zero();
    if (a.q_in_lds) return *reinterpret_cast<const Frag*>(lds_q + ((size_t)head * 16 + r) * qrow + chunk * EPF);
    return r < n_rows ? tw_load_frag(q_global + (size_t)head * D + chunk * EPF) : Elem<T>::zero();
  };
  // Loads carry no condition on the page: a key outside the sequence or the window is read from page 0 (every
  // pool has one), its score is selected away and its value set to zero by the masks of the edge tile it lies
  // in (a tile that is not an edge tile has no such key), so whatever that page holds never reaches a result.
  // The K fragments of a key tile are requested one tile ahead (while the tile before is mixed and multiplied
  // with its values), the V quads of a tile before the barrier that publishes its raw scores: a tile then waits
  // for memory once, not twice, and mostly not at all. KP fragments a head fit the registers kept for that
  // (head sizes up to 128 in bfloat16, 64 in float32); longer heads load their fragments where they are used.
  constexpr int KP = AHEAD ? 4 : 1;
  const bool ahead = AHEAD && steps <= KP;
  Frag kpre[KVN][KP];
  // Page numbers are looked up a tile before the loads that need them, so that no load waits for a lookup.
  const int shift = a.page_shift;
  auto page_of = [&](int p) { return shift >= 0 ? p >> shift : p / P; };
  auto in_page = [&](int p) { return shift >= 0 ? p & (P - 1) : p % P; };
  auto key_page = [&](int v) -> int {
    const int p = key_tile(v) * 16 + r;
    return (v < tile_hi && p < kv_len && (p >= lo || p < keep)) ? table[page_of(p)] : -1;
  };
  auto value_page = [&](int v) -> int {
    const int p = key_tile(v) * 16 + 4 * g;
    return (v < tile_hi && p < kv_len && (p + 3 >= lo || p < keep)) ? table[page_of(p)] : -1;
  };
  auto request_keys = [&](int v, int page) {
    if constexpr (!AHEAD) return;
    const int p = key_tile(v) * 16 + r;
#pragma unroll
    for (int i = 0; i < KVN; ++i) {
      const int head = wave * HPW + i;                     // (SHARE: the wave's first head stands for all)
      const int kvh = (head < H ? head : 0) / heads_per_kv;
      const T* k_row = keys + (((size_t)(page < 0 ? 0 : page) * a.G + kvh) * P + in_page(p)) * D;
#pragma unroll
      for (int st = 0; st < KP; ++st) {
        const int chunk = st * 4 + g;
        kpre[i][st] = chunk < chunks ? tw_load_frag(k_row + chunk * EPF) : Elem<T>::zero();
      }
    }
  };
  int kpage = key_page(tile_lo);
  if (ahead) request_keys(tile_lo, kpage);
  int kpage_next = key_page(tile_lo + 1);
  int vpage = value_page(tile_lo);
  int buf = 0;
  for (int kt = tile_lo; kt < tile_hi; ++kt, buf ^= 1) {
    const int p0 = key_tile(kt) * 16;
    // A tile whose 16 keys every row of the query tile sees (none beyond the first row's position, none before
    // the last row's window) needs no masks; most tiles of a long window are such.
    const bool interior = p0 + 15 <= pos0 && (a.window == 0 || p0 >= pos0 + n_rows - a.window || p0 + 15 < keep);
    // ---- raw scores of this wave's heads ---------------------------------------------------------------
    f32x4 raw_own[HPW];
    {
      const int p = p0 + r;
      const int page = kpage;
#pragma unroll
      for (int i = 0; i < HPW; ++i) {
        const int head = wave * HPW + i;
        raw_own[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (head < H) {
          f32x4 s = {0.f, 0.f, 0.f, 0.f};
          if (AHEAD && ahead) {
#pragma unroll
            for (int st = 0; st < KP; ++st) {
              const int chunk = st * 4 + g;
              if (st < steps) {
                tw_mma16(s, kpre[SHARE ? 0 : i][st], q_frag(head, chunk));
              }
            }
          } else {
            const int kvh = head / heads_per_kv;
            const T* k_row = keys + (((size_t)(page < 0 ? 0 : page) * a.G + kvh) * P + in_page(p)) * D;
            for (int st = 0; st < steps; ++st) {
              const int chunk = st * 4 + g;
              const bool in = chunk < chunks;
              const Frag kf = (page >= 0 && in) ? tw_load_frag(k_row + chunk * EPF) : Elem<T>::zero();
              tw_mma16(s, kf, q_frag(head, chunk));
            }
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) s[e] = s[e] * a.scale - slope[i] * (float)(t_row - (p0 + 4 * g + e));
          raw_own[i] = s;
        }
      }
    }
    // ---- this tile's values, then the next tile's keys: both are on their way during the mixing -----------------
    const int pv = p0 + 4 * g;
    Quad vq[KVN][VT];
#pragma unroll
    for (int i = 0; i < KVN; ++i) {
      const int head = wave * HPW + i;
      const int kvh = (head < H ? head : 0) / heads_per_kv;
      const T* v_base = values + ((size_t)(vpage < 0 ? 0 : vpage) * a.G + kvh) * E * P + in_page(pv);
#pragma unroll
      for (int dt = 0; dt < VT; ++dt) {
        if (dt < dts) vq[i][dt] = *reinterpret_cast<const Quad*>(v_base + (size_t)(dt * 16 + r) * P);
      }
    }
    if (ahead) request_keys(kt + 1, kpage_next);
    kpage = kpage_next;
    kpage_next = key_page(kt + 2);
    vpage = value_page(kt + 1);          // (this tile's quads are in registers already)
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      const int head = wave * HPW + i;
      if (head < H) lds_s[((size_t)buf * H + head) * 64 + lane] = raw_own[i];
    }
    __syncthreads();
    // ---- mix, mask, online softmax, O^T += V^T P^T ------------------------------------------------------------
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      const int head = wave * HPW + i;
      if (head < H) {
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
        const float* talk_row = lds_talk + head * H;
        const f32x4* raw_lane = lds_s + (size_t)buf * H * 64 + lane;
        int other = 0;
        for (; other + 4 <= H; other += 4) {               // four heads' reads in flight at a time
          const f32x4 r0 = raw_lane[(other + 0) * 64], r1 = raw_lane[(other + 1) * 64];
          const f32x4 r2 = raw_lane[(other + 2) * 64], r3 = raw_lane[(other + 3) * 64];
          const float w0 = talk_row[other], w1 = talk_row[other + 1], w2 = talk_row[other + 2], w3 = talk_row[other + 3];
#pragma unroll
          for (int e = 0; e < 4; ++e) s[e] += w0 * r0[e] + w1 * r1[e] + w2 * r2[e] + w3 * r3[e];
        }
        for (; other < H; ++other) {
          const float w = talk_row[other];
          const f32x4 raw = raw_lane[other * 64];
#pragma unroll
          for (int e = 0; e < 4; ++e) s[e] += w * raw[e];
        }
        float mx = -INFINITY;
        if (!interior) {
          const int lo_row = a.window > 0 ? t_row - a.window + 1 : 0;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int p = p0 + 4 * g + e;
            const bool ok = p < kv_len && p <= t_row && (p >= lo_row || p < keep);
            s[e] = ok ? s[e] : -INFINITY;
          }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) mx = fmaxf(mx, s[e]);
        mx = tw_rows_max(mx);
        const float m_new = fmaxf(m[i], mx);
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = mx_exp<T>(m[i] - m_use);
        f32x4 pr;
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pr[e] = mx_exp<T>(s[e] - m_use);
          sum += pr[e];
        }
        sum = tw_rows_sum(sum);
        l[i] = l[i] * alpha + sum;
        m[i] = m_new;
        // the output sums are rescaled only when some row's maximum has moved (a branch the whole wave takes alike)
        const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.f) != 0;
#pragma unroll
        for (int dt = 0; dt < VT; ++dt) {
          if (dt < dts) {
            Quad v = vq[SHARE ? 0 : i][dt];
            if (!interior) {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (pv + e >= kv_len || (pv + e < lo && pv + e >= keep)) v[e] = tw_from_float<T>(0.f);
            }
            if (rescale) {
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[i][dt][e] *= alpha;
            }
            tw_mma16_k4(acc[i][dt], v, pr);
          }
        }
      }
    }
  }

  // ---- results: lane (r, g) holds out[row r][16 dt + 4 g + e] ------------------------------------------------------
#pragma unroll
  for (int i = 0; i < HPW; ++i) {
    const int head = wave * HPW + i;
    if (head >= H || r >= n_rows) continue;
    if (a.splits == 1) {
      const float inv = l[i] > 0.f ? a.out_scale / l[i] : 0.f;
      T* dst = (T*)a.out + (size_t)(q0 + tile * 16 + r) * a.ldo + (size_t)head * E;
#pragma unroll
      for (int dt = 0; dt < VT; ++dt)
        if (dt < dts)
#pragma unroll
          for (int e = 0; e < 4; ++e) dst[dt * 16 + 4 * g + e] = tw_from_float<T>(acc[i][dt][e] * inv);
    } else if (r < a.rows_kept) {
      float* dst = a.part + (((((size_t)blockIdx.y * gridDim.x + tile) * a.splits + blockIdx.z) * H + head) * a.rows_kept + r) * (E + 2);
#pragma unroll
      for (int dt = 0; dt < VT; ++dt)
        if (dt < dts)
#pragma unroll
          for (int e = 0; e < 4; ++e) dst[dt * 16 + 4 * g + e] = acc[i][dt][e];
      if (g == 0) {
        dst[E] = m[i];
        dst[E + 1] = l[i];
      }
    }
  }
}

// Merge the partial results of a tile's key ranges, in index order. grid (tiles, n_seqs, H).
template <typename T>
__global__ __launch_bounds__(256) void attn_mixed_merge_kernel(MixedAttnArgs a) {
  const int seq = a.seq0 + blockIdx.y, head = blockIdx.z, tile = blockIdx.x;
  const int q0 = a.q_start[seq], q_len = a.q_start[seq + 1] - q0;
  if (tile * 16 >= q_len) return;
  const int n_rows = min(min(16, q_len - tile * 16), a.rows_kept);
  const int E = a.E;
  const size_t stride = (size_t)a.H * a.rows_kept * (E + 2);          // between key ranges
  const float* tile_base = a.part + ((((size_t)blockIdx.y * gridDim.x + tile) * a.splits) * a.H + head) * a.rows_kept * (E + 2);
  for (int i = threadIdx.x; i < n_rows * E; i += blockDim.x) {
    const int row = i / E, d = i % E;
    const float* base = tile_base + (size_t)row * (E + 2);
    float m = -INFINITY;
    for (int s = 0; s < a.splits; ++s) m = fmaxf(m, base[s * stride + E]);
    const float m_use = m == -INFINITY ? 0.f : m;
    float l = 0.f, o = 0.f;
    for (int s = 0; s < a.splits; ++s) {
      const float f = mx_exp<T>(base[s * stride + E] - m_use);
      l += base[s * stride + E + 1] * f;
      o += base[s * stride + d] * f;
    }
    const float inv = l > 0.f ? a.out_scale / l : 0.f;
    ((T*)a.out)[(size_t)(q0 + tile * 16 + row) * a.ldo + (size_t)head * E + d] = tw_from_float<T>(o * inv);
  }
}

template <typename T, int HPW, int VT, int WMAX, bool AHEAD, bool SHARE, bool EXACT = false>
static int mixed_launch(const MixedAttnArgs& a, int n_seqs, int tiles, int waves, size_t lds, hipStream_t stream) {
  auto kernel = attn_mixed_kernel<T, HPW, VT, WMAX, AHEAD, SHARE, EXACT>;
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
  }
  kernel<<<dim3(tiles, n_seqs, a.splits), waves * 64, lds, stream>>>(a);
  return TW_LAUNCH_RESULT();
}

template <typename T>
static int mixed_dispatch(const MixedAttnArgs& args, int n_seqs, int max_q_len, hipStream_t stream) {
  const int tiles = tw_div_up(max_q_len, 16);
  // Heads a wave: one up to 8 heads, two above (workgroups of up to 8 waves up to 16 heads). What a wave does once
  // a key tile (page lookups, addresses, loads of keys and values) is paid once for both heads where they share a
  // key/value head, and fewer waves wait at the tile's barrier. The output sums of a wave's heads live in its registers.
  // (measured at 2,048 tokens, heads of 128: 8 heads 164 us with one head a wave, 218 with two; 12 heads 338 and
  // 295; 16 heads 431 and 271; four heads a wave ran out of registers and was slower than two at 16 and 32 heads)
  const int per_kv = args.H / args.G;
  const int hpw = args.H <= 8 ? 1 : 2;
  const int waves = tw_div_up(args.H, hpw);
  const bool share = hpw == 2 && per_kv % 2 == 0;
  MixedAttnArgs a = args;
  a.q_in_lds = mx_lds_bytes<T>(a.H, a.D, true) <= 150 * 1024 ? 1 : 0;
  a.rows_kept = max_q_len == 1 ? 1 : 16;
  a.page_shift = (a.P & (a.P - 1)) == 0 ? __builtin_ctz(a.P) : -1;
  const size_t lds = mx_lds_bytes<T>(a.H, a.D, a.q_in_lds != 0);
  TW_REQUIRE(waves <= 16 && lds <= 150 * 1024);
  int code;
  // (the sizes of most models: compile-time instances for values of 128 beside keys of four MFMA steps)
  const bool exact = a.D == 16 * Elem<T>::kPerFrag && a.E == 128;
#define TW_MIXED(HPW_, VT_, WMAX_, AHEAD_)                                                                          \
  (exact && VT_ == 8 && AHEAD_                                                                                      \
     ? (share ? mixed_launch<T, HPW_, VT_, WMAX_, AHEAD_, (HPW_ > 1), (VT_ == 8 && AHEAD_)>(a, n_seqs, tiles, waves, lds, stream)  \
              : mixed_launch<T, HPW_, VT_, WMAX_, AHEAD_, false, (VT_ == 8 && AHEAD_)>(a, n_seqs, tiles, waves, lds, stream))      \
     : (share ? mixed_launch<T, HPW_, VT_, WMAX_, AHEAD_, (HPW_ > 1)>(a, n_seqs, tiles, waves, lds, stream)          \
              : mixed_launch<T, HPW_, VT_, WMAX_, AHEAD_, false>(a, n_seqs, tiles, waves, lds, stream)))
  if (hpw == 1)
    code = a.E <= 64 ? TW_MIXED(1, 4, 8, true) : a.E <= 128 ? TW_MIXED(1, 8, 8, true) : TW_MIXED(1, 16, 8, true);
  else if (waves <= 8)
    code = a.E <= 64 ? TW_MIXED(2, 4, 8, true) : a.E <= 128 ? TW_MIXED(2, 8, 8, true) : TW_MIXED(2, 16, 8, true);
  else                          // more than 16 heads: up to 16 waves, half the registers each
    code = a.E <= 64 ? TW_MIXED(2, 4, 16, false) : a.E <= 128 ? TW_MIXED(2, 8, 16, false) : TW_MIXED(2, 16, 16, false);
#undef TW_MIXED
  if (code != 0 || a.splits == 1) return code;
  attn_mixed_merge_kernel<T><<<dim3(tiles, n_seqs, a.H), 256, 0, stream>>>(a);
  return TW_LAUNCH_RESULT();
}

// Key ranges for one-token sequences: enough workgroups to spread over the chip, each with at least 4 key tiles.
extern "C" int tw_attn_mixed_splits(int n_seqs, int max_kv_len) {
  if (n_seqs <= 0) return 1;
  const int tiles = tw_div_up(max_kv_len, 16);
  int want = 1024 / n_seqs;
  int most = tiles / 4;
  int s = want < most ? want : most;
  if (s > 64) s = 64;
  return s < 1 ? 1 : s;
}

// Key ranges for prompt portions: only where the row tiles alone would leave most of the chip idle and a tile
// has keys enough to share out (each range at least 8 key tiles).
extern "C" int tw_attn_mixed_prefill_splits(int n_tokens, int n_seqs, int max_kv_len) {
  const int tiles = tw_div_up(n_tokens, 16) + n_seqs;
  const int key_tiles = tw_div_up(max_kv_len, 16);
  int s = 384 / (tiles > 0 ? tiles : 1);
  if (s > key_tiles / 8) s = key_tiles / 8;
  if (s > 8) s = 8;
  return s < 1 ? 1 : s;
}

extern "C" long tw_attn_mixed_workspace_floats(int n_seqs, int max_q_len, int q_heads, int value_dim, int splits) {
  const long tiles = tw_div_up(max_q_len, 16);
  return (long)n_seqs * tiles * splits * q_heads * (max_q_len == 1 ? 1 : 16) * (value_dim + 2);
}

extern "C" int tw_attn_mixed(int dtype, const void* q, long ldq, const void* keys, const void* values,
                             const int* block_table, int table_stride, const int* q_start, const int* kv_len,
                             int seq0, int n_seqs, int max_q_len, void* out, long ldo, const float* talk,
                             const float* sink, const float* slopes, float* workspace, long workspace_floats,
                             int q_heads, int kv_heads, int key_dim, int value_dim, int page_size, int window,
                             int keep_first, float scale, float out_scale, int splits, hipStream_t stream) {
  TW_REQUIRE(q && keys && values && block_table && q_start && kv_len && out);
  TW_REQUIRE(n_seqs >= 0 && seq0 >= 0 && max_q_len >= 1 && splits >= 1 && window >= 0 && keep_first >= 0);
  TW_REQUIRE(q_heads >= 1 && q_heads <= 32 && kv_heads >= 1 && q_heads % kv_heads == 0);
  TW_REQUIRE(key_dim % 16 == 0 && key_dim >= 16 && key_dim <= 256 && value_dim % 16 == 0 && value_dim >= 16 && value_dim <= 256);
  TW_REQUIRE(page_size > 0 && page_size % 4 == 0);
  TW_REQUIRE(ldq >= (long)q_heads * key_dim && ldo >= (long)q_heads * value_dim);
  TW_REQUIRE((uintptr_t)q % 16 == 0 && (uintptr_t)keys % 16 == 0 && (uintptr_t)values % 16 == 0);
  const int esize = dtype == TW_DTYPE_BF16 ? 2 : 4;
  TW_REQUIRE((ldq * esize) % 16 == 0);
  if (splits > 1) {
    TW_REQUIRE(workspace != nullptr);
    TW_REQUIRE(workspace_floats >= tw_attn_mixed_workspace_floats(n_seqs, max_q_len, q_heads, value_dim, splits));
  }
  if (n_seqs == 0) return 0;
  MixedAttnArgs a{q, ldq, keys, values, block_table, table_stride, q_start, kv_len, seq0, out, ldo, talk, sink, slopes,
                  workspace, scale, out_scale, q_heads, kv_heads, key_dim, value_dim, page_size, window, splits, keep_first, -1, 16, 1};
  if (dtype == TW_DTYPE_BF16) return mixed_dispatch<bf16_t>(a, n_seqs, max_q_len, stream);
  if (dtype == TW_DTYPE_F32) return mixed_dispatch<float>(a, n_seqs, max_q_len, stream);
  return TW_ERR_BAD_ARGUMENT;
}

// ---- new keys and values into the pages (no rotation; values transposed inside a page) --------------------------
template <typename T>
__global__ void kv_store_kernel(const T* __restrict__ src, long ld, int k_col, int v_col, const int* __restrict__ slots,
                                T* __restrict__ keys, T* __restrict__ values, int G, int D, int E, int P) {
  const int n = blockIdx.x;
  const int slot = slots[n];
  if (slot < 0) return;
  const int page = slot / P, at = slot % P;
  const T* row = src + (size_t)n * ld;
  for (int i = threadIdx.x; i < G * D; i += blockDim.x) {
    const int kvh = i / D, d = i % D;
    keys[(((size_t)page * G + kvh) * P + at) * D + d] = row[k_col + i];
  }
  for (int i = threadIdx.x; i < G * E; i += blockDim.x) {
    const int kvh = i / E, d = i % E;
    values[(((size_t)page * G + kvh) * E + d) * P + at] = row[v_col + i];
  }
}

extern "C" int tw_kv_store(int dtype, const void* src, long ld, int k_col, int v_col, const int* slots, void* keys,
                           void* values, int n, int kv_heads, int key_dim, int value_dim, int page_size,
                           hipStream_t stream) {
  TW_REQUIRE(src && slots && keys && values && n >= 0 && kv_heads > 0 && key_dim > 0 && value_dim > 0 && page_size > 0);
  TW_REQUIRE(k_col >= 0 && v_col >= 0 && ld >= k_col + (long)kv_heads * key_dim && ld >= v_col + (long)kv_heads * value_dim);
  if (n == 0) return 0;
  if (dtype == TW_DTYPE_BF16)
    kv_store_kernel<bf16_t><<<n, 128, 0, stream>>>((const bf16_t*)src, ld, k_col, v_col, slots, (bf16_t*)keys, (bf16_t*)values,
                                                    kv_heads, key_dim, value_dim, page_size);
  else if (dtype == TW_DTYPE_F32)
    kv_store_kernel<float><<<n, 128, 0, stream>>>((const float*)src, ld, k_col, v_col, slots, (float*)keys, (float*)values,
                                                  kv_heads, key_dim, value_dim, page_size);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}
