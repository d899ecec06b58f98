// A feed-forward of routed experts: every token runs the `top` experts with the largest router scores.
//
//   z = W_router h (float32)      s = sigmoid(z)      chosen: the `top` largest (the lowest index wins a tie)
//   out = sum over the chosen experts e of  expert_e(s_e * h)         (the score multiplies the expert's INPUT)
//   expert(y): down( glu(gate y, up y) ), glu as TW_GLU_SWISH_LIMITED with the experts' limit
//
// A second kind of expert and of weighting (`kind` 1 of tw_moe_experts, `mode` 1 of tw_moe_route):
//   z = W_router h + b        chosen: the `top` largest      p = softmax over the chosen logits alone
//   out = sum over the chosen experts e of  p_e * expert_e(h)         (the weight multiplies the expert's OUTPUT)
//   expert(y): down( gelu(up y) ), the exact gelu y Phi(y); no gate matrix
//
// A step runs in six launches whose shapes depend only on the number of rows: route; plan (every expert's rows are
// laid out one expert after the other, each expert's share padded to whole tiles of 16 rows; which expert a tile
// belongs to is a table on the device, tiles nobody uses say -1); gather (the scaled, rounded input rows in that
// order); two grouped products on the matrix unit, one workgroup a (tile, range of columns), whose weights are the
// tile's expert's; combine (each token adds its experts' rows in the order it chose them). No launch waits for the
// host, so the whole runs inside a captured graph.
//
// The experts' matrices lie stacked, K padded to a multiple of 32 by zeros and rows to a multiple of 16, in the order the
// matrix unit's fragments are read: [X][rows / 16][K / (4 EPF)][piece 0..3][row 0..15][EPF] (EPF: the elements of 16
// bytes), so that a wave's load of one fragment is 1 KB of consecutive memory (eight cache lines; row-major, its 16 rows
// are 16 lines, and the loads queue for the cache's tag lookups):
//   gate, up [X][Fd][Cd], down [X][C16][Fd]   (Fd, Cd: the inner size and the width rounded up to 32, C16: the width
//   rounded up to 16). The gathered rows and the activations between the two products lie the same way.
#include "gemm_shared.h"

#define TW_MOE_MAX_EXPERTS 1024
#define TW_MOE_TILE 16
#define TW_MOE_WIDE 4                 /* tiles a workgroup takes at once in steps of many rows */
#define TW_MOE_SPLITK_TILES 64        /* up to this many tiles a step, the waves of a workgroup split K */

// ---- route ---------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ h, long ld_h, const float* __restrict__ router,
                                                        const float* __restrict__ bias, int mode, int C, int X, int top,
                                                        int* __restrict__ ids, float* __restrict__ weights) {
  __shared__ float z[TW_MOE_MAX_EXPERTS];
  const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* x = h + (size_t)row * ld_h;
  // A wave forms two experts' logits at a time, four elements a lane and load, eight loads in flight before the first
  // is used: a logit is a chain of loads from memory, and their latency is all it costs.
  const bool vec = C % 4 == 0 && ld_h % 4 == 0 && ((uintptr_t)h % 16 == 0) && ((uintptr_t)router % 16 == 0);
  for (int e = 2 * wave; e < X; e += 8) {
    const float* w0 = router + (size_t)e * C;
    const float* w1 = router + (size_t)min(e + 1, X - 1) * C;
    float s0 = 0.f, s1 = 0.f;
    if (vec) {
#pragma unroll 4
      for (int c = 4 * lane; c < C; c += 256) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(w0 + c);
        const f32x4 b = *reinterpret_cast<const f32x4*>(w1 + c);
        float xv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) xv[j] = tw_to_float(x[c + j]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          s0 = __fmaf_rn(a[j], xv[j], s0);
          s1 = __fmaf_rn(b[j], xv[j], s1);
        }
      }
    } else {
      for (int c = lane; c < C; c += 64) {
        const float xv = tw_to_float(x[c]);
        s0 = __fmaf_rn(w0[c], xv, s0);
        s1 = __fmaf_rn(w1[c], xv, s1);
      }
    }
    s0 = tw_wave_sum(s0);
    s1 = tw_wave_sum(s1);
    if (lane == 0) {
      z[e] = s0 + (bias ? bias[e] : 0.f);
      if (e + 1 < X) z[e + 1] = s1 + (bias ? bias[e + 1] : 0.f);
    }
  }
  __syncthreads();
  if (wave != 0) return;
  for (int r = 0; r < top; ++r) {
    float best = -INFINITY;
    int at = 0x7fffffff;
    for (int e = lane; e < X; e += 64) {
      const float v = z[e];
      if (v > best || (v == best && e < at)) { best = v; at = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, TW_WAVE);
      const int oa = __shfl_xor(at, o, TW_WAVE);
      if (ov > best || (ov == best && oa < at)) { best = ov; at = oa; }
    }
    if (lane == 0) {
      ids[(size_t)row * top + r] = at;
      weights[(size_t)row * top + r] = mode == 1 ? best : 1.f / (1.f + expf(-best));
      z[at] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  if (mode == 1 && lane == 0) {
    // the softmax over the chosen logits alone (the first chosen is the largest), in the order they were chosen
    float* w = weights + (size_t)row * top;
    const float first = w[0];
    float sum = 0.f;
    for (int r = 0; r < top; ++r) {
      w[r] = expf(w[r] - first);
      sum += w[r];
    }
    for (int r = 0; r < top; ++r) w[r] = w[r] / sum;
  }
}

extern "C" int tw_moe_route(int dtype, const void* h, long ld_h, const float* router, const float* bias, int mode, int n, int C,
                            int X, int top, int* ids, float* weights, hipStream_t stream) {
  TW_REQUIRE(h && router && ids && weights && n >= 0 && C > 0 && ld_h >= C && (mode == 0 || mode == 1));
  TW_REQUIRE(X > 0 && X <= TW_MOE_MAX_EXPERTS && top > 0 && top <= X);
  if (n == 0) return 0;
  if (dtype == TW_DTYPE_BF16)
    moe_route_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)h, ld_h, router, bias, mode, C, X, top, ids, weights);
  else if (dtype == TW_DTYPE_F32)
    moe_route_kernel<float><<<n, 256, 0, stream>>>((const float*)h, ld_h, router, bias, mode, C, X, top, ids, weights);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- plan ----------------------------------------------------------------------------------------------------
// items = n * top pairs (token, choice). pos[item]: the pair's row in the experts' order; src_item[row]: the pair of a
// row, -1 for padding; tile_expert[tile]: the expert of rows 16 tile .., -1 for a tile behind the last one in use.
// Which of an expert's rows a pair gets depends on the order the atomics arrive in; no result depends on it, since
// every row is computed for itself and a token adds its rows in the order of its choices.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int* __restrict__ ids, int items, int X, int* __restrict__ pos,
                                                        int* __restrict__ src_item, int* __restrict__ tile_expert,
                                                        int capacity, int tiles, int unit) {
  __shared__ int count[TW_MOE_MAX_EXPERTS];
  __shared__ int offset[TW_MOE_MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < X; e += blockDim.x) count[e] = 0;
  for (int r = threadIdx.x; r < capacity; r += blockDim.x) src_item[r] = -1;
  for (int t = threadIdx.x; t < tiles; t += blockDim.x) tile_expert[t] = -1;
  __syncthreads();
  for (int i = threadIdx.x; i < items; i += blockDim.x) pos[i] = atomicAdd(&count[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < X; ++e) {
      offset[e] = at;
      at += (count[e] + unit - 1) / unit * unit;
    }
    offset[X] = at;
  }
  __syncthreads();
  for (int e = threadIdx.x; e < X; e += blockDim.x)
    for (int t = offset[e] / TW_MOE_TILE; t < offset[e + 1] / TW_MOE_TILE; ++t) tile_expert[t] = e;
  for (int i = threadIdx.x; i < items; i += blockDim.x) {
    const int row = offset[ids[i]] + pos[i];
    pos[i] = row;
    src_item[row] = i;
  }
}

// The rows an expert's share is padded to: one tile, or, once the experts have a tile's rows each on average, the
// TW_MOE_WIDE tiles that one workgroup of the grouped products then takes against one read of the expert's matrices.
static int moe_unit(long items, int X) { return items >= (long)TW_MOE_TILE * X ? TW_MOE_TILE * TW_MOE_WIDE : TW_MOE_TILE; }

extern "C" long tw_moe_capacity(long items, int X) {
  // rows the experts' order can take: every expert's share rounded up to whole units (never fewer for more items)
  const long unit = moe_unit(items, X);
  return (items + (long)X * (unit - 1) + unit - 1) / unit * unit;
}

extern "C" int tw_moe_plan(const int* ids, int items, int X, int* pos, int* src_item, int* tile_expert, int capacity,
                           hipStream_t stream) {
  TW_REQUIRE(ids && pos && src_item && tile_expert && items >= 0 && X > 0 && X <= TW_MOE_MAX_EXPERTS);
  TW_REQUIRE(capacity >= tw_moe_capacity(items, X) && capacity % TW_MOE_TILE == 0);
  if (items == 0) return 0;
  moe_plan_kernel<<<1, 1024, 0, stream>>>(ids, items, X, pos, src_item, tile_expert, capacity, capacity / TW_MOE_TILE,
                                          moe_unit(items, X));
  return TW_LAUNCH_RESULT();
}

// ---- gather: xs[row] = round(weight * h[token]) in the experts' order, zeros in padding rows and behind C ----------
template <typename T>
__global__ __launch_bounds__(256) void moe_gather_kernel(const T* __restrict__ h, long ld_h, const float* __restrict__ weights,
                                                         const int* __restrict__ src_item, const int* __restrict__ tile_expert,
                                                         T* __restrict__ xs, int C, int Cd, int top) {
  const int row = blockIdx.x;
  if (tile_expert[row / TW_MOE_TILE] < 0) return;
  const int item = src_item[row];
  constexpr int EPF = Elem<T>::kPerFrag;
  // element c of the row: tile row / 16, step c / (4 EPF), piece c / EPF % 4, row row % 16 of the piece
  T* dst = xs + (size_t)(row / TW_MOE_TILE) * Cd * TW_MOE_TILE + (row % TW_MOE_TILE) * EPF;
  auto at = [](int c) { return (size_t)(c / EPF) * TW_MOE_TILE * EPF + c % EPF; };
  if (item < 0) {
    for (int c = threadIdx.x; c < Cd; c += blockDim.x) dst[at(c)] = tw_from_float<T>(0.f);
    return;
  }
  const float w = weights ? weights[item] : 1.f;          // (no weights: they multiply the experts' outputs instead)
  const T* src = h + (size_t)(item / top) * ld_h;
  for (int c = threadIdx.x; c < Cd; c += blockDim.x) dst[at(c)] = tw_from_float<T>(c < C ? w * tw_to_float(src[c]) : 0.f);
}

// ---- the grouped products ---------------------------------------------------------------------------------------
// One workgroup: a tile of 16 rows against 4 waves x NT x 16 columns of its expert's matrix W[ex] ([N][K], K a multiple
// of 32). GLU: W and W2 are gate and up, the result glu(gate, up) goes out in the compute type; otherwise the float32
// product. Operands go from memory straight into fragments (lane = 16 * piece + row reads 16 bytes).
// SPLITK (steps of few rows, where the tiles in use are too few to fill the chip and every one streams its expert's whole
// matrix): the four waves share one range of NT x 16 columns and take every fourth step over K each; their sums meet in
// LDS and are added in the order of the waves.
// MT > 1 (steps of many rows, whose experts' shares are padded to MT tiles): a workgroup takes MT tiles of one expert
// against every fragment of the expert's matrices it reads.
template <int N> struct MoeCount { static constexpr int value = N; };
// ACT 0: the float32 product; 1: gate and up with the limited swish; 2: one matrix with the exact gelu (1 and 2 write the
// next product's rows in the compute type).
template <typename T, int ACT, int NT, bool SPLITK = false, int MT = 1>
__global__ __launch_bounds__(256) void moe_grouped_kernel(const T* __restrict__ A, long lda, const T* __restrict__ W,
                                                          const T* __restrict__ W2, const int* __restrict__ tile_expert,
                                                          void* __restrict__ out, long ldo, int N, int K, float limit) {
  constexpr int EPF = Elem<T>::kPerFrag;
  constexpr bool GLU = ACT == 1;
  const int tile = blockIdx.x * MT;
  const int ex = tile_expert[tile];
  if (ex < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int col0 = (SPLITK ? blockIdx.y : blockIdx.y * 4 + wave) * 16 * NT;
  if (col0 >= N) return;
  constexpr int KSTEP = 4 * EPF;
  constexpr int BLK = 64 * EPF;                      // elements of one step's fragment of a tile: lane l's at l * EPF
  constexpr int k_stride = (SPLITK ? 4 : 1) * BLK;    // (k counts the elements of a tile's fragments, step after step)
  const int k_first = SPLITK ? wave * BLK : 0;
  const size_t tile_elems = (size_t)K * TW_MOE_TILE;  // all steps of one tile of 16 rows
  const int n_blocks = (N + 15) / 16;
  const T* a_ptr = A + (size_t)tile * tile_elems + lane * EPF;
  const T* w_ptr[NT];
  const T* w2_ptr[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const size_t at = ((size_t)ex * n_blocks + min(col0 / 16 + t, n_blocks - 1)) * tile_elems + lane * EPF;
    w_ptr[t] = W + at;
    w2_ptr[t] = GLU ? W2 + at : nullptr;
  }
  f32x4 acc[MT][NT], acc2[MT][NT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[m][t] = acc2[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  // U steps' operands are on their way before the first is used: what bounds this loop is the latency of memory
  auto steps = [&](int k, auto count) {
    constexpr int U = decltype(count)::value;
    typename Elem<T>::Frag a[U][MT], b[U][NT], b2[U][NT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int m = 0; m < MT; ++m) a[u][m] = tw_load_frag(a_ptr + (size_t)m * tile_elems + k + u * k_stride);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        b[u][t] = tw_load_frag(w_ptr[t] + k + u * k_stride);
        if (GLU) b2[u][t] = tw_load_frag(w2_ptr[t] + k + u * k_stride);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          tw_mma16(acc[m][t], a[u][m], b[u][t]);
          if (GLU) tw_mma16(acc2[m][t], a[u][m], b2[u][t]);
        }
  };
  constexpr int U = MT > 1 ? 2 : GLU ? 4 : (NT > 2 ? 4 : 8);
  int k = k_first;
  const int k_end = (int)tile_elems;
  for (; k + (U - 1) * k_stride < k_end; k += U * k_stride) steps(k, MoeCount<U>());
  for (; k < k_end; k += k_stride) steps(k, MoeCount<1>());
  static_assert(!SPLITK || MT == 1);
  if constexpr (SPLITK) {
    __shared__ f32x4 part[GLU ? 2 : 1][3][NT][64];
    if (wave > 0) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        part[0][wave - 1][t][lane] = acc[0][t];
        if (GLU) part[GLU ? 1 : 0][wave - 1][t][lane] = acc2[0][t];
      }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        acc[0][t] += part[0][w][t][lane];
        if (GLU) acc2[0][t] += part[GLU ? 1 : 0][w][t][lane];
      }
  }
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int col = col0 + t * 16 + r;
      if (col >= N) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (ACT != 0) {
          // the activations are the next product's rows: in fragment order too (ldo: the elements of a row)
          const size_t at = (size_t)(tile + m) * ldo * TW_MOE_TILE + ((size_t)(col / EPF) * TW_MOE_TILE + 4 * g + j) * EPF + col % EPF;
          const float z = acc[m][t][j];
          ((T*)out)[at] = tw_from_float<T>(GLU ? tw_swish_limited(z, acc2[m][t][j], limit)
                                               : 0.5f * z * (1.f + erff(z * 0.70710678118654752f)));
        } else {
          ((float*)out)[(size_t)((tile + m) * TW_MOE_TILE + 4 * g + j) * ldo + col] = acc[m][t][j];
        }
      }
    }
}

// ---- combine: x[token] += its experts' rows, in the order of its choices ------------------------------------------
// A workgroup takes 1,024 columns of a row, four a thread where rows and addresses allow 16-byte accesses.
// weights (or null): a factor on each of the token's rows; accumulate 0: x is written, not added to. more (or null):
// float32 [splits][n][C] partial sums of something else that belongs to the same result (a shared expert's last product
// with its K ranges not yet added up): added here, in index order, before the experts' rows.
template <bool VEC>
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ x, long ld_x, const float* __restrict__ ys,
                                                          long ld_y, const int* __restrict__ pos, int C, int top,
                                                          const float* __restrict__ weights, int accumulate,
                                                          const float* __restrict__ more, int splits, size_t more_stride) {
  const int row = blockIdx.x;
  const int c = blockIdx.y * 1024 + threadIdx.x * 4;
  if (c >= C) return;
  if constexpr (VEC) {
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    if (more)
      for (int s = 0; s < splits; ++s) sum += *reinterpret_cast<const f32x4*>(more + s * more_stride + (size_t)row * C + c);
    for (int r = 0; r < top; ++r) {
      const f32x4 y = *reinterpret_cast<const f32x4*>(ys + (size_t)pos[(size_t)row * top + r] * ld_y + c);
      if (weights) sum += weights[(size_t)row * top + r] * y;
      else sum += y;
    }
    f32x4* dst = reinterpret_cast<f32x4*>(x + (size_t)row * ld_x + c);
    if (accumulate) *dst += sum;
    else *dst = sum;
  } else {
    for (int j = 0; j < 4 && c + j < C; ++j) {
      float sum = 0.f;
      if (more)
        for (int s = 0; s < splits; ++s) sum += more[s * more_stride + (size_t)row * C + c + j];
      for (int r = 0; r < top; ++r)
        sum += (weights ? weights[(size_t)row * top + r] : 1.f) * ys[(size_t)pos[(size_t)row * top + r] * ld_y + c + j];
      if (accumulate) x[(size_t)row * ld_x + c + j] += sum;
      else x[(size_t)row * ld_x + c + j] = sum;
    }
  }
}

// h [n][C] (compute type) -> x [n][C] float32 += the routed experts' results. ids, weights [n * top] come from
// tw_moe_route. Scratch: pos [n * top], src_item [capacity], tile_expert [capacity / 16] (int32), xs [capacity][Cd],
// act [capacity][Fd] (compute type), ys [capacity][C] (float32), capacity = tw_moe_capacity(n * top, X).
extern "C" int tw_moe_experts(int dtype, const void* h, long ld_h, const int* ids, const float* weights, int n, int top, int X,
                              const void* gate, const void* up, const void* down, int C, int Cd, int Fd, float limit,
                              int* pos, int* src_item, int* tile_expert, void* xs, void* act, float* ys, int capacity,
                              float* x, long ld_x, int kind, int accumulate, const float* more, int more_splits,
                              hipStream_t stream) {
  TW_REQUIRE(h && ids && weights && up && down && pos && src_item && tile_expert && xs && act && ys && x);
  TW_REQUIRE((kind == 0 && gate) || kind == 1);
  TW_REQUIRE(more == nullptr || more_splits > 0);
  if (kind == 1) gate = up;            // (never read: the alignment test below wants a pointer)
  TW_REQUIRE(n >= 0 && top > 0 && C > 0 && Cd >= C && Cd % 32 == 0 && Fd > 0 && Fd % 32 == 0 && ld_h >= C && ld_x >= C);
  TW_REQUIRE((uintptr_t)xs % 16 == 0 && (uintptr_t)act % 16 == 0 && (uintptr_t)gate % 16 == 0 && (uintptr_t)up % 16 == 0 &&
             (uintptr_t)down % 16 == 0);
  if (n == 0) return 0;
  const int code = tw_moe_plan(ids, n * top, X, pos, src_item, tile_expert, capacity, stream);
  if (code) return code;
  const int tiles = capacity / TW_MOE_TILE;
  const dim3 glu_grid(tiles, tw_div_up(Fd, 4 * 16 * 2)), down_grid(tiles, tw_div_up(C, 4 * 16 * 4));
  // few rows: most tiles hold one or two rows and each streams its expert's matrices once; the waves then split K
  const bool few = tiles <= TW_MOE_SPLITK_TILES;
  const dim3 glu_few(tiles, tw_div_up(Fd, 16 * 2)), down_few(tiles, tw_div_up(C, 16 * 2));
  const bool wide = moe_unit((long)n * top, X) == TW_MOE_TILE * TW_MOE_WIDE;
  TW_REQUIRE(!wide || capacity % (TW_MOE_TILE * TW_MOE_WIDE) == 0);
  const dim3 glu_wide(tiles / TW_MOE_WIDE, tw_div_up(Fd, 4 * 16 * 2)), down_wide(tiles / TW_MOE_WIDE, tw_div_up(C, 4 * 16 * 2));
  if (dtype == TW_DTYPE_BF16) {
    typedef bf16_t T;
    moe_gather_kernel<T><<<capacity, 256, 0, stream>>>((const T*)h, ld_h, kind == 0 ? weights : nullptr, src_item, tile_expert,
                                                       (T*)xs, C, Cd, top);
    if (few) {
      if (kind == 0)
        moe_grouped_kernel<T, 1, 2, true><<<glu_few, 256, 0, stream>>>((const T*)xs, Cd, (const T*)gate, (const T*)up,
                                                                       tile_expert, act, Fd, Fd, Cd, limit);
      else
        moe_grouped_kernel<T, 2, 2, true><<<glu_few, 256, 0, stream>>>((const T*)xs, Cd, (const T*)up, nullptr,
                                                                       tile_expert, act, Fd, Fd, Cd, 0.f);
      moe_grouped_kernel<T, 0, 2, true><<<down_few, 256, 0, stream>>>((const T*)act, Fd, (const T*)down, nullptr,
                                                                         tile_expert, ys, C, C, Fd, 0.f);
    } else if (wide) {
      if (kind == 0)
        moe_grouped_kernel<T, 1, 2, false, TW_MOE_WIDE><<<glu_wide, 256, 0, stream>>>(
            (const T*)xs, Cd, (const T*)gate, (const T*)up, tile_expert, act, Fd, Fd, Cd, limit);
      else
        moe_grouped_kernel<T, 2, 2, false, TW_MOE_WIDE><<<glu_wide, 256, 0, stream>>>(
            (const T*)xs, Cd, (const T*)up, nullptr, tile_expert, act, Fd, Fd, Cd, 0.f);
      moe_grouped_kernel<T, 0, 2, false, TW_MOE_WIDE><<<down_wide, 256, 0, stream>>>(
          (const T*)act, Fd, (const T*)down, nullptr, tile_expert, ys, C, C, Fd, 0.f);
    } else {
      if (kind == 0)
        moe_grouped_kernel<T, 1, 2><<<glu_grid, 256, 0, stream>>>((const T*)xs, Cd, (const T*)gate, (const T*)up,
                                                                  tile_expert, act, Fd, Fd, Cd, limit);
      else
        moe_grouped_kernel<T, 2, 2><<<glu_grid, 256, 0, stream>>>((const T*)xs, Cd, (const T*)up, nullptr,
                                                                  tile_expert, act, Fd, Fd, Cd, 0.f);
      moe_grouped_kernel<T, 0, 4><<<down_grid, 256, 0, stream>>>((const T*)act, Fd, (const T*)down, nullptr,
                                                                    tile_expert, ys, C, C, Fd, 0.f);
    }
  } else if (dtype == TW_DTYPE_F32) {
    typedef float T;
    moe_gather_kernel<T><<<capacity, 256, 0, stream>>>((const T*)h, ld_h, kind == 0 ? weights : nullptr, src_item, tile_expert,
                                                       (T*)xs, C, Cd, top);
    if (few) {
      if (kind == 0)
        moe_grouped_kernel<T, 1, 2, true><<<glu_few, 256, 0, stream>>>((const T*)xs, Cd, (const T*)gate, (const T*)up,
                                                                       tile_expert, act, Fd, Fd, Cd, limit);
      else
        moe_grouped_kernel<T, 2, 2, true><<<glu_few, 256, 0, stream>>>((const T*)xs, Cd, (const T*)up, nullptr,
                                                                       tile_expert, act, Fd, Fd, Cd, 0.f);
      moe_grouped_kernel<T, 0, 2, true><<<down_few, 256, 0, stream>>>((const T*)act, Fd, (const T*)down, nullptr,
                                                                         tile_expert, ys, C, C, Fd, 0.f);
    } else if (wide) {
      if (kind == 0)
        moe_grouped_kernel<T, 1, 2, false, TW_MOE_WIDE><<<glu_wide, 256, 0, stream>>>(
            (const T*)xs, Cd, (const T*)gate, (const T*)up, tile_expert, act, Fd, Fd, Cd, limit);
      else
        moe_grouped_kernel<T, 2, 2, false, TW_MOE_WIDE><<<glu_wide, 256, 0, stream>>>(
            (const T*)xs, Cd, (const T*)up, nullptr, tile_expert, act, Fd, Fd, Cd, 0.f);
      moe_grouped_kernel<T, 0, 2, false, TW_MOE_WIDE><<<down_wide, 256, 0, stream>>>(
          (const T*)act, Fd, (const T*)down, nullptr, tile_expert, ys, C, C, Fd, 0.f);
    } else {
      if (kind == 0)
        moe_grouped_kernel<T, 1, 2><<<glu_grid, 256, 0, stream>>>((const T*)xs, Cd, (const T*)gate, (const T*)up,
                                                                  tile_expert, act, Fd, Fd, Cd, limit);
      else
        moe_grouped_kernel<T, 2, 2><<<glu_grid, 256, 0, stream>>>((const T*)xs, Cd, (const T*)up, nullptr,
                                                                  tile_expert, act, Fd, Fd, Cd, 0.f);
      moe_grouped_kernel<T, 0, 4><<<down_grid, 256, 0, stream>>>((const T*)act, Fd, (const T*)down, nullptr,
                                                                    tile_expert, ys, C, C, Fd, 0.f);
    }
  } else {
    return TW_ERR_BAD_ARGUMENT;
  }
  const dim3 combine_grid(n, tw_div_up(C, 1024));
  const size_t more_stride = (size_t)n * C;
  if (C % 4 == 0 && ld_x % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)ys % 16 == 0 && (uintptr_t)more % 16 == 0)
    moe_combine_kernel<true><<<combine_grid, 256, 0, stream>>>(x, ld_x, ys, C, pos, C, top, kind == 1 ? weights : nullptr, accumulate,
                                                               more, more_splits, more_stride);
  else
    moe_combine_kernel<false><<<combine_grid, 256, 0, stream>>>(x, ld_x, ys, C, pos, C, top, kind == 1 ? weights : nullptr, accumulate,
                                                                more, more_splits, more_stride);
  return TW_LAUNCH_RESULT();
}
