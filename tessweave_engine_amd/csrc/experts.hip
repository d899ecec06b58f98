// A feed-forward of routed experts: every token runs the `top` experts with the largest router scores.
//
//   z = W_router h (float32)      s = sigmoid(z)      chosen: the `top` largest (the lowest index wins a tie)
//   out = sum over the chosen experts e of  expert_e(s_e * h)         (the score multiplies the expert's INPUT)
//   expert(y): down( glu(gate y, up y) ), glu as TW_GLU_SWISH_LIMITED with the experts' limit
//
// A step runs in six launches whose shapes depend only on the number of rows: route; plan (every expert's rows are
// laid out one expert after the other, each expert's share padded to whole tiles of 16 rows; which expert a tile
// belongs to is a table on the device, tiles nobody uses say -1); gather (the scaled, rounded input rows in that
// order); two grouped products on the matrix unit, one workgroup a (tile, range of columns), whose weights are the
// tile's expert's; combine (each token adds its experts' rows in the order it chose them). No launch waits for the
// host, so the whole runs inside a captured graph.
//
// The experts' matrices lie stacked, row-major, with K padded to a multiple of 32 by zeros:
//   gate, up [X][Fd][Cd], down [X][C][Fd]   (Fd, Cd: the inner size and the width rounded up to 32).
#include "gemm_shared.h"

#define TW_MOE_MAX_EXPERTS 1024
#define TW_MOE_TILE 16

// ---- route ---------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(const T* __restrict__ h, long ld_h, const float* __restrict__ router,
                                                        int C, int X, int top, int* __restrict__ ids,
                                                        float* __restrict__ weights) {
  __shared__ float z[TW_MOE_MAX_EXPERTS];
  const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* x = h + (size_t)row * ld_h;
  for (int e = wave; e < X; e += 4) {
    const float* w = router + (size_t)e * C;
    float sum = 0.f;
    for (int c = lane; c < C; c += 64) sum = __fmaf_rn(w[c], tw_to_float(x[c]), sum);
    sum = tw_wave_sum(sum);
    if (lane == 0) z[e] = sum;
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
      weights[(size_t)row * top + r] = 1.f / (1.f + expf(-best));
      z[at] = -INFINITY;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
}

extern "C" int tw_moe_route(int dtype, const void* h, long ld_h, const float* router, int n, int C, int X, int top, int* ids,
                            float* weights, hipStream_t stream) {
  TW_REQUIRE(h && router && ids && weights && n >= 0 && C > 0 && ld_h >= C);
  TW_REQUIRE(X > 0 && X <= TW_MOE_MAX_EXPERTS && top > 0 && top <= X);
  if (n == 0) return 0;
  if (dtype == TW_DTYPE_BF16)
    moe_route_kernel<bf16_t><<<n, 256, 0, stream>>>((const bf16_t*)h, ld_h, router, C, X, top, ids, weights);
  else if (dtype == TW_DTYPE_F32)
    moe_route_kernel<float><<<n, 256, 0, stream>>>((const float*)h, ld_h, router, C, X, top, ids, weights);
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
                                                        int capacity, int tiles) {
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
      at += (count[e] + TW_MOE_TILE - 1) / TW_MOE_TILE * TW_MOE_TILE;
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

extern "C" long tw_moe_capacity(long items, int X) {
  // rows the experts' order can take: every expert's share rounded up to whole tiles
  return (items + (long)X * (TW_MOE_TILE - 1) + TW_MOE_TILE - 1) / TW_MOE_TILE * TW_MOE_TILE;
}

extern "C" int tw_moe_plan(const int* ids, int items, int X, int* pos, int* src_item, int* tile_expert, int capacity,
                           hipStream_t stream) {
  TW_REQUIRE(ids && pos && src_item && tile_expert && items >= 0 && X > 0 && X <= TW_MOE_MAX_EXPERTS);
  TW_REQUIRE(capacity >= tw_moe_capacity(items, X) && capacity % TW_MOE_TILE == 0);
  if (items == 0) return 0;
  moe_plan_kernel<<<1, 1024, 0, stream>>>(ids, items, X, pos, src_item, tile_expert, capacity, capacity / TW_MOE_TILE);
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
  T* dst = xs + (size_t)row * Cd;
  if (item < 0) {
    for (int c = threadIdx.x; c < Cd; c += blockDim.x) dst[c] = tw_from_float<T>(0.f);
    return;
  }
  const float w = weights[item];
  const T* src = h + (size_t)(item / top) * ld_h;
  for (int c = threadIdx.x; c < Cd; c += blockDim.x) dst[c] = tw_from_float<T>(c < C ? w * tw_to_float(src[c]) : 0.f);
}

// ---- the grouped products ---------------------------------------------------------------------------------------
// One workgroup: a tile of 16 rows against 4 waves x NT x 16 columns of its expert's matrix W[ex] ([N][K], K a multiple
// of 32). GLU: W and W2 are gate and up, the result glu(gate, up) goes out in the compute type; otherwise the float32
// product. Operands go from memory straight into fragments (lane = 16 * piece + row reads 16 bytes).
template <typename T, bool GLU, int NT>
__global__ __launch_bounds__(256) void moe_grouped_kernel(const T* __restrict__ A, long lda, const T* __restrict__ W,
                                                          const T* __restrict__ W2, const int* __restrict__ tile_expert,
                                                          void* __restrict__ out, long ldo, int N, int K, float limit) {
  constexpr int EPF = Elem<T>::kPerFrag;
  const int tile = blockIdx.x;
  const int ex = tile_expert[tile];
  if (ex < 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int col0 = (blockIdx.y * 4 + wave) * 16 * NT;
  if (col0 >= N) return;
  const T* a_ptr = A + (size_t)(tile * TW_MOE_TILE + r) * lda + g * EPF;
  const T* w_ptr[NT];
  const T* w2_ptr[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int col = min(col0 + t * 16 + r, N - 1);
    w_ptr[t] = W + ((size_t)ex * N + col) * K + g * EPF;
    w2_ptr[t] = GLU ? W2 + ((size_t)ex * N + col) * K + g * EPF : nullptr;
  }
  f32x4 acc[NT], acc2[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = acc2[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
  for (int k = 0; k < K; k += 4 * EPF) {
    const typename Elem<T>::Frag a = tw_load_frag(a_ptr + k);
    typename Elem<T>::Frag b[NT], b2[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      b[t] = tw_load_frag(w_ptr[t] + k);
      if (GLU) b2[t] = tw_load_frag(w2_ptr[t] + k);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      tw_mma16(acc[t], a, b[t]);
      if (GLU) tw_mma16(acc2[t], a, b2[t]);
    }
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int col = col0 + t * 16 + r;
    if (col >= N) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const size_t at = (size_t)(tile * TW_MOE_TILE + 4 * g + j) * ldo + col;
      if (GLU) ((T*)out)[at] = tw_from_float<T>(tw_swish_limited(acc[t][j], acc2[t][j], limit));
      else ((float*)out)[at] = acc[t][j];
    }
  }
}

// ---- combine: x[token] += its experts' rows, in the order of its choices ------------------------------------------
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ x, long ld_x, const float* __restrict__ ys,
                                                          long ld_y, const int* __restrict__ pos, int C, int top) {
  const int row = blockIdx.x;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float sum = 0.f;
    for (int r = 0; r < top; ++r) sum += ys[(size_t)pos[(size_t)row * top + r] * ld_y + c];
    x[(size_t)row * ld_x + c] += sum;
  }
}

// h [n][C] (compute type) -> x [n][C] float32 += the routed experts' results. ids, weights [n * top] come from
// tw_moe_route. Scratch: pos [n * top], src_item [capacity], tile_expert [capacity / 16] (int32), xs [capacity][Cd],
// act [capacity][Fd] (compute type), ys [capacity][C] (float32), capacity = tw_moe_capacity(n * top, X).
extern "C" int tw_moe_experts(int dtype, const void* h, long ld_h, const int* ids, const float* weights, int n, int top, int X,
                              const void* gate, const void* up, const void* down, int C, int Cd, int Fd, float limit,
                              int* pos, int* src_item, int* tile_expert, void* xs, void* act, float* ys, int capacity,
                              float* x, long ld_x, hipStream_t stream) {
  TW_REQUIRE(h && ids && weights && gate && up && down && pos && src_item && tile_expert && xs && act && ys && x);
  TW_REQUIRE(n >= 0 && top > 0 && C > 0 && Cd >= C && Cd % 32 == 0 && Fd > 0 && Fd % 32 == 0 && ld_h >= C && ld_x >= C);
  TW_REQUIRE((uintptr_t)xs % 16 == 0 && (uintptr_t)act % 16 == 0 && (uintptr_t)gate % 16 == 0 && (uintptr_t)up % 16 == 0 &&
             (uintptr_t)down % 16 == 0);
  if (n == 0) return 0;
  const int code = tw_moe_plan(ids, n * top, X, pos, src_item, tile_expert, capacity, stream);
  if (code) return code;
  const int tiles = capacity / TW_MOE_TILE;
  const dim3 glu_grid(tiles, tw_div_up(Fd, 4 * 16 * 2)), down_grid(tiles, tw_div_up(C, 4 * 16 * 4));
  if (dtype == TW_DTYPE_BF16) {
    typedef bf16_t T;
    moe_gather_kernel<T><<<capacity, 256, 0, stream>>>((const T*)h, ld_h, weights, src_item, tile_expert, (T*)xs, C, Cd, top);
    moe_grouped_kernel<T, true, 2><<<glu_grid, 256, 0, stream>>>((const T*)xs, Cd, (const T*)gate, (const T*)up, tile_expert,
                                                                 act, Fd, Fd, Cd, limit);
    moe_grouped_kernel<T, false, 4><<<down_grid, 256, 0, stream>>>((const T*)act, Fd, (const T*)down, nullptr, tile_expert,
                                                                  ys, C, C, Fd, 0.f);
  } else if (dtype == TW_DTYPE_F32) {
    typedef float T;
    moe_gather_kernel<T><<<capacity, 256, 0, stream>>>((const T*)h, ld_h, weights, src_item, tile_expert, (T*)xs, C, Cd, top);
    moe_grouped_kernel<T, true, 2><<<glu_grid, 256, 0, stream>>>((const T*)xs, Cd, (const T*)gate, (const T*)up, tile_expert,
                                                                 act, Fd, Fd, Cd, limit);
    moe_grouped_kernel<T, false, 4><<<down_grid, 256, 0, stream>>>((const T*)act, Fd, (const T*)down, nullptr, tile_expert,
                                                                  ys, C, C, Fd, 0.f);
  } else {
    return TW_ERR_BAD_ARGUMENT;
  }
  moe_combine_kernel<<<n, 256, 0, stream>>>(x, ld_x, ys, C, pos, C, top);
  return TW_LAUNCH_RESULT();
}
