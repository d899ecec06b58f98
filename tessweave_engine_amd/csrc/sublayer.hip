// Kernels of a layer arrangement that norms AFTER each sum:
//
//   x <- w * unit(alpha * x + scale * y),  unit(v) = v / sqrt(mean(v^2) + eps)
//
// x is the float32 residual stream, y a sublayer's float32 result (or split-K partial sums that are added up
// here, in index order), scale an optional per-channel factor, w the norm's weight. The normed row is written
// back to x and, rounded once, to `out` in the compute type, which is what the next sublayer's products read.
// Also here: the square of relu, in place, for a feed-forward without a gate.
#include "tw_common.h"

struct ResidualNormArgs {
  float* x;                 // [n][hidden]
  const float* y; long ldy; // [n][ldy] or null
  const float* add; int splits; size_t add_stride;   // [splits][n][hidden] or null
  const float* scale;       // [hidden] or null
  const float* w;           // [hidden]
  void* out;                // [n][hidden], compute type, or null
  int hidden;
  float alpha, eps;
};

// PER groups of four consecutive elements a thread, the row in registers between the two passes.
template <typename T, int PER>
__global__ __launch_bounds__(1024) void residual_norm_vec4_kernel(ResidualNormArgs a) {
  __shared__ float lds[16];
  const int row = blockIdx.x;
  const int chunks = a.hidden / 4;
  float* x = a.x + (size_t)row * a.hidden;
  f32x4 v[PER];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    v[i] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (c < chunks) {
      f32x4 yv = {0.f, 0.f, 0.f, 0.f};
      if (a.add) {
        for (int s = 0; s < a.splits; ++s)
          yv += *reinterpret_cast<const f32x4*>(a.add + s * a.add_stride + (size_t)row * a.hidden + 4 * c);
      } else if (a.y) {
        yv = *reinterpret_cast<const f32x4*>(a.y + (size_t)row * a.ldy + 4 * c);
      }
      if (a.scale) yv *= *reinterpret_cast<const f32x4*>(a.scale + 4 * c);
      const f32x4 xv = *reinterpret_cast<const f32x4*>(x + 4 * c);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[i][e] = __fmaf_rn(a.alpha, xv[e], yv[e]);
        ss = __fmaf_rn(v[i][e], v[i][e], ss);
      }
    }
  }
  const float total = tw_block_sum(ss, lds);
  const float rinv = 1.f / sqrtf(total / (float)a.hidden + a.eps);
  T* out = a.out ? (T*)a.out + (size_t)row * a.hidden : nullptr;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = threadIdx.x + i * blockDim.x;
    if (c < chunks) {
      const f32x4 wv = *reinterpret_cast<const f32x4*>(a.w + 4 * c);
      f32x4 r;
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = v[i][e] * rinv * wv[e];
      *reinterpret_cast<f32x4*>(x + 4 * c) = r;
      if (out) {
#pragma unroll
        for (int e = 0; e < 4; ++e) out[4 * c + e] = tw_from_float<T>(r[e]);
      }
    }
  }
}

// Any row length: the sums are parked in x between the two passes (a thread reads back only what it wrote).
template <typename T>
__global__ void residual_norm_kernel(ResidualNormArgs a) {
  __shared__ float lds[16];
  const int row = blockIdx.x;
  float* x = a.x + (size_t)row * a.hidden;
  float ss = 0.f;
  for (int c = threadIdx.x; c < a.hidden; c += blockDim.x) {
    float yv = 0.f;
    if (a.add) {
      for (int s = 0; s < a.splits; ++s) yv += a.add[s * a.add_stride + (size_t)row * a.hidden + c];
    } else if (a.y) {
      yv = a.y[(size_t)row * a.ldy + c];
    }
    if (a.scale) yv *= a.scale[c];
    const float v = __fmaf_rn(a.alpha, x[c], yv);
    x[c] = v;
    ss = __fmaf_rn(v, v, ss);
  }
  const float total = tw_block_sum(ss, lds);
  const float rinv = 1.f / sqrtf(total / (float)a.hidden + a.eps);
  T* out = a.out ? (T*)a.out + (size_t)row * a.hidden : nullptr;
  for (int c = threadIdx.x; c < a.hidden; c += blockDim.x) {
    const float r = x[c] * rinv * a.w[c];
    x[c] = r;
    if (out) out[c] = tw_from_float<T>(r);
  }
}

template <typename T>
static void residual_norm_launch(const ResidualNormArgs& a, int n, hipStream_t stream) {
  const bool aligned = a.hidden % 4 == 0 && (uintptr_t)a.x % 16 == 0 && (uintptr_t)a.w % 16 == 0 &&
                       (!a.y || ((uintptr_t)a.y % 16 == 0 && a.ldy % 4 == 0)) &&
                       (!a.add || ((uintptr_t)a.add % 16 == 0 && a.add_stride % 4 == 0)) &&
                       (!a.scale || (uintptr_t)a.scale % 16 == 0);
  const int chunks = a.hidden / 4;
  if (aligned && chunks <= 4096) {
    const int per = chunks <= 1024 ? 1 : (chunks <= 2048 ? 2 : 4);
    int threads = (chunks + per - 1) / per;
    threads = (threads + 63) / 64 * 64;
    if (per == 1) residual_norm_vec4_kernel<T, 1><<<n, threads, 0, stream>>>(a);
    else if (per == 2) residual_norm_vec4_kernel<T, 2><<<n, threads, 0, stream>>>(a);
    else residual_norm_vec4_kernel<T, 4><<<n, threads, 0, stream>>>(a);
  } else {
    residual_norm_kernel<T><<<n, 256, 0, stream>>>(a);
  }
}

extern "C" int tw_residual_norm(int out_dtype, float* x, const float* y, long ldy, const float* add, int splits,
                                long add_stride, const float* scale, const float* w, void* out, int n, int hidden,
                                float alpha, float eps, hipStream_t stream) {
  TW_REQUIRE(x && w && n >= 0 && hidden > 0 && eps > 0.f);
  TW_REQUIRE(add == nullptr || (splits > 0 && add_stride >= (long)n * hidden));
  TW_REQUIRE(y == nullptr || ldy >= hidden);
  if (n == 0) return 0;
  ResidualNormArgs a{x, add ? nullptr : y, ldy, add, splits, (size_t)add_stride, scale, w, out, hidden, alpha, eps};
  if (out_dtype == TW_DTYPE_BF16) residual_norm_launch<bf16_t>(a, n, stream);
  else if (out_dtype == TW_DTYPE_F32) residual_norm_launch<float>(a, n, stream);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- x <- max(x, 0)^2 in place ---------------------------------------------------------------------------
template <typename T>
__global__ void relu_squared_kernel(T* __restrict__ x, long ld, int cols, long total) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long row = i / cols;
  const int col = (int)(i % cols);
  T* p = x + row * ld + col;
  const float v = fmaxf(tw_to_float(*p), 0.f);
  *p = tw_from_float<T>(v * v);
}

// The same from split-K partial sums of the product before (float32 [splits][n][cols], added in index order): one
// rounding, and no kernel of its own for the sums.
template <typename T>
__global__ void relu_squared_sums_kernel(const float* __restrict__ partial, int splits, T* __restrict__ x, long ld, int cols,
                                         long total) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  float v = 0.f;
  for (int s = 0; s < splits; ++s) v += partial[(size_t)s * total + i];
  v = fmaxf(v, 0.f);
  x[(i / cols) * ld + i % cols] = tw_from_float<T>(v * v);
}

extern "C" int tw_relu_squared(int dtype, void* x, long ld, int n, int cols, const float* partial, int splits,
                               hipStream_t stream) {
  TW_REQUIRE(x && n >= 0 && cols > 0 && ld >= cols && (partial == nullptr || splits > 0));
  if (n == 0) return 0;
  const long total = (long)n * cols;
  const int blocks = tw_div_up(total, 256);
  if (partial) {
    if (dtype == TW_DTYPE_BF16) relu_squared_sums_kernel<bf16_t><<<blocks, 256, 0, stream>>>(partial, splits, (bf16_t*)x, ld, cols, total);
    else if (dtype == TW_DTYPE_F32) relu_squared_sums_kernel<float><<<blocks, 256, 0, stream>>>(partial, splits, (float*)x, ld, cols, total);
    else return TW_ERR_BAD_ARGUMENT;
    return TW_LAUNCH_RESULT();
  }
  if (dtype == TW_DTYPE_BF16) relu_squared_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, ld, cols, total);
  else if (dtype == TW_DTYPE_F32) relu_squared_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, ld, cols, total);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- a norm on the sublayer's RESULT: x <- x + mult * w * unit(y) -------------------------------------------------
// y is a sublayer's float32 result (or split-K partial sums that are added up here, in index order); its statistic is
// float32; the sum goes back into the float32 stream x and, rounded once, to `out` in the compute type, which is what
// the next sublayer's products read (such an arrangement's sublayers read the stream itself). A block a row, four
// elements a thread and pass where rows and addresses allow; the row of y stays in registers between the two passes
// up to 4,096 elements, longer rows are read again.
struct AddNormedArgs {
  float* x;
  const float* y; long ldy;
  const float* add; int splits; size_t add_stride;
  const float* w;
  void* out;
  int hidden;
  float mult, eps;
};

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void add_normed_kernel(AddNormedArgs a) {
  __shared__ float lds[16];
  constexpr int W = VEC ? 4 : 1;
  constexpr int KEEP = 4;
  const int row = blockIdx.x;
  const int units = a.hidden / W;
  float* x = a.x + (size_t)row * a.hidden;
  auto load = [&](int u, float* v) {
#pragma unroll
    for (int e = 0; e < W; ++e) v[e] = 0.f;
    if (a.add) {
      for (int s = 0; s < a.splits; ++s) {
        const float* p = a.add + s * a.add_stride + (size_t)row * a.hidden + (size_t)u * W;
        if (VEC) {
          const f32x4 t = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
          for (int e = 0; e < W; ++e) v[e] += t[e];
        } else {
          v[0] += p[0];
        }
      }
    } else {
      const float* p = a.y + (size_t)row * a.ldy + (size_t)u * W;
      if (VEC) {
        const f32x4 t = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
        for (int e = 0; e < W; ++e) v[e] = t[e];
      } else {
        v[0] = p[0];
      }
    }
  };
  float kept[KEEP][W];
  float ss = 0.f;
  int i = 0;
  for (int u = threadIdx.x; u < units; u += blockDim.x, ++i) {
    float v[W];
    load(u, v);
#pragma unroll
    for (int e = 0; e < W; ++e) ss = __fmaf_rn(v[e], v[e], ss);
    if (i < KEEP) {
#pragma unroll
      for (int e = 0; e < W; ++e) kept[i][e] = v[e];
    }
  }
  const float total = tw_block_sum(ss, lds);
  const float f = a.mult / sqrtf(total / (float)a.hidden + a.eps);
  T* out = a.out ? (T*)a.out + (size_t)row * a.hidden : nullptr;
  i = 0;
  for (int u = threadIdx.x; u < units; u += blockDim.x, ++i) {
    float v[W];
    if (i < KEEP) {
#pragma unroll
      for (int e = 0; e < W; ++e) v[e] = kept[i][e];
    } else {
      load(u, v);
    }
#pragma unroll
    for (int e = 0; e < W; ++e) {
      const int c = u * W + e;
      const float r = __fmaf_rn(v[e] * f, a.w[c], x[c]);
      x[c] = r;
      if (out) out[c] = tw_from_float<T>(r);
    }
  }
}

extern "C" int tw_add_normed(int out_dtype, float* x, const float* y, long ldy, const float* add, int splits, long add_stride,
                             const float* w, void* out, int n, int hidden, float mult, float eps, hipStream_t stream) {
  TW_REQUIRE(x && w && (y || add) && n >= 0 && hidden > 0 && eps > 0.f);
  TW_REQUIRE(add == nullptr || (splits > 0 && add_stride >= (long)n * hidden));
  TW_REQUIRE(add != nullptr || ldy >= hidden);
  if (n == 0) return 0;
  AddNormedArgs a{x, add ? nullptr : y, ldy, add, splits, (size_t)add_stride, w, out, hidden, mult, eps};
  const bool vec = hidden % 4 == 0 && (add ? ((uintptr_t)add % 16 == 0 && add_stride % 4 == 0)
                                           : ((uintptr_t)y % 16 == 0 && ldy % 4 == 0));
  if (out_dtype == TW_DTYPE_BF16) {
    if (vec) add_normed_kernel<bf16_t, true><<<n, 256, 0, stream>>>(a);
    else add_normed_kernel<bf16_t, false><<<n, 256, 0, stream>>>(a);
  } else if (out_dtype == TW_DTYPE_F32) {
    if (vec) add_normed_kernel<float, true><<<n, 256, 0, stream>>>(a);
    else add_normed_kernel<float, false><<<n, 256, 0, stream>>>(a);
  } else {
    return TW_ERR_BAD_ARGUMENT;
  }
  return TW_LAUNCH_RESULT();
}

// ---- activations of a plain product, in place: kind 1 max(x, 0)^2 (above), 2 the exact gelu, x Phi(x) -------------
__device__ __forceinline__ float sl_act(float v, int kind) {
  if (kind == 2) return 0.5f * v * (1.f + erff(v * 0.70710678118654752f));
  v = fmaxf(v, 0.f);
  return v * v;
}

template <typename T>
__global__ void activation_kernel(T* __restrict__ x, long ld, int cols, long total, const float* __restrict__ partial, int splits,
                                  int kind) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  T* p = x + (i / cols) * ld + i % cols;
  float v = 0.f;
  if (partial) {
    for (int s = 0; s < splits; ++s) v += partial[(size_t)s * total + i];
  } else {
    v = tw_to_float(*p);
  }
  *p = tw_from_float<T>(sl_act(v, kind));
}

extern "C" int tw_activation(int dtype, void* x, long ld, int n, int cols, const float* partial, int splits, int kind,
                             hipStream_t stream) {
  TW_REQUIRE(x && n >= 0 && cols > 0 && ld >= cols && (partial == nullptr || splits > 0) && (kind == 1 || kind == 2));
  if (n == 0) return 0;
  const long total = (long)n * cols;
  const int blocks = tw_div_up(total, 256);
  if (dtype == TW_DTYPE_BF16) activation_kernel<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)x, ld, cols, total, partial, splits, kind);
  else if (dtype == TW_DTYPE_F32) activation_kernel<float><<<blocks, 256, 0, stream>>>((float*)x, ld, cols, total, partial, splits, kind);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- out <- out * sigmoid(gate), element by element (an output gate in front of the output product) ---------------
template <typename T, typename G>
__global__ void sigmoid_gate_kernel(T* __restrict__ out, long ld_out, const G* __restrict__ gate, long ld_g, int cols, long total) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const long row = i / cols;
  const int col = (int)(i % cols);
  T* p = out + row * ld_out + col;
  const float z = tw_to_float(gate[row * ld_g + col]);
  *p = tw_from_float<T>(tw_to_float(*p) / (1.f + expf(-z)));
}

extern "C" int tw_sigmoid_gate(int dtype, void* out, long ld_out, const void* gate, long ld_g, int gate_f32, int n, int cols,
                               hipStream_t stream) {
  TW_REQUIRE(out && gate && n >= 0 && cols > 0 && ld_out >= cols && ld_g >= cols);
  if (n == 0) return 0;
  const long total = (long)n * cols;
  const int blocks = tw_div_up(total, 256);
  if (dtype == TW_DTYPE_BF16 && gate_f32)
    sigmoid_gate_kernel<bf16_t, float><<<blocks, 256, 0, stream>>>((bf16_t*)out, ld_out, (const float*)gate, ld_g, cols, total);
  else if (dtype == TW_DTYPE_BF16)
    sigmoid_gate_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, ld_out, (const bf16_t*)gate, ld_g, cols, total);
  else if (dtype == TW_DTYPE_F32)
    sigmoid_gate_kernel<float, float><<<blocks, 256, 0, stream>>>((float*)out, ld_out, (const float*)gate, ld_g, cols, total);
  else return TW_ERR_BAD_ARGUMENT;
  return TW_LAUNCH_RESULT();
}

// ---- x <- cap * tanh(x / cap) over float32 values (a soft cap of the logits) ---------------------------------------
__global__ void softcap_values_kernel(float* __restrict__ x, long total, float cap) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) x[i] = cap * tanhf(x[i] / cap);
}

extern "C" int tw_softcap_values(float* x, long total, float cap, hipStream_t stream) {
  TW_REQUIRE(x && total >= 0 && cap > 0.f);
  if (total == 0) return 0;
  softcap_values_kernel<<<tw_div_up(total, 256), 256, 0, stream>>>(x, total, cap);
  return TW_LAUNCH_RESULT();
}
