// Elementwise chains of the Llama decoder layer around the projections (gfx950): one pass over the
// activations each instead of the eight (RMSNorm) or two (SiLU * up) torch kernels upstream runs.
//
//   rd_add_rms_norm   h = x + delta (optional; the residual update of the layer before)
//                     y = weight * cast(h_f32 * rsqrt(mean(h_f32^2) + eps))
//                     modeling_llama.py:27-32 (LlamaRMSNorm.forward), :196, :198 (the += updates)
//   rd_silu_mul       y = silu(gate) * up, gate and up the two halves of one fused projection
//                     modeling_llama.py:84-85 (LlamaMLP.forward)
//   rd_silu_add       the two elementwise steps of the drafter head, one launch each:
//                     mode 0  y = x + silu(z)   ResBlock.forward (modeling_drafter.py:38-39)
//                     mode 1  y = silu(x + z)   the recurrent state update (modeling_drafter.py:192-197),
//                             written to up to two places (the state, and its half of the
//                             [context, state] input of the head, modeling_drafter.py:199)
//
// Rounding follows the tensors' dtype at the points where upstream materialises a tensor: the sum
// h, the normalised value before the gain, the activation before the product.  The mean of squares
// is accumulated in float32 in a fixed order (per-thread partials, wave, workgroup), which is not
// torch's reduction order: results agree to float32 rounding of that mean.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "rd_common.h"

namespace {

constexpr int kThreads = 256;

template <typename T> struct Cvt;
template <> struct Cvt<float> {
  static __device__ float up(float v) { return v; }
  static __device__ float down(float v) { return v; }
};
template <> struct Cvt<__hip_bfloat16> {
  static __device__ float up(__hip_bfloat16 v) { return __bfloat162float(v); }
  static __device__ __hip_bfloat16 down(float v) { return __float2bfloat16(v); }
};
template <> struct Cvt<__half> {
  static __device__ float up(__half v) { return __half2float(v); }
  static __device__ __half down(float v) { return __float2half(v); }
};

template <typename T>
struct alignas(16) Vec {
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

__device__ inline float block_sum(float v, float* s_red) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = v;
  __syncthreads();
  float r = 0.f;
  for (int w = 0; w < kThreads / 64; ++w) r += s_red[w];  // fixed order
  return r;
}

// One workgroup per row; the row stays in registers between the two passes (VPT vectors of 16
// bytes per thread).
template <typename T, int VPT>
__global__ __launch_bounds__(kThreads) void add_rms_norm_kernel(
    const T* __restrict__ x, int64_t x_stride, const T* __restrict__ delta, int64_t d_stride,
    const T* __restrict__ weight, T* __restrict__ y, int64_t y_stride, T* __restrict__ h_out,
    int64_t h_stride, int cols, float eps) {
#pragma clang fp contract(off)
  using V = Vec<T>;
  constexpr int N = V::N;
  __shared__ float s_red[kThreads / 64];
  const int64_t row = blockIdx.x;
  const int n_vec = cols / N;
  float h[VPT][N];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int vi = k * kThreads + threadIdx.x;
    if (vi < n_vec) {
      const V a = *reinterpret_cast<const V*>(x + row * x_stride + (int64_t)vi * N);
      if (delta) {
        const V d = *reinterpret_cast<const V*>(delta + row * d_stride + (int64_t)vi * N);
        V s;
#pragma unroll
        for (int e = 0; e < N; ++e) {
          s.v[e] = Cvt<T>::down(Cvt<T>::up(a.v[e]) + Cvt<T>::up(d.v[e]));
          h[k][e] = Cvt<T>::up(s.v[e]);
        }
        if (h_out) *reinterpret_cast<V*>(h_out + row * h_stride + (int64_t)vi * N) = s;
      } else {
#pragma unroll
        for (int e = 0; e < N; ++e) h[k][e] = Cvt<T>::up(a.v[e]);
      }
#pragma unroll
      for (int e = 0; e < N; ++e) ss += h[k][e] * h[k][e];
    }
  }
  const float mean = block_sum(ss, s_red) / (float)cols;
  const float inv = rsqrtf(mean + eps);
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int vi = k * kThreads + threadIdx.x;
    if (vi < n_vec) {
      const V w = *reinterpret_cast<const V*>(weight + (int64_t)vi * N);
      V o;
#pragma unroll
      for (int e = 0; e < N; ++e) {
        const float normed = Cvt<T>::up(Cvt<T>::down(h[k][e] * inv));
        o.v[e] = Cvt<T>::down(Cvt<T>::up(w.v[e]) * normed);
      }
      *reinterpret_cast<V*>(y + row * y_stride + (int64_t)vi * N) = o;
    }
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void silu_mul_kernel(
    const T* __restrict__ gate, const T* __restrict__ up, int64_t in_stride, T* __restrict__ y,
    int64_t y_stride, int cols) {
#pragma clang fp contract(off)
  using V = Vec<T>;
  constexpr int N = V::N;
  const int64_t row = blockIdx.y;
  const int vi = blockIdx.x * kThreads + threadIdx.x;
  if (vi >= cols / N) return;
  const V g = *reinterpret_cast<const V*>(gate + row * in_stride + (int64_t)vi * N);
  const V u = *reinterpret_cast<const V*>(up + row * in_stride + (int64_t)vi * N);
  V o;
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const float gv = Cvt<T>::up(g.v[e]);
    const float act = Cvt<T>::up(Cvt<T>::down(gv / (1.0f + expf(-gv))));
    o.v[e] = Cvt<T>::down(act * Cvt<T>::up(u.v[e]));
  }
  *reinterpret_cast<V*>(y + row * y_stride + (int64_t)vi * N) = o;
}

template <typename T, int MODE>
__global__ __launch_bounds__(kThreads) void silu_add_kernel(
    const T* __restrict__ x, int64_t x_stride, const T* __restrict__ z, int64_t z_stride, T* __restrict__ y,
    int64_t y_stride, T* __restrict__ y2, int64_t y2_stride, int cols) {
#pragma clang fp contract(off)
  using V = Vec<T>;
  constexpr int N = V::N;
  const int64_t row = blockIdx.y;
  const int vi = blockIdx.x * kThreads + threadIdx.x;
  if (vi >= cols / N) return;
  const V a = *reinterpret_cast<const V*>(x + row * x_stride + (int64_t)vi * N);
  const V b = *reinterpret_cast<const V*>(z + row * z_stride + (int64_t)vi * N);
  V o;
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const float av = Cvt<T>::up(a.v[e]), bv = Cvt<T>::up(b.v[e]);
    if (MODE == 0) {
      const float act = Cvt<T>::up(Cvt<T>::down(bv / (1.0f + expf(-bv))));
      o.v[e] = Cvt<T>::down(av + act);
    } else {
      const float s = Cvt<T>::up(Cvt<T>::down(av + bv));
      o.v[e] = Cvt<T>::down(s / (1.0f + expf(-s)));
    }
  }
  *reinterpret_cast<V*>(y + row * y_stride + (int64_t)vi * N) = o;
  if (y2 != nullptr) *reinterpret_cast<V*>(y2 + row * y2_stride + (int64_t)vi * N) = o;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T>
int launch_norm(const void* x, int64_t x_stride, const void* delta, int64_t d_stride, const void* weight,
                void* y, int64_t y_stride, void* h_out, int64_t h_stride, int64_t rows, int cols, float eps,
                hipStream_t s) {
  constexpr int N = Vec<T>::N;
  const int vpt = (cols / N + kThreads - 1) / kThreads;
#define RD_NORM(VPT)                                                                                      \
  do { rd::ScopedTiming rd_t("add_rms_norm_kernel", s);                                                   \
    hipLaunchKernelGGL((add_rms_norm_kernel<T, VPT>), dim3(rows), dim3(kThreads), 0, s,                    \
                       reinterpret_cast<const T*>(x), x_stride, reinterpret_cast<const T*>(delta), d_stride, \
                       reinterpret_cast<const T*>(weight), reinterpret_cast<T*>(y), y_stride,              \
                       reinterpret_cast<T*>(h_out), h_stride, cols, eps); } while (0)
  if (vpt <= 1) RD_NORM(1);
  else if (vpt <= 2) RD_NORM(2);
  else if (vpt <= 4) RD_NORM(4);
  else RD_NORM(8);
#undef RD_NORM
  return rd::check_launch("rd_add_rms_norm");
}

}  // namespace

extern "C" int rd_add_rms_norm(const void* x, int64_t x_row_stride, const void* delta,
                               int64_t delta_row_stride, const void* weight, void* y,
                               int64_t y_row_stride, void* h_out, int64_t h_row_stride, int dtype,
                               int64_t rows, int cols, float eps, void* stream) {
  RD_REQUIRE(rows > 0 && cols > 0 && rows <= 2147483647LL, RD_EINVAL, "rd_add_rms_norm: bad sizes (rows %lld cols %d)",
             (long long)rows, cols);
  RD_REQUIRE(dtype == RD_F32 || dtype == RD_BF16 || dtype == RD_F16, RD_EINVAL, "rd_add_rms_norm: unknown dtype %d", dtype);
  const int vec = dtype == RD_F32 ? 4 : 8;
  RD_REQUIRE(cols % vec == 0 && cols <= 8 * kThreads * vec, RD_ELIMIT,
             "rd_add_rms_norm: cols %d must be a multiple of %d and at most %d", cols, vec, 8 * kThreads * vec);
  RD_REQUIRE(x && weight && y, RD_EINVAL, "rd_add_rms_norm: null pointer");
  RD_REQUIRE(!h_out || delta, RD_EINVAL, "rd_add_rms_norm: h_out without delta");
  RD_REQUIRE(aligned16(x) && aligned16(delta) && aligned16(weight) && aligned16(y) && aligned16(h_out), RD_EINVAL,
             "rd_add_rms_norm: pointers must be 16-byte aligned");
  RD_REQUIRE(x_row_stride % vec == 0 && y_row_stride % vec == 0 && (!delta || delta_row_stride % vec == 0) &&
                 (!h_out || h_row_stride % vec == 0) && x_row_stride >= cols && y_row_stride >= cols,
             RD_EINVAL, "rd_add_rms_norm: row strides must be multiples of %d elements and at least cols", vec);
  hipStream_t s = rd::as_stream(stream);
  switch (dtype) {
    case RD_F32: return launch_norm<float>(x, x_row_stride, delta, delta_row_stride, weight, y, y_row_stride, h_out, h_row_stride, rows, cols, eps, s);
    case RD_BF16: return launch_norm<__hip_bfloat16>(x, x_row_stride, delta, delta_row_stride, weight, y, y_row_stride, h_out, h_row_stride, rows, cols, eps, s);
    default: return launch_norm<__half>(x, x_row_stride, delta, delta_row_stride, weight, y, y_row_stride, h_out, h_row_stride, rows, cols, eps, s);
  }
}

extern "C" int rd_silu_mul(const void* gate, const void* up, int64_t in_row_stride, void* y,
                           int64_t y_row_stride, int dtype, int64_t rows, int cols, void* stream) {
  RD_REQUIRE(rows > 0 && cols > 0 && rows <= 65535 * 1024LL, RD_EINVAL, "rd_silu_mul: bad sizes (rows %lld cols %d)",
             (long long)rows, cols);
  RD_REQUIRE(dtype == RD_F32 || dtype == RD_BF16 || dtype == RD_F16, RD_EINVAL, "rd_silu_mul: unknown dtype %d", dtype);
  const int vec = dtype == RD_F32 ? 4 : 8;
  RD_REQUIRE(cols % vec == 0, RD_ELIMIT, "rd_silu_mul: cols %d must be a multiple of %d", cols, vec);
  RD_REQUIRE(gate && up && y, RD_EINVAL, "rd_silu_mul: null pointer");
  RD_REQUIRE(aligned16(gate) && aligned16(up) && aligned16(y) && in_row_stride % vec == 0 && y_row_stride % vec == 0 &&
                 in_row_stride >= cols && y_row_stride >= cols, RD_EINVAL, "rd_silu_mul: alignment or strides");
  RD_REQUIRE(rows <= 65535, RD_ELIMIT, "rd_silu_mul: rows %lld > 65535", (long long)rows);
  hipStream_t s = rd::as_stream(stream);
  const dim3 grid((cols / vec + kThreads - 1) / kThreads, (unsigned)rows);
  {
    rd::ScopedTiming rd_t("silu_mul_kernel", s);
    switch (dtype) {
      case RD_F32: hipLaunchKernelGGL(silu_mul_kernel<float>, grid, dim3(kThreads), 0, s, reinterpret_cast<const float*>(gate), reinterpret_cast<const float*>(up), in_row_stride, reinterpret_cast<float*>(y), y_row_stride, cols); break;
      case RD_BF16: hipLaunchKernelGGL(silu_mul_kernel<__hip_bfloat16>, grid, dim3(kThreads), 0, s, reinterpret_cast<const __hip_bfloat16*>(gate), reinterpret_cast<const __hip_bfloat16*>(up), in_row_stride, reinterpret_cast<__hip_bfloat16*>(y), y_row_stride, cols); break;
      default: hipLaunchKernelGGL(silu_mul_kernel<__half>, grid, dim3(kThreads), 0, s, reinterpret_cast<const __half*>(gate), reinterpret_cast<const __half*>(up), in_row_stride, reinterpret_cast<__half*>(y), y_row_stride, cols); break;
    }
  }
  return rd::check_launch("rd_silu_mul");
}

extern "C" int rd_silu_add(const void* x, int64_t x_row_stride, const void* z, int64_t z_row_stride,
                           void* y, int64_t y_row_stride, void* y2, int64_t y2_row_stride, int mode,
                           int dtype, int64_t rows, int cols, void* stream) {
  RD_REQUIRE(rows > 0 && cols > 0 && rows <= 65535, RD_EINVAL, "rd_silu_add: bad sizes (rows %lld cols %d)",
             (long long)rows, cols);
  RD_REQUIRE(mode == 0 || mode == 1, RD_EINVAL, "rd_silu_add: unknown mode %d", mode);
  RD_REQUIRE(dtype == RD_F32 || dtype == RD_BF16 || dtype == RD_F16, RD_EINVAL, "rd_silu_add: unknown dtype %d", dtype);
  const int vec = dtype == RD_F32 ? 4 : 8;
  RD_REQUIRE(cols % vec == 0, RD_ELIMIT, "rd_silu_add: cols %d must be a multiple of %d", cols, vec);
  RD_REQUIRE(x && z && y, RD_EINVAL, "rd_silu_add: null pointer");
  RD_REQUIRE(aligned16(x) && aligned16(z) && aligned16(y) && aligned16(y2) && x_row_stride % vec == 0 &&
                 z_row_stride % vec == 0 && y_row_stride % vec == 0 && (!y2 || y2_row_stride % vec == 0) &&
                 x_row_stride >= cols && z_row_stride >= cols && y_row_stride >= cols && (!y2 || y2_row_stride >= cols),
             RD_EINVAL, "rd_silu_add: alignment or strides");
  hipStream_t s = rd::as_stream(stream);
  const dim3 grid((cols / vec + kThreads - 1) / kThreads, (unsigned)rows);
#define RD_SA(T, MODE)                                                                                   \
  hipLaunchKernelGGL((silu_add_kernel<T, MODE>), grid, dim3(kThreads), 0, s, reinterpret_cast<const T*>(x), \
                     x_row_stride, reinterpret_cast<const T*>(z), z_row_stride, reinterpret_cast<T*>(y),  \
                     y_row_stride, reinterpret_cast<T*>(y2), y2_row_stride, cols)
  {
    rd::ScopedTiming rd_t("silu_add_kernel", s);
    if (mode == 0) {
      switch (dtype) {
        case RD_F32: RD_SA(float, 0); break;
        case RD_BF16: RD_SA(__hip_bfloat16, 0); break;
        default: RD_SA(__half, 0); break;
      }
    } else {
      switch (dtype) {
        case RD_F32: RD_SA(float, 1); break;
        case RD_BF16: RD_SA(__hip_bfloat16, 1); break;
        default: RD_SA(__half, 1); break;
      }
    }
  }
#undef RD_SA
  return rd::check_launch("rd_silu_add");
}
