// Norm-after-sum layers with a 32-bit residual stream, and the xIELU activation.
//
//   scaled_add_norm:  z = alpha * x + y;  x' = z / sqrt(mean(z^2) + eps) * g      (g: ONE number for all coordinates)
//
// x is the fp32 residual stream and is replaced in place (or written to `out32`); `outc` receives a copy in the
// compute dtype T (bf16 / fp32), the operand of the next projection. y is a sublayer's output in T (null: zero).
// All arithmetic is fp32. One workgroup per token; any width.
//
//   xielu:  z > 0: softplus(p) z^2 + z/2;   z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2,  (p, q) = act[0..1]
#include "common.hpp"

namespace {

template <typename T> DEVINL float ldf(const T* p, size_t i);
template <> DEVINL float ldf<bf16_t>(const bf16_t* p, size_t i) { return bf2f(p[i]); }
template <> DEVINL float ldf<float>(const float* p, size_t i) { return p[i]; }
template <typename T> DEVINL void stf(T* p, size_t i, float v);
template <> DEVINL void stf<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f2bf(v); }
template <> DEVINL void stf<float>(float* p, size_t i, float v) { p[i] = v; }

template <typename T>
__global__ void __launch_bounds__(256) scaled_add_norm_kernel(const float* x, const T* __restrict__ y,
                                                               const T* __restrict__ gain, float* out32,
                                                               T* __restrict__ outc, int W, float alpha, float eps) {
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float z = alpha * x[row + i];
    if (y) z += ldf<T>(y, row + i);
    out32[row + i] = z;  // the thread that wrote an element is the one that reads it back below
    ss += z * z;
  }
  ss = block_sum(ss, red);
  const float r = ldf<T>(gain, 0) / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) {
    const float v = out32[row + i] * r;
    out32[row + i] = v;
    if (outc) stf<T>(outc, row + i, v);
  }
}

// Rows of up to 256 * NV elements: the sums stay in registers between the two passes (one read and one write of
// the stream instead of two of each).
template <typename T, int NV>
__global__ void __launch_bounds__(256) scaled_add_norm_reg_kernel(const float* x, const T* __restrict__ y,
                                                                   const T* __restrict__ gain, float* out32,
                                                                   T* __restrict__ outc, int W, float alpha,
                                                                   float eps) {
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * W;
  float z[NV], ss = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + 256 * j;
    z[j] = 0.f;
    if (i < W) {
      z[j] = alpha * x[row + i];
      if (y) z[j] += ldf<T>(y, row + i);
      ss += z[j] * z[j];
    }
  }
  ss = block_sum(ss, red);
  const float r = ldf<T>(gain, 0) / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + 256 * j;
    if (i < W) {
      const float v = z[j] * r;
      out32[row + i] = v;
      if (outc) stf<T>(outc, row + i, v);
    }
  }
}

DEVINL float softplusf(float x) { return x > 20.f ? x : log1pf(expf(x)); }

template <typename T>
__global__ void __launch_bounds__(256) xielu_kernel(const T* __restrict__ z, const T* __restrict__ act,
                                                     T* __restrict__ out, int64_t n) {
  const float ap = softplusf(ldf<T>(act, 0)), an = 0.5f + softplusf(ldf<T>(act, 1));
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float v = ldf<T>(z, i);
    const float r = v > 0.f ? ap * v * v + 0.5f * v : an * (expm1f(v) - v) + 0.5f * v;
    stf<T>(out, i, r);
  }
}

}  // namespace

// dt: 0 = bf16, 1 = fp32 (type of y, gain, outc)
extern "C" int areal_scaled_add_norm(const float* x, const void* y, const void* gain, float* out32, void* outc,
                                     int T, int W, float alpha, float eps, int dt, hipStream_t st) {
  if (T == 0) return 0;
  if (W <= 0) return -1;
#define LAUNCH(KERNEL, TT)                                                                                       \
  hipLaunchKernelGGL(KERNEL, dim3(T), dim3(256), 0, st, x, (const TT*)y, (const TT*)gain, out32, (TT*)outc, W, alpha, eps)
#define PICK(TT)                                                                  \
  do {                                                                            \
    if (W <= 256 * 4) LAUNCH((scaled_add_norm_reg_kernel<TT, 4>), TT);            \
    else if (W <= 256 * 8) LAUNCH((scaled_add_norm_reg_kernel<TT, 8>), TT);       \
    else if (W <= 256 * 16) LAUNCH((scaled_add_norm_reg_kernel<TT, 16>), TT);     \
    else if (W <= 256 * 32) LAUNCH((scaled_add_norm_reg_kernel<TT, 32>), TT);     \
    else LAUNCH(scaled_add_norm_kernel<TT>, TT);                                  \
  } while (0)
  if (dt == 0) PICK(bf16_t);
  else PICK(float);
#undef PICK
#undef LAUNCH
  return (int)hipGetLastError();
}

extern "C" int areal_xielu(const void* z, const void* act, void* out, int64_t n, int dt, hipStream_t st) {
  if (n == 0) return 0;
  const int64_t want = (n + 255) / 256;
  const dim3 grid((unsigned)(want < 4096 ? want : 4096));
  if (dt == 0)
    hipLaunchKernelGGL(xielu_kernel<bf16_t>, grid, dim3(256), 0, st, (const bf16_t*)z, (const bf16_t*)act,
                       (bf16_t*)out, n);
  else
    hipLaunchKernelGGL(xielu_kernel<float>, grid, dim3(256), 0, st, (const float*)z, (const float*)act, (float*)out,
                       n);
  return (int)hipGetLastError();
}
