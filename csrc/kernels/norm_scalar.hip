// RMS norm with ONE gain for all coordinates, on a sublayer's output:
//   resid += c * y / sqrt(mean(y^2) + eps)        (c = gain * residual multiplier)
// in one launch per residual step: the row of y is read once into registers,
// the f32 residual stream is updated in place and, when the next sublayer's
// GEMMs want it, written again in the activation dtype. The row sum is taken in
// f32 in a fixed order for a given width, so a row's result does not depend on
// the batch around it.
#include "seqmix.h"

#define NS_MAXV 32          // values per thread held in registers (d <= 256 * 32)

template <typename TY, int NV>
__global__ __launch_bounds__(256) void scalar_rms_add_kernel(
    float* __restrict__ resid, const TY* __restrict__ y, float c, float eps,
    bf16_t* __restrict__ h, int d) {
  __shared__ float red[8];
  const size_t base = (size_t)blockIdx.x * d;
  float v[NV];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int col = threadIdx.x + i * 256;
    v[i] = col < d ? Act<TY>::ld(y + base + col) : 0.f;
    s += v[i] * v[i];
  }
  s = block_sum(s, red);
  const float r = c * rsqrtf(s / (float)d + eps);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int col = threadIdx.x + i * 256;
    if (col < d) {
      const float o = resid[base + col] + v[i] * r;
      resid[base + col] = o;
      if (h) h[base + col] = f2bf(o);
    }
  }
}

__global__ __launch_bounds__(256) void scalar_rms_norm_kernel(
    const float* __restrict__ x, const int64_t* __restrict__ row_idx, float g, float eps,
    float* __restrict__ y, int d) {
  __shared__ float red[8];
  const size_t src = (size_t)(row_idx ? row_idx[blockIdx.x] : blockIdx.x) * d;
  const size_t dst = (size_t)blockIdx.x * d;
  float s = 0.f;
  for (int c = threadIdx.x; c < d; c += 256) { const float v = x[src + c]; s += v * v; }
  s = block_sum(s, red);
  const float r = g * rsqrtf(s / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += 256) y[dst + c] = x[src + c] * r;
}

extern "C" int loqa_scalar_rms_add(void* resid, const void* y, int y_dt, float c, float eps, void* h,
                                   int rows, int d, hipStream_t st) {
  if (rows <= 0) return 0;
  if (d <= 0 || d > 256 * NS_MAXV) return (int)hipErrorInvalidValue;
#define GO(TY, NV)                                                                            \
  hipLaunchKernelGGL((scalar_rms_add_kernel<TY, NV>), dim3(rows), dim3(256), 0, st, (float*)resid, \
                     (const TY*)y, c, eps, (bf16_t*)h, d)
#define BY_WIDTH(TY)                                                                          \
  do {                                                                                        \
    if (d <= 512) GO(TY, 2); else if (d <= 2048) GO(TY, 8); else GO(TY, NS_MAXV);             \
  } while (0)
  if (y_dt == 0) BY_WIDTH(bf16_t); else BY_WIDTH(float);
#undef BY_WIDTH
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_scalar_rms_norm(const void* x, const void* row_idx, float g, float eps, void* y,
                                    int rows, int d, hipStream_t st) {
  if (rows <= 0) return 0;
  hipLaunchKernelGGL(scalar_rms_norm_kernel, dim3(rows), dim3(256), 0, st, (const float*)x,
                     (const int64_t*)row_idx, g, eps, (float*)y, d);
  return (int)hipGetLastError();
}
