// Dynamic-Tanh normalisation: y = tanh(alpha x) * w + b. No statistics, so the
// kernels are elementwise; the fused form carries the f32 residual stream:
//   resid += dyt(y; post)   and, in the same pass,   h = dyt(resid; next)
// which is one read of the sublayer output, one read-modify-write of the
// residual and one write of the next sublayer's input.
#include "seqmix.h"

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void dyt_norm_kernel(
    const TI* __restrict__ x, const int64_t* __restrict__ row_idx, const float* __restrict__ w,
    const float* __restrict__ b, float alpha, TO* __restrict__ y, int rows, int d) {
  const int r = blockIdx.x;
  const size_t src = (size_t)(row_idx ? row_idx[r] : r) * d;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < d; c += gridDim.y * blockDim.x)
    Act<TO>::st(y + (size_t)r * d + c, tanh_f(alpha * Act<TI>::ld(x + src + c)) * w[c] + b[c]);
}

template <typename TY, typename TO>
__global__ __launch_bounds__(256) void dyt_add_norm_kernel(
    float* __restrict__ resid, const TY* __restrict__ y, const float* __restrict__ w1,
    const float* __restrict__ b1, float a1, const float* __restrict__ w2,
    const float* __restrict__ b2, float a2, TO* __restrict__ h, int d) {
  const size_t base = (size_t)blockIdx.x * d;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < d; c += gridDim.y * blockDim.x) {
    const float v = resid[base + c] + (tanh_f(a1 * Act<TY>::ld(y + base + c)) * w1[c] + b1[c]);
    resid[base + c] = v;
    if (h) Act<TO>::st(h + base + c, tanh_f(a2 * v) * w2[c] + b2[c]);
  }
}

extern "C" int loqa_dyt_norm(const void* x, int x_dt, const void* row_idx, const void* w,
                             const void* b, float alpha, void* y, int y_dt, int rows, int d,
                             hipStream_t st) {
  if (rows <= 0) return 0;
  const int thr = d >= 256 ? 256 : 64 * ((d + 63) / 64);
  // a decode step has few rows: the columns spread over workgroups as well
  const int gy = rows >= 512 ? 1 : (d + thr - 1) / thr;
#define GO(TI, TO)                                                                           \
  hipLaunchKernelGGL((dyt_norm_kernel<TI, TO>), dim3(rows, gy), dim3(thr), 0, st, (const TI*)x, \
                     (const int64_t*)row_idx, (const float*)w, (const float*)b, alpha, (TO*)y, rows, d)
  if (x_dt == 0 && y_dt == 0) GO(bf16_t, bf16_t);
  else if (x_dt == 0) GO(bf16_t, float);
  else if (y_dt == 0) GO(float, bf16_t);
  else GO(float, float);
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_dyt_add_norm(void* resid, const void* y, int y_dt, const void* w1,
                                 const void* b1, float a1, const void* w2, const void* b2, float a2,
                                 void* h, int h_dt, int rows, int d, hipStream_t st) {
  if (rows <= 0) return 0;
  const int thr = d >= 256 ? 256 : 64 * ((d + 63) / 64);
  const int gy = rows >= 512 ? 1 : (d + thr - 1) / thr;
#define GO(TY, TO)                                                                              \
  hipLaunchKernelGGL((dyt_add_norm_kernel<TY, TO>), dim3(rows, gy), dim3(thr), 0, st, (float*)resid, \
                     (const TY*)y, (const float*)w1, (const float*)b1, a1, (const float*)w2,    \
                     (const float*)b2, a2, (TO*)h, d)
  if (y_dt == 0 && h_dt == 0) GO(bf16_t, bf16_t);
  else if (y_dt == 0) GO(bf16_t, float);
  else if (h_dt == 0) GO(float, bf16_t);
  else GO(float, float);
#undef GO
  return (int)hipGetLastError();
}
