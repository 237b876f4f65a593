// Decayed linear attention ("lightning") with a carried state, and the gated
// RMS norm that follows it.
//
// Per sequence and head:  S_t = decay_h * S_{t-1} + k_t v_t^T,  o_t = S_t^T q_t,
// q, k, v = SiLU of the projection columns. S [D, Dv] lives in f32 state slots
// between steps.
//
// lightning_scan_kernel: one workgroup per (sequence, head, 32 value columns).
// The columns of S evolve independently, so the grid splits Dv freely. A
// thread holds S[d, e] for one column e and every 8th row d in registers; the
// step's tokens are staged 16 at a time in LDS (SiLU applied once), the
// recurrence then runs token by token in f32 in the order of the definition,
// and the 8 row-partials of o_t are summed in a fixed order. A prompt portion,
// a single decode token, or any cut of a prompt therefore gives the same bits.
#include "seqmix.h"

#define LS_EC 32        // value columns per workgroup
#define LS_DP 8         // row partitions (threads per column)
#define LS_TC 16        // tokens staged per round

template <typename T, int MAXD>   // D <= LS_DP * MAXD
__global__ __launch_bounds__(LS_EC * LS_DP) void lightning_scan_kernel(
    const T* __restrict__ qkv, long ld, int H, int D, int Dv, float* __restrict__ state,
    const int* __restrict__ state_slots, const int* __restrict__ cu_q,
    const int* __restrict__ positions, const float* __restrict__ decay, float* __restrict__ o) {
  extern __shared__ float lds[];
  float* qs = lds;                         // [TC][D]
  float* ks = qs + LS_TC * D;              // [TC][D]
  float* vs = ks + LS_TC * D;              // [TC][EC]
  float* red = vs + LS_TC * LS_EC;         // [TC][DP][EC]
  const int b = blockIdx.x, h = blockIdx.y, e0 = blockIdx.z * LS_EC;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (q1 <= q0) return;
  const int e = threadIdx.x % LS_EC, dp = threadIdx.x / LS_EC;
  const bool col = e0 + e < Dv;
  const float lam = decay[h];
  float* Sg = state + (((size_t)state_slots[b] * H + h) * D) * Dv + e0 + e;
  const bool fresh = positions[q0] == 0;
  float S[MAXD];
#pragma unroll
  for (int i = 0; i < MAXD; ++i) {
    const int d = dp + LS_DP * i;
    S[i] = (!fresh && col && d < D) ? Sg[(size_t)d * Dv] : 0.f;
  }
  const size_t qoff = (size_t)h * D, koff = (size_t)H * D + (size_t)h * D;
  const size_t voff = 2 * (size_t)H * D + (size_t)h * Dv + e0;
  for (int t0 = q0; t0 < q1; t0 += LS_TC) {
    const int nt = min(LS_TC, q1 - t0);
    __syncthreads();
    for (int i = threadIdx.x; i < nt * D; i += blockDim.x) {
      const int tt = i / D, d = i - tt * D;
      const T* row = qkv + (size_t)(t0 + tt) * ld;
      qs[i] = silu_f(Act<T>::ld(row + qoff + d));
      ks[i] = silu_f(Act<T>::ld(row + koff + d));
    }
    for (int i = threadIdx.x; i < nt * LS_EC; i += blockDim.x) {
      const int tt = i / LS_EC, c = i - tt * LS_EC;
      vs[i] = e0 + c < Dv ? silu_f(Act<T>::ld(qkv + (size_t)(t0 + tt) * ld + voff + c)) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float v = vs[tt * LS_EC + e];
      const float* kq = ks + tt * D;
      const float* qq = qs + tt * D;
      float part = 0.f;
#pragma unroll
      for (int i = 0; i < MAXD; ++i) {
        const int d = dp + LS_DP * i;
        if (d < D) {
          S[i] = lam * S[i] + kq[d] * v;
          part += S[i] * qq[d];
        }
      }
      red[(tt * LS_DP + dp) * LS_EC + e] = part;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nt * LS_EC; i += blockDim.x) {
      const int tt = i / LS_EC, c = i - tt * LS_EC;
      if (e0 + c < Dv) {
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < LS_DP; ++k) s += red[(tt * LS_DP + k) * LS_EC + c];
        o[(size_t)(t0 + tt) * H * Dv + (size_t)h * Dv + e0 + c] = s;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < MAXD; ++i) {
    const int d = dp + LS_DP * i;
    if (col && d < D) Sg[(size_t)d * Dv] = S[i];
  }
}

// y = rmsnorm(o) * w * sigmoid(gate), one workgroup per row (all heads together).
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(
    const float* __restrict__ o, const float* __restrict__ w, const TG* __restrict__ gate, long ldg,
    float eps, TO* __restrict__ y, int n) {
  __shared__ float scratch[4];
  const size_t r = blockIdx.x;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float v = o[r * n + c];
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += blockDim.x)
    Act<TO>::st(y + r * n + c, o[r * n + c] * inv * w[c] * sigmoid_f(Act<TG>::ld(gate + r * ldg + c)));
}

extern "C" int loqa_lightning_scan(const void* qkv, int dt, long ld, int H, int D, int Dv,
                                   void* state, int nslots, const void* state_slots,
                                   const void* cu_q, const void* positions, const void* decay,
                                   void* o, int B, int T, hipStream_t st) {
  if (T <= 0 || B <= 0) return 0;
  if (D > LS_DP * 32 || D <= 0 || Dv <= 0) return (int)hipErrorInvalidValue;
  (void)nslots;
  const dim3 grid(B, H, (Dv + LS_EC - 1) / LS_EC), block(LS_EC * LS_DP);
  const size_t smem = (size_t)(2 * LS_TC * D + LS_TC * LS_EC + LS_TC * LS_DP * LS_EC) * 4;
#define GO(TT, MD)                                                                             \
  hipLaunchKernelGGL((lightning_scan_kernel<TT, MD>), grid, block, smem, st, (const TT*)qkv, ld, H, \
                     D, Dv, (float*)state, (const int*)state_slots, (const int*)cu_q,          \
                     (const int*)positions, (const float*)decay, (float*)o)
  const int md = D <= 64 ? 8 : (D <= 128 ? 16 : 32);
  if (dt == 0) { if (md == 8) GO(bf16_t, 8); else if (md == 16) GO(bf16_t, 16); else GO(bf16_t, 32); }
  else { if (md == 8) GO(float, 8); else if (md == 16) GO(float, 16); else GO(float, 32); }
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_gated_rmsnorm(const void* o, const void* w, const void* gate, int g_dt, long ldg,
                                  float eps, void* y, int y_dt, int T, int n, hipStream_t st) {
  if (T <= 0) return 0;
#define GO(TG, TO)                                                                            \
  hipLaunchKernelGGL((gated_rmsnorm_kernel<TG, TO>), dim3(T), dim3(256), 0, st, (const float*)o, \
                     (const float*)w, (const TG*)gate, ldg, eps, (TO*)y, n)
  if (g_dt == 0 && y_dt == 0) GO(bf16_t, bf16_t);
  else if (g_dt == 0) GO(bf16_t, float);
  else if (y_dt == 0) GO(float, bf16_t);
  else GO(float, float);
#undef GO
  return (int)hipGetLastError();
}
