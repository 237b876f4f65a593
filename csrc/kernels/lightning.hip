// Decayed linear attention ("lightning") with a carried state, and the gated
// RMS norm that follows it.
//
// Per sequence and head:  S_t = decay_h * S_{t-1} + k_t v_t^T,  o_t = S_t^T q_t,
// q, k, v = SiLU of the projection columns. S [D, Dv] lives in f32 state slots
// between steps.
//
// lightning_scan_kernel: one workgroup per (sequence, head, 32 value columns).
// The columns of S evolve independently, so the grid splits Dv freely. A
// thread holds S[d, e] for one column e and a contiguous run of MAXD rows d in
// registers (16 threads per column, 8 waves: two per SIMD, so one wave's LDS and
// cross-lane latencies hide behind the other's arithmetic). The step's tokens are staged TC at a time
// in LDS (SiLU applied once, rows zero-padded to 16 MAXD so the recurrence reads
// them as float4); the raw values of the next TC tokens are already in flight
// in registers while the current ones are processed. The recurrence runs token
// by token in f32 in the order of the definition; the 16 row-partials of o_t
// are summed in a fixed order (pairs inside a wave, then the 8 waves). A prompt
// portion, a single decode token, or any cut of a prompt gives the same bits.
#include "seqmix.h"

#define LS_EC 32        // value columns per workgroup
#define LS_DP 16        // row partitions (threads per column)
#define LS_THREADS (LS_EC * LS_DP)
#define LS_WAVES (LS_THREADS / 64)

template <typename T, int MAXD, int TC>   // D <= LS_DP * MAXD
__global__ __launch_bounds__(LS_EC * LS_DP) void lightning_scan_kernel(
    const T* __restrict__ qkv, long ld, int H, int D, int Dv, float* __restrict__ state,
    const int* __restrict__ state_slots, const int* __restrict__ cu_q,
    const int* __restrict__ positions, const float* __restrict__ decay, float* __restrict__ o) {
  constexpr int DPAD = LS_DP * MAXD;            // padded row length in LDS
  constexpr int NPT = TC * DPAD / LS_THREADS;   // staged q (and k) values per thread
  constexpr int NVT = TC * LS_EC / LS_THREADS;  // staged v values per thread
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* qs = lds;                         // [TC][DPAD]
  float* ks = qs + TC * DPAD;              // [TC][DPAD]
  float* vs = ks + TC * DPAD;              // [TC][EC]
  float* red = vs + TC * LS_EC;            // [TC][LS_WAVES][EC]
  const int b = blockIdx.x, h = blockIdx.y, e0 = blockIdx.z * LS_EC;
  const int q0 = cu_q[b], q1 = cu_q[b + 1];
  if (q1 <= q0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int e = tid % LS_EC, dp = tid / LS_EC;
  const bool col = e0 + e < Dv;
  const float lam = decay[h];
  float* Sg = state + (((size_t)state_slots[b] * H + h) * D) * Dv + e0 + e;
  const bool fresh = positions[q0] == 0;
  float S[MAXD];
#pragma unroll
  for (int i = 0; i < MAXD; ++i) {
    const int d = dp * MAXD + i;
    S[i] = (!fresh && col && d < D) ? Sg[(size_t)d * Dv] : 0.f;
  }
  const size_t qoff = (size_t)h * D, koff = (size_t)H * D + (size_t)h * D;
  const size_t voff = 2 * (size_t)H * D + (size_t)h * Dv + e0;
  float rq[NPT], rk[NPT], rv[NVT];
  auto fetch = [&](int t0) {               // raw projections of tokens t0 .. t0 + TC
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
      const int i = tid + LS_THREADS * j, tt = i / DPAD, d = i % DPAD;
      const bool ok = t0 + tt < q1 && d < D;
      const T* row = qkv + (size_t)(ok ? t0 + tt : q0) * ld;
      rq[j] = ok ? Act<T>::ld(row + qoff + d) : 0.f;
      rk[j] = ok ? Act<T>::ld(row + koff + d) : 0.f;
    }
#pragma unroll
    for (int j = 0; j < NVT; ++j) {
      const int i = tid + LS_THREADS * j, tt = i / LS_EC, c = i % LS_EC;
      const bool ok = t0 + tt < q1 && e0 + c < Dv;
      rv[j] = ok ? Act<T>::ld(qkv + (size_t)(t0 + tt) * ld + voff + c) : 0.f;
    }
  };
  fetch(q0);
  for (int t0 = q0; t0 < q1; t0 += TC) {
    const int nt = min(TC, q1 - t0);
    __syncthreads();                       // the previous round's LDS is consumed
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
      qs[tid + LS_THREADS * j] = silu_f(rq[j]);   // silu(0) = 0 keeps the padding zero
      ks[tid + LS_THREADS * j] = silu_f(rk[j]);
    }
#pragma unroll
    for (int j = 0; j < NVT; ++j) vs[tid + LS_THREADS * j] = silu_f(rv[j]);
    __syncthreads();
    if (t0 + TC < q1) fetch(t0 + TC);      // in flight during the recurrence below
    // two tokens per trip: the second token's LDS reads and read-out sums are
    // independent of the first's, so they overlap its latency (only the S
    // updates chain); four partial sums per token in a fixed order
#pragma unroll 2
    for (int tt = 0; tt < nt; ++tt) {
      const float v = vs[tt * LS_EC + e];
      const float4* k4 = reinterpret_cast<const float4*>(ks + tt * DPAD + dp * MAXD);
      const float4* q4 = reinterpret_cast<const float4*>(qs + tt * DPAD + dp * MAXD);
      float p0 = 0.f, p1 = 0.f, p2 = 0.f, p3 = 0.f;
#pragma unroll
      for (int i = 0; i < MAXD / 4; ++i) {
        const float4 kk = k4[i], qq = q4[i];
        S[4 * i] = lam * S[4 * i] + kk.x * v;         p0 += S[4 * i] * qq.x;
        S[4 * i + 1] = lam * S[4 * i + 1] + kk.y * v; p1 += S[4 * i + 1] * qq.y;
        S[4 * i + 2] = lam * S[4 * i + 2] + kk.z * v; p2 += S[4 * i + 2] * qq.z;
        S[4 * i + 3] = lam * S[4 * i + 3] + kk.w * v; p3 += S[4 * i + 3] * qq.w;
      }
      float part = (p0 + p1) + (p2 + p3);
      part += __shfl_xor(part, 32, 64);    // the wave's two row partitions
      if (lane < 32) red[(tt * LS_WAVES + wave) * LS_EC + e] = part;
    }
    __syncthreads();
    for (int i = tid; i < nt * LS_EC; i += LS_THREADS) {
      const int tt = i / LS_EC, c = i % LS_EC;
      if (e0 + c < Dv) {
        const float* r = red + tt * LS_WAVES * LS_EC + c;
        float sum = r[0];
#pragma unroll
        for (int w = 1; w < LS_WAVES; ++w) sum += r[w * LS_EC];
        o[(size_t)(t0 + tt) * H * Dv + (size_t)h * Dv + e0 + c] = sum;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < MAXD; ++i) {
    const int d = dp * MAXD + i;
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
  if (D > LS_DP * 16 || D <= 0 || Dv <= 0) return (int)hipErrorInvalidValue;
  (void)nslots;
  const dim3 grid(B, H, (Dv + LS_EC - 1) / LS_EC), block(LS_EC * LS_DP);
#define GO(TT, MD, TCC)                                                                          \
  hipLaunchKernelGGL((lightning_scan_kernel<TT, MD, TCC>), grid, block,                          \
                     (size_t)(2 * TCC * LS_DP * MD + TCC * LS_EC + TCC * LS_WAVES * LS_EC) * 4, st, \
                     (const TT*)qkv, ld, H, D, Dv, (float*)state, (const int*)state_slots,       \
                     (const int*)cu_q, (const int*)positions, (const float*)decay, (float*)o)
  const int md = D <= 64 ? 4 : (D <= 128 ? 8 : 16);
  if (dt == 0) { if (md == 4) GO(bf16_t, 4, 16); else if (md == 8) GO(bf16_t, 8, 16); else GO(bf16_t, 16, 16); }
  else { if (md == 4) GO(float, 4, 16); else if (md == 8) GO(float, 8, 16); else GO(float, 16, 16); }
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
