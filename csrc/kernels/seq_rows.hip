// Per-sequence row state of decoders whose mixers look one or a few tokens
// back without a cache: token shift (a learned blend with the previous
// token's row) and short causal convolutions on projected rows.
//
// The state lives in f32 slots, one per live sequence: prev[slot][d] (the last
// mixer input) and tail[slot][taps - 1][C] (the last projected rows). Inside a
// feed the earlier rows are read from the batch itself, before the feed's first
// token from the slot; a sequence at position 0 reads zeros, so a reused slot
// needs no clearing. Readers and the writer of a slot are different launches
// (token_shift / conv_norm_rope_append read, seq_state_save writes afterwards),
// so a step never sees half-updated state.
//
// conv_norm_rope_append_kernel (one workgroup per token) is everything between
// the q | k projection GEMM and attention: convolution in f32 (weights stored
// tap-major, [taps][C]), v = convolved k, RMS norm over the whole q and the
// whole k projection, rotate-half rotary positions on the first `dims` entries
// of every head, k into its page [blocks][BLK][G D] and v into its transposed
// page [blocks][G D][BLK] (the layout attention reads). The v8 form gives a thread 8
// neighbouring channels (16-byte loads and stores, all taps' loads in flight at
// once); the scalar form takes any sizes.
#include "seqmix.h"

__device__ __forceinline__ int seq_of_row(const int* __restrict__ cu_q, int B, int t) {
  int b = 0;
  while (b + 1 < B && t >= cu_q[b + 1]) ++b;
  return b;
}

template <typename TO>
__global__ __launch_bounds__(256) void token_shift_kernel(
    const float* __restrict__ x, const float* __restrict__ mu, const float* __restrict__ prev,
    int nslots, const int* __restrict__ slots, const int* __restrict__ cu_q,
    const int* __restrict__ pos, int B, int d, TO* __restrict__ h) {
  const int t = blockIdx.x;
  const size_t base = (size_t)t * d;
  const float* before = nullptr;
  if (t < cu_q[B]) {
    const int b = seq_of_row(cu_q, B, t);
    if (t > cu_q[b]) before = x + base - d;
    else if (pos[t] > 0) before = prev + (size_t)min(max(slots[b], 0), nslots - 1) * d;
  }
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < d; c += gridDim.y * blockDim.x) {
    const float xv = x[base + c];
    const float pv = before ? before[c] : 0.f;
    Act<TO>::st(h + base + c, xv + (pv - xv) * mu[c]);
  }
}

// One workgroup column block per sequence; a thread owns a column and walks the
// tail rows upwards, so it never reads a row it has already replaced.
template <typename TU>
__global__ __launch_bounds__(256) void seq_state_save_kernel(
    const float* __restrict__ x, int d, const TU* __restrict__ u, int ldu, float* __restrict__ prev,
    float* __restrict__ tail, int nslots, int keep, int C, const int* __restrict__ slots,
    const int* __restrict__ cu_q, const int* __restrict__ pos) {
  const int b = blockIdx.x;
  const int q0 = cu_q[b], q1 = cu_q[b + 1], n = q1 - q0;
  if (n <= 0) return;
  const int slot = min(max(slots[b], 0), nslots - 1);
  const bool fresh = pos[q0] == 0;
  const int c0 = blockIdx.y * blockDim.x + threadIdx.x, step = gridDim.y * blockDim.x;
  if (prev)
    for (int c = c0; c < d; c += step) prev[(size_t)slot * d + c] = x[(size_t)(q1 - 1) * d + c];
  float* ts = tail + (size_t)slot * keep * C;
  for (int c = c0; c < C; c += step)
    for (int i = 0; i < keep; ++i) {
      const int r = n - keep + i;                 // row of the feed that lands in tail row i
      float v;
      if (r >= 0) v = Act<TU>::ld(u + (size_t)(q0 + r) * ldu + c);
      else v = fresh ? 0.f : ts[(size_t)(i + n) * C + c];
      ts[(size_t)i * C + c] = v;
    }
}

template <typename TU, typename TO>
__global__ __launch_bounds__(256) void conv_norm_rope_append_kernel(
    const TU* __restrict__ u, int ldu, const float* __restrict__ cw, int taps,
    const float* __restrict__ tail, int nslots, const int* __restrict__ sslots,
    const int* __restrict__ cu_q, const int* __restrict__ pos, int B,
    const float* __restrict__ qn, const float* __restrict__ kn, float eps,
    const float* __restrict__ cs, int max_pos, int dims, int H, int G, int D,
    TO* __restrict__ kc, TO* __restrict__ vc, long cache_rows, int blk,
    const int* __restrict__ kvslots,
    TO* __restrict__ q) {
  extern __shared__ float y[];                    // the convolved q | k row
  __shared__ float red[8];
  const int t = blockIdx.x;
  if (t >= cu_q[B]) return;
  const int b = seq_of_row(cu_q, B, t);
  const int i = t - cu_q[b], p = pos[t], keep = taps - 1;
  const int Cq = H * D, Ck = G * D, C = Cq + Ck;
  const float* ts = tail + (size_t)min(max(sslots[b], 0), nslots - 1) * keep * C;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
      const int s = keep - j;                     // how many tokens back this tap reads
      if (p - s < 0) continue;                    // before the sequence's start
      const float uv = i - s >= 0 ? Act<TU>::ld(u + (size_t)(t - s) * ldu + c)
                                  : ts[(size_t)(keep + i - s) * C + c];
      acc += cw[(size_t)j * C + c] * uv;
    }
    y[c] = acc;
    if (c < Cq) sq += acc * acc; else sk += acc * acc;
  }
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  const float rq = rsqrtf(sq / (float)Cq + eps), rk = rsqrtf(sk / (float)Ck + eps);
  const int half = dims / 2;
  const float* csp = cs + (size_t)min(max(p, 0), max_pos - 1) * dims;     // [half][2]
  const long slot = kvslots[t];
  const bool store = slot >= 0 && slot < cache_rows;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    const bool isq = c < Cq;
    const int cc = isq ? c : c - Cq, e = cc % D;
    const float r = isq ? rq : rk;
    const float* nw = isq ? qn : kn;
    float v = y[c] * r * nw[cc];
    if (e < dims) {
      const int f = e < half ? e : e - half;
      const int pc = e < half ? c + half : c - half, pcc = e < half ? cc + half : cc - half;
      const float o = y[pc] * r * nw[pcc];
      const float co = csp[2 * f], si = csp[2 * f + 1];
      v = e < half ? v * co - o * si : v * co + o * si;
    }
    if (isq) Act<TO>::st(q + (size_t)t * Cq + c, v);
    else if (store) {
      Act<TO>::st(kc + (size_t)slot * Ck + cc, v);
      Act<TO>::st(vc + ((size_t)(slot / blk) * Ck + cc) * blk + slot % blk, y[c]);
    }
  }
}


template <typename T> struct Row8;
template <> struct Row8<bf16_t> {
  static __device__ __forceinline__ void ld(const bf16_t* p, float* f) {
    unpack8(*reinterpret_cast<const uint4*>(p), f);
  }
  static __device__ __forceinline__ void st(bf16_t* p, const float* f) {
    *reinterpret_cast<uint4*>(p) = pack8(f);
  }
};
template <> struct Row8<float> {
  static __device__ __forceinline__ void ld(const float* p, float* f) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
  }
  static __device__ __forceinline__ void st(float* p, const float* f) {
    *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(f[4], f[5], f[6], f[7]);
  }
};

// D, ldu and so C are multiples of 8: a thread's 8 channels lie in one head.
template <typename TU, typename TO>
__global__ __launch_bounds__(1024) void conv_norm_rope_append_v8_kernel(
    const TU* __restrict__ u, int ldu, const float* __restrict__ cw, int taps,
    const float* __restrict__ tail, int nslots, const int* __restrict__ sslots,
    const int* __restrict__ cu_q, const int* __restrict__ pos, int B,
    const float* __restrict__ qn, const float* __restrict__ kn, float eps,
    const float* __restrict__ cs, int max_pos, int dims, int H, int G, int D,
    TO* __restrict__ kc, TO* __restrict__ vc, long cache_rows, int blk,
    const int* __restrict__ kvslots,
    TO* __restrict__ q) {
  extern __shared__ float y[];
  __shared__ float red[16];
  const int t = blockIdx.x;
  if (t >= cu_q[B]) return;
  const int b = seq_of_row(cu_q, B, t);
  const int i = t - cu_q[b], p = pos[t], keep = taps - 1;
  const int Cq = H * D, Ck = G * D, C = Cq + Ck;
  const float* ts = tail + (size_t)min(max(sslots[b], 0), nslots - 1) * keep * C;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x * 8; c < C; c += blockDim.x * 8) {
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    if (i >= keep) {                             // every tap lies inside the feed: no branch
#pragma unroll 4
      for (int j = 0; j < taps; ++j) {
        float uv[8], w[8];
        Row8<TU>::ld(u + (size_t)(t - keep + j) * ldu + c, uv);
        Row8<float>::ld(cw + (size_t)j * C + c, w);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += w[e] * uv[e];
      }
    } else {
      for (int j = max(0, keep - p); j < taps; ++j) {     // taps before position 0 read zeros
        const int s = keep - j;
        float uv[8], w[8];
        if (i - s >= 0) Row8<TU>::ld(u + (size_t)(t - s) * ldu + c, uv);
        else Row8<float>::ld(ts + (size_t)(keep + i - s) * C + c, uv);
        Row8<float>::ld(cw + (size_t)j * C + c, w);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += w[e] * uv[e];
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { y[c + e] = acc[e]; ss += acc[e] * acc[e]; }
    if (c < Cq) sq += ss; else sk += ss;
  }
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  const float rq = rsqrtf(sq / (float)Cq + eps), rk = rsqrtf(sk / (float)Ck + eps);
  const int half = dims / 2;
  const float* csp = cs + (size_t)min(max(p, 0), max_pos - 1) * dims;
  const long slot = kvslots[t];
  const bool store = slot >= 0 && slot < cache_rows;
  for (int c = threadIdx.x * 8; c < C; c += blockDim.x * 8) {
    const bool isq = c < Cq;
    const int cc = isq ? c : c - Cq, e0 = cc % D;
    const float r = isq ? rq : rk;
    const float* nw = isq ? qn : kn;
    float w[8], v[8], raw[8];
    Row8<float>::ld(nw + cc, w);
#pragma unroll
    for (int e = 0; e < 8; ++e) { raw[e] = y[c + e]; v[e] = raw[e] * r * w[e]; }
    if (e0 < dims) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int d = e0 + e;
        if (d >= dims) continue;
        const int f = d < half ? d : d - half;
        const int off = d < half ? half : -half;
        const float o = y[c + e + off] * r * nw[cc + e + off];
        const float co = csp[2 * f], si = csp[2 * f + 1];
        v[e] = d < half ? v[e] * co - o * si : v[e] * co + o * si;
      }
    }
    if (isq) Row8<TO>::st(q + (size_t)t * Cq + c, v);
    else if (store) {
      Row8<TO>::st(kc + (size_t)slot * Ck + cc, v);
      TO* vp = vc + ((size_t)(slot / blk) * Ck + cc) * blk + slot % blk;
#pragma unroll
      for (int e = 0; e < 8; ++e) Act<TO>::st(vp + (size_t)e * blk, raw[e]);
    }
  }
}

extern "C" int loqa_token_shift(const void* x, const void* mu, const void* prev, int nslots,
                                const void* slots, const void* cu_q, const void* pos, int B, int T,
                                int d, void* h, int h_dt, hipStream_t st) {
  if (T <= 0) return 0;
  if (B <= 0 || d <= 0 || nslots <= 0) return (int)hipErrorInvalidValue;
  const int thr = d >= 256 ? 256 : 64 * ((d + 63) / 64);
  const dim3 grid(T, T >= 512 ? 1 : (d + thr - 1) / thr);
#define GO(TO)                                                                                 \
  hipLaunchKernelGGL(token_shift_kernel<TO>, grid, dim3(thr), 0, st, (const float*)x,          \
                     (const float*)mu, (const float*)prev, nslots, (const int*)slots,          \
                     (const int*)cu_q, (const int*)pos, B, d, (TO*)h)
  if (h_dt == 0) GO(bf16_t); else GO(float);
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_seq_state_save(const void* x, int d, const void* u, int u_dt, int ldu,
                                   void* prev, void* tail, int nslots, int keep, int C,
                                   const void* slots, const void* cu_q, const void* pos, int B,
                                   hipStream_t st) {
  if (B <= 0) return 0;
  if (nslots <= 0 || keep < 0 || C <= 0) return (int)hipErrorInvalidValue;
  const int w = C > d ? C : d;
  const dim3 grid(B, (w + 255) / 256);
#define GO(TU)                                                                                 \
  hipLaunchKernelGGL(seq_state_save_kernel<TU>, grid, dim3(256), 0, st, (const float*)x, d,    \
                     (const TU*)u, ldu, (float*)prev, (float*)tail, nslots, keep, C,           \
                     (const int*)slots, (const int*)cu_q, (const int*)pos)
  if (u_dt == 0) GO(bf16_t); else GO(float);
#undef GO
  return (int)hipGetLastError();
}

extern "C" int loqa_conv_norm_rope_append(
    const void* u, int u_dt, int ldu, const void* cw, int taps, const void* tail, int nslots,
    const void* sslots, const void* cu_q, const void* pos, int B, int T, const void* qn,
    const void* kn, float eps, const void* cs, int max_pos, int dims, int H, int G, int D, void* kc,
    void* vc, int blk, int nblocks, const void* kvslots, void* q, int o_dt, hipStream_t st) {
  if (T <= 0) return 0;
  const long C = (long)(H + G) * D;
  if (B <= 0 || taps < 1 || nslots <= 0 || dims < 0 || dims > D || dims % 2 || C * 4 > 64 * 1024 ||
      max_pos <= 0)
    return (int)hipErrorInvalidValue;
  const long rows = (long)blk * nblocks;
  const bool v8 = D % 8 == 0 && ldu % 8 == 0;
  int thr = 256;
  if (v8) {
    thr = (int)((C / 8 + 63) / 64) * 64;
    if (thr > 1024) thr = 1024;
  }
#define ARGS(TU, TO)                                                                            \
  (const TU*)u, ldu, (const float*)cw, taps, (const float*)tail, nslots, (const int*)sslots,    \
      (const int*)cu_q, (const int*)pos, B, (const float*)qn, (const float*)kn, eps,            \
      (const float*)cs, max_pos, dims, H, G, D, (TO*)kc, (TO*)vc, rows, blk,                   \
      (const int*)kvslots,                                                                      \
      (TO*)q
#define GO(TU, TO)                                                                              \
  do {                                                                                          \
    if (v8)                                                                                     \
      hipLaunchKernelGGL((conv_norm_rope_append_v8_kernel<TU, TO>), dim3(T), dim3(thr), C * 4,  \
                         st, ARGS(TU, TO));                                                     \
    else                                                                                        \
      hipLaunchKernelGGL((conv_norm_rope_append_kernel<TU, TO>), dim3(T), dim3(256), C * 4, st, \
                         ARGS(TU, TO));                                                         \
  } while (0)
  if (u_dt == 0 && o_dt == 0) GO(bf16_t, bf16_t);
  else if (u_dt == 1 && o_dt == 1) GO(float, float);
  else return (int)hipErrorInvalidValue;
#undef GO
#undef ARGS
  return (int)hipGetLastError();
}
