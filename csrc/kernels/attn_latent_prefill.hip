// Prompt-pass latent attention on the matrix cores (bf16).
//
// For passes with many query rows the folded form (attn_latent.hip) would pay
// R + Dr multiply-adds per score and R per value entry; here the keys and
// values are first materialised per head from the gathered latent rows (two
// vendor GEMMs: k_un = W_uk c, v = W_uv c), and a flash kernel in the manner of
// attention.hip's attn_fwd_kernel runs over [key, head, DK] / [key, head, DV]:
//   S^T = K Q^T (v_mfma_f32_32x32x16_bf16, the query on the MFMA lane so the
//   online softmax is in-register), O^T += V^T P^T with the exp2'ed S^T as the
//   B operand and V^T read from LDS with transposed reads.
// Differences from the Llama kernel: DK != DV (rotary part only in the keys),
// zero-padded head sizes (DK, DV are the next instantiated sizes), the causal
// bound comes from each row's absolute position, and a learned per-head sink
// joins the softmax denominator at the end.
//
// Helpers: latent_gather_kernel copies each sequence's latent rows from its
// pages into contiguous [sum L, R] / [sum L, Dr] buffers; latent_kfill_kernel
// writes the shared rotary key part into every head's key row;
// rope_pairs_kernel rotates the queries' rotary part in place.
#include "seqmix.h"

#define LP_THREADS 256
#define LP_WAVES 4
#define LP_TILE 64

typedef short lp_v4s __attribute__((ext_vector_type(4)));

struct LatPrefillParams {
  const bf16_t* q; long q_st;       // [T, H, DK]
  const bf16_t* k;                  // [sum L, H, DK]
  const bf16_t* v;                  // [sum L, H, DV]
  bf16_t* o;                        // [T, H, DV]
  const int* cu_q; const int* cu_k; const int* pos;
  const float* sink; float scale_log2;
  int H;
};

template <int DK, int DV>
struct LatPrefillSmem {
  bf16_t k[LP_TILE][DK + 8];
  bf16_t v[LP_TILE][DV + 32];
};

template <int DK, int DV>
__global__ __launch_bounds__(LP_THREADS) void latent_prefill_kernel(LatPrefillParams p) {
  __shared__ __attribute__((aligned(16))) LatPrefillSmem<DK, DV> sm;
  constexpr int NS = DK / 16, NDT = DV / 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = lane >> 5;
  const int head = blockIdx.y, b = blockIdx.z;
  const int q0 = p.cu_q[b], qlen = p.cu_q[b + 1] - q0;
  const int row_lo = blockIdx.x * (LP_WAVES * 32);
  if (row_lo >= qlen) return;
  const int row_hi = min(qlen - 1, row_lo + LP_WAVES * 32 - 1);
  const int k0 = p.cu_k[b], klen = p.cu_k[b + 1] - k0;
  const int qi = row_lo + wave * 32 + (lane & 31);
  const bool valid = qi < qlen;
  const int qpos = p.pos[q0 + (valid ? qi : row_hi)];
  const int kend = min(klen, p.pos[q0 + row_hi] + 1);     // positions grow along a sequence

  bf16x8 qf[NS];
  {
    const bf16_t* qrow = p.q + (size_t)(q0 + (valid ? qi : row_hi)) * p.q_st + (size_t)head * DK;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      uint4 v = valid ? *reinterpret_cast<const uint4*>(qrow + 16 * s + 8 * h) : make_uint4(0, 0, 0, 0);
      qf[s] = *reinterpret_cast<bf16x8*>(&v);
    }
  }
  float16v acc[NDT];
#pragma unroll
  for (int i = 0; i < NDT; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
  float m_run = -1e30f, l_run = 0.f;
  constexpr int CHK = DK / 8, CHV = DV / 8;
  const size_t kst = (size_t)p.H * DK, vst = (size_t)p.H * DV;
  const bf16_t* kbase = p.k + (size_t)k0 * kst + (size_t)head * DK;
  const bf16_t* vbase = p.v + (size_t)k0 * vst + (size_t)head * DV;

  // K / V tiles go through registers: the next tile's 16-byte chunks are
  // requested before this tile's math and stored to LDS after it
  constexpr int NKC = LP_TILE * CHK / LP_THREADS, NVC = LP_TILE * CHV / LP_THREADS;
  uint4 pk[NKC], pv[NVC];
  auto fetch = [&](int kt) {
#pragma unroll
    for (int j = 0; j < NKC; ++j) {
      const int c = threadIdx.x + LP_THREADS * j, kr = c / CHK, cc = (c - kr * CHK) * 8;
      pk[j] = kt + kr < kend ? *reinterpret_cast<const uint4*>(kbase + (size_t)(kt + kr) * kst + cc)
                             : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < NVC; ++j) {
      const int c = threadIdx.x + LP_THREADS * j, kr = c / CHV, cc = (c - kr * CHV) * 8;
      pv[j] = kt + kr < kend ? *reinterpret_cast<const uint4*>(vbase + (size_t)(kt + kr) * vst + cc)
                             : make_uint4(0, 0, 0, 0);
    }
  };
  fetch(0);
  for (int kt = 0; kt < kend; kt += LP_TILE) {
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NKC; ++j) {
      const int c = threadIdx.x + LP_THREADS * j, kr = c / CHK, cc = (c - kr * CHK) * 8;
      *reinterpret_cast<uint4*>(&sm.k[kr][cc]) = pk[j];
    }
#pragma unroll
    for (int j = 0; j < NVC; ++j) {
      const int c = threadIdx.x + LP_THREADS * j, kr = c / CHV, cc = (c - kr * CHV) * 8;
      *reinterpret_cast<uint4*>(&sm.v[kr][cc]) = pv[j];
    }
    __syncthreads();
    if (kt + LP_TILE < kend) fetch(kt + LP_TILE);

    float16v st[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int j = 0; j < 16; ++j) st[t][j] = 0.f;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(&sm.k[32 * t + (lane & 31)][16 * s + 8 * h]);
        st[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[s], st[t], 0, 0, 0);
      }
    }
    bf16x8 pf[2][2];
    {
      float mx = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int key = kt + 32 * t + (j & 3) + 8 * (j >> 2) + 4 * h;
          float sv = st[t][j] * p.scale_log2;
          if (key >= kend || key > qpos) sv = -INFINITY;
          st[t][j] = sv;
          mx = fmaxf(mx, sv);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run, mx);
      const float alpha = exp2f(m_run - m_new);
      float ls = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float e = exp2f(st[t][8 * s2 + j] - m_new);
            ls += e;
            pf[t][s2][j] = (__bf16)e;
          }
      ls += __shfl_xor(ls, 32, 64);
      l_run = l_run * alpha + ls;
      m_run = m_new;
#pragma unroll
      for (int i = 0; i < NDT; ++i)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[i][j] *= alpha;
    }
    const int g = lane >> 4, li = lane & 15;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const int c0 = 32 * dt + 16 * (g & 1) + 4 * (li & 3);
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const int kb = 32 * t + 16 * s2 + 4 * h + (li >> 2);
          const lp_v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) lp_v4s*)(&sm.v[kb][c0]));
          const lp_v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) lp_v4s*)(&sm.v[kb + 8][c0]));
          short8 a8;
          a8[0] = lo[0]; a8[1] = lo[1]; a8[2] = lo[2]; a8[3] = lo[3];
          a8[4] = hi[0]; a8[5] = hi[1]; a8[6] = hi[2]; a8[7] = hi[3];
          acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<bf16x8*>(&a8),
                                                            pf[t][s2], acc[dt], 0, 0, 0);
        }
    }
  }
  if (!valid) return;
  // the sink joins the denominator only (log2 domain, like the scores)
  float f = 1.f, den = l_run;
  if (p.sink) {
    const float sk = p.sink[head] * 1.4426950408889634f;
    const float M = fmaxf(m_run, sk);
    f = exp2f(m_run - M);
    den = l_run * f + exp2f(sk - M);
  }
  const float inv = den > 0.f ? f / den : 0.f;
  bf16_t* orow = p.o + ((size_t)(q0 + qi) * p.H + head) * DV;
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int g4 = 0; g4 < 4; ++g4) {
      const int d0 = 32 * dt + 8 * g4 + 4 * h;
      uint2 w;
      w.x = pack_bf16x2(acc[dt][4 * g4] * inv, acc[dt][4 * g4 + 1] * inv);
      w.y = pack_bf16x2(acc[dt][4 * g4 + 2] * inv, acc[dt][4 * g4 + 3] * inv);
      *reinterpret_cast<uint2*>(orow + d0) = w;
    }
}

// Latent rows of every sequence, gathered from its pages in position order.
__global__ __launch_bounds__(256) void latent_gather_kernel(
    const bf16_t* __restrict__ cache, int blk, const int* __restrict__ bt, int max_blocks,
    const int* __restrict__ cu_k, int R, int Dr, bf16_t* __restrict__ cl, bf16_t* __restrict__ kr) {
  const int b = blockIdx.y;
  const int k0 = cu_k[b], L = cu_k[b + 1] - k0;
  const int W = R + Dr;
  for (int j = blockIdx.x * 4 + (threadIdx.x >> 6); j < L; j += gridDim.x * 4) {
    const bf16_t* src = cache + ((size_t)bt[(size_t)b * max_blocks + j / blk] * blk + j % blk) * W;
    for (int c = threadIdx.x & 63; c < W; c += 64) {
      if (c < R) cl[(size_t)(k0 + j) * R + c] = src[c];
      else kr[(size_t)(k0 + j) * Dr + (c - R)] = src[c];
    }
  }
}

// k[j, h, D + i] = kr[j, i]: the shared rotary key part into every head's row.
__global__ __launch_bounds__(256) void latent_kfill_kernel(bf16_t* __restrict__ k,
                                                           const bf16_t* __restrict__ kr, int H,
                                                           int DKp, int D, int Dr) {
  const size_t j = blockIdx.x;
  for (int i = threadIdx.x; i < H * Dr; i += blockDim.x) {
    const int hh = i / Dr, c = i - hh * Dr;
    k[(j * H + hh) * DKp + D + c] = kr[j * Dr + c];
  }
}

// x[t, h, off + 2i], x[t, h, off + 2i + 1] rotated by the angle of (pos[t], i).
__global__ __launch_bounds__(256) void rope_pairs_kernel(bf16_t* __restrict__ x, long st_t, long st_h,
                                                         int H, int off, int dims,
                                                         const int* __restrict__ pos,
                                                         const float* __restrict__ cs, int max_pos) {
  const size_t t = blockIdx.x;
  const int p = min(max(pos[t], 0), max_pos - 1);
  const float* csr = cs + (size_t)p * dims;
  const int half = dims / 2;
  for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
    const int hh = i / half, pr = i - hh * half;
    bf16_t* e = x + t * st_t + (size_t)hh * st_h + off + 2 * pr;
    const float c = csr[2 * pr], s = csr[2 * pr + 1];
    const float u = bf2f(e[0]), v = bf2f(e[1]);
    e[0] = f2bf(u * c - v * s);
    e[1] = f2bf(v * c + u * s);
  }
}

extern "C" int loqa_latent_gather(const void* cache, int blk, const void* bt, int max_blocks,
                                  const void* cu_k, int B, int max_len, int R, int Dr, void* cl,
                                  void* kr, hipStream_t st) {
  if (B <= 0 || max_len <= 0) return 0;
  const dim3 grid(min(1024, (max_len + 3) / 4), B);
  hipLaunchKernelGGL(latent_gather_kernel, grid, dim3(256), 0, st, (const bf16_t*)cache, blk,
                     (const int*)bt, max_blocks, (const int*)cu_k, R, Dr, (bf16_t*)cl, (bf16_t*)kr);
  return (int)hipGetLastError();
}

extern "C" int loqa_latent_kfill(void* k, const void* kr, int L, int H, int DKp, int D, int Dr,
                                 hipStream_t st) {
  if (L <= 0) return 0;
  hipLaunchKernelGGL(latent_kfill_kernel, dim3(L), dim3(256), 0, st, (bf16_t*)k, (const bf16_t*)kr, H,
                     DKp, D, Dr);
  return (int)hipGetLastError();
}

extern "C" int loqa_rope_pairs(void* x, long st_t, long st_h, int T, int H, int off, int dims,
                               const void* pos, const void* cs, int max_pos, hipStream_t st) {
  if (T <= 0 || dims <= 0) return 0;
  hipLaunchKernelGGL(rope_pairs_kernel, dim3(T), dim3(256), 0, st, (bf16_t*)x, st_t, st_h, H, off,
                     dims, (const int*)pos, (const float*)cs, max_pos);
  return (int)hipGetLastError();
}

// DK in {64, 128, 192, 256}, DV in {64, 128}: callers pad head sizes up.
extern "C" int loqa_latent_prefill(const void* q, long q_st, const void* k, const void* v, void* o,
                                   const void* cu_q, const void* cu_k, const void* pos,
                                   const void* sink, float scale, int B, int H, int max_q, int DK,
                                   int DV, hipStream_t st) {
  if (B <= 0 || H <= 0 || max_q <= 0) return 0;
  LatPrefillParams p;
  p.q = (const bf16_t*)q; p.q_st = q_st; p.k = (const bf16_t*)k; p.v = (const bf16_t*)v;
  p.o = (bf16_t*)o; p.cu_q = (const int*)cu_q; p.cu_k = (const int*)cu_k; p.pos = (const int*)pos;
  p.sink = (const float*)sink; p.scale_log2 = scale * 1.4426950408889634f; p.H = H;
  const dim3 grid((max_q + LP_WAVES * 32 - 1) / (LP_WAVES * 32), H, B);
#define GO(A, C)                                                                              \
  if (DK == A && DV == C) {                                                                   \
    hipLaunchKernelGGL((latent_prefill_kernel<A, C>), grid, dim3(LP_THREADS), 0, st, p);      \
    return (int)hipGetLastError();                                                            \
  }
  GO(64, 64) GO(128, 64) GO(192, 64) GO(256, 64) GO(64, 128) GO(128, 128) GO(192, 128) GO(256, 128)
#undef GO
  return (int)hipErrorInvalidValue;
}
