// Latent (compressed-KV) attention over a paged latent cache.
//
// Every token caches ONE row [R latent | Dr rotary key part] shared by all
// heads; queries arrive already folded into latent space (qa = W_uk^T q), so
//   score(h, t, j) = (qa[h,t] . c_j + rot(qr[t,h]) . kr_j) * scale
//   out[h, t]      = sum_j softmax_j(score)[j] * c_j      (W_uv is applied after)
// with an optional learned sink per head that only joins the denominator.
//
// latent_append_kernel: RMS-norm of the latent part, interleaved rotary on the
//   key part (pairs 2i, 2i+1 of the first `dims` entries), store at the slot.
// latent_attn_kernel: one workgroup per (query token, group of 4 heads,
//   key split). Key tiles are staged once in LDS (f32, odd row stride) for the
//   group's heads; each wave owns one head: a lane scores one key of the tile,
//   the online softmax runs across the wave, and for P.C each lane owns output
//   entries r = lane + 64 i. Prompt portions, single decode tokens and mixed
//   batches take this same kernel: a row's result depends only on its own
//   sequence's pages, in key order. Long contexts with few query rows split
//   the keys over workgroups; latent_combine_kernel merges the partials.
#include "seqmix.h"

#define LAT_THREADS 256
#define LAT_WAVES 4
#define LAT_MAXR 8      // R <= 64 * LAT_MAXR

template <typename T>
__global__ __launch_bounds__(128) void latent_append_kernel(
    const T* __restrict__ z, long ldz, const float* __restrict__ nw, float eps,
    const int* __restrict__ pos, const float* __restrict__ cs, int max_pos, T* __restrict__ cache,
    long cache_rows, const int* __restrict__ slots, int R, int Dr, int dims) {
  __shared__ float scratch[2];
  const int t = blockIdx.x;
  const int slot = slots[t];
  if (slot < 0 || slot >= cache_rows) return;      // padding row (uniform for the block)
  const T* zr = z + (size_t)t * ldz;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float v = Act<T>::ld(zr + i);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)R + eps);
  T* row = cache + (size_t)slot * (R + Dr);
  for (int i = threadIdx.x; i < R; i += blockDim.x)
    Act<T>::st(row + i, Act<T>::ld(zr + i) * inv * nw[i]);
  const int p = min(max(pos[t], 0), max_pos - 1);
  const float* csr = cs + (size_t)p * dims;          // [dims/2][2]
  for (int i = threadIdx.x; i < Dr; i += blockDim.x) {
    float o;
    if (i < dims) {
      const float c = csr[(i >> 1) * 2], s = csr[(i >> 1) * 2 + 1];
      const float u = Act<T>::ld(zr + R + (i & ~1)), v = Act<T>::ld(zr + R + (i | 1));
      o = (i & 1) ? v * c + u * s : u * c - v * s;
    } else {
      o = Act<T>::ld(zr + R + i);
    }
    Act<T>::st(row + R + i, o);
  }
}

struct LatAttnParams {
  const void* qa; long qa_st, qa_sh;     // [H, T, R] strides in elements (token, head)
  const void* qr; long qr_st, qr_sh;     // [T, H, Dr]
  const void* cache; int blk;
  const int* cu_q; const int* ctx; const int* bt; int max_blocks;
  const int* pos; const float* cs; int max_pos;
  const float* sink; float scale;
  int B, H, T, R, Dr, dims;
  void* out;                             // [H, T, R]
  int num_splits, KT;
  float* ws;                             // [splits, T, H, R + 2] when num_splits > 1
};

template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void latent_attn_kernel(LatAttnParams p) {
  extern __shared__ float lds[];
  const int W = p.R + p.Dr, Ws = W | 1, KT = p.KT;
  float* ktile = lds;                         // [KT][Ws]
  float* qs = ktile + (size_t)KT * Ws;        // [4][W]
  float* ps = qs + LAT_WAVES * W;             // [4][KT]
  const int t = blockIdx.x, split = blockIdx.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h_raw = blockIdx.y * LAT_WAVES + wave;
  const bool live = h_raw < p.H;
  const int h = live ? h_raw : p.H - 1;       // idle waves shadow a head, write nothing
  T* out = (T*)p.out + ((size_t)h * p.T + t) * p.R;
  float* wsr = p.num_splits > 1
      ? p.ws + (((size_t)split * p.T + t) * p.H + h) * (p.R + 2) : nullptr;

  int nk = 0, b = 0;
  if (t < p.cu_q[p.B]) {
    while (b + 1 < p.B && t >= p.cu_q[b + 1]) ++b;
    nk = min(p.pos[t] + 1, p.ctx[b]);
  }
  int k0 = 0, k1 = nk;
  if (p.num_splits > 1) {
    const int per = ((nk + p.num_splits - 1) / p.num_splits + KT - 1) / KT * KT;
    k0 = min(nk, split * per);
    k1 = min(nk, k0 + per);
  }
  // the wave's query in LDS, pre-scaled; its rotary part rotated here
  {
    const T* qa = (const T*)p.qa + (size_t)t * p.qa_st + (size_t)h * p.qa_sh;
    const T* qr = (const T*)p.qr + (size_t)t * p.qr_st + (size_t)h * p.qr_sh;
    const int pp = min(max(p.pos[t], 0), p.max_pos - 1);
    const float* csr = p.cs + (size_t)pp * p.dims;
    for (int i = lane; i < W; i += 64) {
      float v;
      if (i < p.R) {
        v = Act<T>::ld(qa + i);
      } else {
        const int j = i - p.R;
        if (j < p.dims) {
          const float c = csr[(j >> 1) * 2], s = csr[(j >> 1) * 2 + 1];
          const float u = Act<T>::ld(qr + (j & ~1)), w = Act<T>::ld(qr + (j | 1));
          v = (j & 1) ? w * c + u * s : u * c - w * s;
        } else {
          v = Act<T>::ld(qr + j);
        }
      }
      qs[wave * W + i] = v * p.scale;
    }
  }
  float m = -INFINITY, l = 0.f;
  float acc[LAT_MAXR];
#pragma unroll
  for (int i = 0; i < LAT_MAXR; ++i) acc[i] = 0.f;
  const T* cache = (const T*)p.cache;
  const int* bt = p.bt + (size_t)b * p.max_blocks;
  for (int kt = k0; kt < k1; kt += KT) {
    __syncthreads();                          // the previous tile is consumed
    for (int j = wave; j < KT; j += LAT_WAVES) {
      const int key = kt + j;
      float* dst = ktile + (size_t)j * Ws;
      if (key < k1) {
        const T* src = cache + ((size_t)bt[key / p.blk] * p.blk + key % p.blk) * W;
        for (int c = lane; c < W; c += 64) dst[c] = Act<T>::ld(src + c);
      } else {
        for (int c = lane; c < W; c += 64) dst[c] = 0.f;
      }
    }
    __syncthreads();
    float s = -INFINITY;
    if (lane < KT && kt + lane < k1) {
      const float* kr = ktile + (size_t)lane * Ws;
      const float* q = qs + wave * W;
      float a = 0.f;
      for (int c = 0; c < W; ++c) a += q[c] * kr[c];
      s = a;
    }
    const float mn = fmaxf(m, wave_max(s));   // finite: the tile holds >= 1 key
    const float pj = s == -INFINITY ? 0.f : expf(s - mn);
    const float corr = m == -INFINITY ? 0.f : expf(m - mn);
    l = l * corr + wave_sum(pj);
    m = mn;
    if (lane < KT) ps[wave * KT + lane] = pj;
    __syncthreads();                          // ps visible to the wave's other lanes
#pragma unroll
    for (int i = 0; i < LAT_MAXR; ++i) acc[i] *= corr;
    const int nj = min(KT, k1 - kt);
    for (int j = 0; j < nj; ++j) {
      const float pv = ps[wave * KT + j];
      const float* cr = ktile + (size_t)j * Ws;
#pragma unroll
      for (int i = 0; i < LAT_MAXR; ++i) {
        const int r = lane + 64 * i;
        if (r < p.R) acc[i] += pv * cr[r];
      }
    }
  }
  if (!live) return;
  if (wsr) {                                  // partial of this key split
    if (lane == 0) { wsr[0] = m; wsr[1] = l; }
#pragma unroll
    for (int i = 0; i < LAT_MAXR; ++i) {
      const int r = lane + 64 * i;
      if (r < p.R) wsr[2 + r] = acc[i];
    }
    return;
  }
  float M = m, den = l, f = 1.f;
  if (p.sink) {
    const float sk = p.sink[h];
    M = fmaxf(m, sk);
    f = m == -INFINITY ? 0.f : expf(m - M);
    den = l * f + expf(sk - M);
  }
  const float inv = den > 0.f ? f / den : 0.f;
#pragma unroll
  for (int i = 0; i < LAT_MAXR; ++i) {
    const int r = lane + 64 * i;
    if (r < p.R) Act<T>::st(out + r, acc[i] * inv);
  }
}

// The same computation for even R and R + Dr (every real configuration), laid
// out for throughput: the key tile sits in LDS in the activation dtype (twice
// the keys per tile for bf16), the score of a key is split over two lanes (each
// half of the wave takes half of the row, read two entries at a time, two
// independent accumulators), and for P.C a lane owns pairs of output entries.
#define LAT_MAXP 8      // R <= 128 * LAT_MAXP
#define LAT_MAXCH 10    // 16-byte chunks of a key tile per thread

template <typename T> struct Pair;
template <> struct Pair<bf16_t> {
  static __device__ __forceinline__ float2 ld(const bf16_t* p) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
    return make_float2(__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u));
  }
};
template <> struct Pair<float> {
  static __device__ __forceinline__ float2 ld(const float* p) {
    return *reinterpret_cast<const float2*>(p);
  }
};

template <typename T>
__global__ __launch_bounds__(LAT_THREADS) void latent_attn2_kernel(LatAttnParams p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int W = p.R + p.Dr, Ws = W + 2, KT = p.KT;      // KT <= 32; Ws / 2 odd or even: rows shift banks
  float* qs = lds;                                      // [4][W] f32, pre-scaled
  float* ps = qs + LAT_WAVES * W;                       // [4][KT]
  T* ktile = reinterpret_cast<T*>(ps + LAT_WAVES * KT); // [KT][Ws]
  const int t = blockIdx.x, split = blockIdx.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h_raw = blockIdx.y * LAT_WAVES + wave;
  const bool live = h_raw < p.H;
  const int h = live ? h_raw : p.H - 1;
  T* out = (T*)p.out + ((size_t)h * p.T + t) * p.R;
  float* wsr = p.num_splits > 1
      ? p.ws + (((size_t)split * p.T + t) * p.H + h) * (p.R + 2) : nullptr;
  int nk = 0, b = 0;
  if (t < p.cu_q[p.B]) {
    while (b + 1 < p.B && t >= p.cu_q[b + 1]) ++b;
    nk = min(p.pos[t] + 1, p.ctx[b]);
  }
  int k0 = 0, k1 = nk;
  if (p.num_splits > 1) {
    const int per = ((nk + p.num_splits - 1) / p.num_splits + KT - 1) / KT * KT;
    k0 = min(nk, split * per);
    k1 = min(nk, k0 + per);
  }
  {
    const T* qa = (const T*)p.qa + (size_t)t * p.qa_st + (size_t)h * p.qa_sh;
    const T* qr = (const T*)p.qr + (size_t)t * p.qr_st + (size_t)h * p.qr_sh;
    const int pp = min(max(p.pos[t], 0), p.max_pos - 1);
    const float* csr = p.cs + (size_t)pp * p.dims;
    for (int i = lane; i < W; i += 64) {
      float v;
      if (i < p.R) {
        v = Act<T>::ld(qa + i);
      } else {
        const int j = i - p.R;
        if (j < p.dims) {
          const float c = csr[(j >> 1) * 2], s = csr[(j >> 1) * 2 + 1];
          const float u = Act<T>::ld(qr + (j & ~1)), w = Act<T>::ld(qr + (j | 1));
          v = (j & 1) ? w * c + u * s : u * c - w * s;
        } else {
          v = Act<T>::ld(qr + j);
        }
      }
      qs[wave * W + i] = v * p.scale;
    }
  }
  float m = -INFINITY, l = 0.f;
  float2 acc[LAT_MAXP];
#pragma unroll
  for (int i = 0; i < LAT_MAXP; ++i) acc[i] = make_float2(0.f, 0.f);
  const T* cache = (const T*)p.cache;
  const int* bt = p.bt + (size_t)b * p.max_blocks;
  const int key_l = lane & 31, half = lane >> 5;
  // the two halves of a row, in pairs: [0, hp) and [hp, W / 2)
  const int npair = W >> 1, hp = (npair + 1) >> 1;
  const int c_lo = half ? hp : 0, c_hi = half ? npair : hp;
  // Staging. Rows that are multiples of 16 bytes move as 16-byte chunks: the
  // tile's page lookups are done once (row offsets in LDS), then every thread
  // issues its chunks back to back, and the NEXT tile's chunks are in flight in
  // registers while this tile is scored. Other row sizes go 4 bytes at a time.
  long long* rowoff = reinterpret_cast<long long*>(ktile + (size_t)KT * Ws);   // [KT]
  const int epc = 16 / (int)sizeof(T);                  // entries per chunk
  const bool vec = (W % epc) == 0;
  const int cpr = W / epc, nch = KT * cpr;
  uint4 pre[LAT_MAXCH];
  auto plan_rows = [&](int kt) {
    if (threadIdx.x < KT) {
      const int key = kt + threadIdx.x;
      rowoff[threadIdx.x] = key < k1
          ? (long long)(((size_t)bt[key / p.blk] * p.blk + key % p.blk) * W) : -1ll;
    }
  };
  auto fetch = [&]() {
#pragma unroll
    for (int j = 0; j < LAT_MAXCH; ++j) {
      const int c = threadIdx.x + LAT_THREADS * j;
      pre[j] = make_uint4(0, 0, 0, 0);
      if (c < nch) {
        const int row = c / cpr, cc = c - row * cpr;
        const long long off = rowoff[row];
        if (off >= 0) pre[j] = *reinterpret_cast<const uint4*>(cache + off + cc * epc);
      }
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int j = 0; j < LAT_MAXCH; ++j) {
      const int c = threadIdx.x + LAT_THREADS * j;
      if (c < nch) {
        const int row = c / cpr, cc = c - row * cpr;
        uint32_t* dst = reinterpret_cast<uint32_t*>(ktile + (size_t)row * Ws + cc * epc);
        dst[0] = pre[j].x; dst[1] = pre[j].y; dst[2] = pre[j].z; dst[3] = pre[j].w;
      }
    }
  };
  if (vec && k0 < k1) {
    plan_rows(k0);
    __syncthreads();
    fetch();
  }
  for (int kt = k0; kt < k1; kt += KT) {
    __syncthreads();
    if (vec) {
      commit();
      if (kt + KT < k1) plan_rows(kt + KT);
    } else {
      for (int j = wave; j < KT; j += LAT_WAVES) {
        const int key = kt + j;
        uint32_t* dst = reinterpret_cast<uint32_t*>(ktile + (size_t)j * Ws);
        if (key < k1) {
          const T* src = cache + ((size_t)bt[key / p.blk] * p.blk + key % p.blk) * W;
          if (sizeof(T) == 2) {
            const uint32_t* s32 = reinterpret_cast<const uint32_t*>(src);
            for (int c = lane; c < npair; c += 64) dst[c] = s32[c];
          } else {
            const float* sf = reinterpret_cast<const float*>(src);
            float* df = reinterpret_cast<float*>(dst);
            for (int c = lane; c < W; c += 64) df[c] = sf[c];
          }
        }
      }
    }
    __syncthreads();
    if (vec && kt + KT < k1) fetch();
    float s = -INFINITY;
    const bool has = key_l < KT && kt + key_l < k1;
    if (has) {
      const T* kr = ktile + (size_t)key_l * Ws;
      const float* q = qs + wave * W;
      float a0 = 0.f, a1 = 0.f;
#pragma unroll 8
      for (int c = c_lo; c < c_hi; ++c) {    // 8 pairs in flight: LDS latency overlaps the FMAs
        const float2 kk = Pair<T>::ld(kr + 2 * c);
        const float2 qq = *reinterpret_cast<const float2*>(q + 2 * c);
        a0 += qq.x * kk.x;
        a1 += qq.y * kk.y;
      }
      s = a0 + a1;
    }
    {
      const float o = __shfl_xor(s, 32, 64);        // the other half of the row
      if (has) s += o;
    }
    const float mn = fmaxf(m, wave_max(s));
    const float pj = (has && half == 0) ? expf(s - mn) : 0.f;
    const float corr = m == -INFINITY ? 0.f : expf(m - mn);
    l = l * corr + wave_sum(pj);
    m = mn;
    if (lane < KT) ps[wave * KT + lane] = pj;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < LAT_MAXP; ++i) { acc[i].x *= corr; acc[i].y *= corr; }
    const int nj = min(KT, k1 - kt);
#pragma unroll 4
    for (int j = 0; j < nj; ++j) {
      const float pv = ps[wave * KT + j];
      const T* cr = ktile + (size_t)j * Ws;
#pragma unroll
      for (int i = 0; i < LAT_MAXP; ++i) {
        const int r = 2 * (lane + 64 * i);
        if (r < p.R) {
          const float2 cc = Pair<T>::ld(cr + r);
          acc[i].x += pv * cc.x;
          acc[i].y += pv * cc.y;
        }
      }
    }
  }
  if (!live) return;
  if (wsr) {
    if (lane == 0) { wsr[0] = m; wsr[1] = l; }
#pragma unroll
    for (int i = 0; i < LAT_MAXP; ++i) {
      const int r = 2 * (lane + 64 * i);
      if (r < p.R) { wsr[2 + r] = acc[i].x; wsr[3 + r] = acc[i].y; }
    }
    return;
  }
  float M = m, den = l, f = 1.f;
  if (p.sink) {
    const float sk = p.sink[h];
    M = fmaxf(m, sk);
    f = m == -INFINITY ? 0.f : expf(m - M);
    den = l * f + expf(sk - M);
  }
  const float inv = den > 0.f ? f / den : 0.f;
#pragma unroll
  for (int i = 0; i < LAT_MAXP; ++i) {
    const int r = 2 * (lane + 64 * i);
    if (r < p.R) {
      Act<T>::st(out + r, acc[i].x * inv);
      Act<T>::st(out + r + 1, acc[i].y * inv);
    }
  }
}

// out[h, t] from the key splits' (m, l, acc) partials, merged in split order.
// One wave per (token, head): lane s first turns split s's (m, l) into its
// weight e^{m_s - M} (M = the largest m, or the sink), then the partial
// accumulators stream through in split order, four splits in flight.
template <typename T>
__global__ __launch_bounds__(64) void latent_combine_kernel(
    const float* __restrict__ ws, const float* __restrict__ sink, T* __restrict__ out, int Tn, int H,
    int R, int S) {
  __shared__ float fs[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const size_t stride = (size_t)Tn * H * (R + 2);
  const float* base = ws + ((size_t)t * H + h) * (R + 2);
  const float ms = lane < S ? base[lane * stride] : -INFINITY;
  const float ls = lane < S ? base[lane * stride + 1] : 0.f;
  float M = wave_max(ms);
  if (sink) M = fmaxf(M, sink[h]);
  const float f = ms == -INFINITY ? 0.f : expf(ms - M);
  fs[lane] = f;
  float den = wave_sum(ls * f);
  if (sink) den += expf(sink[h] - M);
  __syncthreads();
  float acc[LAT_MAXR];
#pragma unroll
  for (int i = 0; i < LAT_MAXR; ++i) acc[i] = 0.f;
  // unconditional (clamped) loads, so several splits' rows are in flight at once
#pragma unroll 4
  for (int s = 0; s < S; ++s) {
    const float* w = base + s * stride + 2;
    const float fw = fs[s];
    float v[LAT_MAXR];
#pragma unroll
    for (int i = 0; i < LAT_MAXR; ++i) v[i] = w[min(lane + 64 * i, R - 1)];
#pragma unroll
    for (int i = 0; i < LAT_MAXR; ++i) acc[i] += v[i] * fw;
  }
  const float inv = den > 0.f ? 1.f / den : 0.f;
#pragma unroll
  for (int i = 0; i < LAT_MAXR; ++i) {
    const int r = lane + 64 * i;
    if (r < R) Act<T>::st(out + ((size_t)h * Tn + t) * R + r, acc[i] * inv);
  }
}

extern "C" int loqa_latent_append(const void* z, int dt, long ldz, const void* nw, float eps,
                                  const void* pos, const void* cs, int max_pos, void* cache, int blk,
                                  int nblocks, const void* slots, int T, int R, int Dr, int dims,
                                  hipStream_t st) {
  if (T <= 0) return 0;
  const long rows = (long)blk * nblocks;
  if (dt == 0)
    hipLaunchKernelGGL(latent_append_kernel<bf16_t>, dim3(T), dim3(128), 0, st, (const bf16_t*)z,
                       ldz, (const float*)nw, eps, (const int*)pos, (const float*)cs, max_pos,
                       (bf16_t*)cache, rows, (const int*)slots, R, Dr, dims);
  else
    hipLaunchKernelGGL(latent_append_kernel<float>, dim3(T), dim3(128), 0, st, (const float*)z, ldz,
                       (const float*)nw, eps, (const int*)pos, (const float*)cs, max_pos,
                       (float*)cache, rows, (const int*)slots, R, Dr, dims);
  return (int)hipGetLastError();
}

extern "C" int loqa_latent_attention(
    const void* qa, long qa_st, long qa_sh, const void* qr, long qr_st, long qr_sh, int dt,
    const void* cache, int blk, int nblocks, const void* cu_q, const void* ctx, const void* bt,
    int max_blocks, const void* pos, const void* cs, int max_pos, const void* sink, float scale,
    int B, int H, int T, int R, int Dr, int dims, void* out, int num_splits, void* ws,
    hipStream_t st) {
  if (T <= 0 || H <= 0) return 0;
  if (R > 64 * LAT_MAXR || R <= 0 || B <= 0) return (int)hipErrorInvalidValue;
  if (num_splits > 1 && !ws) return (int)hipErrorInvalidValue;
  if (num_splits > 64) return (int)hipErrorInvalidValue;      // one combine lane per split
  LatAttnParams p;
  p.qa = qa; p.qa_st = qa_st; p.qa_sh = qa_sh; p.qr = qr; p.qr_st = qr_st; p.qr_sh = qr_sh;
  p.cache = cache; p.blk = blk; p.cu_q = (const int*)cu_q; p.ctx = (const int*)ctx;
  p.bt = (const int*)bt; p.max_blocks = max_blocks; p.pos = (const int*)pos;
  p.cs = (const float*)cs; p.max_pos = max_pos; p.sink = (const float*)sink; p.scale = scale;
  p.B = B; p.H = H; p.T = T; p.R = R; p.Dr = Dr; p.dims = dims; p.out = out;
  p.num_splits = num_splits < 1 ? 1 : num_splits; p.ws = (float*)ws;
  const int W = R + Dr, Ws = W | 1;
  if (W % 2 == 0 && R % 2 == 0 && R <= 128 * LAT_MAXP) {
    const size_t esz = dt == 0 ? 2 : 4;
    int KT2 = 32;
    const size_t chunks_per_row = ((size_t)W * esz + 15) / 16;
    while (KT2 > 4 && ((size_t)(LAT_WAVES * W + LAT_WAVES * KT2) * 4 + (size_t)KT2 * (W + 2) * esz +
                       KT2 * 8 > 60 * 1024 || KT2 * chunks_per_row > (size_t)LAT_THREADS * LAT_MAXCH))
      KT2 >>= 1;
    const size_t smem2 = (size_t)(LAT_WAVES * W + LAT_WAVES * KT2) * 4 + (size_t)KT2 * (W + 2) * esz +
                         KT2 * 8 + 8;
    if (smem2 <= 64 * 1024 && KT2 * chunks_per_row <= (size_t)LAT_THREADS * LAT_MAXCH) {
      p.KT = KT2;
      const dim3 grid2(T, (H + LAT_WAVES - 1) / LAT_WAVES, p.num_splits);
      if (dt == 0) hipLaunchKernelGGL(latent_attn2_kernel<bf16_t>, grid2, dim3(LAT_THREADS), smem2, st, p);
      else hipLaunchKernelGGL(latent_attn2_kernel<float>, grid2, dim3(LAT_THREADS), smem2, st, p);
      int rc2 = (int)hipGetLastError();
      if (rc2 || p.num_splits == 1) return rc2;
      if (dt == 0)
        hipLaunchKernelGGL(latent_combine_kernel<bf16_t>, dim3(T, H), dim3(64), 0, st,
                           (const float*)ws, (const float*)sink, (bf16_t*)out, T, H, R, p.num_splits);
      else
        hipLaunchKernelGGL(latent_combine_kernel<float>, dim3(T, H), dim3(64), 0, st,
                           (const float*)ws, (const float*)sink, (float*)out, T, H, R, p.num_splits);
      return (int)hipGetLastError();
    }
  }
  int KT = 64;
  while (KT > 4 && ((size_t)KT * Ws + LAT_WAVES * W + LAT_WAVES * KT) * 4 > 60 * 1024) KT >>= 1;
  p.KT = KT;
  const size_t smem = ((size_t)KT * Ws + LAT_WAVES * W + LAT_WAVES * KT) * 4;
  if (smem > 64 * 1024) return (int)hipErrorInvalidValue;
  const dim3 grid(T, (H + LAT_WAVES - 1) / LAT_WAVES, p.num_splits);
  if (dt == 0) hipLaunchKernelGGL(latent_attn_kernel<bf16_t>, grid, dim3(LAT_THREADS), smem, st, p);
  else hipLaunchKernelGGL(latent_attn_kernel<float>, grid, dim3(LAT_THREADS), smem, st, p);
  int rc = (int)hipGetLastError();
  if (rc || p.num_splits == 1) return rc;
  if (dt == 0)
    hipLaunchKernelGGL(latent_combine_kernel<bf16_t>, dim3(T, H), dim3(64), 0, st, (const float*)ws,
                       (const float*)sink, (bf16_t*)out, T, H, R, p.num_splits);
  else
    hipLaunchKernelGGL(latent_combine_kernel<float>, dim3(T, H), dim3(64), 0, st, (const float*)ws,
                       (const float*)sink, (float*)out, T, H, R, p.num_splits);
  return (int)hipGetLastError();
}
