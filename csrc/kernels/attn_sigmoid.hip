// Attention without softmax over paged K / V: a visible key weighs
//   w = sigmoid(q . k * scale + bias[h])            (f32, not normalised over keys)
// and head h's output  sum_j w_j v_j  is multiplied by sigmoid(gate[t][h]).
// Visibility: key j <= the query's position p, and with `chunk` > 0 only keys of
// p's own chunk (j / chunk == p / chunk, chunks counted from the sequence's
// position 0 - not from where a prompt was cut). K and V pages are
// [blocks][BLK][G * D]; rows find their sequence through cu_q and their keys
// through the block table, so prompt portions, decode tokens and mixed batches
// are one launch.
//
// Two forms:
//  * sigmoid_attn_rows_kernel (any dtype, any head size): a wave per (token,
//    head), four heads per workgroup. Lanes take one key each for the scores
//    (f32 dot products, 16-byte loads of the key row), the weights of up to 64
//    keys go through LDS, then lanes take output columns and add the weighted
//    value rows in ascending key order. This is the decode form and the exact
//    f32 form.
//  * sigmoid_attn_mfma_kernel (bf16, D = 64 / 128): a workgroup per (16-row
//    query tile of one sequence, key/value head); its waves share the staged K
//    and (transposed) V tiles of 32 keys in LDS and take the query heads of the
//    group in turn. S^T = K Q^T and O^T = V^T P^T run on
//    v_mfma_f32_16x16x32_bf16; the key order inside a 32-key step is permuted
//    so that the score accumulators ARE the P^T operand (no shuffles). Scores,
//    sigmoid and the output accumulators are f32.
#include "seqmix.h"

struct SigAttnParams {
  const void* q; const void* kc; const void* vc; int blk; long cache_rows;
  const int* cu_q; const int* ctx; const int* bt; int max_blocks; const int* pos;
  const float* bias; const void* gate; int gate_ld; float scale; int chunk;
  int B, T, H, G, D; void* o;
};

__device__ __forceinline__ int chunk_start(int p, int chunk) {
  return chunk > 0 ? (p / chunk) * chunk : 0;
}

template <typename T>
__global__ __launch_bounds__(256) void sigmoid_attn_rows_kernel(SigAttnParams p) {
  extern __shared__ float lds[];                 // per wave: D floats of q, 64 weights
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x, h = blockIdx.y * 4 + wave;
  if (t >= p.cu_q[p.B] || h >= p.H) return;
  int b = 0;
  while (b + 1 < p.B && t >= p.cu_q[b + 1]) ++b;
  const int D = p.D, GD = p.G * D, g = h / (p.H / p.G);
  float* qs = lds + wave * (D + 64);
  float* ws = qs + D;
  const T* q = (const T*)p.q + (size_t)t * p.H * D + (size_t)h * D;
  for (int e = lane; e < D; e += 64) qs[e] = Act<T>::ld(q + e);
  __builtin_amdgcn_wave_barrier();
  const int pq = p.pos[t];
  const int lo = chunk_start(pq, p.chunk), hi = min(pq, p.ctx[b] - 1);
  const int* bt = p.bt + (size_t)b * p.max_blocks;
  const float hb = p.bias[h];
  const T* kc = (const T*)p.kc;
  const T* vc = (const T*)p.vc;
  constexpr int NV = 4;                          // output columns per lane (D <= 256)
  float acc[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = 0.f;
  for (int k0 = lo; k0 <= hi; k0 += 64) {
    const int j = k0 + lane;
    float w = 0.f;
    if (j <= hi) {
      const long row = (long)bt[j / p.blk] * p.blk + j % p.blk;
      const T* kr = kc + (size_t)min(max(row, 0L), p.cache_rows - 1) * GD + (size_t)g * D;
      float s = 0.f;
      if (sizeof(T) == 2 && D % 8 == 0) {        // 16-byte loads of the key row
        for (int e = 0; e < D; e += 8) {
          float f[8];
          unpack8(*reinterpret_cast<const uint4*>(kr + e), f);
#pragma unroll
          for (int i = 0; i < 8; ++i) s += qs[e + i] * f[i];
        }
      } else {
        for (int e = 0; e < D; ++e) s += qs[e] * Act<T>::ld(kr + e);
      }
      w = sigmoid_f(s * p.scale + hb);
    }
    ws[lane] = w;                                // a wave's LDS accesses stay in program order
    __builtin_amdgcn_wave_barrier();
    const int nk = min(64, hi - k0 + 1);
    for (int kk = 0; kk < nk; ++kk) {
      const int jj = k0 + kk;
      const long row = (long)bt[jj / p.blk] * p.blk + jj % p.blk;
      const T* vr = vc + (size_t)min(max(row, 0L), p.cache_rows - 1) * GD + (size_t)g * D;
      const float wk = ws[kk];
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int e = lane + 64 * i;
        if (e < D) acc[i] += wk * Act<T>::ld(vr + e);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  float gt = 1.f;
  if (p.gate) gt = sigmoid_f(Act<T>::ld((const T*)p.gate + (size_t)t * p.gate_ld + h));
  T* o = (T*)p.o + (size_t)t * p.H * D + (size_t)h * D;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int e = lane + 64 * i;
    if (e < D) Act<T>::st(o + e, acc[i] * gt);
  }
}

// ------------------------------------------------------------ matrix cores
#define SA_KT 32                                 // keys per step
#define SA_VP 8                                  // padding (elements) of a transposed V row

template <int D, int UPW>
__global__ __launch_bounds__(256) void sigmoid_attn_mfma_kernel(SigAttnParams p, int tiles_per_seq,
                                                                int heads_per_wg) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[SA_KT][D + 8];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[D][SA_KT + SA_VP];
  const int b = blockIdx.x / tiles_per_seq, tile = blockIdx.x % tiles_per_seq;
  const int q0 = p.cu_q[b], n = p.cu_q[b + 1] - q0;
  if (tile * 16 >= n) return;
  const int t0 = q0 + tile * 16, nv = min(16, n - tile * 16);
  const int g = blockIdx.y, rep = p.H / p.G;
  const int h_first = g * rep + blockIdx.z * heads_per_wg;
  const int h_end = min(g * rep + rep, h_first + heads_per_wg);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int fr = lane & 15, fq = lane >> 4;
  const int GD = p.G * D, HD = p.H * D;
  const bf16_t* kc = (const bf16_t*)p.kc;
  const bf16_t* vc = (const bf16_t*)p.vc;
  const int* bt = p.bt + (size_t)b * p.max_blocks;
  const int ctx = p.ctx[b];
  const int p0 = p.pos[t0];                      // rows of a feed hold consecutive positions
  const int pq = p0 + min(fr, nv - 1);           // this lane's query (clamped rows repeat the last)
  const int lo_q = chunk_start(pq, p.chunk);
  const int kbeg = chunk_start(p0, p.chunk), kend = min(p0 + nv - 1, ctx - 1);

  // this wave's heads: h_first + wave, + 4, ...; their query fragments and accumulators
  bf16x8 qf[UPW][D / 32];
  float4v oacc[UPW][D / 16];
  float hb[UPW];
  const bf16_t* qrow = (const bf16_t*)p.q + (size_t)(t0 + min(fr, nv - 1)) * HD + fq * 8;
#pragma unroll
  for (int u = 0; u < UPW; ++u) {
    const int h = min(h_first + wave + 4 * u, p.H - 1);
    hb[u] = p.bias[h];
#pragma unroll
    for (int ks = 0; ks < D / 32; ++ks)
      qf[u][ks] = *reinterpret_cast<const bf16x8*>(qrow + (size_t)h * D + 32 * ks);
#pragma unroll
    for (int et = 0; et < D / 16; ++et) oacc[u][et] = float4v{0.f, 0.f, 0.f, 0.f};
  }

  for (int k0 = kbeg; k0 <= kend; k0 += SA_KT) {
    __syncthreads();                             // the previous step's tiles are consumed
    // stage 32 key rows: K as it is, V transposed; 16-byte chunks of 8 entries
    for (int i = threadIdx.x; i < SA_KT * (D / 8); i += 256) {
      const int key = i / (D / 8), ch = (i % (D / 8)) * 8;
      const int j = k0 + key;
      uint4 kv = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
      if (j <= kend) {
        const long row = min(max((long)bt[j / p.blk] * p.blk + j % p.blk, 0L), p.cache_rows - 1);
        kv = *reinterpret_cast<const uint4*>(kc + (size_t)row * GD + (size_t)g * D + ch);
        vv = *reinterpret_cast<const uint4*>(vc + (size_t)row * GD + (size_t)g * D + ch);
      }
      *reinterpret_cast<uint4*>(&Ks[key][ch]) = kv;
      const bf16_t* ve = reinterpret_cast<const bf16_t*>(&vv);
#pragma unroll
      for (int e = 0; e < 8; ++e) Vt[ch + e][key] = ve[e];
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < UPW; ++u) {
      if (h_first + wave + 4 * u >= h_end) continue;        // wave-uniform
      // S^T tiles: keys k0 + 16 kt + 4 fq + i against query fr
      float4v s[2];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        s[kt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < D / 32; ++ks) {
          const bf16x8 a = *reinterpret_cast<const bf16x8*>(&Ks[16 * kt + fr][32 * ks + fq * 8]);
          s[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[u][ks], s[kt], 0, 0, 0);
        }
      }
      // weights in f32, then the P^T operand: slot kk < 4 is key 4 fq + kk,
      // slot kk >= 4 is key 16 + 4 fq + kk - 4 (the V^T operand uses the same order)
      float w[2][4];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int j = k0 + 16 * kt + 4 * fq + i;
          const bool seen = j <= pq && j >= lo_q;
          w[kt][i] = seen ? sigmoid_f(s[kt][i] * p.scale + hb[u]) : 0.f;
        }
      uint4 pu;
      pu.x = pack_bf16x2(w[0][0], w[0][1]); pu.y = pack_bf16x2(w[0][2], w[0][3]);
      pu.z = pack_bf16x2(w[1][0], w[1][1]); pu.w = pack_bf16x2(w[1][2], w[1][3]);
      const bf16x8 pw = *reinterpret_cast<const bf16x8*>(&pu);
#pragma unroll
      for (int et = 0; et < D / 16; ++et) {
        const uint2 v0 = *reinterpret_cast<const uint2*>(&Vt[16 * et + fr][4 * fq]);
        const uint2 v1 = *reinterpret_cast<const uint2*>(&Vt[16 * et + fr][16 + 4 * fq]);
        uint4 va = make_uint4(v0.x, v0.y, v1.x, v1.y);
        oacc[u][et] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *reinterpret_cast<const bf16x8*>(&va), pw, oacc[u][et], 0, 0, 0);
      }
    }
  }
  // oacc[u][et][i]: output column 16 et + 4 fq + i of query row fr
  if (fr >= nv) return;
  const int t = t0 + fr;
#pragma unroll
  for (int u = 0; u < UPW; ++u) {
    const int h = h_first + wave + 4 * u;
    if (h >= h_end) continue;
    float gt = 1.f;
    if (p.gate) gt = sigmoid_f(bf2f(((const bf16_t*)p.gate)[(size_t)t * p.gate_ld + h]));
    bf16_t* o = (bf16_t*)p.o + (size_t)t * HD + (size_t)h * D;
#pragma unroll
    for (int et = 0; et < D / 16; ++et) {
      uint2 pk;
      pk.x = pack_bf16x2(oacc[u][et][0] * gt, oacc[u][et][1] * gt);
      pk.y = pack_bf16x2(oacc[u][et][2] * gt, oacc[u][et][3] * gt);
      *reinterpret_cast<uint2*>(o + 16 * et + 4 * fq) = pk;
    }
  }
}

extern "C" int loqa_sigmoid_attention(
    const void* q, int dt, const void* kc, const void* vc, int blk, int nblocks, const void* cu_q,
    const void* ctx, const void* bt, int max_blocks, const void* pos, const void* bias,
    const void* gate, int gate_ld, float scale, int chunk, int B, int T, int H, int G, int D,
    int max_q, int mfma, void* o, hipStream_t st) {
  if (T <= 0) return 0;
  if (B <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || D > 256 || blk <= 0 || nblocks <= 0 ||
      chunk < 0)
    return (int)hipErrorInvalidValue;
  SigAttnParams p;
  p.q = q; p.kc = kc; p.vc = vc; p.blk = blk; p.cache_rows = (long)blk * nblocks;
  p.cu_q = (const int*)cu_q; p.ctx = (const int*)ctx; p.bt = (const int*)bt;
  p.max_blocks = max_blocks; p.pos = (const int*)pos; p.bias = (const float*)bias; p.gate = gate;
  p.gate_ld = gate_ld; p.scale = scale; p.chunk = chunk; p.B = B; p.T = T; p.H = H; p.G = G;
  p.D = D; p.o = o;
  if (mfma && dt == 0 && (D == 64 || D == 128) && max_q > 0) {
    const int rep = H / G;
    const int zs = (rep + 15) / 16;                        // at most 16 heads per workgroup
    const int hpw = (rep + zs - 1) / zs;
    const int upw = (hpw + 3) / 4;
    const int tiles = (max_q + 15) / 16;
    const dim3 grid(B * tiles, G, zs);
#define GO(DD, UU)                                                                              \
  hipLaunchKernelGGL((sigmoid_attn_mfma_kernel<DD, UU>), grid, dim3(256), 0, st, p, tiles, hpw)
    if (D == 64) { if (upw <= 1) GO(64, 1); else if (upw == 2) GO(64, 2); else GO(64, 4); }
    else { if (upw <= 1) GO(128, 1); else if (upw == 2) GO(128, 2); else GO(128, 4); }
#undef GO
    return (int)hipGetLastError();
  }
  const dim3 grid(T, (H + 3) / 4);
  const size_t lds = 4 * (size_t)(D + 64) * sizeof(float);
  if (dt == 0)
    hipLaunchKernelGGL(sigmoid_attn_rows_kernel<bf16_t>, grid, dim3(256), lds, st, p);
  else
    hipLaunchKernelGGL(sigmoid_attn_rows_kernel<float>, grid, dim3(256), lds, st, p);
  return (int)hipGetLastError();
}
