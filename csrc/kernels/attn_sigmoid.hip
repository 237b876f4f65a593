// Attention without softmax over paged K / V: a visible key weighs
//   w = sigmoid(q . k * scale + bias[h])            (f32, not normalised over keys)
// and head h's output  sum_j w_j v_j  is multiplied by sigmoid(gate[t][h]).
// Visibility: key j <= the query's position p, and with `chunk` > 0 only keys of
// p's own chunk (j / chunk == p / chunk, chunks counted from the sequence's
// position 0 - not from where a prompt was cut). K pages are
// [blocks][BLK][G * D]; V pages are stored transposed, [blocks][G * D][BLK]: the
// value product sums over keys, so both the decode form (a lane owns output
// columns and reads a column's keys of a page as one 16- or 32-byte run) and
// the matrix-core form (whose V operand wants a column's consecutive keys) read
// them without a transposition of their own. Rows find their sequence through
// cu_q and their keys through the block table, so prompt portions, decode
// tokens and mixed batches are one launch.
//
// Three forms:
//  * sigmoid_attn_rows_kernel (any dtype, any head size): a wave per (token,
//    head), four heads per workgroup. Lanes take one key each for the scores
//    (f32 dot products), the weights of up to 64 keys go through LDS, then
//    lanes take output columns and add the weighted value rows in ascending
//    key order. The form for head sizes the others do not take.
//  * sigmoid_attn_keys_kernel (any dtype, D a power of two): the decode form
//    and the exact f32 form; see there.
//  * sigmoid_attn_mfma_kernel (bf16, D = 64 / 128): a workgroup per (64 query
//    rows of one sequence, key/value head); each wave owns a 16-row tile and
//    carries the group's query heads in registers, all waves share the staged
//    K and (transposed) V tiles of 64 keys in LDS (the next tile's rows are in
//    flight in registers), and a wave skips the steps that lie before its
//    rows' chunk or after them. S^T = K Q^T and O^T = V^T P^T run on
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
  constexpr int NV = 8;                          // output columns per lane (D <= 512)
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
      const long page = min(max((long)bt[jj / p.blk], 0L), p.cache_rows / p.blk - 1);
      const T* vr = vc + ((size_t)page * GD + (size_t)g * D) * p.blk + jj % p.blk;
      const float wk = ws[kk];
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int e = lane + 64 * i;
        if (e < D) acc[i] += wk * Act<T>::ld(vr + (size_t)e * p.blk);
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


// ------------------------------------------------------------ few rows, many keys
template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> {
  static __device__ __forceinline__ void ld(const bf16_t* p, float* f) {
    unpack8(*reinterpret_cast<const uint4*>(p), f);
  }
};
template <> struct Vec8<float> {
  static __device__ __forceinline__ void ld(const float* p, float* f) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
  }
};

// The decode form (D a power of two, 8 .. 512; pages of 8 .. 64 keys that
// divide 64): a workgroup per (token, key/value head) serves up to RH query
// heads of the group, so every K row and V column run is read once for all of
// them. The visible keys go in 64-key windows aligned to multiples of 64 (so a
// window is whole pages), dealt to the workgroup's waves in turn. Scores: a
// lane takes one key and all RH heads (16-byte loads of the key row against the
// queries in LDS). Values: a lane owns output columns (D / 64 of them; for
// D < 64 the lanes split into 64 / D groups that take pages in turn) and adds,
// page by page, its column's keys weighted from LDS. The partial sums meet
// through shuffles (groups) and LDS (waves) in a fixed order. Which wave, lane
// and step a key lands on depends only on its position in the sequence.
template <typename T, int RH, int DC, int BK>
__global__ __launch_bounds__(RH <= 4 ? 1024 : 512) void sigmoid_attn_keys_kernel(
    SigAttnParams p, int heads_per_wg) {
  extern __shared__ float lds[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, NW = blockDim.x >> 6;
  const int t = blockIdx.x, g = blockIdx.y;
  if (t >= p.cu_q[p.B]) return;
  int b = 0;
  while (b + 1 < p.B && t >= p.cu_q[b + 1]) ++b;
  const int D = DC ? DC : p.D;                   // head sizes 64 and 128 unroll fully
  const int GD = p.G * D, HD = p.H * D, rep = p.H / p.G;
  const int blk = BK ? BK : p.blk;               // 16-key pages unroll fully
  const int h_first = g * rep + blockIdx.z * heads_per_wg;
  const int nh = min(heads_per_wg, g * rep + rep - h_first);
  float* qs = lds;                               // [RH][D]
  float* red = qs + RH * D;                      // [NW][RH][D]
  float* wts = red + NW * RH * D + wave * RH * 64;           // per wave [RH][64] weights
  const T* q = (const T*)p.q + (size_t)t * HD + (size_t)h_first * D;
  for (int i = threadIdx.x; i < nh * D; i += blockDim.x) qs[i] = Act<T>::ld(q + i);
  __syncthreads();
  const int pq = p.pos[t];
  const int lo = chunk_start(pq, p.chunk), hi = min(pq, p.ctx[b] - 1);
  const int* bt = p.bt + (size_t)b * p.max_blocks;
  const long npages = p.cache_rows / blk;
  const T* kc = (const T*)p.kc;
  const T* vc = (const T*)p.vc;
  // value phase: column(s) of this lane, and which pages of a window its group takes
  const int groups = D >= 64 ? 1 : 64 / D, grp = D >= 64 ? 0 : lane / D;
  const int e0 = D >= 64 ? lane : lane % D, cpl = D >= 64 ? D / 64 : 1;
  float hb[RH];
#pragma unroll
  for (int r = 0; r < RH; ++r) hb[r] = p.bias[min(h_first + r, p.H - 1)];
  float acc[RH][8];
#pragma unroll
  for (int r = 0; r < RH; ++r)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[r][i] = 0.f;
  for (int win = lo / 64 + wave; hi >= lo && win <= hi / 64; win += NW) {
    const int k0 = 64 * win, j = k0 + lane;
    const bool live = j >= lo && j <= hi;
    float sc[RH];
#pragma unroll
    for (int r = 0; r < RH; ++r) sc[r] = 0.f;
    if (live) {
      const long row = min(max((long)bt[j / blk] * blk + j % blk, 0L), p.cache_rows - 1);
      const T* kr = kc + (size_t)row * GD + (size_t)g * D;
#pragma unroll(DC ? DC / 8 : 4)
      for (int e = 0; e < D; e += 8) {
        float f[8];
        Vec8<T>::ld(kr + e, f);
#pragma unroll
        for (int r = 0; r < RH; ++r)
#pragma unroll
          for (int i = 0; i < 8; ++i) sc[r] += qs[r * D + e + i] * f[i];
      }
    }
#pragma unroll
    for (int r = 0; r < RH; ++r)
      wts[r * 64 + lane] = live && r < nh ? sigmoid_for<T>(sc[r] * p.scale + hb[r]) : 0.f;
    __builtin_amdgcn_wave_barrier();
    // every page of the window, visible or not (keys out of sight weigh zero; a
    // page past the last key repeats the last one): no branch, so the page
    // lookups and then all loads are in flight together
    const int npw = 64 / blk;                    // pages per window
    long pgid[8];
#pragma unroll
    for (int a = 0; a < 8; ++a) {
      const int pg = grp + a * groups;
      pgid[a] = pg < npw ? min(max((long)bt[min(k0 + pg * blk, hi) / blk], 0L), npages - 1) : 0;
    }
#pragma unroll
    for (int a = 0; a < 8; ++a) {
      const int pg = grp + a * groups;
      if (pg >= npw) break;
      const T* vp = vc + ((size_t)pgid[a] * GD + (size_t)g * D + e0) * blk;
#pragma unroll
      for (int ci = 0; ci < 8; ++ci) {
        if (ci >= cpl) break;
#pragma unroll(BK ? BK / 8 : 1)
        for (int c8 = 0; c8 < blk; c8 += 8) {
          float f[8];
          Vec8<T>::ld(vp + (size_t)ci * 64 * blk + c8, f);
#pragma unroll
          for (int r = 0; r < RH; ++r) {
            const float* w = wts + r * 64 + pg * blk + c8;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[r][ci] += w[i] * f[i];
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  for (int off = D; off < 64; off <<= 1)         // D < 64: the page groups of a column
#pragma unroll
    for (int r = 0; r < RH; ++r) acc[r][0] += __shfl_xor(acc[r][0], off, 64);
  if (grp == 0)
#pragma unroll
    for (int r = 0; r < RH; ++r)
#pragma unroll
      for (int ci = 0; ci < 8; ++ci)
        if (ci < cpl) red[(wave * RH + r) * D + e0 + 64 * ci] = acc[r][ci];
  __syncthreads();
  for (int i = threadIdx.x; i < nh * D; i += blockDim.x) {
    const int r = i / D, e = i % D, h = h_first + r;
    float v = 0.f;
    for (int w = 0; w < NW; ++w) v += red[(w * RH + r) * D + e];       // waves in order
    float gt = 1.f;
    if (p.gate) gt = sigmoid_f(Act<T>::ld((const T*)p.gate + (size_t)t * p.gate_ld + h));
    Act<T>::st((T*)p.o + (size_t)t * HD + (size_t)h * D + e, v * gt);
  }
}

// ------------------------------------------------------------ matrix cores
#define SA_KT 64                                 // keys staged per step (two 32-key MFMA sub-steps)
#define SA_VP 8                                  // padding (elements) of a V^T row: 16-byte aligned rows
#define SA_ROWS 64                               // query rows per workgroup: one 16-row tile per wave
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#define SA_MAXPG 2048                            // page ids of a workgroup's key range kept in LDS

// NH = query heads a wave carries (all of them against its own 16-row tile).
template <int D, int NH>
__global__ __launch_bounds__(256) void sigmoid_attn_mfma_kernel(SigAttnParams p, int blocks_per_seq,
                                                                int heads_per_wg, int per_rb) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[SA_KT][D + 8];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[D][SA_KT + SA_VP];
  __shared__ int pgs[SA_MAXPG];
  constexpr int NCH = SA_KT * (D / 8) / 256;     // 16-byte chunks a thread stages per tile
  // workgroups start in the order of their ids: the row blocks go last first (a
  // block late in its chunk has the most keys), with a block's (key/value head,
  // head split) workgroups side by side, so the long workgroups start early and
  // the short ones fill in behind them
  const int rb = gridDim.x / per_rb - 1 - blockIdx.x / per_rb, sub_id = blockIdx.x % per_rb;
  const int b = rb / blocks_per_seq, blk_i = rb % blocks_per_seq;
  const int q0 = p.cu_q[b], n = p.cu_q[b + 1] - q0;
  if (blk_i * SA_ROWS >= n) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int fr = lane & 15, fq = lane >> 4;
  const int r0 = blk_i * SA_ROWS;                               // first row of the block in the feed
  const int nb = min(SA_ROWS, n - r0);                          // rows of the block
  const int nv = max(0, min(16, nb - 16 * wave));               // rows of this wave's tile
  const int g = sub_id % p.G, rep = p.H / p.G;
  const int h_first = g * rep + (sub_id / p.G) * heads_per_wg;
  const int h_end = min(g * rep + rep, h_first + heads_per_wg);
  const int GD = p.G * D, HD = p.H * D;
  const bf16_t* kc = (const bf16_t*)p.kc;
  const bf16_t* vc = (const bf16_t*)p.vc;
  const int* bt = p.bt + (size_t)b * p.max_blocks;
  const long npages = p.cache_rows / p.blk;
  const int p0 = p.pos[q0 + r0];                 // rows of a feed hold consecutive positions
  const int kbeg = chunk_start(p0, p.chunk), kend = min(p0 + nb - 1, p.ctx[b] - 1);
  // this wave's tile: positions pw0 .. pw1; this lane's query (clamped rows repeat the last)
  const int pw0 = p0 + 16 * wave, pw1 = pw0 + max(nv, 1) - 1;
  const int wlo = chunk_start(pw0, p.chunk);
  const int pq = pw0 + min(fr, max(nv, 1) - 1);
  const int lo_q = chunk_start(pq, p.chunk);

  bf16x8 qf[NH][D / 32];
  float4v oacc[NH][D / 16];
  float hb[NH];
  const int trow = q0 + r0 + min(16 * wave + min(fr, max(nv, 1) - 1), nb - 1);
  const bf16_t* qrow = (const bf16_t*)p.q + (size_t)trow * HD + fq * 8;
#pragma unroll
  for (int u = 0; u < NH; ++u) {
    const int h = min(h_first + u, p.H - 1);
    hb[u] = p.bias[h];
#pragma unroll
    for (int ks = 0; ks < D / 32; ++ks)
      qf[u][ks] = *reinterpret_cast<const bf16x8*>(qrow + (size_t)h * D + 32 * ks);
#pragma unroll
    for (int et = 0; et < D / 16; ++et) oacc[u][et] = float4v{0.f, 0.f, 0.f, 0.f};
  }

  // staging: thread -> NCH 16-byte chunks of K (key, 8 entries) and of V^T
  // (column, 8 keys of a page); the next tile's chunks are requested before this
  // tile's MFMAs and land in LDS after them. Steps are aligned to multiples of
  // 64 keys, so a step is whole pages. (Keys past the last one repeat it or read
  // the rest of its page: their weights are zero. No branch, so the block-table
  // lookups and then all loads are in flight together.)
  // The pages of the workgroup's key range are looked up once, into LDS, so a
  // step's loads do not wait for a block-table read (ranges of more than
  // SA_MAXPG pages read the table directly).
  const int bsh = __ffs(p.blk) - 1, bmask = p.blk - 1;       // pages hold a power of two of keys
  const int kb0 = (kbeg / SA_KT) * SA_KT, pg0 = kb0 >> bsh;
  const int npg = (kend >> bsh) - pg0 + 1;
  const bool in_lds = npg <= SA_MAXPG;
  if (in_lds)
    for (int i = threadIdx.x; i < npg; i += 256)
      pgs[i] = (int)min(max((long)bt[pg0 + i], 0L), npages - 1);
  __syncthreads();
  const int kpp = p.blk / 8;                     // 8-key runs per page
  u32x4 kreg[NCH], vreg[NCH];                    // (plain vectors: these stay in registers)
#define SA_PAGE(J) (in_lds ? (long)pgs[((J) >> bsh) - pg0]                                      \
                           : min(max((long)bt[(J) >> bsh], 0L), npages - 1))
#define SA_FETCH(K0)                                                                            \
  {                                                                                             \
    long kof_[NCH], vof_[NCH];                                                                  \
    _Pragma("unroll") for (int c = 0; c < NCH; ++c) {                                           \
      const int i_ = threadIdx.x + 256 * c;                                                     \
      const int j_ = min((K0) + i_ / (D / 8), kend);                                            \
      kof_[c] = ((SA_PAGE(j_) << bsh) + (j_ & bmask)) * GD + (long)g * D + (i_ % (D / 8)) * 8;  \
      const int e_ = i_ / 8, run_ = i_ % 8;                                                     \
      const long pg_ = SA_PAGE(min((K0) + run_ * 8, kend));                                     \
      vof_[c] = ((pg_ * GD + (long)g * D + e_) << bsh) + (run_ % kpp) * 8;                      \
    }                                                                                           \
    _Pragma("unroll") for (int c = 0; c < NCH; ++c) {                                           \
      kreg[c] = *reinterpret_cast<const u32x4*>(kc + kof_[c]);                                  \
      vreg[c] = *reinterpret_cast<const u32x4*>(vc + vof_[c]);                                  \
    }                                                                                           \
  }
  SA_FETCH(kb0)
  for (int k0 = kb0; k0 <= kend; k0 += SA_KT) {
    __syncthreads();                             // the previous step's tiles are consumed
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int i = threadIdx.x + 256 * c;
      *reinterpret_cast<u32x4*>(&Ks[i / (D / 8)][(i % (D / 8)) * 8]) = kreg[c];
      *reinterpret_cast<u32x4*>(&Vt[i / 8][(i % 8) * 8]) = vreg[c];
    }
    __syncthreads();
    if (k0 + SA_KT <= kend) { SA_FETCH(k0 + SA_KT) }
    if (nv == 0) continue;
#pragma unroll
    for (int sub = 0; sub < SA_KT / 32; ++sub) {
      const int ks0 = k0 + 32 * sub;             // first key of this 32-key sub-step
      // nothing of it is visible to the wave's rows: after them or before their chunk
      if (ks0 > pw1 || ks0 + 32 <= wlo) continue;
      // S^T tiles: keys ks0 + 16 kt + 4 fq + i against query fr; a K fragment
      // read from LDS serves every head the wave carries
      float4v sc[NH][2];
#pragma unroll
      for (int u = 0; u < NH; ++u) sc[u][0] = sc[u][1] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int ks = 0; ks < D / 32; ++ks) {
          const bf16x8 a = *reinterpret_cast<const bf16x8*>(
              &Ks[32 * sub + 16 * kt + fr][32 * ks + fq * 8]);
#pragma unroll
          for (int u = 0; u < NH; ++u)
            sc[u][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[u][ks], sc[u][kt], 0, 0, 0);
        }
      // weights in f32, then the P^T operands: slot kk < 4 is key 4 fq + kk,
      // slot kk >= 4 is key 16 + 4 fq + kk - 4 (the V^T operand uses the same order)
      bf16x8 pw[NH];
#pragma unroll
      for (int u = 0; u < NH; ++u) {
        float w[2][4];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int j = ks0 + 16 * kt + 4 * fq + i;
            const bool seen = j <= pq && j >= lo_q;
            w[kt][i] = seen ? sigmoid_fast(sc[u][kt][i] * p.scale + hb[u]) : 0.f;
          }
        const u32x4 pu = {pack_bf16x2(w[0][0], w[0][1]), pack_bf16x2(w[0][2], w[0][3]),
                          pack_bf16x2(w[1][0], w[1][1]), pack_bf16x2(w[1][2], w[1][3])};
        pw[u] = __builtin_bit_cast(bf16x8, pu);
      }
#pragma unroll
      for (int et = 0; et < D / 16; ++et) {
        const u32x2 v0 = *reinterpret_cast<const u32x2*>(&Vt[16 * et + fr][32 * sub + 4 * fq]);
        const u32x2 v1 = *reinterpret_cast<const u32x2*>(&Vt[16 * et + fr][32 * sub + 16 + 4 * fq]);
        const u32x4 va = {v0.x, v0.y, v1.x, v1.y};
#pragma unroll
        for (int u = 0; u < NH; ++u)
          oacc[u][et] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              __builtin_bit_cast(bf16x8, va), pw[u], oacc[u][et], 0, 0, 0);
      }
    }
  }
#undef SA_FETCH
#undef SA_PAGE
  // oacc[u][et][i]: output column 16 et + 4 fq + i of query row fr
  if (fr >= nv) return;
  const int t = q0 + r0 + 16 * wave + fr;
#pragma unroll
  for (int u = 0; u < NH; ++u) {
    const int h = h_first + u;
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
  if (B <= 0 || H <= 0 || G <= 0 || H % G || D <= 0 || D > 512 || blk <= 0 || nblocks <= 0 ||
      chunk < 0)
    return (int)hipErrorInvalidValue;
  SigAttnParams p;
  p.q = q; p.kc = kc; p.vc = vc; p.blk = blk; p.cache_rows = (long)blk * nblocks;
  p.cu_q = (const int*)cu_q; p.ctx = (const int*)ctx; p.bt = (const int*)bt;
  p.max_blocks = max_blocks; p.pos = (const int*)pos; p.bias = (const float*)bias; p.gate = gate;
  p.gate_ld = gate_ld; p.scale = scale; p.chunk = chunk; p.B = B; p.T = T; p.H = H; p.G = G;
  p.D = D; p.o = o;
  const bool pages_ok = 64 % blk == 0 && blk % 8 == 0;      // a 64-key window is whole pages of 8-key runs
  if (mfma && dt == 0 && (D == 64 || D == 128) && max_q > 0 && pages_ok) {
    const int rep = H / G;
    const int hmax = D == 64 ? 8 : 4;                      // heads a wave can carry in registers
    const int blocks = (max_q + SA_ROWS - 1) / SA_ROWS;
    int zs = (rep + hmax - 1) / hmax;
    int hpw = (rep + zs - 1) / zs;
    // a short batch fills the chip through more, narrower workgroups: the query
    // heads of a group spread over workgroups (K / V tiles come from L2 again)
    while (hpw > 1 && (long)B * blocks * G * zs < 512) {
      hpw = (hpw + 1) / 2;
      zs = (rep + hpw - 1) / hpw;
    }
    const dim3 grid(B * blocks * G * zs, 1, 1);
#define GO(DD, NN)                                                                              \
  hipLaunchKernelGGL((sigmoid_attn_mfma_kernel<DD, NN>), grid, dim3(256), 0, st, p, blocks, hpw, G * zs)
    if (D == 64) {
      if (hpw <= 1) GO(64, 1); else if (hpw == 2) GO(64, 2); else if (hpw <= 4) GO(64, 4);
      else GO(64, 8);
    } else {
      if (hpw <= 1) GO(128, 1); else if (hpw == 2) GO(128, 2); else GO(128, 4);
    }
#undef GO
    return (int)hipGetLastError();
  }
  if (D >= 8 && (D & (D - 1)) == 0 && pages_ok) {
    const int rep = H / G;
    int rh = rep < 8 ? rep : 8;
    if (rh * D > 2048) rh = 2048 / D;
    // waves = key windows in flight; LDS holds (1 + waves) RH D floats
    const int nw = rh * D <= 512 && rh <= 4 ? 16 : rh * D <= 1024 ? 8 : 4;
    const int zs = (rep + rh - 1) / rh;
    const int hpw = (rep + zs - 1) / zs;
    const int RH = hpw <= 1 ? 1 : hpw == 2 ? 2 : hpw <= 4 ? 4 : 8;
    const dim3 grid(T, G, zs);
    const size_t lds = ((size_t)(1 + nw) * RH * D + nw * (RH + 1) * 64) * sizeof(float);
#define GO(TT, RR, DD, BB)                                                                      \
  hipLaunchKernelGGL((sigmoid_attn_keys_kernel<TT, RR, DD, BB>), grid, dim3(64 * nw), lds, st, p, hpw)
#define BY_D(TT, RR)                                                                            \
  do {                                                                                          \
    if (D == 64 && blk == 16) GO(TT, RR, 64, 16);                                               \
    else if (D == 128 && blk == 16) GO(TT, RR, 128, 16);                                        \
    else GO(TT, RR, 0, 0);                                                                      \
  } while (0)
#define BY_RH(TT)                                                                               \
  do {                                                                                          \
    if (RH == 1) BY_D(TT, 1); else if (RH == 2) BY_D(TT, 2); else if (RH == 4) BY_D(TT, 4);     \
    else BY_D(TT, 8);                                                                           \
  } while (0)
    if (dt == 0) BY_RH(bf16_t); else BY_RH(float);
#undef BY_RH
#undef BY_D
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
