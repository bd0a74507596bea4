// Sigmoid-weighted attention over a sliding window of a paged key / value cache plus mean-pooled blocks behind it.
//
//   rope_pairs_cache:  q, k with the neighbouring pairs (2i, 2i + 1) of their first `rdims` numbers per head turned
//                      by the step's angles cs [T, rdims / 2, 2] = (cos, sin); q out in fp32, k / v into the pages
//   pool_update:       for every block of `pool` positions whose last position the step wrote, the mean key and mean
//                      value of the block's cached rows, in fp32, into the pooled caches
//   pool_window_attn:  out[t, h] = sum over visible keys of sigmoid(q . k * scale + pb[h]) * v; the row at position i
//                      sees the positions j with 0 <= i - j < window (all j <= i when window = 0) and the pooled rows
//                      of the blocks b with b * pool + pool - 1 <= i - window. No softmax, nothing is normalised.
//
// Pooled row of block b of a sequence: page = block_table[(b * pool) / bs], rank (b * pool % bs) / pool inside it
// (two blocks that start in the same page are at least `pool` positions apart, so their ranks differ); the pooled
// caches are [pages, ceil(bs / pool), G * dim | G * vdim] in the pages' storage type (the means are formed in fp32
// and rounded once, as the keys and values themselves are when they are cached).
#include "anytype.h"
#include "seqrows.h"

template <typename T>
__global__ __launch_bounds__(256) void rope_pairs_cache_kernel(const T* __restrict__ proj, int64_t ldp, int off_q,
                                                               int off_k, int off_v, const float* __restrict__ cs,
                                                               int rdims, float* __restrict__ qout,
                                                               T* __restrict__ kc, T* __restrict__ vc,
                                                               const int64_t* __restrict__ slots, int H, int G,
                                                               int dim, int vdim) {
  const int t = blockIdx.x;
  const T* row = proj + (int64_t)t * ldp;
  const float* ang = cs ? cs + (int64_t)t * rdims : nullptr;  // rdims / 2 pairs of (cos, sin)
  const int64_t slot = slots[t];
  const int nq = H * dim, nk = G * dim, nv = G * vdim;
  for (int e = threadIdx.x; e < nq + nk; e += blockDim.x) {
    const bool isq = e < nq;
    const int i = isq ? e : e - nq;
    const int d = i % dim;
    const T* src = row + (isq ? off_q : off_k) + i;
    float v = El<T>::ld(src);
    if (d < rdims) {
      const float c = ang[(d >> 1) * 2], s = ang[(d >> 1) * 2 + 1];
      const float o = El<T>::ld((d & 1) ? src - 1 : src + 1);
      v = (d & 1) ? fmaf(v, c, o * s) : fmaf(v, c, -o * s);
    }
    if (isq) qout[(int64_t)t * nq + i] = v;
    else if (slot >= 0) El<T>::st(kc + slot * nk + i, v);
  }
  if (slot >= 0)
    for (int i = threadIdx.x; i < nv; i += blockDim.x) vc[slot * nv + i] = row[off_v + i];
}

void launch_rope_pairs_cache(const void* proj, int64_t ldp, int off_q, int off_k, int off_v, const void* cs, int rdims,
                             void* qout, void* kc, void* vc, const void* slots, int T_, int H, int G, int dim, int vdim,
                             int dt, hipStream_t st) {
  if (T_ == 0) return;
  if (rdims < 0 || rdims % 2 || rdims > dim) throw std::runtime_error("rope_pairs_cache: bad rotated dimensions");
  DISPATCH_T(dt, T, (rope_pairs_cache_kernel<T><<<T_, 256, 0, st>>>(
      (const T*)proj, ldp, off_q, off_k, off_v, rdims ? (const float*)cs : nullptr, rdims, (float*)qout, (T*)kc, (T*)vc,
      (const int64_t*)slots, H, G, dim, vdim)));
  HIP_CHECK_LAUNCH();
}

__device__ __forceinline__ int64_t pool_row(const int* btr, int blk, int pool, int bs, int per) {
  const int p = blk * pool;
  return (int64_t)btr[p / bs] * per + (p % bs) / pool;
}

// grid (B, blocks a portion can complete): workgroup (b, n) takes block p0 / pool + n of sequence b
template <typename T>
__global__ __launch_bounds__(256) void pool_update_kernel(const T* __restrict__ kc, const T* __restrict__ vc,
                                                          T* __restrict__ kp, T* __restrict__ vp,
                                                          const int* __restrict__ bt, int maxb,
                                                          const int* __restrict__ cu, const int* __restrict__ ctx,
                                                          int nk, int nv, int bs, int pool, int per) {
  const int b = blockIdx.x;
  const int qlen = cu[b + 1] - cu[b], L = ctx[b];
  if (qlen <= 0 || L <= 0) return;
  const int p0 = L - qlen;
  const int blk = p0 / pool + blockIdx.y;
  if (blk >= L / pool) return;  // p0 <= blk * pool + pool - 1 < L: the step wrote the block's last position
  const int* btr = bt + (int64_t)b * maxb;
  const int64_t dst = pool_row(btr, blk, pool, bs, per);
  const float inv = 1.0f / (float)pool;
  for (int c = threadIdx.x; c < nk + nv; c += blockDim.x) {
    const bool isk = c < nk;
    const int cc = isk ? c : c - nk;
    const int n = isk ? nk : nv;
    const T* src = isk ? kc : vc;
    float a = 0.f;
    for (int i = 0; i < pool; ++i) {
      const int j = blk * pool + i;
      a += El<T>::ld(src + ((int64_t)btr[j / bs] * bs + j % bs) * n + cc);
    }
    El<T>::st((isk ? kp : vp) + dst * n + cc, a * inv);
  }
}

void launch_pool_update(const void* kc, const void* vc, void* kp, void* vp, const void* bt, int maxb, const void* cu,
                        const void* ctx, int B, int max_qlen, int nk, int nv, int bs, int pool, int per, int dt,
                        hipStream_t st) {
  if (B == 0 || pool <= 0) return;
  const int ny = max_qlen / pool + 1;
  if (B > 65535 * 32 || ny > 65535) throw std::runtime_error("pool_update: grid too large");
  dim3 g(B, ny);
  DISPATCH_T(dt, T, (pool_update_kernel<T><<<g, 256, 0, st>>>((const T*)kc, (const T*)vc, (T*)kp, (T*)vp,
                                                              (const int*)bt, maxb, (const int*)cu, (const int*)ctx,
                                                              nk, nv, bs, pool, per)));
  HIP_CHECK_LAUNCH();
}

// Vector kernel (any shape, either storage type). Workgroup: one row t, one key group g, up to NWT of its query
// heads, one chunk of value columns. The row's visible keys are numbered u = 0 .. nb + nwin - 1: first the nb pooled
// blocks, then the window's positions. KB of them are staged in LDS as fp32 at a time; wave w scores them for head w
// with lanes over keys and leaves the weights in LDS; then the waves split the value columns between them, each
// accumulating its columns for all heads of the workgroup, so a value row is read once per workgroup.
template <typename T, int NWT, int NR2>
__global__ void pool_window_attn_kernel(const float* __restrict__ q, const T* __restrict__ kc,
                                        const T* __restrict__ vc, const T* __restrict__ kp,
                                        const T* __restrict__ vp, const int* __restrict__ bt, int maxb,
                                        const int* __restrict__ cu, const int* __restrict__ ctx,
                                        const float* __restrict__ pb, void* __restrict__ out, int out_f32, int B, int H,
                                        int G, int dim, int vdim, int bs, float scale, int window, int pool, int per,
                                        int KB, int Dp, int hchunks, int RVchunk) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  float* tile = reinterpret_cast<float*>(smem);   // [KB][Dp] keys
  float* qs = tile + (size_t)KB * Dp;              // [NWT][dim] queries times scale
  float* ps = qs + (size_t)NWT * dim;              // [NWT][KB] weights of the staged keys
  int64_t* srow = reinterpret_cast<int64_t*>((reinterpret_cast<uintptr_t>(ps + (size_t)NWT * KB) + 7) & ~(uintptr_t)7);
  const int t = blockIdx.x, wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int rep = H / G;
  const int g = blockIdx.y / hchunks;
  const int hl0 = (blockIdx.y % hchunks) * NWT;
  const bool live = hl0 + wv < rep;
  const int h = g * rep + hl0 + wv;
  const int v0 = blockIdx.z * RVchunk;
  const int RV = min(RVchunk, vdim - v0);
  const int cs = NR2 * 64;
  const int c0 = wv * cs + lane;
  const RowSeq r = row_seq(cu, ctx, B, t);
  float acc[NWT][NR2];
#pragma unroll
  for (int hh = 0; hh < NWT; ++hh)
#pragma unroll
    for (int i = 0; i < NR2; ++i) acc[hh][i] = 0.f;
  if (r.pos >= 0) {
    float* qw = qs + (size_t)wv * dim;
    float* p = ps + (size_t)wv * KB;
    float bias = 0.f;
    if (live) {
      const float* qsrc = q + ((int64_t)t * H + h) * dim;
      for (int d = lane; d < dim; d += 64) qw[d] = qsrc[d] * scale;
      bias = pb[h];
    }
    const int jlo = window > 0 ? max(0, r.pos - window + 1) : 0;
    const int nb = (pool > 0 && window > 0 && r.pos - window + 1 >= pool) ? (r.pos - window + 1) / pool : 0;
    const int total = nb + (r.pos - jlo + 1);
    const int* btr = bt + (int64_t)r.b * maxb;
    const int64_t krow = (int64_t)G * dim, vrow = (int64_t)G * vdim;
    for (int u0 = 0; u0 < total; u0 += KB) {
      const int nk = min(KB, total - u0);
      __syncthreads();
      for (int kk = threadIdx.x; kk < nk; kk += blockDim.x) {
        const int u = u0 + kk;
        if (u < nb) {
          srow[kk] = -1 - pool_row(btr, u, pool, bs, per);  // negative: a row of the pooled caches
        } else {
          const int j = jlo + (u - nb);
          srow[kk] = (int64_t)btr[j / bs] * bs + j % bs;
        }
      }
      __syncthreads();
      for (int e = threadIdx.x; e < nk * dim; e += blockDim.x) {
        const int kk = e / dim, d = e - kk * dim;
        const int64_t sr = srow[kk];
        tile[(size_t)kk * Dp + d] = El<T>::ld(sr < 0 ? kp + (-1 - sr) * krow + (int64_t)g * dim + d
                                                     : kc + sr * krow + (int64_t)g * dim + d);
      }
      __syncthreads();
      if (live) {
        for (int kk = lane; kk < nk; kk += 64) {
          const float* row = tile + (size_t)kk * Dp;
          float a0 = 0.f, a1 = 0.f;
          int d = 0;
          for (; d + 1 < dim; d += 2) {
            a0 = fmaf(qw[d], row[d], a0);
            a1 = fmaf(qw[d + 1], row[d + 1], a1);
          }
          if (d < dim) a0 = fmaf(qw[d], row[d], a0);
          p[kk] = 1.0f / (1.0f + expf(-((a0 + a1) + bias)));
        }
      } else {
        for (int kk = lane; kk < nk; kk += 64) p[kk] = 0.f;
      }
      __syncthreads();
      constexpr int VK = 8;
      for (int k0 = 0; k0 < nk; k0 += VK) {
        float vv[VK][NR2];
#pragma unroll
        for (int j = 0; j < VK; ++j) {
          const int64_t sr = srow[min(k0 + j, nk - 1)];
#pragma unroll
          for (int i = 0; i < NR2; ++i) {
            const int c = c0 + 64 * i;
            float v = 0.f;
            if (c < RV) {
              const int64_t col = (int64_t)g * vdim + v0 + c;
              v = El<T>::ld(sr < 0 ? vp + (-1 - sr) * vrow + col : vc + sr * vrow + col);
            }
            vv[j][i] = v;
          }
        }
#pragma unroll
        for (int j = 0; j < VK; ++j) {
          if (k0 + j < nk) {
#pragma unroll
            for (int hh = 0; hh < NWT; ++hh) {
              const float pj = ps[hh * KB + k0 + j];
#pragma unroll
              for (int i = 0; i < NR2; ++i) acc[hh][i] = fmaf(pj, vv[j][i], acc[hh][i]);
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int hh = 0; hh < NWT; ++hh) {
    if (hl0 + hh < rep) {
      const int64_t o = ((int64_t)t * H + g * rep + hl0 + hh) * vdim + v0;
#pragma unroll
      for (int i = 0; i < NR2; ++i) {
        const int c = c0 + 64 * i;
        if (c < RV) {
          if (out_f32) ((float*)out)[o + c] = acc[hh][i];
          else ((bf16_t*)out)[o + c] = f2bf(acc[hh][i]);
        }
      }
    }
  }
}

template <typename T>
static void pool_window_attn_t(const void* q, const void* kc, const void* vc, const void* kp, const void* vp,
                               const void* bt, int maxb, const void* cu, const void* ctx, const void* pb, void* out,
                               int out_f32, int T_, int B, int H, int G, int dim, int vdim, int bs, float scale,
                               int window, int pool, int per, hipStream_t st) {
  const int rep = H / G;
  const int NW = rep >= 8 ? 8 : (rep > 2 ? 4 : rep);
  const int hchunks = (rep + NW - 1) / NW;
  const int Dp = dim | 1;  // an odd row stride: lanes score neighbouring keys without bank conflicts
  int KB = 64;
  auto bytes = [&](int kb) { return ((size_t)kb * Dp + (size_t)NW * (dim + kb)) * 4 + (size_t)kb * 8 + 16; };
  while (KB > 8 && bytes(KB) > 60 * 1024) KB >>= 1;
  if (bytes(KB) > 60 * 1024) throw std::runtime_error("pool_window_attn: head dimension too large for LDS");
  int nr2 = 1;
  while (nr2 < 4 && NW * nr2 * 2 <= 16 && NW * nr2 * 64 < vdim) nr2 <<= 1;
  const int RVchunk = std::min(vdim, NW * nr2 * 64);
  const int zch = (vdim + RVchunk - 1) / RVchunk;
  if (G * hchunks > 65535 || zch > 65535) throw std::runtime_error("pool_window_attn: too many heads");
  dim3 g(T_, G * hchunks, zch);
#define LAUNCH_PW(NW_, NR_)                                                                                         \
  pool_window_attn_kernel<T, NW_, NR_><<<g, NW_ * 64, bytes(KB), st>>>(                                             \
      (const float*)q, (const T*)kc, (const T*)vc, (const T*)kp, (const T*)vp, (const int*)bt, maxb,                \
      (const int*)cu, (const int*)ctx, (const float*)pb, out, out_f32, B, H, G, dim, vdim, bs, scale, window, pool, \
      per, KB, Dp, hchunks, RVchunk)
#define LAUNCH_PW_NR(NW_)                \
  do {                                   \
    if (nr2 == 1) LAUNCH_PW(NW_, 1);     \
    else if (nr2 == 2) LAUNCH_PW(NW_, 2); \
    else LAUNCH_PW(NW_, 4);              \
  } while (0)
  if (NW == 1) LAUNCH_PW_NR(1);
  else if (NW == 2) LAUNCH_PW_NR(2);
  else if (NW == 4) LAUNCH_PW_NR(4);
  else {
    if (nr2 == 1) LAUNCH_PW(8, 1);
    else LAUNCH_PW(8, 2);
  }
#undef LAUNCH_PW_NR
#undef LAUNCH_PW
}

// dt: storage type of the paged caches; out_f32: the output rows are fp32 (else bf16)
void launch_pool_window_attn(const void* q, const void* kc, const void* vc, const void* kp, const void* vp,
                             const void* bt, int maxb, const void* cu, const void* ctx, const void* pb, void* out,
                             int out_f32, int T_, int B, int H, int G, int dim, int vdim, int bs, float scale,
                             int window, int pool, int per, int dt, hipStream_t st) {
  if (T_ == 0 || B == 0) return;
  if (G < 1 || H % G) throw std::runtime_error("pool_window_attn: heads must be a multiple of the key/value heads");
  if (window < 0 || pool < 0 || (pool > 0 && (window == 0 || per < (bs + pool - 1) / pool)))
    throw std::runtime_error("pool_window_attn: bad window / pool");
  DISPATCH_T(dt, T, (pool_window_attn_t<T>(q, kc, vc, kp, vp, bt, maxb, cu, ctx, pb, out, out_f32, T_, B, H, G, dim,
                                           vdim, bs, scale, window, pool, per, st)));
  HIP_CHECK_LAUNCH();
}

// The same attention on the matrix cores, for bf16 pages with key size 32, 64 or 128 and a value size that is a
// multiple of 8: prompt portions and single rows alike. One workgroup serves one key/value group, GE of its query
// heads and 64 * NS / GE query rows of one sequence: its 64 * NS slots enumerate (row, head) pairs, slot s -> row
// s / GE, head s % GE, so a key tile is staged in LDS once for the whole head group. The rows' visible keys are
// numbered u = 0 .. nb + ntok - 1 for the workgroup: first the pooled blocks the LAST row sees, then the positions
// from the FIRST row's window start to the last row; a tile is 64 of them, whatever they are, and the mask tells each
// row which of them it sees. Products are the swapped ones,
//   S^T[key][slot] = K . Q^T   (A = K rows from LDS, B = Q^T fragments in registers)
//   O^T[c][slot]  += V^T . P^T (A = V^T by transposing LDS reads, B = P^T straight from the S^T accumulators)
// with the fp32 queries and the fp32 weights entering as value + remainder (two bf16 numbers, two matrix
// instructions), so scores and weighted sums are those of 32-bit operands. There is no softmax: a weight is
// sigmoid(score + bias) and the sums over keys are plain sums - so the keys can be split over workgroups at will
// (nsplit > 1: each writes its partial sums, fp32, and pool_attn_reduce adds them in order), which is what gives a
// step of single rows enough workgroups. The next tile's 16-byte chunks are fetched into registers while this one is
// computed from LDS.
template <int DK, int NVT, int NS>
__global__ __launch_bounds__(256, 2) void pool_window_attn_mfma_kernel(
    const float* __restrict__ q, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
    const bf16_t* __restrict__ kp, const bf16_t* __restrict__ vp, const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, const float* __restrict__ pb,
    void* __restrict__ out, int out_f32, float* __restrict__ part, int nsplit, int64_t part_stride, int H, int G,
    int GE, int vdim, int bs, float scale, int window, int pool, int per, int nvch) {
  constexpr int BKV = 64;
  constexpr int LDK = DK + 16;
  constexpr int VCH = NVT * 16;
  constexpr int LDV = VCH + 16;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[BKV * LDK];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[BKV * LDV];
  const int rep = H / G;
  const int rows_per_wg = 64 * NS / GE;
  const int rb = blockIdx.x / nsplit, sp = blockIdx.x % nsplit, by = blockIdx.y, b = blockIdx.z;
  const int vch = by % nvch, hy = by / nvch;
  const int kvh = hy / (rep / GE);
  const int h0 = kvh * rep + (hy % (rep / GE)) * GE;
  const int t0 = cu_q[b], qlen = cu_q[b + 1] - t0;
  const int r0 = rb * rows_per_wg;
  if (r0 >= qlen || ctx_lens[b] <= 0) return;
  const int p0 = ctx_lens[b] - qlen;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int li = lane & 15, g = lane >> 4;
  const int v0 = vch * VCH;
  const int64_t vrow = (int64_t)G * vdim;
  const int voff = kvh * vdim + v0;
  constexpr float kLog2e = 1.4426950408889634f;

  int row[NS], hd[NS], qpos[NS], grp_first[NS], grp_last[NS];
  bool valid[NS], grp_rows[NS], grp_full[NS];
  float bias2[NS];
  s16x8 qf[NS][DK / 32], ql[NS][DK / 32];
  f32x4 o[NS][NVT];
  bool wave_rows = false;
#pragma unroll
  for (int n = 0; n < NS; ++n) {
    const int gs = (w * NS + n) * 16, slot = gs + li;
    row[n] = r0 + slot / GE;
    hd[n] = h0 + slot % GE;
    valid[n] = slot < rows_per_wg * GE && row[n] < qlen;
    qpos[n] = p0 + (valid[n] ? row[n] : 0);
    grp_rows[n] = r0 + gs / GE < qlen && gs < rows_per_wg * GE;
    grp_full[n] = r0 + (gs + 15) / GE < qlen && gs + 15 < rows_per_wg * GE;  // every slot of the group holds a row
    grp_first[n] = p0 + min(qlen - 1, r0 + gs / GE);  // (the same in every lane)
    grp_last[n] = p0 + min(qlen - 1, r0 + (gs + 15) / GE);
    wave_rows = wave_rows || grp_rows[n];
    bias2[n] = pb[valid[n] ? hd[n] : h0] * kLog2e;
    const float* qp = q + ((int64_t)(t0 + (valid[n] ? row[n] : 0)) * H + (valid[n] ? hd[n] : h0)) * DK + 8 * g;
#pragma unroll
    for (int ks = 0; ks < DK / 32; ++ks)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x = qp[32 * ks + j];
        const bf16_t hi = f2bf(x);
        qf[n][ks][j] = (short)hi;
        ql[n][ks][j] = (short)f2bf(x - bf2f(hi));
      }
#pragma unroll
    for (int i = 0; i < NVT; ++i) o[n][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const float scale2 = scale * kLog2e;
  const int pf = p0 + r0, pl = p0 + min(qlen, r0 + rows_per_wg) - 1;  // positions of the first and last row
  const int jlo = window > 0 ? max(0, pf - window + 1) : 0;
  const int nb = (pool > 0 && window > 0 && pl - window + 1 >= pool) ? (pl - window + 1) / pool : 0;
  const int total = nb + (pl - jlo + 1);
  const int tiles = (total + BKV - 1) / BKV, tps = (tiles + nsplit - 1) / nsplit;
  const int u_begin = sp * tps * BKV, u_end = min(total, (sp + 1) * tps * BKV);
  const int* bt = block_tables + (int64_t)b * max_blocks;
  constexpr int CHK = DK / 8, CHV = VCH / 8;
  static_assert((BKV * CHK) % 256 == 0 && (BKV * CHV) % 256 == 0, "whole 16-byte chunks per thread");
  constexpr int NCK = BKV * CHK / 256, NCV = BKV * CHV / 256;
  u16x8 kr[NCK], vr[NCV];
  // the cache row of visible key u: a pooled row (negative) or a page row
  auto src_row = [&](int u) -> int64_t {
    if (u < nb) return -1 - pool_row(bt, u, pool, bs, per);
    const int j = jlo + (u - nb);
    return (int64_t)bt[j / bs] * bs + j % bs;
  };
  auto load_tile = [&](int u0) {
#pragma unroll
    for (int j = 0; j < NCK; ++j) {
      const int c = threadIdx.x + 256 * j;
      const int64_t sl = src_row(min(u0 + c / CHK, total - 1));
      const bf16_t* base = sl < 0 ? kp + ((-1 - sl) * G + kvh) * DK : kc + (sl * G + kvh) * DK;
      kr[j] = *reinterpret_cast<const u16x8*>(base + (c % CHK) * 8);
    }
#pragma unroll
    for (int j = 0; j < NCV; ++j) {
      const int c = threadIdx.x + 256 * j;
      const int ch = c % CHV;
      const int64_t sl = src_row(min(u0 + c / CHV, total - 1));
      const bf16_t* base = sl < 0 ? vp + (-1 - sl) * vrow + voff : vc + sl * vrow + voff;
      u16x8 val = {0, 0, 0, 0, 0, 0, 0, 0};
      if (v0 + ch * 8 < vdim) val = *reinterpret_cast<const u16x8*>(base + ch * 8);
      vr[j] = val;
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int j = 0; j < NCK; ++j) {
      const int c = threadIdx.x + 256 * j;
      *reinterpret_cast<u16x8*>(&Ks[(c / CHK) * LDK + (c % CHK) * 8]) = kr[j];
    }
#pragma unroll
    for (int j = 0; j < NCV; ++j) {
      const int c = threadIdx.x + 256 * j;
      *reinterpret_cast<u16x8*>(&Vs[(c / CHV) * LDV + (c % CHV) * 8]) = vr[j];
    }
  };
  auto compute_tile = [&](int u0) {
    // what the tile is to each slot group: 0 nothing of it is seen (weights zero), 1 some of it (masked), 2 all of it
    // by every row of the group (no mask). A tile of pooled rows and positions both is masked.
    int see[NS];
    bool any = false;
    const int ul = u0 + BKV - 1;
#pragma unroll
    for (int n = 0; n < NS; ++n) {
      see[n] = grp_rows[n] ? 1 : 0;
      if (ul < nb) {  // pooled rows only
        if (u0 * pool + pool - 1 > grp_last[n] - window) see[n] = 0;
        else if (grp_full[n] && ul < u_end && ul * pool + pool - 1 <= grp_first[n] - window) see[n] = see[n] ? 2 : 0;
      } else if (u0 >= nb) {  // positions only
        const int j0 = jlo + (u0 - nb), j1 = j0 + BKV - 1;
        if (j0 > grp_last[n] || (window > 0 && grp_first[n] - j1 >= window)) see[n] = 0;
        else if (grp_full[n] && ul < u_end && j1 <= grp_first[n] && (window == 0 || grp_last[n] - j0 < window))
          see[n] = see[n] ? 2 : 0;
      }
      any = any || see[n] != 0;
    }
    if (!any) return;
    f32x4 s[NS][4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
      for (int n = 0; n < NS; ++n) s[n][kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < DK / 32; ++ks) {
        const s16x8 kf = *reinterpret_cast<const s16x8*>(&Ks[(kt * 16 + li) * LDK + 32 * ks + 8 * g]);
#pragma unroll
        for (int n = 0; n < NS; ++n) {
          s[n][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[n][ks], s[n][kt], 0, 0, 0);
          s[n][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, ql[n][ks], s[n][kt], 0, 0, 0);
        }
      }
    }
    // S^T accumulators: lane (li, g) holds slot li's scores for the keys u0 + 16 kt + 4 g + i
    s16x8 pf_[NS][2], pl_[NS][2];
    auto weights = [&](int n, auto whole_c) {
      constexpr bool WHOLE = decltype(whole_c)::value;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = __builtin_amdgcn_exp2f(-fmaf(s[n][kt][i], scale2, bias2[n]));
          float p = __builtin_amdgcn_rcpf(1.0f + e);
          if constexpr (!WHOLE) {
            const int u = u0 + kt * 16 + 4 * g + i;
            bool vis = u < u_end;
            if (u < nb) {
              vis = vis && u * pool + pool - 1 <= qpos[n] - window;
            } else {
              const int j = jlo + (u - nb);
              vis = vis && j <= qpos[n] && (window == 0 || qpos[n] - j < window);
            }
            p = vis ? p : 0.f;
          }
          const bf16_t hi = f2bf(p);
          pf_[n][kt >> 1][(kt & 1) * 4 + i] = (short)hi;
          pl_[n][kt >> 1][(kt & 1) * 4 + i] = (short)f2bf(p - bf2f(hi));
        }
    };
#pragma unroll
    for (int n = 0; n < NS; ++n) {
      if (see[n] == 0) {
        const s16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        pf_[n][0] = pf_[n][1] = pl_[n][0] = pl_[n][1] = z;
      } else if (see[n] == 2) {
        weights(n, std::true_type{});
      } else {
        weights(n, std::false_type{});
      }
    }
    const int tq = li >> 2, tp = li & 3;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
      for (int dt = 0; dt < NVT; ++dt) {
        const bf16_t* a0 = &Vs[(32 * ks + 4 * g + tq) * LDV + dt * 16 + 4 * tp];
        const bf16_t* a1 = a0 + 16 * LDV;
        const s16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(a0));
        const s16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(a1));
        const s16x8 vf = {x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
#pragma unroll
        for (int n = 0; n < NS; ++n) {
          o[n][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf_[n][ks], o[n][dt], 0, 0, 0);
          o[n][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl_[n][ks], o[n][dt], 0, 0, 0);
        }
      }
    }
  };
  if (u_end > u_begin) load_tile(u_begin);
  for (int u0 = u_begin; u0 < u_end; u0 += BKV) {
    __syncthreads();  // every wave is done reading the previous tile
    store_tile();
    __syncthreads();
    if (u0 + BKV < u_end) load_tile(u0 + BKV);
    if (wave_rows) compute_tile(u0);
  }
#pragma unroll
  for (int n = 0; n < NS; ++n) {
    if (!valid[n]) continue;
    const int64_t at = ((int64_t)(t0 + row[n]) * H + hd[n]) * vdim + v0 + 4 * g;
#pragma unroll
    for (int dt = 0; dt < NVT; ++dt) {
      if (v0 + dt * 16 + 4 * g >= vdim) continue;
      const f32x4 v = o[n][dt];
      if (nsplit > 1) {
        *reinterpret_cast<f32x4*>(part + (int64_t)sp * part_stride + at + dt * 16) = v;
      } else if (out_f32) {
        *reinterpret_cast<f32x4*>((float*)out + at + dt * 16) = v;
      } else {
        *reinterpret_cast<u16x4*>((bf16_t*)out + at + dt * 16) = u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
      }
    }
  }
}

// out[e] = sum over the splits, in order, of part[sp, e]; n a multiple of 4
__global__ __launch_bounds__(256) void pool_attn_reduce_kernel(const float* __restrict__ part, int nsplit,
                                                               int64_t stride, void* __restrict__ out, int out_f32,
                                                               int64_t n) {
  const int64_t e = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (e >= n) return;
  f32x4 a = *reinterpret_cast<const f32x4*>(part + e);
  for (int sp = 1; sp < nsplit; ++sp) a += *reinterpret_cast<const f32x4*>(part + (int64_t)sp * stride + e);
  if (out_f32) *reinterpret_cast<f32x4*>((float*)out + e) = a;
  else *reinterpret_cast<u16x4*>((bf16_t*)out + e) = u16x4{f2bf(a[0]), f2bf(a[1]), f2bf(a[2]), f2bf(a[3])};
}

bool pool_attn_mfma_ok(int dim, int vdim) { return (dim == 32 || dim == 64 || dim == 128) && vdim % 8 == 0; }

// B sequences whose portions have at most max_qlen rows; rows [row0, row0 + rows) of `out` are theirs. nsplit > 1:
// `part` holds nsplit * rows * H * vdim floats.
void launch_pool_window_attn_mfma(const void* q, const void* kc, const void* vc, const void* kp, const void* vp,
                                  const void* bt, int maxb, const void* cu, const void* ctx, const void* pb, void* out,
                                  int out_f32, void* part, int nsplit, int64_t row0, int64_t rows, int B, int max_qlen,
                                  int H, int G, int dim, int vdim, int bs, float scale, int window, int pool, int per,
                                  hipStream_t st) {
  if (B == 0 || max_qlen <= 0 || rows <= 0) return;
  if (G < 1 || H % G) throw std::runtime_error("pool_window_attn: heads must be a multiple of the key/value heads");
  if (!pool_attn_mfma_ok(dim, vdim)) throw std::runtime_error("pool_window_attn: shape not built for the matrix cores");
  if (window < 0 || pool < 0 || (pool > 0 && (window == 0 || per < (bs + pool - 1) / pool)) || nsplit < 1)
    throw std::runtime_error("pool_window_attn: bad window / pool / split");
  const int rep = H / G;
  int GE = 1;
  for (int ge = std::min(rep, 64); ge >= 1; --ge)
    if (rep % ge == 0) {
      GE = ge;
      break;
    }
  const int nvt = vdim > 128 ? 16 : (vdim > 64 ? 8 : 4);
  const int nvch = (vdim + nvt * 16 - 1) / (nvt * 16);
  const bool two_fit = nvt <= 4 || (nvt == 8 && dim != 128);
  const int ns = (two_fit && max_qlen > 64 / GE) ? 2 : 1;
  const int rows_per_wg = 64 * ns / GE;
  const int64_t gy = (int64_t)G * (rep / GE) * nvch;
  const int64_t gx = (int64_t)((max_qlen + rows_per_wg - 1) / rows_per_wg) * nsplit;
  if (gy > 65535 || B > 65535 || gx > 0x7fffffff) throw std::runtime_error("pool_window_attn: grid too large");
  dim3 grid((unsigned)gx, (unsigned)gy, B);
  const int64_t stride = rows * H * vdim;
  // partial sums are addressed by the step's row numbers: shift the base so that row0 lands on the buffer's start
  float* pbase = part ? (float*)part - row0 * H * vdim : nullptr;
#define LAUNCH_PWM(DK_, NVT_, NS_)                                                                                  \
  pool_window_attn_mfma_kernel<DK_, NVT_, NS_><<<grid, 256, 0, st>>>(                                               \
      (const float*)q, (const bf16_t*)kc, (const bf16_t*)vc, (const bf16_t*)kp, (const bf16_t*)vp, (const int*)bt,  \
      maxb, (const int*)cu, (const int*)ctx, (const float*)pb, out, out_f32, pbase, nsplit, stride, H, G, GE, vdim, \
      bs, scale, window, pool, per, nvch)
#define LAUNCH_PWM_D(DK_)                     \
  do {                                        \
    if (nvt == 16) LAUNCH_PWM(DK_, 16, 1);    \
    else if (nvt == 8) {                      \
      if (ns == 2) LAUNCH_PWM(DK_, 8, 2);     \
      else LAUNCH_PWM(DK_, 8, 1);             \
    } else {                                  \
      if (ns == 2) LAUNCH_PWM(DK_, 4, 2);     \
      else LAUNCH_PWM(DK_, 4, 1);             \
    }                                         \
  } while (0)
  if (dim == 32) LAUNCH_PWM_D(32);
  else if (dim == 64) LAUNCH_PWM_D(64);
  else {
    if (nvt == 16) LAUNCH_PWM(128, 16, 1);
    else if (nvt == 8) LAUNCH_PWM(128, 8, 1);
    else if (ns == 2) LAUNCH_PWM(128, 4, 2);
    else LAUNCH_PWM(128, 4, 1);
  }
#undef LAUNCH_PWM_D
#undef LAUNCH_PWM
  HIP_CHECK_LAUNCH();
  if (nsplit > 1) {
    const int64_t n = stride;
    char* obase = (char*)out + row0 * H * vdim * (out_f32 ? 4 : 2);
    pool_attn_reduce_kernel<<<(unsigned)((n / 4 + 255) / 256), 256, 0, st>>>((const float*)part, nsplit, stride, obase,
                                                                            out_f32, n);
    HIP_CHECK_LAUNCH();
  }
}
