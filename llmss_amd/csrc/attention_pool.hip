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
// caches are [pages, ceil(bs / pool), G * dim | G * vdim] fp32.
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
                                                          float* __restrict__ kp, float* __restrict__ vp,
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
    (isk ? kp : vp)[dst * n + cc] = a * inv;
  }
}

void launch_pool_update(const void* kc, const void* vc, void* kp, void* vp, const void* bt, int maxb, const void* cu,
                        const void* ctx, int B, int max_qlen, int nk, int nv, int bs, int pool, int per, int dt,
                        hipStream_t st) {
  if (B == 0 || pool <= 0) return;
  const int ny = max_qlen / pool + 1;
  if (B > 65535 * 32 || ny > 65535) throw std::runtime_error("pool_update: grid too large");
  dim3 g(B, ny);
  DISPATCH_T(dt, T, (pool_update_kernel<T><<<g, 256, 0, st>>>((const T*)kc, (const T*)vc, (float*)kp, (float*)vp,
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
                                        const T* __restrict__ vc, const float* __restrict__ kp,
                                        const float* __restrict__ vp, const int* __restrict__ bt, int maxb,
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
        tile[(size_t)kk * Dp + d] = sr < 0 ? kp[(-1 - sr) * krow + (int64_t)g * dim + d]
                                           : El<T>::ld(kc + sr * krow + (int64_t)g * dim + d);
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
              v = sr < 0 ? vp[(-1 - sr) * vrow + col] : El<T>::ld(vc + sr * vrow + col);
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
      (const float*)q, (const T*)kc, (const T*)vc, (const float*)kp, (const float*)vp, (const int*)bt, maxb,        \
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
