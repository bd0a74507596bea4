// Softmax attention with a sink, a soft cap, partial rotary positions and head mixing, over a paged key/value cache
// whose key and value widths may differ.
//
//   s_h(i, j) = cap * tanh(scale * q_h(i) . k_g(j) / cap)          (cap 0: no cap)          g = h / (H / G)
//   p_h(i, j) = exp(s_h(i, j)) / (1 + sum_j' exp(s_h(i, j')))      j' over the causal keys: a sink of score 0
//   w_h(i, j) = sum_h' talk[h, h'] p_h'(i, j)                      (talk absent: w = p)
//   out_h(i)  = sum_j w_h(i, j) v_g(j)
//
// Mixing weights across heads commutes with the weighted sum over keys: out_h(i) = sum_h' talk[h, h'] O_h'(i)[g]
// with O_h'(i)[c] = sum_j p_h'(i, j) v_c(j) the weighted sum of head h''s weights over the values of group c. So
// the attention kernel runs an ordinary one-pass online softmax per head and accumulates against the whole value
// row of a key (all G groups side by side, as the cache stores it), and a small second kernel mixes. Without a
// talk matrix only the head's own group is accumulated.
//
// The sink enters the online softmax as its initial state: running maximum 0, running denominator 1, no value.
//
// Options that other designs use: `sink` 0 makes it the ordinary softmax (no unit in the denominator); `chunk` > 0
// lets position i see only the keys from floor(i / chunk) * chunk on (blocks counted from position 0 of the
// sequence); `vshare` > 1 lets that many neighbouring key heads read one value head (the value cache then holds
// G / vshare heads) - differential attention caches the two maps of a key head as two key heads over one value head.
//
// One kernel serves portions of prompts, continued portions and single decoded tokens: a row finds its sequence and
// position through cu / ctx_lens and reads every key, those of its own step too, from the paged cache.
// Scores, softmax and sums are fp32; the cache is read in the model's storage type.
#include "anytype.h"
#include "seqrows.h"

// q (+ bias), k (+ bias) rotated on the first `rot` dimensions of each head (i paired with i + rot / 2) by the
// angle table cs [npos, rot / 2, 2] = (cos, sin) already scaled; v (+ bias) copied. q -> qout fp32 [T, H * dim];
// k, v -> the paged caches at slots[t] (slot < 0: not cached).
template <typename T>
__global__ __launch_bounds__(256) void rope_bias_cache_kernel(const T* __restrict__ proj, int64_t ldp, int off_q,
                                                              int off_k, int off_v, const T* __restrict__ bias,
                                                              const int64_t* __restrict__ positions,
                                                              const float* __restrict__ cs, int npos, int rot,
                                                              float* __restrict__ qout, T* __restrict__ kc,
                                                              T* __restrict__ vc, const int64_t* __restrict__ slots,
                                                              int H, int G, int dim, int vdim) {
  const int t = blockIdx.x;
  int64_t p = positions[t];
  p = p < 0 ? 0 : (p >= npos ? npos - 1 : p);
  const int half = rot >> 1;
  const float* tab = cs + p * (int64_t)half * 2;
  const T* row = proj + (int64_t)t * ldp;
  const int64_t slot = slots[t];
  const int nq = H * dim, nk = G * dim, nv = G * vdim;
  // bias layout: q | k | v
  for (int e = threadIdx.x; e < nq + nk; e += blockDim.x) {
    const bool isk = e >= nq;
    const int idx = isk ? e - nq : e;
    const int d = idx % dim;
    const int base = (isk ? off_k : off_q) + idx - d;
    const T* b = bias ? bias + (isk ? nq : 0) + idx - d : nullptr;
    float val = El<T>::ld(row + base + d) + (b ? El<T>::ld(b + d) : 0.f);
    if (d < rot) {
      const int i = d < half ? d : d - half;
      const int od = d < half ? d + half : d - half;
      const float other = El<T>::ld(row + base + od) + (b ? El<T>::ld(b + od) : 0.f);
      const float c = tab[2 * i], s = tab[2 * i + 1];
      val = d < half ? val * c - other * s : val * c + other * s;
    }
    if (!isk) qout[(int64_t)t * nq + idx] = val;
    else if (slot >= 0) El<T>::st(kc + slot * (int64_t)nk + idx, val);
  }
  if (slot >= 0)
    for (int e = threadIdx.x; e < nv; e += blockDim.x)
      El<T>::st(vc + slot * (int64_t)nv + e,
                El<T>::ld(row + off_v + e) + (bias ? El<T>::ld(bias + nq + nk + e) : 0.f));
}

void launch_rope_bias_cache(const void* proj, int64_t ldp, int off_q, int off_k, int off_v, const void* bias,
                            const void* positions, const void* cs, int npos, int rot, void* qout, void* kc, void* vc,
                            const void* slots, int T_, int H, int G, int dim, int vdim, int dt, hipStream_t st) {
  if (T_ == 0) return;
  if (rot < 0 || rot > dim || (rot & 1)) throw std::runtime_error("rope_bias_cache: rotary dims must be even, <= dim");
  DISPATCH_T(dt, T, (rope_bias_cache_kernel<T><<<T_, 256, 0, st>>>(
      (const T*)proj, ldp, off_q, off_k, off_v, (const T*)bias, (const int64_t*)positions, (const float*)cs, npos, rot,
      (float*)qout, (T*)kc, (T*)vc, (const int64_t*)slots, H, G, dim, vdim)));
  HIP_CHECK_LAUNCH();
}

// Vector kernel (any shape, either storage type; single decoded rows and what the matrix-core kernel below does not
// take). Workgroup: one row t, one key group g, up to NWT of its query heads. Grid (T, G * chunks of heads, chunks of
// value columns). A block of KB keys of group g is staged in LDS once; wave w scores it for head w with lanes over
// keys, updates that head's online softmax and leaves the weights in LDS. Then the waves split the VALUE COLUMNS
// between them: wave w accumulates its slice of columns for ALL heads of the workgroup, so a value row is read once
// per workgroup, straight from the cache, 8 or 16 keys' loads in flight at a time. Value columns v0 .. v0 + RV - 1 of
// the key's whole value row [G * vdim] (all = 1) or of group g's part (all = 0). out [T, H, RVtot] fp32.
template <typename T, int NWT, int NR2, bool WORDS>
__global__ void sink_attn_kernel(const float* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc,
                                 const int* __restrict__ bt, int maxb, const int* __restrict__ cu,
                                 const int* __restrict__ ctx, float* __restrict__ out, int B, int H, int G, int dim,
                                 int vdim, int bs, float scale, float cap, int all, int KB, int Dp, int hchunks,
                                 int RVchunk, int sink, int chunk, int vshare) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);
  float* qs = reinterpret_cast<float*>(smem + (((size_t)KB * Dp * sizeof(T) + 15) & ~(size_t)15));
  float* ps = qs + (size_t)NWT * dim;      // [NWT][KB] weights of the current block of keys
  float* hs = ps + (size_t)NWT * KB;       // [NWT][2]: the block's rescale factor, the final denominator
  // [KB] cache row of each staged key, on the next 8-byte boundary
  int64_t* srow = reinterpret_cast<int64_t*>((reinterpret_cast<uintptr_t>(hs + 2 * NWT) + 7) & ~(uintptr_t)7);
  const int t = blockIdx.x, wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int rep = H / G;
  const int g = blockIdx.y / hchunks;
  const int hl0 = (blockIdx.y % hchunks) * NWT;
  const bool live = hl0 + wv < rep;  // this wave scores a head
  const int h = g * rep + hl0 + wv;
  const int GV = G / vshare;  // value heads
  const int RVtot = all ? GV * vdim : vdim;
  const int v0 = blockIdx.z * RVchunk;
  const int RV = min(RVchunk, RVtot - v0);
  const int64_t vrow = (int64_t)GV * vdim;
  const int voff = (all ? 0 : (g / vshare) * vdim) + v0;
  const int cs = NR2 * 64;  // columns per wave
  constexpr int VK = NR2 >= 4 ? 8 : 16;  // keys whose value loads are in flight together
  const RowSeq r = row_seq(cu, ctx, B, t);
  if (r.pos < 0) {
    for (int hh = 0; hh < NWT && hl0 + hh < rep; ++hh)
      for (int i = threadIdx.x; i < RV; i += blockDim.x) out[((int64_t)t * H + g * rep + hl0 + hh) * RVtot + v0 + i] = 0.f;
    return;
  }
  float* qw = qs + (size_t)wv * dim;
  float* p = ps + (size_t)wv * KB;
  if (live) {
    const float* qsrc = q + ((int64_t)t * H + h) * dim;
    for (int d = lane; d < dim; d += 64) qw[d] = qsrc[d] * scale;
  }
  float acc[NWT][NR2];
#pragma unroll
  for (int hh = 0; hh < NWT; ++hh)
#pragma unroll
    for (int i = 0; i < NR2; ++i) acc[hh][i] = 0.f;
  // the sink: score 0, weight exp(0 - m), no value; without it the first block of keys sets the maximum
  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
  const float icap = cap > 0.f ? 1.0f / cap : 0.f;
  const int* btr = bt + (int64_t)r.b * maxb;
  const int c0 = wv * cs + lane;  // this lane's first column within the chunk
  for (int j0 = chunk > 0 ? (r.pos / chunk) * chunk : 0; j0 <= r.pos; j0 += KB) {
    const int nk = min(KB, r.pos - j0 + 1);
    __syncthreads();
    for (int kk = threadIdx.x; kk < nk; kk += blockDim.x) {
      const int j = j0 + kk;
      srow[kk] = (int64_t)btr[j / bs] * bs + j % bs;
    }
    __syncthreads();
    if (WORDS) {  // rows copied as 4-byte words by all threads, several loads in flight per thread
      const int wpr = dim * (int)sizeof(T) / 4, ldw = Dp * (int)sizeof(T) / 4;
      const unsigned* kw = reinterpret_cast<const unsigned*>(kc);
      unsigned* tw = reinterpret_cast<unsigned*>(tile);
#pragma unroll 4
      for (int e = threadIdx.x; e < nk * wpr; e += blockDim.x) {
        const int kk = e / wpr, wd = e - kk * wpr;
        tw[(size_t)kk * ldw + wd] = kw[(srow[kk] * G + g) * wpr + wd];
      }
    } else {
      for (int e = threadIdx.x; e < nk * dim; e += blockDim.x) {
        const int kk = e / dim, d = e - kk * dim;
        tile[(size_t)kk * Dp + d] = kc[(srow[kk] * G + g) * dim + d];
      }
    }
    __syncthreads();
    if (live) {
      float s = -INFINITY;
      if (lane < nk) {
        const T* row = tile + (size_t)lane * Dp;
        float d_ = 0.f, d2 = 0.f;
        if (WORDS && sizeof(T) == 2) {  // two keys' numbers per LDS read
          const unsigned* rw = reinterpret_cast<const unsigned*>(row);
          for (int w2 = 0; w2 < dim / 2; ++w2) {
            const unsigned u = rw[w2];
            d_ = fmaf(qw[2 * w2], __uint_as_float(u << 16), d_);
            d2 = fmaf(qw[2 * w2 + 1], __uint_as_float(u & 0xffff0000u), d2);
          }
          d_ += d2;
        } else {
          for (int d = 0; d < dim; ++d) d_ = fmaf(qw[d], El<T>::ld(row + d), d_);
        }
        s = cap > 0.f ? cap * tanhf(d_ * icap) : d_;
      }
      const float m_new = fmaxf(m, warp_max(s));
      const float alpha = expf(m - m_new);
      const float pj = lane < nk ? expf(s - m_new) : 0.f;
      l = l * alpha + warp_sum(pj);
      m = m_new;
      if (lane < KB) p[lane] = pj;
      if (lane == 0) hs[2 * wv] = alpha;
    } else {
      if (lane < KB) p[lane] = 0.f;
      if (lane == 0) hs[2 * wv] = 1.f;
    }
    __syncthreads();  // weights, rescale factors and cache rows visible to every wave
#pragma unroll
    for (int hh = 0; hh < NWT; ++hh) {
      const float al = hs[2 * hh];
#pragma unroll
      for (int i = 0; i < NR2; ++i) acc[hh][i] *= al;
    }
    for (int k0 = 0; k0 < nk; k0 += VK) {
      float vv[VK][NR2];
#pragma unroll
      for (int j = 0; j < VK; ++j) {
        const T* row = vc + srow[min(k0 + j, nk - 1)] * vrow + voff;
#pragma unroll
        for (int i = 0; i < NR2; ++i) {
          const int c = c0 + 64 * i;
          vv[j][i] = c < RV ? El<T>::ld(row + c) : 0.f;
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
  if (lane == 0) hs[2 * wv + 1] = l;
  __syncthreads();
#pragma unroll
  for (int hh = 0; hh < NWT; ++hh) {
    if (hl0 + hh < rep) {
      const float inv = 1.0f / hs[2 * hh + 1];
      float* o = out + ((int64_t)t * H + g * rep + hl0 + hh) * RVtot + v0;
#pragma unroll
      for (int i = 0; i < NR2; ++i) {
        const int c = c0 + 64 * i;
        if (c < RV) o[c] = acc[hh][i] * inv;
      }
    }
  }
}

template <typename T>
static void sink_attn_t(const void* q, const void* kc, const void* vc, const void* bt, int maxb, const void* cu,
                        const void* ctx, void* out, int T_, int B, int H, int G, int dim, int vdim, int bs,
                        float scale, float cap, int all, int sink, int chunk, int vshare, hipStream_t st) {
  const int rep = H / G;
  const int NW = rep >= 8 ? 8 : (rep > 2 ? 4 : rep);  // waves = heads per workgroup: 1, 2, 4 or 8
  const int hchunks = (rep + NW - 1) / NW;
  int Dp;  // key row stride in LDS: an odd number of 4-byte words (lanes score neighbouring keys)
  if (sizeof(T) == 2) {
    Dp = (dim + 1) & ~1;
    if (((Dp / 2) & 1) == 0) Dp += 2;
  } else {
    Dp = dim | 1;
  }
  int KB = 64;
  auto bytes = [&](int kb) {
    return (((size_t)kb * Dp * sizeof(T) + 15) & ~(size_t)15) + (size_t)NW * (dim + kb + 2) * 4 + (size_t)kb * 8 + 16;
  };
  while (KB > 8 && bytes(KB) > 60 * 1024) KB >>= 1;
  if (bytes(KB) > 60 * 1024) throw std::runtime_error("sink attention: head dimension too large for LDS");
  const int RVtot = all ? (G / vshare) * vdim : vdim;
  // columns per workgroup: NW waves x NR2 x 64, NR2 in {1, 2, 4} with at most 16 accumulators per lane
  int nr2 = 1;
  while (nr2 < 4 && NW * nr2 * 2 <= 16 && NW * nr2 * 64 < RVtot) nr2 <<= 1;
  const int RVchunk = std::min(RVtot, NW * nr2 * 64);
  const int zch = (RVtot + RVchunk - 1) / RVchunk;
  if (G * hchunks > 65535 || zch > 65535) throw std::runtime_error("sink attention: too many heads");
  dim3 g(T_, G * hchunks, zch);
  // whole 4-byte words per key row, word-aligned rows: the word copy and the two-numbers-per-read dot product
  const bool words = (dim * sizeof(T)) % 4 == 0 && ((uintptr_t)kc % 4) == 0;
#define LAUNCH_SA1(NW_, NR_, WD_)                                                                            \
  sink_attn_kernel<T, NW_, NR_, WD_><<<g, NW_ * 64, bytes(KB), st>>>(                                        \
      (const float*)q, (const T*)kc, (const T*)vc, (const int*)bt, maxb, (const int*)cu, (const int*)ctx,    \
      (float*)out, B, H, G, dim, vdim, bs, scale, cap, all, KB, Dp, hchunks, RVchunk, sink, chunk, vshare)
#define LAUNCH_SA(NW_, NR_)               \
  do {                                    \
    if (words) LAUNCH_SA1(NW_, NR_, true); \
    else LAUNCH_SA1(NW_, NR_, false);     \
  } while (0)
#define LAUNCH_SA_NR(NW_)                \
  do {                                   \
    if (nr2 == 1) LAUNCH_SA(NW_, 1);     \
    else if (nr2 == 2) LAUNCH_SA(NW_, 2); \
    else LAUNCH_SA(NW_, 4);              \
  } while (0)
  if (NW == 1) LAUNCH_SA_NR(1);
  else if (NW == 2) LAUNCH_SA_NR(2);
  else if (NW == 4) LAUNCH_SA_NR(4);
  else {
    if (nr2 == 1) LAUNCH_SA(8, 1);
    else LAUNCH_SA(8, 2);
  }
#undef LAUNCH_SA_NR
#undef LAUNCH_SA
#undef LAUNCH_SA1
}

void launch_sink_attn(const void* q, const void* kc, const void* vc, const void* bt, int maxb, const void* cu,
                      const void* ctx, void* out, int T_, int B, int H, int G, int dim, int vdim, int bs, float scale,
                      float cap, int all, int sink, int chunk, int vshare, int dt, hipStream_t st) {
  if (T_ == 0 || B == 0) return;
  if (G < 1 || H % G) throw std::runtime_error("sink attention: heads must be a multiple of the key/value heads");
  if (vshare < 1 || G % vshare || chunk < 0) throw std::runtime_error("sink attention: bad vshare / chunk");
  DISPATCH_T(dt, T, (sink_attn_t<T>(q, kc, vc, bt, maxb, cu, ctx, out, T_, B, H, G, dim, vdim, bs, scale, cap, all,
                                    sink, chunk, vshare, st)));
  HIP_CHECK_LAUNCH();
}

// The same attention on the matrix cores, for portions of bf16 prompts (key size 32, 64 or 128, value size a
// multiple of 8). One workgroup serves one key/value group, GE of its query heads and 64 * NS / GE query rows of one
// sequence: its 64 * NS "slots" enumerate (row, head) pairs, slot s -> row s / GE, head s % GE, so a key tile is
// staged in LDS once for the whole head group. A wave owns NS groups of 16 neighbouring slots; per group the
// products are the swapped ones,
//   S^T[key][slot] = K . Q^T   (A = K rows from LDS, B = Q^T fragments in registers)
//   O^T[c][slot]  += V^T . P^T (A = V^T by transposing LDS reads, B = P^T straight from the S^T accumulators)
// so a lane owns one slot's softmax row: cap, mask, running maximum (starting at the sink's 0) and sum need two
// shuffles per tile, and a key or value fragment read from LDS feeds the matrix instructions of all NS groups.
// The softmax runs on base-2 exponents (scores times log2 e). A tile that every row of a group sees whole - before
// the group's first position, not before the chunk of its last - skips the mask. Row blocks are taken last first and
// spread evenly over the dies (causal_block_order). (Two tiles in LDS, the next one written while this one is read
// and one barrier per tile, measured the same as one tile and two barriers, and is not kept.)
// The value tile holds VCH = 16 * NVT columns of the key's value row - all groups side by side when the heads'
// weights are mixed afterwards - and blockIdx.y also enumerates the column chunks.
// PRECISE: the fp32 queries and the fp32 softmax weights enter the products as the sum of two bf16 numbers (the
// rounded value and the rounded remainder, two matrix instructions each), so scores and weighted sums are those of
// 32-bit queries and weights; otherwise both are rounded to bf16 once.
template <int DK, int NVT, bool PRECISE, int NS>
__global__ __launch_bounds__(256, 2) void sink_attn_mfma_kernel(
    const float* __restrict__ q, const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
    const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ cu_q, const int* __restrict__ ctx_lens,
    float* __restrict__ out, int H, int G, int GE, int vdim, int bs, float scale, float cap, int all, int nvch,
    int sink, int chunk, int vshare) {
  constexpr int BKV = 64;
  constexpr int LDK = DK + 16;
  constexpr int VCH = NVT * 16;
  constexpr int LDV = VCH + 16;
  __shared__ __attribute__((aligned(16))) bf16_t Ks[BKV * LDK];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[BKV * LDV];
  const int rep = H / G;
  const int rows_per_wg = 64 * NS / GE;
  int bx, by, b;
  causal_block_order(bx, by, b);
  const int vch = by % nvch, hy = by / nvch;
  const int kvh = hy / (rep / GE);
  const int h0 = kvh * rep + (hy % (rep / GE)) * GE;
  const int t0 = cu_q[b], qlen = cu_q[b + 1] - t0;
  const int r0 = bx * rows_per_wg;
  if (r0 >= qlen) return;
  const int p0 = ctx_lens[b] - qlen;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int li = lane & 15, g = lane >> 4;
  const int GV = G / vshare;
  const int RVtot = all ? GV * vdim : vdim;
  const int v0 = vch * VCH;
  const int64_t vrow = (int64_t)GV * vdim;
  const int voff = (all ? 0 : (kvh / vshare) * vdim) + v0;

  // per slot group: the lane's slot, and (the same in every lane) the positions the group's rows span
  int row[NS], hd[NS], qpos[NS], qlo[NS];
  bool valid[NS], grp_rows[NS];
  int grp_first[NS], grp_last[NS], grp_lo[NS], grp_hilo[NS];
  s16x8 qf[NS][DK / 32], ql[NS][PRECISE ? DK / 32 : 1];
  f32x4 o[NS][NVT];
  float m[NS], lsum[NS];
  bool wave_rows = false;
#pragma unroll
  for (int n = 0; n < NS; ++n) {
    const int gs = (w * NS + n) * 16, slot = gs + li;
    row[n] = r0 + slot / GE;
    hd[n] = h0 + slot % GE;
    valid[n] = slot < rows_per_wg * GE && row[n] < qlen;
    qpos[n] = p0 + (valid[n] ? row[n] : 0);
    qlo[n] = chunk > 0 ? (qpos[n] / chunk) * chunk : 0;  // the first key this row sees
    // a group none of whose slots holds a row (a single decoded row fills part of the first) only helps to stage
    grp_rows[n] = r0 + gs / GE < qlen && gs < rows_per_wg * GE;
    wave_rows = wave_rows || grp_rows[n];
    grp_first[n] = p0 + min(qlen - 1, r0 + gs / GE);
    grp_last[n] = p0 + min(qlen - 1, r0 + (gs + 15) / GE);
    grp_lo[n] = chunk > 0 ? (grp_first[n] / chunk) * chunk : 0;
    grp_hilo[n] = chunk > 0 ? (grp_last[n] / chunk) * chunk : 0;
    const float* qp = q + ((int64_t)(t0 + (valid[n] ? row[n] : 0)) * H + (valid[n] ? hd[n] : h0)) * DK + 8 * g;
#pragma unroll
    for (int ks = 0; ks < DK / 32; ++ks)
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x = qp[32 * ks + j];
        const bf16_t hi = f2bf(x);
        qf[n][ks][j] = (short)hi;
        if constexpr (PRECISE) ql[n][ks][j] = (short)f2bf(x - bf2f(hi));
      }
#pragma unroll
    for (int i = 0; i < NVT; ++i) o[n][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    // the sink: score 0, weight exp(0 - m), no value; without it a masked score's stand-in is the starting maximum
    m[n] = sink ? 0.f : -1.0e30f;
    lsum[n] = sink ? 1.f : 0.f;
  }
  constexpr float kLog2e = 1.4426950408889634f;
  const float icap = cap > 0.f ? 1.0f / cap : 0.f;
  const float scale2 = scale * kLog2e;
  const int r_last = min(qlen, r0 + rows_per_wg) - 1;
  const int kv_end = p0 + r_last + 1;
  const int kv_begin = chunk > 0 ? ((p0 + r0) / chunk) * chunk : 0;  // the first row's block starts first
  const int* bt = block_tables + (int64_t)b * max_blocks;
  constexpr int CHK = DK / 8, CHV = VCH / 8;
  // Software pipeline: the next tile's 16-byte chunks are fetched into registers while this tile is computed from
  // LDS, and written to LDS after the next barrier, so a tile does not wait a memory round trip behind the last one.
  static_assert((BKV * CHK) % 256 == 0 && (BKV * CHV) % 256 == 0, "whole 16-byte chunks per thread");
  constexpr int NCK = BKV * CHK / 256, NCV = BKV * CHV / 256;
  u16x8 kr[NCK], vr[NCV];
  auto load_tile = [&](int kv0) {
#pragma unroll
    for (int j = 0; j < NCK; ++j) {
      const int c = threadIdx.x + 256 * j;
      const int r = c / CHK, ch = c % CHK;
      const int key = min(kv0 + r, kv_end - 1);
      const int64_t sl = (int64_t)bt[key / bs] * bs + key % bs;
      kr[j] = *reinterpret_cast<const u16x8*>(kc + (sl * G + kvh) * DK + ch * 8);
    }
#pragma unroll
    for (int j = 0; j < NCV; ++j) {
      const int c = threadIdx.x + 256 * j;
      const int r = c / CHV, ch = c % CHV;
      const int key = min(kv0 + r, kv_end - 1);
      const int64_t sl = (int64_t)bt[key / bs] * bs + key % bs;
      u16x8 val = {0, 0, 0, 0, 0, 0, 0, 0};
      if (v0 + ch * 8 < RVtot) val = *reinterpret_cast<const u16x8*>(vc + sl * vrow + voff + ch * 8);
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
  // one tile of keys from LDS for every slot group of this wave that sees any of it
  auto compute_tile = [&](int kv0) {
    bool act[NS];
    bool any = false;
#pragma unroll
    for (int n = 0; n < NS; ++n) {
      // not wholly in the group's causal future, not wholly before the block of its first row
      act[n] = grp_rows[n] && kv0 <= grp_last[n] && kv0 + BKV > grp_lo[n];
      any = any || act[n];
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
          if constexpr (PRECISE) s[n][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, ql[n][ks], s[n][kt], 0, 0, 0);
        }
      }
    }
    // S^T accumulators: lane (li, g) holds slot li's scores for keys kv0 + 16 kt + 4 g + i.
    // The matrix instructions above and below run for every group of the wave (a fragment from LDS serves them all);
    // a group that sees nothing of the tile gets zero weights, which leave its sums as they are.
    s16x8 pf[NS][2], pl[NS][PRECISE ? 2 : 1];
    auto softmax = [&](int n, auto whole_c, auto cap_c) {
      constexpr bool WHOLE = decltype(whole_c)::value, CAP = decltype(cap_c)::value;
      float mx = m[n];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v;
          if constexpr (CAP) {
            const float x = s[n][kt][i] * scale;
            const float e2 = __expf(2.0f * x * icap);  // tanh(x) = 1 - 2 / (exp(2x) + 1)
            v = cap * (1.0f - 2.0f / (e2 + 1.0f)) * kLog2e;
          } else {
            v = s[n][kt][i] * scale2;
          }
          if constexpr (!WHOLE) {
            const int key = kv0 + kt * 16 + 4 * g + i;
            v = (key <= qpos[n] && key >= qlo[n] && key < kv_end) ? v : -1.0e30f;
          }
          s[n][kt][i] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float alpha = __builtin_amdgcn_exp2f(m[n] - mx);
      m[n] = mx;
      float ps = 0.f;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float p = __builtin_amdgcn_exp2f(s[n][kt][i] - mx);
          if constexpr (!WHOLE) p = s[n][kt][i] > -1.0e29f ? p : 0.f;
          const bf16_t pb = f2bf(p);
          pf[n][kt >> 1][(kt & 1) * 4 + i] = (short)pb;
          if constexpr (PRECISE) {
            ps += p;
            pl[n][kt >> 1][(kt & 1) * 4 + i] = (short)f2bf(p - bf2f(pb));
          } else {
            ps += bf2f(pb);
          }
        }
      ps += __shfl_xor(ps, 16, 64);
      ps += __shfl_xor(ps, 32, 64);
      lsum[n] = lsum[n] * alpha + ps;
#pragma unroll
      for (int i = 0; i < NVT; ++i) o[n][i] *= alpha;
    };
#pragma unroll
    for (int n = 0; n < NS; ++n) {
      if (!act[n]) {
        const s16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        pf[n][0] = pf[n][1] = z;
        if constexpr (PRECISE) pl[n][0] = pl[n][1] = z;
        continue;
      }
      // does every row of the group see the whole tile?
      const bool whole = kv0 + BKV - 1 <= grp_first[n] && kv0 >= grp_hilo[n];
      if (cap > 0.f) softmax(n, std::false_type{}, std::true_type{});
      else if (whole) softmax(n, std::true_type{}, std::false_type{});
      else softmax(n, std::false_type{}, std::false_type{});
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
          o[n][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[n][ks], o[n][dt], 0, 0, 0);
          if constexpr (PRECISE) o[n][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl[n][ks], o[n][dt], 0, 0, 0);
        }
      }
    }
  };
  if (kv_end > kv_begin) load_tile(kv_begin);  // (a padded row has no keys at all)
  for (int kv0 = kv_begin; kv0 < kv_end; kv0 += BKV) {
    __syncthreads();  // every wave is done reading the previous tile
    store_tile();
    __syncthreads();
    if (kv0 + BKV < kv_end) load_tile(kv0 + BKV);
    if (wave_rows) compute_tile(kv0);
  }
#pragma unroll
  for (int n = 0; n < NS; ++n) {
    if (!valid[n]) continue;
    const float inv = 1.0f / lsum[n];
    float* op = out + ((int64_t)(t0 + row[n]) * H + hd[n]) * RVtot + v0 + 4 * g;
#pragma unroll
    for (int dt = 0; dt < NVT; ++dt)
      if (v0 + dt * 16 + 4 * g < RVtot) *reinterpret_cast<f32x4*>(op + dt * 16) = o[n][dt] * inv;
  }
}

// Can the matrix-core kernel take this shape? (bf16 storage is the caller's to check.)
bool sink_attn_mfma_ok(int dim, int vdim) { return (dim == 32 || dim == 64 || dim == 128) && vdim % 8 == 0; }

void launch_sink_attn_mfma(const void* q, const void* kc, const void* vc, const void* bt, int maxb, const void* cu,
                           const void* ctx, void* out, int B, int max_qlen, int H, int G, int dim, int vdim, int bs,
                           float scale, float cap, int all, int sink, int chunk, int vshare, int precise,
                           hipStream_t st) {
  if (B == 0 || max_qlen <= 0) return;
  if (G < 1 || H % G) throw std::runtime_error("sink attention: heads must be a multiple of the key/value heads");
  if (vshare < 1 || G % vshare || chunk < 0) throw std::runtime_error("sink attention: bad vshare / chunk");
  if (!sink_attn_mfma_ok(dim, vdim)) throw std::runtime_error("sink attention: shape not built for the matrix cores");
  const int rep = H / G;
  int GE = 1;
  for (int ge = std::min(rep, 64); ge >= 1; --ge)
    if (rep % ge == 0) {
      GE = ge;
      break;
    }
  const int RVtot = all ? (G / vshare) * vdim : vdim;
  const int nvt = RVtot > 128 ? 16 : (RVtot > 64 ? 8 : 4);
  const int nvch = (RVtot + nvt * 16 - 1) / (nvt * 16);
  // two slot groups per wave where a portion has more rows than one group each would hold (the widest value tile,
  // and 128-wide keys with split queries beside the middle one, keep one: two groups would not fit the registers)
  const bool two_fit = nvt <= 4 || (nvt == 8 && !(dim == 128 && precise));
  const int ns = (two_fit && max_qlen > 64 / GE) ? 2 : 1;
  const int rows_per_wg = 64 * ns / GE;
  const int64_t gy = (int64_t)G * (rep / GE) * nvch;
  if (gy > 65535 || B > 65535) throw std::runtime_error("sink attention: too many heads or sequences");
  dim3 grid((max_qlen + rows_per_wg - 1) / rows_per_wg, (unsigned)gy, B);
#define LAUNCH_SAM2(DK_, NVT_, PR_, NS_)                                                                            \
  sink_attn_mfma_kernel<DK_, NVT_, PR_, NS_><<<grid, 256, 0, st>>>(                                                 \
      (const float*)q, (const bf16_t*)kc, (const bf16_t*)vc, (const int*)bt, maxb, (const int*)cu, (const int*)ctx, \
      (float*)out, H, G, GE, vdim, bs, scale, cap, all, nvch, sink, chunk, vshare)
#define LAUNCH_SAM1(DK_, NVT_, NS_)                                                       \
  do {                                                                                    \
    if (!precise) LAUNCH_SAM2(DK_, NVT_, false, NS_);                                     \
    else LAUNCH_SAM2(DK_, NVT_, true, (DK_ == 128 && NVT_ == 8 && NS_ == 2) ? 1 : NS_);   \
  } while (0)
#define LAUNCH_SAM(DK_)                       \
  do {                                        \
    if (nvt == 16) LAUNCH_SAM1(DK_, 16, 1);   \
    else if (nvt == 8) {                      \
      if (ns == 2) LAUNCH_SAM1(DK_, 8, 2);    \
      else LAUNCH_SAM1(DK_, 8, 1);            \
    } else {                                  \
      if (ns == 2) LAUNCH_SAM1(DK_, 4, 2);    \
      else LAUNCH_SAM1(DK_, 4, 1);            \
    }                                         \
  } while (0)
  if (dim == 32) LAUNCH_SAM(32);
  else if (dim == 64) LAUNCH_SAM(64);
  else LAUNCH_SAM(128);
#undef LAUNCH_SAM
#undef LAUNCH_SAM1
#undef LAUNCH_SAM2
  HIP_CHECK_LAUNCH();
}

// y[t, h * vdim + v] = c * sum_h' talk[h, h'] O[t, h', g(h) * vdim + v]     (talk null: y = c * O[t, h, v])
template <typename T>
__global__ __launch_bounds__(256) void talk_mix_kernel(const float* __restrict__ O, const float* __restrict__ talk,
                                                       float c, T* __restrict__ y, int64_t ldy, int H, int G,
                                                       int vdim) {
  const int t = blockIdx.x;
  const int rep = H / G;
  const int RVtot = talk ? G * vdim : vdim;
  const float* Ot = O + (int64_t)t * H * RVtot;
  if ((vdim & 3) == 0) {  // four columns per thread, 16-byte reads
    for (int e = threadIdx.x * 4; e < H * vdim; e += blockDim.x * 4) {
      const int h = e / vdim, v = e % vdim;
      f32x4 a;
      if (talk) {
        a = f32x4{0.f, 0.f, 0.f, 0.f};
        const int col = (h / rep) * vdim + v;
        for (int hh = 0; hh < H; ++hh) {
          const float w = talk[h * H + hh];
          const f32x4 x = *reinterpret_cast<const f32x4*>(Ot + (int64_t)hh * RVtot + col);
          a[0] = fmaf(w, x[0], a[0]), a[1] = fmaf(w, x[1], a[1]), a[2] = fmaf(w, x[2], a[2]), a[3] = fmaf(w, x[3], a[3]);
        }
      } else {
        a = *reinterpret_cast<const f32x4*>(Ot + (int64_t)h * RVtot + v);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) El<T>::st(y + (int64_t)t * ldy + e + i, a[i] * c);
    }
    return;
  }
  for (int e = threadIdx.x; e < H * vdim; e += blockDim.x) {
    const int h = e / vdim, v = e % vdim;
    float a;
    if (talk) {
      a = 0.f;
      const int col = (h / rep) * vdim + v;
      for (int hh = 0; hh < H; ++hh) a = fmaf(talk[h * H + hh], Ot[(int64_t)hh * RVtot + col], a);
    } else {
      a = Ot[(int64_t)h * RVtot + v];
    }
    El<T>::st(y + (int64_t)t * ldy + e, a * c);
  }
}

void launch_talk_mix(const void* O, const void* talk, float c, void* y, int64_t ldy, int T_, int H, int G, int vdim,
                     int dt, hipStream_t st) {
  if (T_ == 0) return;
  DISPATCH_T(dt, T, (talk_mix_kernel<T><<<T_, 256, 0, st>>>((const float*)O, (const float*)talk, c, (T*)y, ldy, H, G,
                                                            vdim)));
  HIP_CHECK_LAUNCH();
}

// Queries [H, maps, dim] and keys [G, maps, dim] of a projection row, each vector of dim numbers divided by its root
// mean square and multiplied by a weight [dim] (null: left as it is); values [G, vdim]. q -> qout fp32, ordered (key
// head, map, query head within the group), so that with the keys cached as G * maps heads the grouped-query mapping
// "query vector n reads key head n / rep" holds; k, v -> the paged caches at slots[t] (slot < 0: not cached).
// One wave per vector.
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(const T* __restrict__ proj, int64_t ldp, int off_q,
                                                            int off_k, int off_v, const T* __restrict__ qw,
                                                            const T* __restrict__ kw, float eps,
                                                            float* __restrict__ qout, T* __restrict__ kc,
                                                            T* __restrict__ vc, const int64_t* __restrict__ slots,
                                                            int H, int G, int maps, int dim, int vdim) {
  const int t = blockIdx.x, wv = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const T* row = proj + (int64_t)t * ldp;
  const int64_t slot = slots[t];
  const int rep = H / G, nqv = H * maps, nkv = G * maps;
  for (int n = wv; n < nqv + nkv; n += nw) {
    const bool isk = n >= nqv;
    const int idx = isk ? n - nqv : n;
    if (isk && slot < 0) continue;
    const T* src = row + (isk ? off_k : off_q) + (int64_t)idx * dim;
    const T* wt = isk ? kw : qw;
    float inv = 1.f;
    if (wt) {
      float ss = 0.f;
      for (int d = lane; d < dim; d += 64) {
        const float v = El<T>::ld(src + d);
        ss = fmaf(v, v, ss);
      }
      inv = 1.0f / sqrtf(warp_sum(ss) / (float)dim + eps);
    }
    if (isk) {
      T* dst = kc + (slot * nkv + idx) * (int64_t)dim;
      for (int d = lane; d < dim; d += 64)
        El<T>::st(dst + d, wt ? El<T>::ld(src + d) * inv * El<T>::ld(wt + d) : El<T>::ld(src + d));
    } else {
      const int h = idx / maps, mp = idx - h * maps;
      const int g = h / rep, r = h - g * rep;
      float* dst = qout + ((int64_t)t * nqv + (g * maps + mp) * rep + r) * dim;
      for (int d = lane; d < dim; d += 64)
        dst[d] = wt ? El<T>::ld(src + d) * inv * El<T>::ld(wt + d) : El<T>::ld(src + d);
    }
  }
  if (slot >= 0)
    for (int e = threadIdx.x; e < G * vdim; e += blockDim.x) vc[slot * (int64_t)G * vdim + e] = row[off_v + e];
}

// The same for bf16 rows whose vectors are whole 16-byte pieces: dim / 8 neighbouring lanes (a power of two) share a
// vector, each lane reads its eight numbers once, the sum of squares is added up across the lanes of the vector, and the
// result leaves in 16-byte stores (two for a query's eight fp32 numbers).
__global__ __launch_bounds__(256) void qk_norm_cache_vec_kernel(const bf16_t* __restrict__ proj, int64_t ldp,
                                                                int off_q, int off_k, int off_v,
                                                                const bf16_t* __restrict__ qw,
                                                                const bf16_t* __restrict__ kw, float eps,
                                                                float* __restrict__ qout, bf16_t* __restrict__ kc,
                                                                bf16_t* __restrict__ vc,
                                                                const int64_t* __restrict__ slots, int H, int G,
                                                                int maps, int dim, int vdim) {
  const int t = blockIdx.x;
  const int L = dim >> 3;  // lanes per vector
  const int sub = threadIdx.x & (L - 1), per = blockDim.x / L;
  const bf16_t* row = proj + (int64_t)t * ldp;
  const int64_t slot = slots[t];
  const int rep = H / G, nqv = H * maps, nkv = G * maps;
  for (int n = threadIdx.x / L; n < nqv + nkv; n += per) {
    const bool isk = n >= nqv;
    const int idx = isk ? n - nqv : n;
    if (isk && slot < 0) continue;
    const bf16_t* wt = isk ? kw : qw;
    const u16x8 raw = *reinterpret_cast<const u16x8*>(row + (isk ? off_k : off_q) + (int64_t)idx * dim + 8 * sub);
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = bf2f(raw[i]);
    if (wt) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) ss = fmaf(x[i], x[i], ss);
      for (int o = L >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
      const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
      const u16x8 wr = *reinterpret_cast<const u16x8*>(wt + 8 * sub);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = x[i] * inv * bf2f(wr[i]);
    }
    if (isk) {
      u16x8 y;
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = wt ? f2bf(x[i]) : raw[i];
      *reinterpret_cast<u16x8*>(kc + (slot * nkv + idx) * (int64_t)dim + 8 * sub) = y;
    } else {
      const int h = idx / maps, mp = idx - h * maps;
      const int g = h / rep, r = h - g * rep;
      float* dst = qout + ((int64_t)t * nqv + (g * maps + mp) * rep + r) * dim + 8 * sub;
      *reinterpret_cast<f32x4*>(dst) = f32x4{x[0], x[1], x[2], x[3]};
      *reinterpret_cast<f32x4*>(dst + 4) = f32x4{x[4], x[5], x[6], x[7]};
    }
  }
  if (slot >= 0)
    for (int e = threadIdx.x * 8; e < G * vdim; e += blockDim.x * 8)
      *reinterpret_cast<u16x8*>(vc + slot * (int64_t)G * vdim + e) = *reinterpret_cast<const u16x8*>(row + off_v + e);
}

void launch_qk_norm_cache(const void* proj, int64_t ldp, int off_q, int off_k, int off_v, const void* qw,
                          const void* kw, float eps, void* qout, void* kc, void* vc, const void* slots, int T_, int H,
                          int G, int maps, int dim, int vdim, int dt, hipStream_t st) {
  if (T_ == 0) return;
  if (G < 1 || H % G || maps < 1) throw std::runtime_error("qk_norm_cache: heads must be a multiple of the key heads");
  const auto al16 = [](const void* p) { return p == nullptr || ((uintptr_t)p & 15) == 0; };
  if (dt == 0 && dim >= 8 && dim <= 512 && (dim & (dim - 1)) == 0 && (G * vdim) % 8 == 0 && ldp % 8 == 0 &&
      off_q % 8 == 0 && off_k % 8 == 0 && off_v % 8 == 0 && al16(proj) && al16(qw) && al16(kw) && al16(qout) &&
      al16(kc) && al16(vc)) {
    qk_norm_cache_vec_kernel<<<T_, 256, 0, st>>>((const bf16_t*)proj, ldp, off_q, off_k, off_v, (const bf16_t*)qw,
                                                 (const bf16_t*)kw, eps, (float*)qout, (bf16_t*)kc, (bf16_t*)vc,
                                                 (const int64_t*)slots, H, G, maps, dim, vdim);
    HIP_CHECK_LAUNCH();
    return;
  }
  DISPATCH_T(dt, T, (qk_norm_cache_kernel<T><<<T_, 256, 0, st>>>(
      (const T*)proj, ldp, off_q, off_k, off_v, (const T*)qw, (const T*)kw, eps, (float*)qout, (T*)kc, (T*)vc,
      (const int64_t*)slots, H, G, maps, dim, vdim)));
  HIP_CHECK_LAUNCH();
}

// Two maps per head, O fp32 [T, G * 2 * rep, vdim] ordered (key head, map, query head within the group):
//   o = O[map 0] - lam * O[map 1];   y[t, head] = mult * o / sqrt(mean(o^2) + eps)      head = g * rep + r
// One wave per (row, head).
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(const float* __restrict__ O, float lam, float eps,
                                                           float mult, T* __restrict__ y, int64_t ldy, int H, int G,
                                                           int vdim) {
  const int t = blockIdx.x, wv = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  const int rep = H / G;
  for (int h = blockIdx.y * nw + wv; h < H; h += gridDim.y * nw) {
    const int g = h / rep, r = h - g * rep;
    const float* a1 = O + ((int64_t)t * 2 * H + (g * 2) * rep + r) * vdim;
    const float* a2 = a1 + (int64_t)rep * vdim;
    float ss = 0.f;
    for (int c = lane; c < vdim; c += 64) {
      const float o = a1[c] - lam * a2[c];
      ss = fmaf(o, o, ss);
    }
    const float inv = mult / sqrtf(warp_sum(ss) / (float)vdim + eps);
    T* dst = y + (int64_t)t * ldy + (int64_t)h * vdim;
    for (int c = lane; c < vdim; c += 64) El<T>::st(dst + c, (a1[c] - lam * a2[c]) * inv);
  }
}

// The same with vdim / 4 neighbouring lanes (a power of two) to a head: each lane reads its four numbers of both
// maps in 16-byte pieces once and writes its four results in one piece.
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_vec_kernel(const float* __restrict__ O, float lam, float eps,
                                                               float mult, T* __restrict__ y, int64_t ldy, int H,
                                                               int G, int vdim) {
  const int t = blockIdx.x;
  const int L = vdim >> 2, sub = threadIdx.x & (L - 1), per = blockDim.x / L;
  const int rep = H / G;
  for (int h = blockIdx.y * per + threadIdx.x / L; h < H; h += gridDim.y * per) {
    const int g = h / rep, r = h - g * rep;
    const float* a1 = O + ((int64_t)t * 2 * H + (g * 2) * rep + r) * vdim + 4 * sub;
    const f32x4 x1 = *reinterpret_cast<const f32x4*>(a1);
    const f32x4 x2 = *reinterpret_cast<const f32x4*>(a1 + (int64_t)rep * vdim);
    float o[4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[i] = x1[i] - lam * x2[i];
      ss = fmaf(o[i], o[i], ss);
    }
    for (int d = L >> 1; d > 0; d >>= 1) ss += __shfl_xor(ss, d, 64);
    const float inv = mult / sqrtf(ss / (float)vdim + eps);
    T* dst = y + (int64_t)t * ldy + (int64_t)h * vdim + 4 * sub;
    if constexpr (sizeof(T) == 4) {
      *reinterpret_cast<f32x4*>(dst) = f32x4{o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv};
    } else {
      u32x2 pk;
      pk[0] = (unsigned)f2bf(o[0] * inv) | ((unsigned)f2bf(o[1] * inv) << 16);
      pk[1] = (unsigned)f2bf(o[2] * inv) | ((unsigned)f2bf(o[3] * inv) << 16);
      *reinterpret_cast<u32x2*>(dst) = pk;
    }
  }
}

void launch_diff_combine(const void* O, float lam, float eps, float mult, void* y, int64_t ldy, int T_, int H, int G,
                         int vdim, int dt, hipStream_t st) {
  if (T_ == 0) return;
  if (G < 1 || H % G) throw std::runtime_error("diff_combine: heads must be a multiple of the key heads");
  const int L = vdim / 4;
  if (vdim % 4 == 0 && L >= 1 && L <= 64 && (L & (L - 1)) == 0 && ldy % 4 == 0 && ((uintptr_t)O & 15) == 0 &&
      ((uintptr_t)y & 15) == 0) {
    const int per = 256 / L;
    dim3 g(T_, std::min(64, (H + per - 1) / per));
    DISPATCH_T(dt, T, (diff_combine_vec_kernel<T><<<g, 256, 0, st>>>((const float*)O, lam, eps, mult, (T*)y, ldy, H,
                                                                      G, vdim)));
    HIP_CHECK_LAUNCH();
    return;
  }
  dim3 g(T_, std::min(64, (H + 3) / 4));
  DISPATCH_T(dt, T, (diff_combine_kernel<T><<<g, 256, 0, st>>>((const float*)O, lam, eps, mult, (T*)y, ldy, H, G,
                                                                vdim)));
  HIP_CHECK_LAUNCH();
}
