// Latent attention over a paged cache of compressed key/value rows.
//
// A latent-attention layer projects each token to one row c of `R` numbers (RMS-normed), and every head's keys and
// values are linear maps of it (k = W_uk c, v = W_uv c). Only c is cached. With the key projection absorbed into
// the query (qa_h = W_uk_h^T q_h) the scores are qa_h . c_j and the attention output is W_uv_h (sum_j p_j c_j), so
// the kernel below is a multi-query attention whose single key/value head is the latent row itself:
//
//   out[t, h, :] = sum_j softmax_j(scale * qa[t, h, :] . c_j) c_j       j over the keys position(t) may see
//
// Visibility is causal with an optional sliding window: j <= i and i - j < window (window 0 = no limit).
// One kernel serves prompt portions, portions that continue a cached prefix and single decoded tokens: every
// token of the step finds its sequence through cu_q and its position from ctx_lens, and reads all keys - those of
// its own step included - from the paged cache, so a position's result does not depend on how the prompt was cut.
// Scores, softmax and the weighted sum are fp32; the cache is read in the model's storage type.
//
// Work split: one workgroup per token and group of NW heads (one wave per head). A block of KB keys is staged into
// LDS once for all heads of the group; each wave scores it with lanes over keys, does its online-softmax update
// and accumulates with lanes over the R latent dimensions (NR = ceil(R / 64) registers per lane).
#include "anytype.h"

// c = rms_norm(src[t, off : off + R]) * w, written to cache[slot[t], :R] (slot < 0: not cached) in fp32 math.
// rot > 0: the cached row is [c | k_rot], k_rot = src[t, off + R : off + R + rot] with the neighbouring pairs
// (2i, 2i + 1), i < rdims / 2, turned by cs[t, i] = (cos, sin) and the numbers from rdims on passed unchanged; and
// every query head's rotated part - head h holds qdim plain numbers, then rot - is turned the same way into
// qa[t, h, R : R + rot] (qa [T, H, R + rot] in its own type TQ).
template <typename T, typename TQ>
__global__ __launch_bounds__(64) void latent_norm_cache_kernel(const T* __restrict__ src, int64_t lds_, int off,
                                                               const T* __restrict__ w, float eps,
                                                               T* __restrict__ cache, const int64_t* __restrict__ slots,
                                                               int R, int rot, int rdims,
                                                               const float* __restrict__ cs, TQ* __restrict__ qa,
                                                               int off_q, int H, int qdim) {
  const int t = blockIdx.x, lane = threadIdx.x;
  const int64_t slot = slots[t];
  const int half = rdims >> 1, rest = rot - rdims;
  const float* tab = cs + (int64_t)t * half * 2;
  if (rot) {
    const T* q = src + (int64_t)t * lds_ + off_q;
    TQ* dst = qa + (int64_t)t * H * (R + rot) + R;
    for (int e = lane; e < H * half; e += 64) {
      const int h = e / half, i = e - h * half;
      const T* p = q + (int64_t)h * (qdim + rot) + qdim + 2 * i;
      const float u = El<T>::ld(p), v = El<T>::ld(p + 1), c = tab[2 * i], sn = tab[2 * i + 1];
      El<TQ>::st(dst + (int64_t)h * (R + rot) + 2 * i, u * c - v * sn);
      El<TQ>::st(dst + (int64_t)h * (R + rot) + 2 * i + 1, v * c + u * sn);
    }
    for (int e = lane; e < H * rest; e += 64) {
      const int h = e / rest, i = rdims + e - h * rest;
      El<TQ>::st(dst + (int64_t)h * (R + rot) + i, El<T>::ld(q + (int64_t)h * (qdim + rot) + qdim + i));
    }
  }
  if (slot < 0) return;
  const T* s = src + (int64_t)t * lds_ + off;
  float ss = 0.f;
  for (int r = lane; r < R; r += 64) {
    const float v = El<T>::ld(s + r);
    ss += v * v;
  }
  ss = warp_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)R + eps);
  T* dst = cache + slot * (int64_t)(R + rot);
  for (int r = lane; r < R; r += 64) El<T>::st(dst + r, El<T>::ld(s + r) * inv * El<T>::ld(w + r));
  for (int i = lane; i < half; i += 64) {
    const float u = El<T>::ld(s + R + 2 * i), v = El<T>::ld(s + R + 2 * i + 1), c = tab[2 * i], sn = tab[2 * i + 1];
    El<T>::st(dst + R + 2 * i, u * c - v * sn);
    El<T>::st(dst + R + 2 * i + 1, v * c + u * sn);
  }
  for (int i = rdims + lane; i < rot; i += 64) El<T>::st(dst + R + i, El<T>::ld(s + R + i));
}

// dq: storage type of qa (0 bf16, 1 fp32); only read when rot > 0
void launch_latent_norm_cache(const void* src, int64_t ld, int off, const void* w, float eps, void* cache,
                              const void* slots, int T_, int R, int rot, int rdims, const void* cs, void* qa,
                              int off_q, int H, int qdim, int dt, int dq, hipStream_t st) {
  if (T_ == 0) return;
  if (rot < 0 || rdims < 0 || rdims > rot || (rdims & 1))
    throw std::runtime_error("latent_norm_cache: rotated dimensions must be even and fit the rotated part");
  DISPATCH_T(dt, T, DISPATCH_T(rot ? dq : 1, TQ, (latent_norm_cache_kernel<T, TQ><<<T_, 64, 0, st>>>(
      (const T*)src, ld, off, (const T*)w, eps, (T*)cache, (const int64_t*)slots, R, rot, rdims, (const float*)cs,
      (TQ*)qa, off_q, H, qdim))));
  HIP_CHECK_LAUNCH();
}

// cs[t, i] = (cos, sin) of fl(position[t] * freqs[i]): the angle is the fp32 product, its cosine and sine are
// evaluated in double and rounded once
__global__ __launch_bounds__(256) void rope_angles_kernel(const int64_t* __restrict__ positions,
                                                          const float* __restrict__ freqs, float* __restrict__ cs,
                                                          int T_, int half) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= T_ * half) return;
  const int t = e / half, i = e - t * half;
  const float ang = (float)positions[t] * freqs[i];
  double sn, c;
  sincos((double)ang, &sn, &c);
  cs[2 * (int64_t)e] = (float)c;
  cs[2 * (int64_t)e + 1] = (float)sn;
}

void launch_rope_angles(const void* positions, const void* freqs, void* cs, int T_, int half, hipStream_t st) {
  if (T_ == 0 || half == 0) return;
  rope_angles_kernel<<<(T_ * half + 255) / 256, 256, 0, st>>>((const int64_t*)positions, (const float*)freqs,
                                                              (float*)cs, T_, half);
  HIP_CHECK_LAUNCH();
}

template <typename T, int NR>
__global__ void latent_attn_kernel(const float* __restrict__ qa, int64_t ldq, const T* __restrict__ cache,
                                   const int* __restrict__ bt, int maxb, const int* __restrict__ cu_q,
                                   const int* __restrict__ ctx_lens, float* __restrict__ out, int64_t ldo, int B,
                                   int H, int R, int bs, int window, float scale, int KB, int Rp) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int NW = blockDim.x >> 6;
  T* tile = reinterpret_cast<T*>(smem);
  float* qs = reinterpret_cast<float*>(smem + (((size_t)KB * Rp * sizeof(T) + 15) & ~(size_t)15));
  float* ps = qs + (size_t)NW * R;
  const int t = blockIdx.x, wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * NW + wv;
  const bool live = h < H;
  // sequence of token t: the last b with cu_q[b] <= t (empty sequences share a boundary and are skipped)
  int lo = 0, hi = B;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid;
  }
  const int b = lo;
  const int qlen = cu_q[b + 1] - cu_q[b];
  const int pos = ctx_lens[b] - qlen + (t - cu_q[b]);
  float* o = out + (int64_t)t * ldo + (int64_t)h * R;
  if (pos < 0 || t >= cu_q[B]) {  // padded row (no context): zeros
    if (live)
      for (int r = lane; r < R; r += 64) o[r] = 0.f;
    return;
  }
  const int j_lo = window > 0 ? max(0, pos - window + 1) : 0;
  float* q = qs + (size_t)wv * R;
  float* p = ps + (size_t)wv * KB;
  if (live) {
    const float* qsrc = qa + (int64_t)t * ldq + (int64_t)h * R;
    for (int r = lane; r < R; r += 64) q[r] = qsrc[r] * scale;
  }
  float acc[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  const int* btr = bt + (int64_t)b * maxb;
  for (int j0 = j_lo; j0 <= pos; j0 += KB) {
    const int nk = min(KB, pos - j0 + 1);
    __syncthreads();  // the previous block's readers are done (and q is visible)
    for (int kk = wv; kk < nk; kk += NW) {
      const int j = j0 + kk;
      const int64_t slot = (int64_t)btr[j / bs] * bs + j % bs;
      const T* src = cache + slot * R;
      T* dst = tile + (size_t)kk * Rp;
      for (int r = lane; r < R; r += 64) dst[r] = src[r];
    }
    __syncthreads();
    if (live) {
      float s = -INFINITY;
      if (lane < nk) {
        const T* row = tile + (size_t)lane * Rp;
        float d = 0.f;
        for (int r = 0; r < R; ++r) d = fmaf(q[r], El<T>::ld(row + r), d);
        s = d;
      }
      const float m_new = fmaxf(m, warp_max(s));
      const float alpha = expf(m - m_new);
      const float pj = lane < nk ? expf(s - m_new) : 0.f;
      l = l * alpha + warp_sum(pj);
      m = m_new;
      if (lane < KB) p[lane] = pj;
#pragma unroll
      for (int i = 0; i < NR; ++i) acc[i] *= alpha;
    }
    __syncthreads();  // p visible to the whole wave
    if (live) {
      for (int kk = 0; kk < nk; ++kk) {
        const float pj = p[kk];
        const T* row = tile + (size_t)kk * Rp;
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const int r = lane + 64 * i;
          if (r < R) acc[i] = fmaf(pj, El<T>::ld(row + r), acc[i]);
        }
      }
    }
  }
  if (live) {
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int r = lane + 64 * i;
      if (r < R) o[r] = acc[i] * inv;
    }
  }
}

template <typename T>
static void latent_attn_t(const void* qa, int64_t ldq, const void* cache, const void* bt, int maxb, const void* cu_q,
                          const void* ctx_lens, void* out, int64_t ldo, int T_, int B, int H, int R, int bs,
                          int window, float scale, hipStream_t st) {
  const int NW = std::min(H, 8);
  // row stride in LDS: an odd number of 4-byte words, so lanes scoring neighbouring keys hit different banks
  int Rp;
  if (sizeof(T) == 2) {
    Rp = (R + 1) & ~1;
    if (((Rp / 2) & 1) == 0) Rp += 2;
  } else {
    Rp = R | 1;
  }
  int KB = 64;
  auto bytes = [&](int kb) { return (((size_t)kb * Rp * sizeof(T) + 15) & ~(size_t)15) + (size_t)NW * (R + kb) * 4; };
  while (KB > 4 && bytes(KB) > 60 * 1024) KB >>= 1;
  if (bytes(KB) > 60 * 1024) throw std::runtime_error("latent attention: latent rank too large for LDS");
  dim3 g(T_, (H + NW - 1) / NW);
  const int nr = (R + 63) / 64;
#define LAUNCH_LA(NR_)                                                                                              \
  latent_attn_kernel<T, NR_><<<g, NW * 64, bytes(KB), st>>>((const float*)qa, ldq, (const T*)cache, (const int*)bt,  \
                                                            maxb, (const int*)cu_q, (const int*)ctx_lens,            \
                                                            (float*)out, ldo, B, H, R, bs, window, scale, KB, Rp)
  if (nr <= 1) LAUNCH_LA(1);
  else if (nr <= 2) LAUNCH_LA(2);
  else if (nr <= 4) LAUNCH_LA(4);
  else if (nr <= 8) LAUNCH_LA(8);
  else if (nr <= 16) LAUNCH_LA(16);
  else throw std::runtime_error("latent attention: latent rank above 1024");
#undef LAUNCH_LA
}

void launch_latent_attn(const void* qa, int64_t ldq, const void* cache, const void* bt, int maxb, const void* cu_q,
                        const void* ctx_lens, void* out, int64_t ldo, int T_, int B, int H, int R, int bs, int window,
                        float scale, int dt, hipStream_t st) {
  if (T_ == 0 || B == 0) return;
  if (T_ > 0 && (H + 7) / 8 > 65535) throw std::runtime_error("latent attention: too many heads");
  DISPATCH_T(dt, T, (latent_attn_t<T>(qa, ldq, cache, bt, maxb, cu_q, ctx_lens, out, ldo, T_, B, H, R, bs, window,
                                      scale, st)));
  HIP_CHECK_LAUNCH();
}
