// A residual stream kept in fp32: scaled embedding gather and the fused "residual add + RMS norm" whose norm
// weight may be stored around zero (y = x / rms(x) * (offset + w), offset 1) or plainly (offset 0).
//
// The other families keep their residual in bf16 (norm.hip add_norm); designs that define the residual sum in
// 32-bit use these kernels instead: the stream x [T, H] is fp32 and updated in place, only the normed output that
// feeds the matrix products is rounded to the model's storage type.
#include "anytype.h"
#include "seqrows.h"

// x[t, :] = table[ids[t], :] * scale
template <typename T>
__global__ __launch_bounds__(256) void embed_scaled_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                           float* __restrict__ x, int H, int vocab, float scale) {
  const int t = blockIdx.x;
  int64_t id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* src = table + id * (int64_t)H;
  float* dst = x + (int64_t)t * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) dst[c] = El<T>::ld(src + c) * scale;
}

void launch_embed_scaled(const void* ids, const void* table, void* x, int T_, int H, int vocab, float scale, int dt,
                         hipStream_t st) {
  if (T_ == 0) return;
  DISPATCH_T(dt, T, (embed_scaled_kernel<T><<<T_, 256, 0, st>>>((const int64_t*)ids, (const T*)table, (float*)x, H,
                                                                  vocab, scale)));
  HIP_CHECK_LAUNCH();
}

// x[t] += (a[t] + f[t])   (either addend may be absent; a in the storage type)
// y[t]  = x[t] * rsqrt(mean(x[t]^2) + eps) * (woff + w)      (skipped when y is null)
// The sum is formed as x + (a + f): the two sublayer outputs of a parallel block are added to each other first.
// f is either a dense fp32 row b[t], or the still uncombined output of a mixture-of-experts layer (moe.hip):
//   f[t] = sum_j wts[t, j] * ey[place[t * top + j]] (+ shared[t])        j ascending, then the shared expert
// so the expert outputs are weighted, summed and added to the stream in this one pass.
// VEC: H % 4 == 0 and every row 16-byte (fp32) / 8-byte (bf16) aligned - four elements per lane and access.
struct ResidArgs {
  float* x;
  const void* a;
  int64_t lda;
  const float* b;
  int64_t ldb;
  const float* ey;
  const int* place;
  const float* wts;
  int top;
  const void* shared_;
  int64_t lds_;
  const void* w;
  float woff, eps;
  void* y;
  int64_t ldy;
  int H;
};

template <typename T>
__device__ __forceinline__ f32x4 ld4(const T* p);
template <>
__device__ __forceinline__ f32x4 ld4<float>(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
template <>
__device__ __forceinline__ f32x4 ld4<bf16_t>(const bf16_t* p) {
  const u16x4 v = *reinterpret_cast<const u16x4*>(p);
  return f32x4{bf2f(v[0]), bf2f(v[1]), bf2f(v[2]), bf2f(v[3])};
}
template <typename T>
__device__ __forceinline__ void st4(T* p, f32x4 v);
template <>
__device__ __forceinline__ void st4<float>(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }
template <>
__device__ __forceinline__ void st4<bf16_t>(bf16_t* p, f32x4 v) {
  *reinterpret_cast<u16x4*>(p) = u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
}

template <typename T, int V>  // V = elements per lane and access: 4 (vector) or 1
__global__ __launch_bounds__(256) void resid_add_norm_kernel(ResidArgs p) {
  __shared__ float red[16];
  const int t = blockIdx.x, H = p.H;
  float* xr = p.x + (int64_t)t * H;
  const T* ar = p.a ? (const T*)p.a + (int64_t)t * p.lda : nullptr;
  const float* br = p.b ? p.b + (int64_t)t * p.ldb : nullptr;
  const T* sr = p.shared_ ? (const T*)p.shared_ + (int64_t)t * p.lds_ : nullptr;
  const bool moe = p.ey != nullptr;
  const bool add = ar || br || moe;
  float ss = 0.f;
  for (int c = threadIdx.x * V; c < H; c += blockDim.x * V) {
    float v[V];
    if constexpr (V == 4) {
      const f32x4 q = *reinterpret_cast<const f32x4*>(xr + c);
      v[0] = q[0]; v[1] = q[1]; v[2] = q[2]; v[3] = q[3];
    } else {
      v[0] = xr[c];
    }
    if (add) {
      float f[V];
      bool hasf = false;
#pragma unroll
      for (int i = 0; i < V; ++i) f[i] = 0.f;
      if (moe) {
        hasf = true;
        for (int j = 0; j < p.top; ++j) {
          const float wj = p.wts[(int64_t)t * p.top + j];
          const float* er = p.ey + (int64_t)p.place[(int64_t)t * p.top + j] * H + c;
          if constexpr (V == 4) {
            const f32x4 e = *reinterpret_cast<const f32x4*>(er);
#pragma unroll
            for (int i = 0; i < 4; ++i) f[i] = fmaf(wj, e[i], f[i]);
          } else {
            f[0] = fmaf(wj, er[0], f[0]);
          }
        }
        if (sr) {
          if constexpr (V == 4) {
            const f32x4 e = ld4<T>(sr + c);
#pragma unroll
            for (int i = 0; i < 4; ++i) f[i] += e[i];
          } else {
            f[0] += El<T>::ld(sr + c);
          }
        }
      } else if (br) {
        hasf = true;
        if constexpr (V == 4) {
          const f32x4 e = *reinterpret_cast<const f32x4*>(br + c);
          f[0] = e[0]; f[1] = e[1]; f[2] = e[2]; f[3] = e[3];
        } else {
          f[0] = br[c];
        }
      }
      if (ar) {
        float av[V];
        if constexpr (V == 4) {
          const f32x4 e = ld4<T>(ar + c);
          av[0] = e[0]; av[1] = e[1]; av[2] = e[2]; av[3] = e[3];
        } else {
          av[0] = El<T>::ld(ar + c);
        }
#pragma unroll
        for (int i = 0; i < V; ++i) f[i] = hasf ? av[i] + f[i] : av[i];
      }
#pragma unroll
      for (int i = 0; i < V; ++i) v[i] += f[i];
      if constexpr (V == 4) *reinterpret_cast<f32x4*>(xr + c) = f32x4{v[0], v[1], v[2], v[3]};
      else xr[c] = v[0];
    }
#pragma unroll
    for (int i = 0; i < V; ++i) ss += v[i] * v[i];
  }
  if (!p.y) return;
  const float tot = block_sum(ss, red);
  const float r = 1.0f / sqrtf(tot / (float)H + p.eps);
  T* yr = (T*)p.y + (int64_t)t * p.ldy;
  const T* w = (const T*)p.w;
  for (int c = threadIdx.x * V; c < H; c += blockDim.x * V) {
    // each thread re-reads the elements it wrote itself
    if constexpr (V == 4) {
      const f32x4 q = *reinterpret_cast<const f32x4*>(xr + c);
      const f32x4 wv = ld4<T>(w + c);
      st4<T>(yr + c, f32x4{q[0] * r * (p.woff + wv[0]), q[1] * r * (p.woff + wv[1]), q[2] * r * (p.woff + wv[2]),
                           q[3] * r * (p.woff + wv[3])});
    } else {
      El<T>::st(yr + c, xr[c] * r * (p.woff + El<T>::ld(w + c)));
    }
  }
}

void launch_resid_add_norm(void* x, const void* a, int64_t lda, const void* b, int64_t ldb, const void* ey,
                           const void* place, const void* wts, int top, const void* shared_, int64_t lds_,
                           const void* w, float woff, float eps, void* y, int64_t ldy, int T_, int H, int dt,
                           hipStream_t st) {
  if (T_ == 0) return;
  ResidArgs p{(float*)x, a, lda, (const float*)b, ldb, (const float*)ey, (const int*)place, (const float*)wts, top,
              shared_, lds_, w, woff, eps, y, ldy, H};
  const int es = dt == 0 ? 2 : 4;
  auto al = [&](const void* q, int64_t ld, int bytes) { return !q || (((uintptr_t)q | (uintptr_t)(ld * bytes)) % (4 * bytes)) == 0; };
  const bool vec = H % 4 == 0 && al(x, H, 4) && al(a, lda, es) && al(b, ldb, 4) && al(ey, H, 4) && al(shared_, lds_, es) &&
                   al(w, 4, es) && al(y, ldy, es);
  DISPATCH_T(dt, T, {
    if (vec) resid_add_norm_kernel<T, 4><<<T_, 256, 0, st>>>(p);
    else resid_add_norm_kernel<T, 1><<<T_, 256, 0, st>>>(p);
  });
  HIP_CHECK_LAUNCH();
}

// ---- blocks whose norm sits on the sublayer's output, results of the layers averaged over depth, bigram embedding
//
// The layers' results live in hist [slots, T, W] fp32 (slot stride ldh). Layer i works in place on hist[i + 1], which
// the step before has filled with the layer's input.

// hist[0][t] = hist[1][t] = table[ids[t]] * scale + bigram[row],
//   row = (before * mul_prev + ids[t] * mul_cur) mod buckets, or `buckets` (the table's last row) at position 0.
// `before` is the row above inside a portion and prev[slot] for a portion's first row; that workgroup then sets
// prev[slot] to the portion's last token (it has read the old value: one workgroup, a barrier in between).
template <typename T>
__global__ __launch_bounds__(256) void embed_bigram_kernel(const int64_t* __restrict__ ids,
                                                           const int64_t* __restrict__ positions,
                                                           const T* __restrict__ table, float scale,
                                                           const T* __restrict__ bigram, int64_t buckets,
                                                           int64_t mul_prev, int64_t mul_cur, int64_t* __restrict__ prev,
                                                           const int* __restrict__ cu, const int* __restrict__ ctx,
                                                           const int* __restrict__ sslots, int B,
                                                           float* __restrict__ h0, float* __restrict__ h1, int W,
                                                           int vocab) {
  const int t = blockIdx.x;
  const RowSeq r = row_seq(cu, ctx, B, t);
  float* d0 = h0 + (int64_t)t * W;
  float* d1 = h1 + (int64_t)t * W;
  if (r.pos < 0) {  // a padded row
    for (int c = threadIdx.x; c < W; c += blockDim.x) d0[c] = d1[c] = 0.f;
    return;
  }
  auto clampv = [&](int64_t id) { return id < 0 ? (int64_t)0 : (id >= vocab ? (int64_t)vocab - 1 : id); };
  const int64_t id = clampv(ids[t]);
  const int slot = sslots[r.b];
  int64_t before = 0;
  if (r.j > 0) before = clampv(ids[t - 1]);
  else if (r.pos > 0 && slot >= 0) before = prev[slot];
  int64_t row = (before * mul_prev + id * mul_cur) % buckets;
  if (row < 0) row += buckets;
  if (positions[t] == 0) row = buckets;
  if (r.j == 0 && slot >= 0) {
    __syncthreads();  // every thread holds the old value
    if (threadIdx.x == 0) prev[slot] = clampv(ids[t + r.qlen - 1]);
  }
  const T* src = table + id * (int64_t)W;
  const T* bg = bigram + row * (int64_t)W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = fmaf(El<T>::ld(src + c), scale, El<T>::ld(bg + c));
    d0[c] = v;
    d1[c] = v;
  }
}

void launch_embed_bigram(const void* ids, const void* positions, const void* table, float scale, const void* bigram,
                         int64_t buckets, int64_t mul_prev, int64_t mul_cur, void* prev, const void* cu,
                         const void* ctx, const void* sslots, int B, void* h0, void* h1, int T_, int W, int vocab,
                         int dt, hipStream_t st) {
  if (T_ == 0) return;
  if (buckets < 1) throw std::runtime_error("embed_bigram: at least one bucket");
  DISPATCH_T(dt, T, (embed_bigram_kernel<T><<<T_, 256, 0, st>>>(
      (const int64_t*)ids, (const int64_t*)positions, (const T*)table, scale, (const T*)bigram, buckets, mul_prev,
      mul_cur, (int64_t*)prev, (const int*)cu, (const int*)ctx, (const int*)sslots, B, (float*)h0, (float*)h1, W,
      vocab)));
  HIP_CHECK_LAUNCH();
}

// x = hist[n][t] += y[t] / sqrt(mean(y[t]^2) + eps) * w; with dwa also hist[n + 1][t] = sum_{j <= n} dwa[j] hist[j][t]
// (over the updated x). The mean square is summed in fp32 from y in the storage type.
template <typename T, int V>
__global__ __launch_bounds__(256) void resid_norm_add_kernel(float* __restrict__ hist, int64_t ldh, int n,
                                                             const T* __restrict__ y, int64_t ldy,
                                                             const T* __restrict__ w, float eps,
                                                             const float* __restrict__ dwa, int W) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  const T* yr = y + (int64_t)t * ldy;
  float ss = 0.f;
  for (int c = threadIdx.x * V; c < W; c += blockDim.x * V) {
    if constexpr (V == 4) {
      const f32x4 q = ld4<T>(yr + c);
      ss += q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3];
    } else {
      const float q = El<T>::ld(yr + c);
      ss += q * q;
    }
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)W + eps);
  float* xr = hist + (int64_t)n * ldh + (int64_t)t * W;
  float* nx = xr + ldh;
  const float wn = dwa ? dwa[n] : 0.f;
  for (int c = threadIdx.x * V; c < W; c += blockDim.x * V) {
    if constexpr (V == 4) {
      const f32x4 q = ld4<T>(yr + c), wv = ld4<T>(w + c);
      f32x4 x = *reinterpret_cast<const f32x4*>(xr + c);
#pragma unroll
      for (int i = 0; i < 4; ++i) x[i] += q[i] * inv * wv[i];
      *reinterpret_cast<f32x4*>(xr + c) = x;
      if (dwa) {
        f32x4 a = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < n; ++j) {
          const float wj = dwa[j];
          const f32x4 e = *reinterpret_cast<const f32x4*>(hist + (int64_t)j * ldh + (int64_t)t * W + c);
#pragma unroll
          for (int i = 0; i < 4; ++i) a[i] = fmaf(wj, e[i], a[i]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = fmaf(wn, x[i], a[i]);
        *reinterpret_cast<f32x4*>(nx + c) = a;
      }
    } else {
      const float x = xr[c] + El<T>::ld(yr + c) * inv * El<T>::ld(w + c);
      xr[c] = x;
      if (dwa) {
        float a = 0.f;
        for (int j = 0; j < n; ++j) a = fmaf(dwa[j], hist[(int64_t)j * ldh + (int64_t)t * W + c], a);
        nx[c] = fmaf(wn, x, a);
      }
    }
  }
}

void launch_resid_norm_add(void* hist, int64_t ldh, int n, const void* y, int64_t ldy, const void* w, float eps,
                           const void* dwa, int T_, int W, int dt, hipStream_t st) {
  if (T_ == 0) return;
  const int es = dt == 0 ? 2 : 4;
  const bool vec = W % 4 == 0 && ldh % 4 == 0 && ((uintptr_t)hist % 16) == 0 && ((uintptr_t)y % (4 * es)) == 0 &&
                   (ldy * es) % (4 * es) == 0 && ((uintptr_t)w % (4 * es)) == 0;
  DISPATCH_T(dt, T, {
    if (vec) resid_norm_add_kernel<T, 4><<<T_, 256, 0, st>>>((float*)hist, ldh, n, (const T*)y, ldy, (const T*)w, eps,
                                                             (const float*)dwa, W);
    else resid_norm_add_kernel<T, 1><<<T_, 256, 0, st>>>((float*)hist, ldh, n, (const T*)y, ldy, (const T*)w, eps,
                                                         (const float*)dwa, W);
  });
  HIP_CHECK_LAUNCH();
}

// y[t, c] *= sigmoid(src[t, col + c])
template <typename T>
__global__ __launch_bounds__(256) void gate_mul_kernel(T* __restrict__ y, int64_t ldy, const T* __restrict__ src,
                                                       int64_t lds_, int N) {
  const int t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < N; c += gridDim.y * blockDim.x) {
    const float g = El<T>::ld(src + (int64_t)t * lds_ + c);
    T* p = y + (int64_t)t * ldy + c;
    El<T>::st(p, El<T>::ld(p) / (1.0f + expf(-g)));
  }
}

// The same for bf16 rows made of whole 16-byte pieces: eight numbers per thread and access.
__global__ __launch_bounds__(256) void gate_mul_vec_kernel(bf16_t* __restrict__ y, int64_t ldy,
                                                           const bf16_t* __restrict__ src, int64_t lds_, int N) {
  const int t = blockIdx.x;
  for (int c = (blockIdx.y * blockDim.x + threadIdx.x) * 8; c < N; c += gridDim.y * blockDim.x * 8) {
    const u16x8 gv = *reinterpret_cast<const u16x8*>(src + (int64_t)t * lds_ + c);
    u16x8* p = reinterpret_cast<u16x8*>(y + (int64_t)t * ldy + c);
    u16x8 v = *p;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = f2bf(bf2f(v[i]) / (1.0f + expf(-bf2f(gv[i]))));
    *p = v;
  }
}

void launch_gate_mul(void* y, int64_t ldy, const void* src, int64_t lds_, int T_, int N, int dt, hipStream_t st) {
  if (T_ == 0 || N == 0) return;
  if (dt == 0 && N % 8 == 0 && ldy % 8 == 0 && lds_ % 8 == 0 && ((uintptr_t)y & 15) == 0 && ((uintptr_t)src & 15) == 0) {
    dim3 g(T_, std::min(64, (N / 8 + 255) / 256));
    gate_mul_vec_kernel<<<g, 256, 0, st>>>((bf16_t*)y, ldy, (const bf16_t*)src, lds_, N);
    HIP_CHECK_LAUNCH();
    return;
  }
  dim3 g(T_, std::min(64, (N + 255) / 256));
  DISPATCH_T(dt, T, (gate_mul_kernel<T><<<g, 256, 0, st>>>((T*)y, ldy, (const T*)src, lds_, N)));
  HIP_CHECK_LAUNCH();
}
