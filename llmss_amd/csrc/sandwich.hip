// Blocks normed on both sides of a sublayer, over the fp32 residual stream x [T, W]:
//
//   sandwich_add_norm:  x += rms_norm(y * sigmoid(r + rb)) * wpost      y the sublayer's result, r its gate logits
//                       x += add                                        (optional fp32 rows)
//                       h  = rms_norm(x) * wnext                        (optional, in the storage type)
//   token_side_add:     e = table[id, col0 : col0 + d]; g = gelu_tanh(Wg x) * e; y = Wp g;
//                       x += rms_norm(y) * wn, then the same optional `add` and `h`
//
// so a sublayer's closing op also forms the next reader's input, as add_norm does for the uniform families. y is
// either a dense row in the storage type, or the still uncombined output of a mixture-of-experts layer (moe.hip):
// y[t] = sum_j (wts ? wts[t, j] : 1) * ey[place[t * top + j]] (+ shared[t]), j ascending, then the shared expert.
// Norm weights, biases and layer scales are fp32. One workgroup per row; the gated row lives in LDS between the
// pass that sums its squares and the pass that adds it, and the updated x between that pass and the norm.
#include "anytype.h"

struct SandwichArgs {
  float* x;
  const void* y;
  int64_t ldy;
  const float* ey;
  const int* place;
  const float* wts;
  int top;
  const void* shared_;
  int64_t lds_;
  const void* r;
  int64_t ldr;
  const float* rb;
  const float* wpost;
  const float* add;
  const float* wnext;
  void* h;
  int64_t ldh;
  float eps;
  int W;
};

template <typename T, int V>
__device__ __forceinline__ void ldv(const T* p, float* v) {
  if constexpr (V == 4 && sizeof(T) == 4) {
    const f32x4 q = *reinterpret_cast<const f32x4*>(p);
    v[0] = q[0], v[1] = q[1], v[2] = q[2], v[3] = q[3];
  } else if constexpr (V == 4) {
    const u16x4 q = *reinterpret_cast<const u16x4*>(p);
    v[0] = bf2f(q[0]), v[1] = bf2f(q[1]), v[2] = bf2f(q[2]), v[3] = bf2f(q[3]);
  } else {
    v[0] = El<T>::ld(p);
  }
}
template <typename T, int V>
__device__ __forceinline__ void stv(T* p, const float* v) {
  if constexpr (V == 4 && sizeof(T) == 4) {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
  } else if constexpr (V == 4) {
    *reinterpret_cast<u16x4*>(p) = u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
  } else {
    El<T>::st(p, v[0]);
  }
}

// the tail both kernels share: buf holds the updated x row; writes h = rms_norm(x) * wnext
template <typename T, int V>
__device__ __forceinline__ void norm_out(const float* buf, float ss, const SandwichArgs& p, int t, float* red) {
  if (!p.wnext) return;
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)p.W + p.eps);
  T* hr = (T*)p.h + (int64_t)t * p.ldh;
  for (int c = threadIdx.x * V; c < p.W; c += blockDim.x * V) {
    float w[V], o[V];
    ldv<float, V>(p.wnext + c, w);
#pragma unroll
    for (int i = 0; i < V; ++i) o[i] = buf[c + i] * inv * w[i];
    stv<T, V>(hr + c, o);
  }
}

template <typename T, int V>
__global__ __launch_bounds__(256) void sandwich_add_norm_kernel(SandwichArgs p) {
  extern __shared__ __attribute__((aligned(16))) float buf[];
  __shared__ float red[16];
  const int t = blockIdx.x, W = p.W;
  float* xr = p.x + (int64_t)t * W;
  const bool has_y = p.y != nullptr || p.ey != nullptr;
  float inv = 0.f;
  if (has_y) {
    const T* yr = p.y ? (const T*)p.y + (int64_t)t * p.ldy : nullptr;
    const T* sr = p.shared_ ? (const T*)p.shared_ + (int64_t)t * p.lds_ : nullptr;
    const T* rr = p.r ? (const T*)p.r + (int64_t)t * p.ldr : nullptr;
    float ss = 0.f;
    for (int c = threadIdx.x * V; c < W; c += blockDim.x * V) {
      float v[V];
      if (yr) {
        ldv<T, V>(yr + c, v);
      } else {
#pragma unroll
        for (int i = 0; i < V; ++i) v[i] = 0.f;
        for (int j = 0; j < p.top; ++j) {
          const float wj = p.wts ? p.wts[(int64_t)t * p.top + j] : 1.0f;
          float e[V];
          ldv<float, V>(p.ey + (int64_t)p.place[(int64_t)t * p.top + j] * W + c, e);
#pragma unroll
          for (int i = 0; i < V; ++i) v[i] = fmaf(wj, e[i], v[i]);
        }
        if (sr) {
          float e[V];
          ldv<T, V>(sr + c, e);
#pragma unroll
          for (int i = 0; i < V; ++i) v[i] += e[i];
        }
      }
      if (rr) {
        float z[V], b[V];
        ldv<T, V>(rr + c, z);
        ldv<float, V>(p.rb + c, b);
#pragma unroll
        for (int i = 0; i < V; ++i) v[i] = v[i] / (1.0f + expf(-(z[i] + b[i])));
      }
#pragma unroll
      for (int i = 0; i < V; ++i) {
        buf[c + i] = v[i];
        ss = fmaf(v[i], v[i], ss);
      }
    }
    ss = block_sum(ss, red);
    inv = 1.0f / sqrtf(ss / (float)W + p.eps);
  }
  const float* ar = p.add ? p.add + (int64_t)t * W : nullptr;
  float ss2 = 0.f;
  for (int c = threadIdx.x * V; c < W; c += blockDim.x * V) {
    float xv[V];
    ldv<float, V>(xr + c, xv);
    if (has_y) {
      float w[V];
      ldv<float, V>(p.wpost + c, w);
#pragma unroll
      for (int i = 0; i < V; ++i) xv[i] = fmaf(buf[c + i] * inv, w[i], xv[i]);
    }
    if (ar) {
      float a[V];
      ldv<float, V>(ar + c, a);
#pragma unroll
      for (int i = 0; i < V; ++i) xv[i] += a[i];
    }
    if (has_y || ar) stv<float, V>(xr + c, xv);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      buf[c + i] = xv[i];
      ss2 = fmaf(xv[i], xv[i], ss2);
    }
  }
  norm_out<T, V>(buf, ss2, p, t, red);
}

static bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

void launch_sandwich_add_norm(void* x, const void* y, int64_t ldy, const void* ey, const void* place, const void* wts,
                              int top, const void* shared_, int64_t lds_, const void* r, int64_t ldr, const void* rb,
                              const void* wpost, const void* add, const void* wnext, void* h, int64_t ldh, float eps,
                              int T_, int W, int dt, hipStream_t st) {
  if (T_ == 0) return;
  if ((size_t)W * 4 > 64 * 1024) throw std::runtime_error("sandwich_add_norm: rows wider than 16384");
  SandwichArgs p{(float*)x, y, ldy, (const float*)ey, (const int*)place, (const float*)wts, top, shared_, lds_, r, ldr,
                 (const float*)rb, (const float*)wpost, (const float*)add, (const float*)wnext, h, ldh, eps, W};
  const int es = dt == 0 ? 2 : 4;
  const auto alv = [&](const void* q, int64_t ld) { return !q || (((uintptr_t)q % (4 * es)) == 0 && ld % 4 == 0); };
  const bool vec = W % 4 == 0 && al16(x) && al16(ey) && al16(rb) && al16(wpost) && al16(add) && al16(wnext) &&
                   alv(y, ldy) && alv(shared_, lds_) && alv(r, ldr) && alv(h, ldh);
  const size_t lds = (size_t)W * 4;
  DISPATCH_T(dt, T, {
    if (vec) sandwich_add_norm_kernel<T, 4><<<T_, 256, lds, st>>>(p);
    else sandwich_add_norm_kernel<T, 1><<<T_, 256, lds, st>>>(p);
  });
  HIP_CHECK_LAUNCH();
}

struct SideArgs {
  const int64_t* ids;
  const void* table;  // [vocab, ldt] in the storage type
  int64_t ldt;
  int vocab, col0, d;
  const void* wg;  // [d, W]
  const void* wp;  // [W, d]
  const float* wn;
};

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// buf: [W] the x row, then [W] the projected row, then [d] the gated numbers
template <typename T, int V>
__global__ __launch_bounds__(512) void token_side_add_kernel(SandwichArgs p, SideArgs s) {
  extern __shared__ __attribute__((aligned(16))) float buf[];
  __shared__ float red[16];
  const int t = blockIdx.x, W = p.W, d = s.d;
  float* xs = buf;
  float* ys = buf + W;
  float* gs = ys + W;
  float* xr = p.x + (int64_t)t * W;
  for (int c = threadIdx.x * V; c < W; c += blockDim.x * V) {
    float v[V];
    ldv<float, V>(xr + c, v);
#pragma unroll
    for (int i = 0; i < V; ++i) xs[c + i] = v[i];
  }
  __syncthreads();
  int64_t id = s.ids[t];
  id = id < 0 ? 0 : (id >= s.vocab ? s.vocab - 1 : id);
  const T* er = (const T*)s.table + id * s.ldt + s.col0;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  for (int j = wv; j < d; j += nw) {  // a wave per gate row, lanes over the width
    const T* wr = (const T*)s.wg + (int64_t)j * W;
    float a = 0.f;
    for (int c = lane * V; c < W; c += 64 * V) {
      float w[V];
      ldv<T, V>(wr + c, w);
#pragma unroll
      for (int i = 0; i < V; ++i) a = fmaf(w[i], xs[c + i], a);
    }
    a = warp_sum(a);
    if (lane == 0) gs[j] = gelu_tanh_f(a) * El<T>::ld(er + j);
  }
  __syncthreads();
  float ss = 0.f;
  const bool rows16 = sizeof(T) == 2 && d % 8 == 0 && ((uintptr_t)s.wp & 15) == 0;  // 16-byte reads of a bf16 row
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const T* wr = (const T*)s.wp + (int64_t)c * d;
    float a = 0.f, a2 = 0.f;
    if (rows16) {
      for (int j = 0; j < d; j += 8) {
        const u16x8 w8 = *reinterpret_cast<const u16x8*>(wr + j);
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
          a = fmaf(bf2f(w8[i]), gs[j + i], a);
          a2 = fmaf(bf2f(w8[i + 1]), gs[j + i + 1], a2);
        }
      }
      a += a2;
    } else {
      for (int j = 0; j < d; ++j) a = fmaf(El<T>::ld(wr + j), gs[j], a);
    }
    ys[c] = a;
    ss = fmaf(a, a, ss);
  }
  ss = block_sum(ss, red);  // (its barriers also make ys visible)
  const float inv = 1.0f / sqrtf(ss / (float)W + p.eps);
  const float* ar = p.add ? p.add + (int64_t)t * W : nullptr;
  float ss2 = 0.f;
  for (int c = threadIdx.x * V; c < W; c += blockDim.x * V) {
    float xv[V], w[V];
    ldv<float, V>(s.wn + c, w);
#pragma unroll
    for (int i = 0; i < V; ++i) xv[i] = fmaf(ys[c + i] * inv, w[i], xs[c + i]);
    if (ar) {
      float a[V];
      ldv<float, V>(ar + c, a);
#pragma unroll
      for (int i = 0; i < V; ++i) xv[i] += a[i];
    }
    stv<float, V>(xr + c, xv);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      xs[c + i] = xv[i];
      ss2 = fmaf(xv[i], xv[i], ss2);
    }
  }
  norm_out<T, V>(xs, ss2, p, t, red);
}

void launch_token_side_add(void* x, const void* ids, const void* table, int64_t ldt, int vocab, int col0, int d,
                           const void* wg, const void* wp, const void* wn, const void* add, const void* wnext, void* h,
                           int64_t ldh, float eps, int T_, int W, int dt, hipStream_t st) {
  if (T_ == 0) return;
  const size_t lds = ((size_t)2 * W + d) * 4;
  if (lds > 64 * 1024) throw std::runtime_error("token_side_add: rows too wide");
  SandwichArgs p{};
  p.x = (float*)x; p.add = (const float*)add; p.wnext = (const float*)wnext; p.h = h; p.ldh = ldh; p.eps = eps; p.W = W;
  SideArgs s{(const int64_t*)ids, table, ldt, vocab, col0, d, wg, wp, (const float*)wn};
  const int es = dt == 0 ? 2 : 4;
  const bool vec = W % 4 == 0 && al16(x) && al16(wn) && al16(add) && al16(wnext) && ((uintptr_t)wg % (4 * es)) == 0 &&
                   (!h || (((uintptr_t)h % (4 * es)) == 0 && ldh % 4 == 0));
  DISPATCH_T(dt, T, {
    if (vec) token_side_add_kernel<T, 4><<<T_, 512, lds, st>>>(p, s);
    else token_side_add_kernel<T, 1><<<T_, 512, lds, st>>>(p, s);
  });
  HIP_CHECK_LAUNCH();
}
