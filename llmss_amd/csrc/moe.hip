// Mixture-of-experts feed-forward: routing, grouping of (token, expert) pairs and the grouped expert GEMMs.
//
//   z = W_router h (fp32, gemm_any)                                   [T, E]
//   moe_route:   s = sigmoid(z); the `top` experts with the largest s + correction are chosen (ties: the lower
//                index); weights = chosen s / (their sum + 1e-20)     -> idx [T, top] int32, wts [T, top] fp32
//   moe_group:   pairs p = t * top + j are bucketed by expert: off [E + 1], order [P] (pair at each sorted row),
//                place [P] (sorted row of each pair) and a flat list of row tiles (expert, first row; 64 or 128 rows each) so the
//                grouped GEMMs launch a grid whose size is known on the host (ceil(P / rows) + E tiles at most)
//   moe_gate_up: act[r, f] = glu(h[token(r)] . gate_e[f], h[token(r)] . up_e[f])   for sorted row r of expert e
//   moe_down:    y[r, n] = act[r, :] . down_e[n, :]                   (fp32)
//   moe_combine: out[t, :] = sum_j wts[t, j] * y[place[t * top + j], :] (+ shared[t, :])   (fp32, j ascending;
//                no wts: the plain sum, for layers whose weights went onto the experts' inputs in moe_gate_up)
//
// Expert activation (clamped, gated): g = min(g, limit), u = clamp(u, -limit, limit),
// glu = g * sigmoid(alpha * g) * (u + 1). glu_clamp applies the same to a dense [T, 2F] gate|up product (the
// shared expert, which runs through the ordinary GEMMs).
//
// Nothing here synchronises with the host: group sizes stay on the device, so a decode step with experts can be
// captured into a HIP graph. Every pair's row is computed alone, so a token's result does not depend on what else
// is in the step.
#include "anytype.h"
#include "tile_valu.h"

__device__ __forceinline__ float glu_clamped(float g, float u, float limit, float alpha) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + 1.f);
}
// silu: the plain gated form silu(g) * u, no clamps
__device__ __forceinline__ float glu_value(float g, float u, float limit, float alpha, int silu) {
  return silu ? g / (1.f + expf(-g)) * u : glu_clamped(g, u, limit, alpha);
}

// ------------------------------------------------------------------------------------------------ routing
// one wave per token; lanes over experts
__global__ __launch_bounds__(64) void moe_route_kernel(const float* __restrict__ z, const float* __restrict__ corr,
                                                       int* __restrict__ idx, float* __restrict__ wts, int E, int top,
                                                       int norm) {
  extern __shared__ float sc[];  // [E] scores, [E] choice values
  float* ch = sc + E;
  const int t = blockIdx.x, lane = threadIdx.x;
  for (int e = lane; e < E; e += 64) {
    const float s = 1.f / (1.f + expf(-z[(int64_t)t * E + e]));
    sc[e] = s;
    ch[e] = s + (corr ? corr[e] : 0.f);
  }
  __syncthreads();
  float sum = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = ch[e];
      if (v > best || (v == best && e < bi)) {
        best = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) {
        best = ov;
        bi = oi;
      }
    }
    if (bi >= E) bi = 0;  // every value NaN: keep indices in range
    const float s = sc[bi];
    sum += s;
    if (lane == 0) {
      idx[(int64_t)t * top + j] = bi;
      wts[(int64_t)t * top + j] = s;
      ch[bi] = -INFINITY;
    }
    __syncthreads();
  }
  if (!norm) return;  // the chosen scores themselves
  const float inv = 1.f / (sum + 1e-20f);
  for (int j = lane; j < top; j += 64) wts[(int64_t)t * top + j] *= inv;
}

void launch_moe_route(const void* z, const void* corr, void* idx, void* wts, int T_, int E, int top, int norm,
                      hipStream_t st) {
  if (T_ == 0) return;
  if (top > E || top <= 0) throw std::runtime_error("moe_route: top must be in [1, experts]");
  moe_route_kernel<<<T_, 64, 2 * E * sizeof(float), st>>>((const float*)z, (const float*)corr, (int*)idx, (float*)wts,
                                                           E, top, norm);
  HIP_CHECK_LAUNCH();
}

// Router logits and routing in one launch, for steps of few tokens (a decode step): one workgroup per token, its waves
// share the experts' dot products z_e = h . W_r[e] (fp32 accumulation over lanes), then the token is routed
// as moe_route_kernel does. A prompt's thousands of tokens take the matrix-core GEMM and moe_route instead.
template <typename T>
__global__ __launch_bounds__(1024) void moe_router_kernel(const T* __restrict__ h, int64_t ldh, const T* __restrict__ wr,
                                                         const float* __restrict__ corr, int* __restrict__ idx,
                                                         float* __restrict__ wts, int E, int K, int top, bool vec,
                                                         int norm) {
  extern __shared__ float sc[];  // [E] scores, [E] choice values
  float* ch = sc + E;
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, nw = blockDim.x >> 6;
  const T* x = h + (int64_t)t * ldh;
  for (int e = wv; e < E; e += nw) {
    const T* w = wr + (int64_t)e * K;
    float acc = 0.f;
    if (vec) {  // K % 8 == 0, rows 16-byte aligned (bf16) - eight elements per lane and access
      for (int k = lane * 8; k < K; k += 512) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = fmaf(El<T>::ld(x + k + i), El<T>::ld(w + k + i), acc);
      }
    } else {
      for (int k = lane; k < K; k += 64) acc = fmaf(El<T>::ld(x + k), El<T>::ld(w + k), acc);
    }
    acc = warp_sum(acc);
    if (lane == 0) {
      const float s = 1.f / (1.f + expf(-acc));
      sc[e] = s;
      ch[e] = s + (corr ? corr[e] : 0.f);
    }
  }
  __syncthreads();
  float sum = 0.f;
  for (int j = 0; j < top; ++j) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = ch[e];
      if (v > best || (v == best && e < bi)) {
        best = v;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > best || (ov == best && oi < bi)) {
        best = ov;
        bi = oi;
      }
    }
    if (bi >= E) bi = 0;
    const float s = sc[bi];
    sum += s;
    __syncthreads();  // every wave has read ch before the winner is struck out
    if (tid == 0) {
      idx[(int64_t)t * top + j] = bi;
      wts[(int64_t)t * top + j] = s;
      ch[bi] = -INFINITY;
    }
    __syncthreads();
  }
  if (!norm) return;
  const float inv = 1.f / (sum + 1e-20f);
  for (int j = tid; j < top; j += blockDim.x) wts[(int64_t)t * top + j] *= inv;
}

void launch_moe_router(const void* h, int64_t ldh, const void* wr, const void* corr, void* idx, void* wts, int T_,
                       int E, int K, int top, int dt, int norm, hipStream_t st) {
  if (T_ == 0) return;
  if (top > E || top <= 0) throw std::runtime_error("moe_router: top must be in [1, experts]");
  const int es = dt == 0 ? 2 : 4;
  const bool vec = K % 8 == 0 && ((uintptr_t)h % 16) == 0 && ((uintptr_t)wr % 16) == 0 && (ldh * es) % 16 == 0;
  const int threads = E >= 16 ? 1024 : (E >= 8 ? 512 : 256);  // a wave per expert up to 16 waves
  DISPATCH_T(dt, T, (moe_router_kernel<T><<<T_, threads, 2 * E * sizeof(float), st>>>(
                        (const T*)h, ldh, (const T*)wr, (const float*)corr, (int*)idx, (float*)wts, E, K, top, vec,
                        norm)));
  HIP_CHECK_LAUNCH();
}

// ------------------------------------------------------------------------------------------------ grouping
// One workgroup. meta = [ntiles | off[E + 1] | tile_expert[maxt] | tile_row0[maxt]], order [P], place [P].
__global__ __launch_bounds__(1024) void moe_group_kernel(const int* __restrict__ idx, int P, int E, int maxt,
                                                         int* __restrict__ meta, int* __restrict__ order,
                                                         int* __restrict__ place, int tile_rows) {
  extern __shared__ int sm[];  // cnt[E], cur[E]
  int* cnt = sm;
  int* cur = sm + E;
  int* off = meta + 1;
  int* tile_e = meta + 1 + (E + 1);
  int* tile_r = tile_e + maxt;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) atomicAdd(&cnt[idx[p]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int o = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      off[e] = o;
      cur[e] = o;
      for (int r = 0; r < cnt[e]; r += tile_rows) {
        if (nt < maxt) {
          tile_e[nt] = e;
          tile_r[nt] = o + r;
        }
        ++nt;
      }
      o += cnt[e];
    }
    off[E] = o;
    meta[0] = nt < maxt ? nt : maxt;
  }
  __syncthreads();
  // rows within an expert take whatever order the atomics give: every pair's row is computed on its own, so the
  // values do not depend on where the row lands
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    const int o = atomicAdd(&cur[idx[p]], 1);
    order[o] = p;
    place[p] = o;
  }
}

void launch_moe_group(const void* idx, int P, int E, int maxt, void* meta, void* order, void* place, int tile_rows,
                      hipStream_t st) {
  if (P == 0) return;
  if (tile_rows <= 0) throw std::runtime_error("moe_group: tile rows");
  if (E > 4096) throw std::runtime_error("moe_group: more than 4096 experts");
  moe_group_kernel<<<1, 1024, 2 * E * sizeof(int), st>>>((const int*)idx, P, E, maxt, (int*)meta, (int*)order,
                                                          (int*)place, tile_rows);
  HIP_CHECK_LAUNCH();
}

// ------------------------------------------------------------------------------------------------ grouped GEMMs
// grid (ceil(F / 64), maxt): tile y of the list covers sorted rows [row0, min(row0 + 64, off[e + 1])) of expert e.
template <typename T>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const T* __restrict__ h, int64_t ldh,
                                                          const T* __restrict__ wg, const T* __restrict__ wu,
                                                          const int* __restrict__ meta, const int* __restrict__ order,
                                                          T* __restrict__ act, int E, int maxt, int top, int F, int K,
                                                          float limit, float alpha, const float* __restrict__ pw,
                                                          int silu) {
  __shared__ float As[TV_BK][TV_LD];
  __shared__ float Gs[TV_BK][TV_LD];
  __shared__ float Us[TV_BK][TV_LD];
  if ((int)blockIdx.y >= meta[0]) return;
  const int* off = meta + 1;
  const int e = meta[1 + (E + 1) + blockIdx.y];
  const int row0 = meta[1 + (E + 1) + maxt + blockIdx.y];
  const int rows = min(TV_BM, off[e + 1] - row0);
  const int n0 = blockIdx.x * TV_BN;
  const int tid = threadIdx.x;
  const T* G = wg + (int64_t)e * F * K;
  const T* U = wu + (int64_t)e * F * K;
  const int r = tid >> 2, kq = (tid & 3) * 4;
  const T* arow = r < rows ? h + (int64_t)(order[row0 + r] / top) * ldh : nullptr;
  const int n = n0 + r;
  float ag[4][4] = {}, au[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += TV_BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + kq + i;
      const bool kin = k < K;
      As[kq + i][r] = (arow && kin) ? El<T>::ld(arow + k) : 0.f;
      Gs[kq + i][r] = (n < F && kin) ? El<T>::ld(G + (int64_t)n * K + k) : 0.f;
      Us[kq + i][r] = (n < F && kin) ? El<T>::ld(U + (int64_t)n * K + k) : 0.f;
    }
    __syncthreads();
    tv_mac(ag, As, Gs, tid);
    tv_mac(au, As, Us, tid);
    __syncthreads();
  }
  const int tx = tid & 15, ty = tid >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = ty * 4 + i;
    if (m >= rows) continue;
    const float sw = pw ? pw[order[row0 + m]] : 1.0f;  // the pair's weight on the expert's input
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int f = n0 + tx * 4 + j;
      if (f < F) El<T>::st(act + (int64_t)(row0 + m) * F + f, glu_value(ag[i][j] * sw, au[i][j] * sw, limit, alpha, silu));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(const T* __restrict__ act, const T* __restrict__ wd,
                                                       const int* __restrict__ meta, float* __restrict__ y, int E,
                                                       int maxt, int N, int F) {
  __shared__ float As[TV_BK][TV_LD];
  __shared__ float Bs[TV_BK][TV_LD];
  if ((int)blockIdx.y >= meta[0]) return;
  const int* off = meta + 1;
  const int e = meta[1 + (E + 1) + blockIdx.y];
  const int row0 = meta[1 + (E + 1) + maxt + blockIdx.y];
  const int rows = min(TV_BM, off[e + 1] - row0);
  const int n0 = blockIdx.x * TV_BN;
  const int tid = threadIdx.x;
  const T* W = wd + (int64_t)e * N * F;
  const int r = tid >> 2, kq = (tid & 3) * 4;
  const T* arow = r < rows ? act + (int64_t)(row0 + r) * F : nullptr;
  const int n = n0 + r;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < F; k0 += TV_BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int k = k0 + kq + i;
      const bool kin = k < F;
      As[kq + i][r] = (arow && kin) ? El<T>::ld(arow + k) : 0.f;
      Bs[kq + i][r] = (n < N && kin) ? El<T>::ld(W + (int64_t)n * F + k) : 0.f;
    }
    __syncthreads();
    tv_mac(acc, As, Bs, tid);
    __syncthreads();
  }
  const int tx = tid & 15, ty = tid >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = ty * 4 + i;
    if (m >= rows) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = n0 + tx * 4 + j;
      if (c < N) y[(int64_t)(row0 + m) * N + c] = acc[i][j];
    }
  }
}

void launch_moe_gate_up(const void* h, int64_t ldh, const void* wg, const void* wu, const void* meta,
                        const void* order, void* act, int E, int maxt, int top, int F, int K, float limit,
                        float alpha, int dt, const void* pw, int silu, hipStream_t st) {
  if (maxt <= 0) return;
  if (maxt > 65535) throw std::runtime_error("moe_gate_up: too many row tiles");
  dim3 g((F + TV_BN - 1) / TV_BN, maxt);
  DISPATCH_T(dt, T, (moe_gate_up_kernel<T><<<g, 256, 0, st>>>((const T*)h, ldh, (const T*)wg, (const T*)wu,
                                                               (const int*)meta, (const int*)order, (T*)act, E, maxt,
                                                               top, F, K, limit, alpha, (const float*)pw, silu)));
  HIP_CHECK_LAUNCH();
}

void launch_moe_down(const void* act, const void* wd, const void* meta, void* y, int E, int maxt, int N, int F,
                     int dt, hipStream_t st) {
  if (maxt <= 0) return;
  if (maxt > 65535) throw std::runtime_error("moe_down: too many row tiles");
  dim3 g((N + TV_BN - 1) / TV_BN, maxt);
  DISPATCH_T(dt, T, (moe_down_kernel<T><<<g, 256, 0, st>>>((const T*)act, (const T*)wd, (const int*)meta, (float*)y,
                                                            E, maxt, N, F)));
  HIP_CHECK_LAUNCH();
}

// ------------------------------------------------------------------------------------------------ combine
template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ place,
                                                          const float* __restrict__ wts, const T* __restrict__ shared_,
                                                          int64_t lds_, float* __restrict__ out, int N, int top) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < N; c += blockDim.x) {
    float a = 0.f;
    for (int j = 0; j < top; ++j)
      a = fmaf(wts ? wts[(int64_t)t * top + j] : 1.0f, y[(int64_t)place[(int64_t)t * top + j] * N + c], a);
    if (shared_) a += El<T>::ld(shared_ + (int64_t)t * lds_ + c);
    out[(int64_t)t * N + c] = a;
  }
}

void launch_moe_combine(const void* y, const void* place, const void* wts, const void* shared_, int64_t lds_,
                        void* out, int T_, int N, int top, int dt, hipStream_t st) {
  if (T_ == 0) return;
  DISPATCH_T(dt, T, (moe_combine_kernel<T><<<T_, 256, 0, st>>>((const float*)y, (const int*)place, (const float*)wts,
                                                                (const T*)shared_, lds_, (float*)out, N, top)));
  HIP_CHECK_LAUNCH();
}

// ------------------------------------------------------------------------------------------------ dense GLU
// out[t, f] = glu(gu[t, f], gu[t, F + f])
template <typename T>
__global__ __launch_bounds__(256) void glu_clamp_kernel(const T* __restrict__ gu, int64_t ldg, T* __restrict__ out,
                                                        int64_t ldo, int F, float limit, float alpha) {
  const int t = blockIdx.x;
  const T* g = gu + (int64_t)t * ldg;
  for (int f = threadIdx.x; f < F; f += blockDim.x)
    El<T>::st(out + (int64_t)t * ldo + f, glu_clamped(El<T>::ld(g + f), El<T>::ld(g + F + f), limit, alpha));
}

void launch_glu_clamp(const void* gu, int64_t ldg, void* out, int64_t ldo, int T_, int F, float limit, float alpha,
                      int dt, hipStream_t st) {
  if (T_ == 0) return;
  DISPATCH_T(dt, T, (glu_clamp_kernel<T><<<T_, 256, 0, st>>>((const T*)gu, ldg, (T*)out, ldo, F, limit, alpha)));
  HIP_CHECK_LAUNCH();
}
