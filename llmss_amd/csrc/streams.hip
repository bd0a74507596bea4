// Residual streams with learned connections, causal convolutions over time with a per-sequence tail, gated group
// norms and a gated activation - the memory-bound glue of per-layer designs whose blocks run one after the other.
//
// Streams: the residual is S copies x_1 .. x_S [S, T, W] in fp32. A sublayer reads u = sum_s in[s] x_s, normed,
// and its output y is written back as x_t <- sum_s mix[s, t] x_s + c * out[t] * y for all t at once. S = 1 with
// in = out = mix = 1 is the ordinary pre-norm residual, so designs without extra streams use the same kernels.
// One pass does both: the write-back of the previous sublayer and the read + norm of the next.
//
// Convolution tail: a causal convolution of `taps` taps needs the last taps - 1 inputs of the sequence when a step
// starts past position 0. They live in a per-sequence state slot [slots, taps - 1, C] in fp32 and are renewed by a
// second launch after the convolution has read the old ones. A portion that starts at position 0 reads zeros,
// whatever its slot held before: a slot handed to a new sequence needs no clearing.
#include "anytype.h"
#include "seqrows.h"

#define MAX_STREAMS 8
#define MAX_TAIL 16
#define CONV_CPT 4  // channels per thread of the convolution kernel

// x[s, t, :] = table[ids[t], :] (+ pos_table[positions[t], :]) for every stream s
template <typename T>
__global__ __launch_bounds__(256) void embed_streams_kernel(const int64_t* __restrict__ ids,
                                                            const int64_t* __restrict__ positions,
                                                            const T* __restrict__ table, const T* __restrict__ ptab,
                                                            float* __restrict__ x, int S, int T_, int W, int vocab,
                                                            int npos) {
  const int t = blockIdx.x;
  int64_t id = ids[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  int64_t p = positions[t];
  p = p < 0 ? 0 : (p >= npos ? npos - 1 : p);
  const T* src = table + id * (int64_t)W;
  const T* ps = ptab ? ptab + p * (int64_t)W : nullptr;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = El<T>::ld(src + c);
    if (ps) v += El<T>::ld(ps + c);
    for (int s = 0; s < S; ++s) x[((int64_t)s * T_ + t) * W + c] = v;
  }
}

void launch_embed_streams(const void* ids, const void* positions, const void* table, const void* ptab, void* x, int S,
                          int T_, int W, int vocab, int npos, int dt, hipStream_t st) {
  if (T_ == 0) return;
  DISPATCH_T(dt, T, (embed_streams_kernel<T><<<T_, 256, 0, st>>>((const int64_t*)ids, (const int64_t*)positions,
                                                                   (const T*)table, (const T*)ptab, (float*)x, S, T_,
                                                                   W, vocab, npos)));
  HIP_CHECK_LAUNCH();
}

// Row t. If y: x_s <- sum_r mix[r, s] x_r + c * outw[s] * y[t] for all s at once.
// If w: u = sum_s inw[s] x_s (inw null: the plain sum), h[t] = norm(u) * w, with
// rms = 0: (u - mean) / sqrt(var + eps), var the mean squared deviation; rms = 1: u / sqrt(mean(u^2) + eps).
// TH: storage type of h (the model's, or float when a convolution follows).
template <typename T, typename TH>
__global__ __launch_bounds__(256) void stream_add_norm_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                              int64_t ldy, const float* __restrict__ mix,
                                                              const float* __restrict__ outw, float c,
                                                              const float* __restrict__ inw, const T* __restrict__ w,
                                                              float eps, int rms, TH* __restrict__ h, int64_t ldh,
                                                              int S, int T_, int W) {
  extern __shared__ float u_s[];  // W floats, then 32 for the reductions
  float* red = u_s + W;
  const int t = blockIdx.x;
  float msum = 0.f;
  for (int col = threadIdx.x; col < W; col += blockDim.x) {
    float xs[MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s)
      if (s < S) xs[s] = x[((int64_t)s * T_ + t) * W + col];
    if (y) {
      const float yv = El<T>::ld(y + (int64_t)t * ldy + col) * c;
      float nx[MAX_STREAMS];
#pragma unroll
      for (int s = 0; s < MAX_STREAMS; ++s) {
        if (s < S) {
          float a = 0.f;
          for (int r = 0; r < S; ++r) a = fmaf(mix[r * S + s], xs[r], a);
          nx[s] = fmaf(outw[s], yv, a);
        }
      }
#pragma unroll
      for (int s = 0; s < MAX_STREAMS; ++s)
        if (s < S) {
          xs[s] = nx[s];
          x[((int64_t)s * T_ + t) * W + col] = nx[s];
        }
    }
    if (w) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < MAX_STREAMS; ++s)
        if (s < S) u = inw ? fmaf(inw[s], xs[s], u) : u + xs[s];
      u_s[col] = u;
      msum += u;
    }
  }
  if (!w) return;
  float mean = 0.f;
  if (!rms) mean = block_sum(msum, red) / (float)W;
  float ss = 0.f;
  for (int col = threadIdx.x; col < W; col += blockDim.x) {
    const float d = u_s[col] - mean;
    ss = fmaf(d, d, ss);
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int col = threadIdx.x; col < W; col += blockDim.x)
    El<TH>::st(h + (int64_t)t * ldh + col, (u_s[col] - mean) * inv * El<T>::ld(w + col));
}

void launch_stream_add_norm(void* x, const void* y, int64_t ldy, const void* mix, const void* outw, float c,
                            const void* inw, const void* w, float eps, int rms, void* h, int64_t ldh, int S, int T_,
                            int W, int dt, int h_f32, hipStream_t st) {
  if (T_ == 0) return;
  if (S < 1 || S > MAX_STREAMS) throw std::runtime_error("stream_add_norm: 1 to 8 streams");
  const size_t lds = (size_t)(W + 32) * 4;
  if (lds > 64 * 1024) throw std::runtime_error("stream_add_norm: width too large for LDS");
#define LAUNCH_SAN(TH_)                                                                                              \
  stream_add_norm_kernel<T, TH_><<<T_, 256, lds, st>>>((float*)x, (const T*)y, ldy, (const float*)mix,                \
                                                       (const float*)outw, c, (const float*)inw, (const T*)w, eps, rms, \
                                                       (TH_*)h, ldh, S, T_, W)
  DISPATCH_T(dt, T, {
    if (h_f32) LAUNCH_SAN(float);
    else LAUNCH_SAN(T);
  });
#undef LAUNCH_SAN
  HIP_CHECK_LAUNCH();
}

// out[t, c] = act((res ? in[t, c] : 0) + sum_k w[c, k] * in_(pos - (taps - 1 - k))[c]); inputs before the portion come
// from the sequence's tail (state[slot, i, c] holds position p0 - (taps - 1) + i), inputs before position 0 are zero.
template <typename TI, typename TW, typename TO>
__global__ __launch_bounds__(256) void causal_conv_kernel(const TI* __restrict__ in, int64_t ldi,
                                                          const TW* __restrict__ w, const float* __restrict__ state,
                                                          const int* __restrict__ cu, const int* __restrict__ ctx,
                                                          const int* __restrict__ sslots, TO* __restrict__ out,
                                                          int64_t ldo, int B, int C, int taps, int res, int silu,
                                                          const TW* __restrict__ bias) {
  const int t = blockIdx.x;
  const RowSeq r = row_seq(cu, ctx, B, t);  // once per workgroup: a thread walks CONV_CPT channels
  const int c_end = min(C, (int)(blockIdx.y + 1) * (int)blockDim.x * CONV_CPT);
  if (r.pos < 0) {
    for (int c = blockIdx.y * blockDim.x * CONV_CPT + threadIdx.x; c < c_end; c += blockDim.x)
      El<TO>::st(out + (int64_t)t * ldo + c, 0.f);
    return;
  }
  const int slot = sslots[r.b];
  const int R = taps - 1;
  for (int c = blockIdx.y * blockDim.x * CONV_CPT + threadIdx.x; c < c_end; c += blockDim.x) {
    float acc = res ? El<TI>::ld(in + (int64_t)t * ldi + c) : 0.f;
    for (int k = 0; k < taps; ++k) {
      const int d = R - k;
      if (r.pos - d < 0) continue;
      float v;
      if (r.j - d >= 0) v = El<TI>::ld(in + (int64_t)(t - d) * ldi + c);
      else v = state[((int64_t)slot * R + (r.j - d + R)) * C + c];
      acc = fmaf(El<TW>::ld(w + (int64_t)c * taps + k), v, acc);
    }
    if (bias) acc += El<TW>::ld(bias + c);
    if (silu) acc = acc / (1.0f + expf(-acc));
    El<TO>::st(out + (int64_t)t * ldo + c, acc);
  }
}

// The same for steps of long portions: a workgroup takes CONV_STRIP neighbouring rows and a thread CH neighbouring
// channels of them (four: 16-byte reads of fp32 rows), so an input is read once (plus the rows before the strip)
// instead of once per tap. The rows are loaded up front, all loads in flight together; the strip's place in its
// sequence is found once and walked from there (looked up again where a sequence ends). Taps are added in the order
// of the kernel above: the same numbers bit for bit. RMAX: the most rows back that a tap may reach (taps - 1).
#define CONV_STRIP 16
template <typename T, int CH>
__device__ __forceinline__ void conv_ld(const T* p, float* v) {
  if constexpr (CH == 4 && sizeof(T) == 4) {
    const f32x4 x = *reinterpret_cast<const f32x4*>(p);
    v[0] = x[0], v[1] = x[1], v[2] = x[2], v[3] = x[3];
  } else if constexpr (CH == 4) {
    const u32x2 x = *reinterpret_cast<const u32x2*>(p);
    v[0] = __uint_as_float(x[0] << 16), v[1] = __uint_as_float(x[0] & 0xffff0000u);
    v[2] = __uint_as_float(x[1] << 16), v[3] = __uint_as_float(x[1] & 0xffff0000u);
  } else {
#pragma unroll
    for (int e = 0; e < CH; ++e) v[e] = El<T>::ld(p + e);
  }
}
template <typename T, int CH>
__device__ __forceinline__ void conv_st(T* p, const float* v) {
  if constexpr (CH == 4 && sizeof(T) == 4) {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
  } else if constexpr (CH == 4) {
    u32x2 x;
    x[0] = (unsigned)f2bf(v[0]) | ((unsigned)f2bf(v[1]) << 16);
    x[1] = (unsigned)f2bf(v[2]) | ((unsigned)f2bf(v[3]) << 16);
    *reinterpret_cast<u32x2*>(p) = x;
  } else {
#pragma unroll
    for (int e = 0; e < CH; ++e) El<T>::st(p + e, v[e]);
  }
}

template <typename TI, typename TW, typename TO, int RMAX, int CH>
__global__ __launch_bounds__(256) void causal_conv_strip_kernel(const TI* __restrict__ in, int64_t ldi,
                                                                const TW* __restrict__ w,
                                                                const float* __restrict__ state,
                                                                const int* __restrict__ cu, const int* __restrict__ ctx,
                                                                const int* __restrict__ sslots, TO* __restrict__ out,
                                                                int64_t ldo, int B, int C, int taps, int res, int silu,
                                                                int T_, const TW* __restrict__ bias) {
  const int t0 = blockIdx.x * CONV_STRIP;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * CH;
  if (c >= C) return;  // (C is a multiple of CH)
  const int R = taps - 1;
  float wd[RMAX + 1][CH];  // wd[d]: the weight of the input d rows back
#pragma unroll
  for (int d = 0; d <= RMAX; ++d)
#pragma unroll
    for (int e = 0; e < CH; ++e) wd[d][e] = d <= R ? El<TW>::ld(w + (int64_t)(c + e) * taps + (R - d)) : 0.f;
  float x[CONV_STRIP + RMAX][CH];  // x[i]: input row t0 - RMAX + i
#pragma unroll
  for (int i = 0; i < CONV_STRIP + RMAX; ++i) {
    const int tt = t0 - RMAX + i;
    if (i >= RMAX - R && tt >= 0 && tt < T_) {
      conv_ld<TI, CH>(in + (int64_t)tt * ldi + c, x[i]);
    } else {
#pragma unroll
      for (int e = 0; e < CH; ++e) x[i][e] = 0.f;
    }
  }
  RowSeq r = row_seq(cu, ctx, B, t0);
#pragma unroll
  for (int i = 0; i < CONV_STRIP; ++i) {
    const int t = t0 + i;
    if (t >= T_) break;
    if (i > 0) {
      ++r.j;
      ++r.pos;
      if (r.j >= r.qlen) r = row_seq(cu, ctx, B, t);
    }
    float acc[CH];
#pragma unroll
    for (int e = 0; e < CH; ++e) acc[e] = 0.f;
    if (r.pos >= 0) {
      if (res) {
#pragma unroll
        for (int e = 0; e < CH; ++e) acc[e] = x[i + RMAX][e];
      }
#pragma unroll
      for (int d = RMAX; d >= 0; --d) {
        if (d > R || r.pos - d < 0) continue;
        float v[CH];
        if (r.j - d >= 0) {
#pragma unroll
          for (int e = 0; e < CH; ++e) v[e] = x[i + RMAX - d][e];
        } else {
          conv_ld<float, CH>(state + ((int64_t)sslots[r.b] * R + (r.j - d + R)) * C + c, v);
        }
#pragma unroll
        for (int e = 0; e < CH; ++e) acc[e] = fmaf(wd[d][e], v[e], acc[e]);
      }
      if (bias) {
#pragma unroll
        for (int e = 0; e < CH; ++e) acc[e] += El<TW>::ld(bias + c + e);
      }
      if (silu) {
#pragma unroll
        for (int e = 0; e < CH; ++e) acc[e] = acc[e] / (1.0f + expf(-acc[e]));
      }
    }
    conv_st<TO, CH>(out + (int64_t)t * ldo + c, acc);
  }
}

// The tail after the step: state[slot, i, c] <- input at position ctx - (taps - 1) + i
template <typename TI>
__global__ __launch_bounds__(256) void conv_tail_kernel(const TI* __restrict__ in, int64_t ldi,
                                                        float* __restrict__ state, const int* __restrict__ cu,
                                                        const int* __restrict__ ctx, const int* __restrict__ sslots,
                                                        int C, int taps) {
  const int b = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int slot = sslots[b], qlen = cu[b + 1] - cu[b], n = ctx[b];
  if (slot < 0 || qlen <= 0 || n <= 0) return;
  const int R = taps - 1, p0 = n - qlen;
  float nv[MAX_TAIL];
#pragma unroll
  for (int i = 0; i < MAX_TAIL; ++i) {
    if (i < R) {
      const int pp = n - R + i;
      float v = 0.f;
      if (pp >= p0) v = El<TI>::ld(in + (int64_t)(cu[b] + pp - p0) * ldi + c);
      else if (pp >= 0) v = state[((int64_t)slot * R + (pp - p0 + R)) * C + c];
      nv[i] = v;
    }
  }
#pragma unroll
  for (int i = 0; i < MAX_TAIL; ++i)
    if (i < R) state[((int64_t)slot * R + i) * C + c] = nv[i];
}

template <typename TI, typename TW, typename TO>
static void causal_conv_t(const void* in, int64_t ldi, const void* w, void* state, const void* cu, const void* ctx,
                          const void* sslots, void* out, int64_t ldo, int T_, int B, int C, int taps, int res,
                          int silu, const void* bias, hipStream_t st) {
  if (T_ >= 256 && T_ >= 8 * B && taps <= 9) {  // portions of eight rows and more on average
    const auto al16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    const bool four = C % 4 == 0 && ldi % 4 == 0 && ldo % 4 == 0 && al16(in) && al16(out) && al16(state);
#define LAUNCH_STRIP(RMAX_, CH_)                                                                                    \
  causal_conv_strip_kernel<TI, TW, TO, RMAX_, CH_><<<g, 256, 0, st>>>(                                              \
      (const TI*)in, ldi, (const TW*)w, (const float*)state, (const int*)cu, (const int*)ctx, (const int*)sslots,   \
      (TO*)out, ldo, B, C, taps, res, silu, T_, (const TW*)bias)
    if (four) {
      dim3 g((T_ + CONV_STRIP - 1) / CONV_STRIP, (C / 4 + 255) / 256);
      if (taps <= 4) LAUNCH_STRIP(3, 4);
      else LAUNCH_STRIP(8, 4);
    } else {
      dim3 g((T_ + CONV_STRIP - 1) / CONV_STRIP, (C + 255) / 256);
      if (taps <= 4) LAUNCH_STRIP(3, 1);
      else LAUNCH_STRIP(8, 1);
    }
#undef LAUNCH_STRIP
  } else {
    dim3 g(T_, (C + 256 * CONV_CPT - 1) / (256 * CONV_CPT));
    causal_conv_kernel<TI, TW, TO><<<g, 256, 0, st>>>((const TI*)in, ldi, (const TW*)w, (const float*)state,
                                                      (const int*)cu, (const int*)ctx, (const int*)sslots, (TO*)out,
                                                      ldo, B, C, taps, res, silu, (const TW*)bias);
  }
  if (taps > 1) {
    dim3 g2(B, (C + 255) / 256);
    conv_tail_kernel<TI><<<g2, 256, 0, st>>>((const TI*)in, ldi, (float*)state, (const int*)cu, (const int*)ctx,
                                             (const int*)sslots, C, taps);
  }
}

// di / dw / dout: storage types of the input, the weights and the output (0 bf16, 1 fp32)
void launch_causal_conv(const void* in, int64_t ldi, const void* w, void* state, const void* cu, const void* ctx,
                        const void* sslots, void* out, int64_t ldo, int T_, int B, int C, int taps, int res, int silu,
                        int di, int dw, int dout, const void* bias, hipStream_t st) {
  if (T_ == 0 || B == 0) return;
  if (taps < 1 || taps - 1 > MAX_TAIL) throw std::runtime_error("causal_conv: 1 to 17 taps");
  if ((C + 255) / 256 > 65535) throw std::runtime_error("causal_conv: too many channels");
  DISPATCH_T(di, TI, DISPATCH_T(dw, TW, DISPATCH_T(dout, TO, (causal_conv_t<TI, TW, TO>(
      in, ldi, w, state, cu, ctx, sslots, out, ldo, T_, B, C, taps, res, silu, bias, st)))));
  HIP_CHECK_LAUNCH();
}

// out[t, g * n + i] = c * o[t, g * n + i] / sqrt(mean_i(o[t, g, :]^2) + eps) * w[i] * act(gate[t, g * n + i])
// act 0: sigmoid, 1: silu. o fp32; gate, w and out in the storage type. wfull: w holds a weight per column, w[g * n +
// i]. first: the gate comes before the norm, out = c * u / sqrt(mean(u^2) + eps) * w with u = o * act(gate).
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ o, int64_t ldo,
                                                               const T* __restrict__ gate, int64_t ldg,
                                                               const T* __restrict__ w, float eps, int act, float c,
                                                               T* __restrict__ out, int64_t ldout, int n, int wfull,
                                                               int first) {
  __shared__ float red[32];
  const int t = blockIdx.x, g = blockIdx.y;
  const float* row = o + (int64_t)t * ldo + (int64_t)g * n;
  const T* gr = gate + (int64_t)t * ldg + (int64_t)g * n;
  const T* wr = wfull ? w + (int64_t)g * n : w;
  auto gate_of = [&](int i) {
    const float z = El<T>::ld(gr + i);
    const float sg = 1.0f / (1.0f + expf(-z));
    return act ? z * sg : sg;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const float u = first ? row[i] * gate_of(i) : row[i];
    ss = fmaf(u, u, ss);
  }
  ss = block_sum(ss, red);
  const float inv = c / sqrtf(ss / (float)n + eps);
  T* dst = out + (int64_t)t * ldout + (int64_t)g * n;
  for (int i = threadIdx.x; i < n; i += blockDim.x)
    El<T>::st(dst + i, row[i] * inv * El<T>::ld(wr + i) * gate_of(i));
}

void launch_gated_group_norm(const void* o, int64_t ldo, const void* gate, int64_t ldg, const void* w, float eps,
                             int act, float c, void* out, int64_t ldout, int T_, int groups, int n, int dt, int wfull,
                             int first, hipStream_t st) {
  if (T_ == 0) return;
  if (groups > 65535) throw std::runtime_error("gated_group_norm: too many groups");
  dim3 g(T_, groups);
  const int threads = n >= 256 ? 256 : ((n + 63) / 64) * 64;
  DISPATCH_T(dt, T, (gated_group_norm_kernel<T><<<g, threads, 0, st>>>((const float*)o, ldo, (const T*)gate, ldg,
                                                                        (const T*)w, eps, act, c, (T*)out, ldout, n,
                                                                        wfull, first)));
  HIP_CHECK_LAUNCH();
}

// out[t, f] = act(gu[t, f]) * gu[t, F + f]; act 0: tanh-form GELU, 1: SiLU
template <typename T>
__global__ __launch_bounds__(256) void glu_act_kernel(const T* __restrict__ gu, int64_t ldg, T* __restrict__ out,
                                                      int64_t ldo, int F, int act) {
  const int t = blockIdx.x;
  for (int f = blockIdx.y * blockDim.x + threadIdx.x; f < F; f += gridDim.y * blockDim.x) {
    const float g = El<T>::ld(gu + (int64_t)t * ldg + f), u = El<T>::ld(gu + (int64_t)t * ldg + F + f);
    float a;
    if (act == 0) a = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    else a = g / (1.0f + expf(-g));
    El<T>::st(out + (int64_t)t * ldo + f, a * u);
  }
}

void launch_glu_act(const void* gu, int64_t ldg, void* out, int64_t ldo, int T_, int F, int act, int dt,
                    hipStream_t st) {
  if (T_ == 0 || F == 0) return;
  dim3 g(T_, std::min(64, (F + 255) / 256));
  DISPATCH_T(dt, T, (glu_act_kernel<T><<<g, 256, 0, st>>>((const T*)gu, ldg, (T*)out, ldo, F, act)));
  HIP_CHECK_LAUNCH();
}

// out[t, f] = act(x[t, f]), no gate. act 0: tanh-form GELU, 1: SiLU, 2: xIELU with the two coefficients (a, b):
//   z > 0: a z^2 + z / 2;   z <= 0: b (exp(z) - 1 - z) + z / 2
__device__ __forceinline__ float act_value(float z, int act, float a, float b) {
  if (act == 0) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
  if (act == 1) return z / (1.0f + expf(-z));
  return z > 0.f ? fmaf(a * z, z, 0.5f * z) : fmaf(b, expm1f(z) - z, 0.5f * z);
}

template <typename T>
__global__ __launch_bounds__(256) void act_fn_kernel(const T* __restrict__ x, int64_t ldx, T* __restrict__ out,
                                                     int64_t ldo, int F, int act, float a, float b) {
  const int t = blockIdx.x;
  for (int f = blockIdx.y * blockDim.x + threadIdx.x; f < F; f += gridDim.y * blockDim.x)
    El<T>::st(out + (int64_t)t * ldo + f, act_value(El<T>::ld(x + (int64_t)t * ldx + f), act, a, b));
}

// 16-byte accesses: eight bf16 or four fp32 numbers per thread and step (rows 16-byte aligned, F a multiple)
template <typename T>
__global__ __launch_bounds__(256) void act_fn_vec_kernel(const T* __restrict__ x, int64_t ldx, T* __restrict__ out,
                                                         int64_t ldo, int F, int act, float a, float b) {
  constexpr int N = 16 / sizeof(T);
  const int t = blockIdx.x;
  for (int f = (blockIdx.y * blockDim.x + threadIdx.x) * N; f < F; f += gridDim.y * blockDim.x * N) {
    if constexpr (sizeof(T) == 2) {
      u16x8 v = *reinterpret_cast<const u16x8*>(x + (int64_t)t * ldx + f);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = f2bf(act_value(bf2f(v[i]), act, a, b));
      *reinterpret_cast<u16x8*>(out + (int64_t)t * ldo + f) = v;
    } else {
      f32x4 v = *reinterpret_cast<const f32x4*>(x + (int64_t)t * ldx + f);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = act_value(v[i], act, a, b);
      *reinterpret_cast<f32x4*>(out + (int64_t)t * ldo + f) = v;
    }
  }
}

void launch_act_fn(const void* x, int64_t ldx, void* out, int64_t ldo, int T_, int F, int act, float a, float b,
                   int dt, hipStream_t st) {
  if (T_ == 0 || F == 0) return;
  const int es = dt == 0 ? 2 : 4, n = 16 / es;
  const bool vec = F % n == 0 && ldx % n == 0 && ldo % n == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0;
  if (vec) {
    dim3 g(T_, std::min(64, (F / n + 255) / 256));
    DISPATCH_T(dt, T, (act_fn_vec_kernel<T><<<g, 256, 0, st>>>((const T*)x, ldx, (T*)out, ldo, F, act, a, b)));
  } else {
    dim3 g(T_, std::min(64, (F + 255) / 256));
    DISPATCH_T(dt, T, (act_fn_kernel<T><<<g, 256, 0, st>>>((const T*)x, ldx, (T*)out, ldo, F, act, a, b)));
  }
  HIP_CHECK_LAUNCH();
}
