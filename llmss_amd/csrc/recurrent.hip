// Linear recurrences over a matrix state per head, carried from token to token in fp32.
//
// Every head keeps a state S [dim, vdim]. Per token, with key k and query q [dim] and value v [vdim]:
//
//   decay (MODE 0):  S <- a S + k v^T                          o = S^T q     a = decay[head], a constant
//   delta (MODE 1):  S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q
//                    k <- k / sqrt(|k|^2 + 1e-6), q <- q / sqrt(|q|^2 + 1e-6) / sqrt(dim)
//                    beta = sigmoid(b), g = exp(-exp(A_log[head]) softplus(a + dt_bias[head]))
//   ssd   (MODE 2):  d = softplus(a + dt_bias[head]); S <- exp(-exp(A_log[head]) d) S + d k v^T
//                    o = S^T q + D[head] v             (k = B, q = C of the head's group, v = the head's input x)
//
// Both updates act on the columns of S independently: column c needs only v[c] and the whole k and q. So a thread
// owns one column, split over 1, 2 or 4 neighbouring lanes (32 to 128 state values in registers each) that reduce
// with shuffles, and a workgroup owns (sequence, head, block of columns). Tokens are walked in order; the
// rows of REC_CT tokens at a time are staged in LDS by the whole workgroup (activation and the per-token scalars
// are applied there). The state is read from the sequence's slot unless the portion starts at position 0 (then it is
// zero, whatever the slot held) and written back at the end. Rows of a padded sequence (no slot) are zeroed.
#include "anytype.h"
#include "seqrows.h"

#define REC_CT 8  // tokens staged at a time
#define REC_NE 6  // staged numbers of a token per thread, at most: 5 of k / q / v and one per-token scalar

// 32 consecutive floats from a 16-byte aligned LDS address
__device__ __forceinline__ void ld32(const float* p, float* r) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(p + 4 * i);
    r[4 * i] = v[0], r[4 * i + 1] = v[1], r[4 * i + 2] = v[2], r[4 * i + 3] = v[3];
  }
}

// Sum over the 1, 2 or 4 neighbouring lanes that share a state column: lane-swap moves inside a quad (data-parallel
// primitives on the vector ALU; no trip through LDS as a general shuffle would take)
__device__ __forceinline__ float quad_swap1(float v) {  // lanes 0 <-> 1, 2 <-> 3
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false));
}
__device__ __forceinline__ float quad_swap2(float v) {  // lanes 0 <-> 2, 1 <-> 3
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false));
}
__device__ __forceinline__ float part_sum(float v, int P) {
  if (P >= 2) v += quad_swap1(v);
  if (P >= 4) v += quad_swap2(v);
  return v;
}

struct RecArgs {
  const void* q;  // [T, ldq]: head g's query at q + g * dim
  const void* k;
  const void* v;  // head h's values at v + h * vdim
  int64_t ldq, ldk, ldv;
  const void* ab;  // delta: per-head inputs a at ab[t * ldab + off_a + h], b at ab[t * ldab + off_b + h]
  int64_t ldab;
  int off_a, off_b;
  const float* decay;    // decay: [H]; delta: A_log [H]
  const float* dt_bias;  // delta: [H]
  float* state;          // [slots, H, dim, vdim]
  const int* cu;
  const int* ctx;
  const int* sslots;
  float* out;  // [T, H * vdim]
  int64_t ldo;
  int H, G, dim, vdim, silu_in;
  int gates_ready;  // delta: a / b already hold g / beta (delta_gates_kernel), nothing left to compute while staging
  const float* skip;  // ssd: D [H]
};

// TQ: storage of q / k / v; TP: storage of a / b. R: state values per lane, P lanes per column. Staging: every
// thread owns up to REC_NE of a token's `per` staged numbers (k [dim], q [dim], v [cols], beta, g); the next REC_CT
// tokens' numbers are fetched into registers before the current ones are computed on, and put into LDS afterwards,
// so the global loads are in flight behind the arithmetic. Threads beyond cols * P only fetch.
template <typename TQ, typename TP, int R, int MODE>
__global__ __launch_bounds__(256) void recurrence_kernel(RecArgs A, int P, int cols) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  // sequences in reverse step order, slowest in the grid: the step's long portions (they come last) are dispatched
  // first, one per SIMD, and the single-token sequences fill in behind them
  const int b = gridDim.z - 1 - blockIdx.z, h = blockIdx.x, zb = blockIdx.y;
  const int dim = A.dim, vdim = A.vdim;
  const int g = h / (A.H / A.G);
  const int qlen = A.cu[b + 1] - A.cu[b];
  if (qlen <= 0) return;
  const int t0 = A.cu[b], n = A.ctx[b], slot = A.sslots[b];
  const int cidx = min((int)threadIdx.x / P, cols - 1);
  const int col = zb * cols + cidx, part = threadIdx.x % P;
  const bool live = col < vdim && (int)threadIdx.x < cols * P;
  if (slot < 0 || n <= 0) {
    if (live && part == 0)
      for (int j = 0; j < qlen; ++j) A.out[(int64_t)(t0 + j) * A.ldo + (int64_t)h * vdim + col] = 0.f;
    return;
  }
  const int p0 = n - qlen;
  const int d0 = part * R;  // this lane's rows of the column: d0 .. d0 + R - 1
  float S[R];
  float* sp = A.state + (((int64_t)slot * A.H + h) * dim) * vdim;
  if (p0 > 0) {  // rows past dim and lanes without a column read a valid address and drop the value
    const int cc = min(col, vdim - 1);
#pragma unroll
    for (int i = 0; i < R; ++i) S[i] = sp[(int64_t)min(d0 + i, dim - 1) * vdim + cc];
#pragma unroll
    for (int i = 0; i < R; ++i) S[i] = (live && d0 + i < dim) ? S[i] : 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < R; ++i) S[i] = 0.f;
  }
  // staged numbers per token: k [dimp], q [dimp], v [cols], beta, g; rows padded to whole 16-byte reads
  const int dimp = (dim + 3) & ~3;
  const int per = (2 * dimp + cols + 2 + 3) & ~3;
  float a_const = 0.f, dtb = 0.f;
  if (MODE == 0) a_const = A.decay[h];
  else {
    a_const = expf(A.decay[h]);
    dtb = A.dt_bias[h];
  }
  const float qmul = MODE == 1 ? 1.0f / sqrtf((float)dim) : 1.0f;
  const float dskip = MODE == 2 ? A.skip[h] : 0.f;
  // this thread's staged numbers: slots 0 .. REC_NE - 2 hold k / q / v entries (storage TQ), the last slot the
  // head's two per-token scalars (storage TP, threads 0 and 1). A slot without an entry points at a valid address
  // all the same, so every load is unconditional and the whole batch is in flight together.
  const TQ* src[REC_NE - 1];
  int64_t ld[REC_NE - 1];
  bool has[REC_NE - 1];
  const TQ* dummy = (const TQ*)A.k + (int64_t)t0 * A.ldk + (int64_t)g * dim;
#pragma unroll
  for (int k = 0; k < REC_NE - 1; ++k) {
    const int e = threadIdx.x + k * blockDim.x;
    has[k] = false, src[k] = dummy, ld[k] = A.ldk;
    if (e < dimp) {
      if (e < dim) has[k] = true, src[k] = dummy + e;
    } else if (e < 2 * dimp) {
      if (e - dimp < dim)
        has[k] = true, ld[k] = A.ldq, src[k] = (const TQ*)A.q + (int64_t)t0 * A.ldq + (int64_t)g * dim + (e - dimp);
    } else if (e < 2 * dimp + cols) {
      const int c = zb * cols + (e - 2 * dimp);
      if (c < vdim) has[k] = true, ld[k] = A.ldv, src[k] = (const TQ*)A.v + (int64_t)t0 * A.ldv + (int64_t)h * vdim + c;
    }
  }
  const bool has_s = MODE >= 1 && threadIdx.x < 2;  // thread 0: beta's input (ssd: the step size's), thread 1: the decay's
  const TP* src_s = has_s ? (const TP*)A.ab + (int64_t)t0 * A.ldab + (threadIdx.x == 0 ? A.off_b : A.off_a) + h : nullptr;
  float pre[REC_CT * REC_NE];
  auto fetch = [&](int j0) {
#pragma unroll
    for (int jj = 0; jj < REC_CT; ++jj) {
      const int64_t tj = min(j0 + jj, qlen - 1);
#pragma unroll
      for (int k = 0; k < REC_NE - 1; ++k) pre[jj * REC_NE + k] = El<TQ>::ld(src[k] + tj * ld[k]);
      if (MODE >= 1) pre[jj * REC_NE + REC_NE - 1] = has_s ? El<TP>::ld(src_s + tj * A.ldab) : 0.f;
    }
  };
  auto put = [&]() {
#pragma unroll
    for (int jj = 0; jj < REC_CT; ++jj) {
#pragma unroll
      for (int k = 0; k < REC_NE - 1; ++k) {
        const int e = threadIdx.x + k * blockDim.x;
        if (e >= 2 * dimp + cols) continue;
        float v = has[k] ? pre[jj * REC_NE + k] : 0.f;
        if (A.silu_in) v = v / (1.0f + (sizeof(TQ) == 2 ? __expf(-v) : expf(-v)));  // bf16 rows: the fast exponential
        sm[jj * per + e] = v;
      }
      if (has_s) {
        float v = pre[jj * REC_NE + REC_NE - 1];
        if (A.gates_ready) {
        } else if (threadIdx.x == 0) {
          if (MODE == 2) {
            const float z = v + dtb;
            v = z > 20.f ? z : log1pf(expf(z));
          } else {
            v = 1.0f / (1.0f + expf(-v));
          }
        } else {
          const float z = v + dtb;
          v = expf(-a_const * (z > 20.f ? z : log1pf(expf(z))));
        }
        sm[jj * per + 2 * dimp + cols + threadIdx.x] = v;
      }
    }
  };
  fetch(0);
  for (int j0 = 0; j0 < qlen; j0 += REC_CT) {
    const int nt = min(REC_CT, qlen - j0);
    __syncthreads();  // the previous tokens' readers are done
    put();
    __syncthreads();
    if (j0 + REC_CT < qlen) fetch(j0 + REC_CT);
    for (int jj = 0; jj < nt; ++jj) {
      const float* ks = sm + jj * per;
      const float* qs = ks + dimp;
      const float vv = ks[2 * dimp + cidx];
      // k and q come from LDS 32 numbers at a time by 16-byte reads issued together (a wave alone on its SIMD has
      // nobody to hide a read's latency behind), sums run in four partial accumulators
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
      if (MODE == 0) {
#pragma unroll
        for (int c0 = 0; c0 < R; c0 += 32) {
          float kr[32], qr[32];
          ld32(ks + d0 + c0, kr);
          ld32(qs + d0 + c0, qr);
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            if (d0 + c0 + i < dim) {
              S[c0 + i] = fmaf(a_const, S[c0 + i], kr[i] * vv);
              o4[i & 3] = fmaf(S[c0 + i], qr[i], o4[i & 3]);
            }
          }
        }
      } else if (MODE == 2) {
        const float dv = ks[2 * dimp + cols] * vv, gg = ks[2 * dimp + cols + 1];
#pragma unroll
        for (int c0 = 0; c0 < R; c0 += 32) {
          float kr[32], qr[32];
          ld32(ks + d0 + c0, kr);
          ld32(qs + d0 + c0, qr);
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            if (d0 + c0 + i < dim) {
              S[c0 + i] = fmaf(gg, S[c0 + i], kr[i] * dv);
              o4[i & 3] = fmaf(S[c0 + i], qr[i], o4[i & 3]);
            }
          }
        }
      } else {
        const float beta = ks[2 * dimp + cols], gg = ks[2 * dimp + cols + 1];
        float kk4[4] = {0.f, 0.f, 0.f, 0.f}, sk4[4] = {0.f, 0.f, 0.f, 0.f}, qq4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c0 = 0; c0 < R; c0 += 32) {
          float kr[32];
          ld32(ks + d0 + c0, kr);
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            if (d0 + c0 + i < dim) {
              kk4[i & 3] = fmaf(kr[i], kr[i], kk4[i & 3]);
              S[c0 + i] *= gg;
              sk4[i & 3] = fmaf(S[c0 + i], kr[i], sk4[i & 3]);
            }
          }
        }
        float kk = (kk4[0] + kk4[1]) + (kk4[2] + kk4[3]), sk = (sk4[0] + sk4[1]) + (sk4[2] + sk4[3]);
        kk = part_sum(kk, P);
        sk = part_sum(sk, P);
        const float kn = 1.0f / sqrtf(kk + 1e-6f);
        const float u = beta * (vv - sk * kn) * kn;
#pragma unroll
        for (int c0 = 0; c0 < R; c0 += 32) {
          float kr[32], qr[32];
          ld32(ks + d0 + c0, kr);
          ld32(qs + d0 + c0, qr);
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            if (d0 + c0 + i < dim) {
              qq4[i & 3] = fmaf(qr[i], qr[i], qq4[i & 3]);
              S[c0 + i] = fmaf(kr[i], u, S[c0 + i]);
              o4[i & 3] = fmaf(S[c0 + i], qr[i], o4[i & 3]);
            }
          }
        }
        float qq = (qq4[0] + qq4[1]) + (qq4[2] + qq4[3]);
        qq = part_sum(qq, P);
        const float qn = qmul / sqrtf(qq + 1e-6f);
#pragma unroll
        for (int i = 0; i < 4; ++i) o4[i] *= qn;
      }
      float o = (o4[0] + o4[1]) + (o4[2] + o4[3]);
      o = part_sum(o, P);
      if (MODE == 2) o = fmaf(dskip, vv, o);
      if (live && part == 0) A.out[(int64_t)(t0 + j0 + jj) * A.ldo + (int64_t)h * vdim + col] = o;
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (d0 + i < dim) sp[(int64_t)(d0 + i) * vdim + col] = S[i];
  }
}

// A column is split over up to 4 lanes (32 state values per lane up to dim 128): more waves share the walk, and the
// state, the staged k / q and the prefetched rows fit the register file without spilling.
template <typename TQ, typename TP, int MODE>
static void recurrence_t(const RecArgs& A, int B, hipStream_t st) {
  const int dim = A.dim, vdim = A.vdim;
  int P = 1;
  while (P < 4 && dim > 32 * P) P <<= 1;
  if (dim > 128 * P) throw std::runtime_error("recurrence: key dimension above 512");
  const int R = dim <= 32 * P ? 32 : (dim <= 64 * P ? 64 : 128);
  const int cols = std::min(vdim, 64 / P);  // a wave of state columns per workgroup: many workgroups fill the chip
  const int dimp = (dim + 3) & ~3;
  const int per = (2 * dimp + cols + 2 + 3) & ~3;
  const int threads = ((std::max(cols * P, (2 * dimp + cols + REC_NE - 2) / (REC_NE - 1)) + 63) / 64) * 64;
  if (threads > 256) throw std::runtime_error("recurrence: too many numbers per token to stage");
  dim3 g(A.H, (vdim + cols - 1) / cols, B);
  if (B > 65535 || g.y > 65535) throw std::runtime_error("recurrence: too many sequences or columns");
  const size_t lds = ((size_t)REC_CT * per + 4 * 128) * 4;  // + room for the last token's reads past its k / q
  if (R == 32) recurrence_kernel<TQ, TP, 32, MODE><<<g, threads, lds, st>>>(A, P, cols);
  else if (R == 64) recurrence_kernel<TQ, TP, 64, MODE><<<g, threads, lds, st>>>(A, P, cols);
  else recurrence_kernel<TQ, TP, 128, MODE><<<g, threads, lds, st>>>(A, P, cols);
}

void launch_recurrence(int mode, const void* q, const void* k, const void* v, int64_t ldq, int64_t ldk, int64_t ldv,
                       const void* ab, int64_t ldab, int off_a, int off_b, const void* decay, const void* dt_bias,
                       void* state, const void* cu, const void* ctx, const void* sslots, void* out, int64_t ldo, int B,
                       int H, int G, int dim, int vdim, int silu_in, int gates_ready, int dq, int dp, const void* skip,
                       hipStream_t st) {
  if (B == 0) return;
  if (G < 1 || H % G) throw std::runtime_error("recurrence: heads must be a multiple of the key heads");
  RecArgs A{q, k, v, ldq, ldk, ldv, ab, ldab, off_a, off_b, (const float*)decay, (const float*)dt_bias, (float*)state,
            (const int*)cu, (const int*)ctx, (const int*)sslots, (float*)out, ldo, H, G, dim, vdim, silu_in, gates_ready,
            (const float*)skip};
  if (mode == 0) DISPATCH_T(dq, TQ, (recurrence_t<TQ, float, 0>(A, B, st)));
  else if (mode == 2) DISPATCH_T(dq, TQ, DISPATCH_T(dp, TP, (recurrence_t<TQ, TP, 2>(A, B, st))));
  else DISPATCH_T(dq, TQ, DISPATCH_T(dp, TP, (recurrence_t<TQ, TP, 1>(A, B, st))));
  HIP_CHECK_LAUNCH();
}

// Steps with long portions prepare what every workgroup of a head would otherwise recompute while staging:
// out[t, c] = silu(in[t, c]) in fp32 (the decay recurrence's q | k | v), and the delta rule's per-token scalars
// gates[t, h] = g = exp(-exp(A_log[h]) softplus(a[t, h] + dt_bias[h])), gates[t, H + h] = beta = sigmoid(b[t, h]).
template <typename T>
__global__ __launch_bounds__(256) void silu_f32_kernel(const T* __restrict__ in, int64_t ldi, float* __restrict__ out,
                                                       int64_t ldo, int n) {
  const int t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < n; c += gridDim.y * blockDim.x) {
    const float v = El<T>::ld(in + (int64_t)t * ldi + c);
    out[(int64_t)t * ldo + c] = v / (1.0f + (sizeof(T) == 2 ? __expf(-v) : expf(-v)));
  }
}

void launch_silu_f32(const void* in, int64_t ldi, void* out, int64_t ldo, int T_, int n, int dt, hipStream_t st) {
  if (T_ == 0 || n == 0) return;
  dim3 g(T_, std::min(32, (n + 255) / 256));
  DISPATCH_T(dt, T, (silu_f32_kernel<T><<<g, 256, 0, st>>>((const T*)in, ldi, (float*)out, ldo, n)));
  HIP_CHECK_LAUNCH();
}

template <typename T>
__global__ __launch_bounds__(256) void delta_gates_kernel(const T* __restrict__ a, const T* __restrict__ b, int64_t ld,
                                                          const float* __restrict__ A_log,
                                                          const float* __restrict__ dt_bias,
                                                          float* __restrict__ gates, int T_, int H) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= T_ * H) return;
  const int t = e / H, h = e - t * H;
  const float z = El<T>::ld(a + (int64_t)t * ld + h) + dt_bias[h];
  gates[(int64_t)t * 2 * H + h] = expf(-expf(A_log[h]) * (z > 20.f ? z : log1pf(expf(z))));
  gates[(int64_t)t * 2 * H + H + h] = 1.0f / (1.0f + expf(-El<T>::ld(b + (int64_t)t * ld + h)));
}

void launch_delta_gates(const void* a, const void* b, int64_t ld, const void* A_log, const void* dt_bias, void* gates,
                        int T_, int H, int dt, hipStream_t st) {
  if (T_ == 0) return;
  DISPATCH_T(dt, T, (delta_gates_kernel<T><<<(T_ * H + 255) / 256, 256, 0, st>>>(
      (const T*)a, (const T*)b, ld, (const float*)A_log, (const float*)dt_bias, (float*)gates, T_, H)));
  HIP_CHECK_LAUNCH();
}
