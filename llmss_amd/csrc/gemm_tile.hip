// bf16 matrix products on the matrix cores for the shapes gemm.hip's plans do not cover: batched per-head products
// over strided views, products that keep an fp32 output, and the grouped expert GEMMs of a mixture-of-experts layer
// (row gather, per-expert weights, the clamped gated activation fused behind the gate / up product).
//
//   C[b][m][n] = sum_k A[b][m][k] * B[b][n][k]        A, B bf16 with k contiguous; C bf16 or fp32
//
// One 64x64 or 128x128 output tile per 256-thread workgroup, k in steps of 64 through LDS, v_mfma_f32_16x16x32_bf16.
// Fragment layout: lane (li = lane % 16, g = lane / 16) holds k = 8g .. 8g + 7 of row li
// (A) or of column li (B); the accumulator holds rows 4g .. 4g + 3 of column li. Rows, columns and the k tail are
// bounds-checked while staging (zero fill), so any M, N, K works; rows that are 16-byte aligned take vector loads.
//
// Modes: PLAIN (batched, strided), GATE_UP (grouped: rows of an expert's tile list, A rows gathered through
// order[] / top, two weight matrices, output glu(gate, up) in bf16) and DOWN (grouped: A = the activation rows,
// fp32 output). The tile list and offsets are those moe_group writes (moe.hip).
#include "anytype.h"

#define GT_BK 64
#define GT_LD 72  // bf16 per LDS row: 144 bytes, keeps ds_read_b128 rows 16-byte aligned and spreads the banks

enum { GT_PLAIN = 0, GT_GATE_UP = 1, GT_DOWN = 2 };

struct GemmTileArgs {
  const bf16_t* A;
  const bf16_t* B;
  const bf16_t* B2;  // GATE_UP: the up weights
  void* C;
  int M, N, K;
  int64_t sAb, sAm, sBb, sBn, sCb, sCm;
  // grouped modes
  const int* meta;
  const int* order;
  int E, maxt, top;
  float limit, alpha;
  const float* pw;  // GATE_UP: weight of each (token, slot) pair on the expert's input (null: 1)
  int silu;         // GATE_UP: silu(g) * u instead of the clamped form
};

__device__ __forceinline__ float glu_clamped_t(float g, float u, float limit, float alpha, int silu) {
  if (silu) return g / (1.f + expf(-g)) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + 1.f);
}

// 8 consecutive k of one row (zero beyond the row / k range)
__device__ __forceinline__ u16x8 gt_load(const bf16_t* row, int k, int K, bool vec) {
  u16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
  if (row) {
    if (vec && k + 8 <= K) {
      v = *reinterpret_cast<const u16x8*>(row + k);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (k + i < K) v[i] = row[k + i];
    }
  }
  return v;
}

// BM x BN output tile per 256-thread workgroup (64x64 or 128x128), waves in a 2x2 grid: each wave owns a
// (BM/2) x (BN/2) block = MB x NB accumulators of 16x16. Per 32 of k a wave reads MB A fragments and NB B
// fragments from LDS for MB * NB MFMAs (two such halves per staged k step of 64). The next k step's global loads are issued into registers before the current
// step's MFMAs and written to LDS after them, so memory latency overlaps the matrix work.
template <int MODE, typename TC, int BM, int BN>
__global__ __launch_bounds__(256) void gemm_tile_kernel(GemmTileArgs p) {
  constexpr int MB = BM / 32, NB = BN / 32;   // 16x16 blocks per wave, rows x columns
  constexpr int CA = BM / 32, CB = BN / 32;   // 16-byte chunks per thread per staged tile
  constexpr bool DUAL = MODE == GT_GATE_UP;
  __shared__ __attribute__((aligned(16))) bf16_t As[BM * GT_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * GT_LD];
  __shared__ __attribute__((aligned(16))) bf16_t B2s[DUAL ? BN * GT_LD : 8];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, li = lane & 15, g = lane >> 4;
  const int wm = (w >> 1) * (BM / 2), wn = (w & 1) * (BN / 2);
  const int n0 = blockIdx.x * BN;
  int m0 = 0, rows = 0, crow0 = 0;
  const bf16_t* A = p.A;
  const bf16_t* B = p.B;
  const bf16_t* B2 = p.B2;
  if constexpr (MODE == GT_PLAIN) {
    m0 = blockIdx.y * BM;
    rows = min(BM, p.M - m0);
    A += (int64_t)blockIdx.z * p.sAb;
    B += (int64_t)blockIdx.z * p.sBb;
  } else {
    if ((int)blockIdx.y >= p.meta[0]) return;
    const int e = p.meta[1 + (p.E + 1) + blockIdx.y];
    crow0 = p.meta[1 + (p.E + 1) + p.maxt + blockIdx.y];
    rows = min(BM, p.meta[1 + e + 1] - crow0);
    B += (int64_t)e * p.sBb;
    if constexpr (DUAL) B2 += (int64_t)e * p.sBb;
  }
  // staging: chunk c = tid + 256 i -> (row c / 8, k offset (c % 8) * 8) of each tile
  const bf16_t* arow[CA];
  const bf16_t* brow[CB];
  const bf16_t* b2row[CB];
  bool avec[CA], bvec[CB], b2vec[CB];
  const int sk = (tid & 7) * 8;
#pragma unroll
  for (int i = 0; i < CA; ++i) {
    const int sr = (tid >> 3) + 32 * i;
    arow[i] = nullptr;
    if (sr < rows) {
      if constexpr (MODE == GT_PLAIN) arow[i] = A + (int64_t)(m0 + sr) * p.sAm;
      else if constexpr (MODE == GT_GATE_UP) arow[i] = A + (int64_t)(p.order[crow0 + sr] / p.top) * p.sAm;
      else arow[i] = A + (int64_t)(crow0 + sr) * p.sAm;
    }
    avec[i] = arow[i] && ((uintptr_t)arow[i] & 15) == 0;
  }
#pragma unroll
  for (int i = 0; i < CB; ++i) {
    const int sr = (tid >> 3) + 32 * i;
    brow[i] = (n0 + sr < p.N) ? B + (int64_t)(n0 + sr) * p.sBn : nullptr;
    bvec[i] = brow[i] && ((uintptr_t)brow[i] & 15) == 0;
    b2row[i] = nullptr;
    b2vec[i] = false;
    if constexpr (DUAL) {
      b2row[i] = (n0 + sr < p.N) ? B2 + (int64_t)(n0 + sr) * p.sBn : nullptr;
      b2vec[i] = b2row[i] && ((uintptr_t)b2row[i] & 15) == 0;
    }
  }
  u16x8 ra[CA], rb[CB], rb2[CB];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < CA; ++i) ra[i] = gt_load(arow[i], k0 + sk, p.K, avec[i]);
#pragma unroll
    for (int i = 0; i < CB; ++i) {
      rb[i] = gt_load(brow[i], k0 + sk, p.K, bvec[i]);
      if constexpr (DUAL) rb2[i] = gt_load(b2row[i], k0 + sk, p.K, b2vec[i]);
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < CA; ++i) *reinterpret_cast<u16x8*>(&As[((tid >> 3) + 32 * i) * GT_LD + sk]) = ra[i];
#pragma unroll
    for (int i = 0; i < CB; ++i) {
      *reinterpret_cast<u16x8*>(&Bs[((tid >> 3) + 32 * i) * GT_LD + sk]) = rb[i];
      if constexpr (DUAL) *reinterpret_cast<u16x8*>(&B2s[((tid >> 3) + 32 * i) * GT_LD + sk]) = rb2[i];
    }
  };

  f32x4 acc[MB][NB], acc2[DUAL ? MB : 1][DUAL ? NB : 1];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      if constexpr (DUAL) acc2[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  fetch(0);
  for (int k0 = 0; k0 < p.K; k0 += GT_BK) {
    __syncthreads();  // the previous step's fragment reads are done
    stash();
    __syncthreads();
    if (k0 + GT_BK < p.K) fetch(k0 + GT_BK);
#pragma unroll
    for (int ks = 0; ks < GT_BK; ks += 32) {
      s16x8 a[MB];
#pragma unroll
      for (int i = 0; i < MB; ++i)
        a[i] = *reinterpret_cast<const s16x8*>(&As[(wm + 16 * i + li) * GT_LD + ks + 8 * g]);
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const s16x8 b = *reinterpret_cast<const s16x8*>(&Bs[(wn + 16 * j + li) * GT_LD + ks + 8 * g]);
#pragma unroll
        for (int i = 0; i < MB; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b, acc[i][j], 0, 0, 0);
        if constexpr (DUAL) {
          const s16x8 b2 = *reinterpret_cast<const s16x8*>(&B2s[(wn + 16 * j + li) * GT_LD + ks + 8 * g]);
#pragma unroll
          for (int i = 0; i < MB; ++i)
            acc2[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b2, acc2[i][j], 0, 0, 0);
        }
      }
    }
  }
  TC* C = (TC*)p.C;
  if constexpr (MODE == GT_PLAIN) C += (int64_t)blockIdx.z * p.sCb;
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int r = wm + 16 * i + 4 * g + q;
      if (r >= rows) continue;
      TC* crow = C + (int64_t)((MODE == GT_PLAIN ? m0 : crow0) + r) * p.sCm;
      float sw = 1.0f;
      if constexpr (MODE == GT_GATE_UP) sw = p.pw ? p.pw[p.order[crow0 + r]] : 1.0f;
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int n = n0 + wn + 16 * j + li;
        if (n >= p.N) continue;
        float v = acc[i][j][q];
        if constexpr (DUAL) v = glu_clamped_t(v * sw, acc2[i][j][q] * sw, p.limit, p.alpha, p.silu);
        El<TC>::st(crow + n, v);
      }
    }
}

void launch_gemm_tile(const void* A, const void* B, void* C, int M, int N, int K, int batch, int64_t sAb, int64_t sAm,
                      int64_t sBb, int64_t sBn, int64_t sCb, int64_t sCm, int dc, hipStream_t st) {
  if (M <= 0 || N <= 0 || batch <= 0) return;
  const int T = (M >= 512 && N >= 128) ? 128 : 64;  // big tiles where there is enough work to fill the chip
  if (batch > 65535 || (M + T - 1) / T > 65535) throw std::runtime_error("gemm_tile: grid too large");
  GemmTileArgs a{};
  a.A = (const bf16_t*)A; a.B = (const bf16_t*)B; a.C = C;
  a.M = M; a.N = N; a.K = K;
  a.sAb = sAb; a.sAm = sAm; a.sBb = sBb; a.sBn = sBn; a.sCb = sCb; a.sCm = sCm;
  dim3 g((N + T - 1) / T, (M + T - 1) / T, batch);
  if (dc != 0 && dc != 1) throw std::runtime_error("gemm_tile: bad output dtype code");
  if (T == 128) {
    if (dc == 0) gemm_tile_kernel<GT_PLAIN, bf16_t, 128, 128><<<g, 256, 0, st>>>(a);
    else gemm_tile_kernel<GT_PLAIN, float, 128, 128><<<g, 256, 0, st>>>(a);
  } else {
    if (dc == 0) gemm_tile_kernel<GT_PLAIN, bf16_t, 64, 64><<<g, 256, 0, st>>>(a);
    else gemm_tile_kernel<GT_PLAIN, float, 64, 64><<<g, 256, 0, st>>>(a);
  }
  HIP_CHECK_LAUNCH();
}

// act[r, f] = glu(h[order[r] / top] . gate_e[f], h[..] . up_e[f]) over the tile list (bf16); tile_rows = the rows
// per tile the list was built with (moe_group): 64 or 128
void launch_moe_gate_up_tile(const void* h, int64_t ldh, const void* wg, const void* wu, const void* meta,
                             const void* order, void* act, int E, int maxt, int top, int F, int K, float limit,
                             float alpha, int tile_rows, const void* pw, int silu, hipStream_t st) {
  if (tile_rows != 64 && tile_rows != 128) throw std::runtime_error("moe_gate_up: tile rows must be 64 or 128");
  if (maxt <= 0) return;
  if (maxt > 65535) throw std::runtime_error("moe_gate_up: too many row tiles");
  GemmTileArgs a{};
  a.A = (const bf16_t*)h; a.B = (const bf16_t*)wg; a.B2 = (const bf16_t*)wu; a.C = act;
  a.N = F; a.K = K; a.sAm = ldh; a.sBb = (int64_t)F * K; a.sBn = K; a.sCm = F;
  a.meta = (const int*)meta; a.order = (const int*)order; a.E = E; a.maxt = maxt; a.top = top;
  a.limit = limit; a.alpha = alpha; a.pw = (const float*)pw; a.silu = silu;
  // 128-row tiles are 64 columns wide here: with two accumulator sets (gate and up) a 128x128 tile leaves one
  // workgroup per CU; at 128x64 two to three fit and hide each other's staging
  dim3 g((F + 63) / 64, maxt);
  if (tile_rows == 128) gemm_tile_kernel<GT_GATE_UP, bf16_t, 128, 64><<<g, 256, 0, st>>>(a);
  else gemm_tile_kernel<GT_GATE_UP, bf16_t, 64, 64><<<g, 256, 0, st>>>(a);
  HIP_CHECK_LAUNCH();
}

// y[r, n] = act[r, :] . down_e[n, :] over the tile list (fp32)
void launch_moe_down_tile(const void* act, const void* wd, const void* meta, void* y, int E, int maxt, int N, int F,
                          int tile_rows, hipStream_t st) {
  if (tile_rows != 64 && tile_rows != 128) throw std::runtime_error("moe_down: tile rows must be 64 or 128");
  if (maxt <= 0) return;
  if (maxt > 65535) throw std::runtime_error("moe_down: too many row tiles");
  GemmTileArgs a{};
  a.A = (const bf16_t*)act; a.B = (const bf16_t*)wd; a.C = y;
  a.N = N; a.K = F; a.sAm = F; a.sBb = (int64_t)N * F; a.sBn = F; a.sCm = N;
  a.meta = (const int*)meta; a.E = E; a.maxt = maxt; a.top = 1;
  dim3 g((N + tile_rows - 1) / tile_rows, maxt);
  if (tile_rows == 128) gemm_tile_kernel<GT_DOWN, float, 128, 128><<<g, 256, 0, st>>>(a);
  else gemm_tile_kernel<GT_DOWN, float, 64, 64><<<g, 256, 0, st>>>(a);
  HIP_CHECK_LAUNCH();
}
