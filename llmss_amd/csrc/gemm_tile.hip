// bf16 matrix products on the matrix cores for the shapes gemm.hip's plans do not cover: batched per-head products
// over strided views, products that keep an fp32 output, and the grouped expert GEMMs of a mixture-of-experts layer
// (row gather, per-expert weights, the clamped gated activation fused behind the gate / up product).
//
//   C[b][m][n] = sum_k A[b][m][k] * B[b][n][k]        A, B bf16 with k contiguous; C bf16 or fp32
//
// One 64x64 output tile per 256-thread workgroup, k in steps of 32 through LDS. Wave w owns rows [16w, 16w + 16) and
// all four 16-column blocks: per k step one A fragment and four B fragments (ds_read_b128 each) feed four
// v_mfma_f32_16x16x32_bf16. Fragment layout: lane (li = lane % 16, g = lane / 16) holds k = 8g .. 8g + 7 of row li
// (A) or of column li (B); the accumulator holds rows 4g .. 4g + 3 of column li. Rows, columns and the k tail are
// bounds-checked while staging (zero fill), so any M, N, K works; rows that are 16-byte aligned take vector loads.
//
// Modes: PLAIN (batched, strided), GATE_UP (grouped: rows of an expert's tile list, A rows gathered through
// order[] / top, two weight matrices, output glu(gate, up) in bf16) and DOWN (grouped: A = the activation rows,
// fp32 output). The tile list and offsets are those moe_group writes (moe.hip).
#include "anytype.h"

#define GT_BM 64
#define GT_BN 64
#define GT_BK 32
#define GT_LD 40  // bf16 per LDS row: 80 bytes, keeps ds_read_b128 rows 16-byte aligned and spreads the banks

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
};

__device__ __forceinline__ float glu_clamped_t(float g, float u, float limit, float alpha) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.f + expf(-alpha * g)) * (u + 1.f);
}

// 8 consecutive k of one row into LDS (zero beyond the row / k range)
__device__ __forceinline__ void gt_stage(bf16_t* dst, const bf16_t* row, int k, int K, bool vec) {
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
  *reinterpret_cast<u16x8*>(dst) = v;
}

template <int MODE, typename TC>
__global__ __launch_bounds__(256) void gemm_tile_kernel(GemmTileArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t As[GT_BM * GT_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[GT_BN * GT_LD];
  __shared__ __attribute__((aligned(16))) bf16_t B2s[MODE == GT_GATE_UP ? GT_BN * GT_LD : 8];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, li = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * GT_BN;
  int m0 = 0, rows = 0, crow0 = 0;
  const bf16_t* A = p.A;
  const bf16_t* B = p.B;
  const bf16_t* B2 = p.B2;
  if constexpr (MODE == GT_PLAIN) {
    m0 = blockIdx.y * GT_BM;
    rows = min(GT_BM, p.M - m0);
    A += (int64_t)blockIdx.z * p.sAb;
    B += (int64_t)blockIdx.z * p.sBb;
  } else {
    if ((int)blockIdx.y >= p.meta[0]) return;
    const int e = p.meta[1 + (p.E + 1) + blockIdx.y];
    crow0 = p.meta[1 + (p.E + 1) + p.maxt + blockIdx.y];
    rows = min(GT_BM, p.meta[1 + e + 1] - crow0);
    B += (int64_t)e * p.sBb;
    if constexpr (MODE == GT_GATE_UP) B2 += (int64_t)e * p.sBb;
  }
  // staging: thread -> (row tid / 4, k chunk (tid % 4) * 8) of each tile
  const int sr = tid >> 2, sk = (tid & 3) * 8;
  const bf16_t* arow = nullptr;
  if (sr < rows) {
    if constexpr (MODE == GT_PLAIN) arow = A + (int64_t)(m0 + sr) * p.sAm;
    else if constexpr (MODE == GT_GATE_UP) arow = A + (int64_t)(p.order[crow0 + sr] / p.top) * p.sAm;
    else arow = A + (int64_t)(crow0 + sr) * p.sAm;
  }
  const bf16_t* brow = (n0 + sr < p.N) ? B + (int64_t)(n0 + sr) * p.sBn : nullptr;
  const bf16_t* b2row = nullptr;
  if constexpr (MODE == GT_GATE_UP) b2row = (n0 + sr < p.N) ? B2 + (int64_t)(n0 + sr) * p.sBn : nullptr;
  const bool avec = arow && ((uintptr_t)arow & 15) == 0;
  const bool bvec = brow && ((uintptr_t)brow & 15) == 0;
  const bool b2vec = b2row && ((uintptr_t)b2row & 15) == 0;

  f32x4 acc[4], acc2[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = acc2[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < p.K; k0 += GT_BK) {
    __syncthreads();
    gt_stage(&As[sr * GT_LD + sk], arow, k0 + sk, p.K, avec);
    gt_stage(&Bs[sr * GT_LD + sk], brow, k0 + sk, p.K, bvec);
    if constexpr (MODE == GT_GATE_UP) gt_stage(&B2s[sr * GT_LD + sk], b2row, k0 + sk, p.K, b2vec);
    __syncthreads();
    const s16x8 a = *reinterpret_cast<const s16x8*>(&As[(16 * w + li) * GT_LD + 8 * g]);
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      const s16x8 b = *reinterpret_cast<const s16x8*>(&Bs[(16 * nb + li) * GT_LD + 8 * g]);
      acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[nb], 0, 0, 0);
      if constexpr (MODE == GT_GATE_UP) {
        const s16x8 b2 = *reinterpret_cast<const s16x8*>(&B2s[(16 * nb + li) * GT_LD + 8 * g]);
        acc2[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b2, acc2[nb], 0, 0, 0);
      }
    }
  }
  TC* C = (TC*)p.C;
  if constexpr (MODE == GT_PLAIN) C += (int64_t)blockIdx.z * p.sCb;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 16 * w + 4 * g + i;
    if (r >= rows) continue;
    TC* crow = C + (int64_t)((MODE == GT_PLAIN ? m0 : crow0) + r) * p.sCm;
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      const int n = n0 + 16 * nb + li;
      if (n >= p.N) continue;
      float v = acc[nb][i];
      if constexpr (MODE == GT_GATE_UP) v = glu_clamped_t(v, acc2[nb][i], p.limit, p.alpha);
      El<TC>::st(crow + n, v);
    }
  }
}

void launch_gemm_tile(const void* A, const void* B, void* C, int M, int N, int K, int batch, int64_t sAb, int64_t sAm,
                      int64_t sBb, int64_t sBn, int64_t sCb, int64_t sCm, int dc, hipStream_t st) {
  if (M <= 0 || N <= 0 || batch <= 0) return;
  if (batch > 65535 || (M + GT_BM - 1) / GT_BM > 65535) throw std::runtime_error("gemm_tile: grid too large");
  GemmTileArgs a{};
  a.A = (const bf16_t*)A; a.B = (const bf16_t*)B; a.C = C;
  a.M = M; a.N = N; a.K = K;
  a.sAb = sAb; a.sAm = sAm; a.sBb = sBb; a.sBn = sBn; a.sCb = sCb; a.sCm = sCm;
  dim3 g((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM, batch);
  if (dc == 0) gemm_tile_kernel<GT_PLAIN, bf16_t><<<g, 256, 0, st>>>(a);
  else if (dc == 1) gemm_tile_kernel<GT_PLAIN, float><<<g, 256, 0, st>>>(a);
  else throw std::runtime_error("gemm_tile: bad output dtype code");
  HIP_CHECK_LAUNCH();
}

// act[r, f] = glu(h[order[r] / top] . gate_e[f], h[..] . up_e[f]) over the tile list (bf16)
void launch_moe_gate_up_tile(const void* h, int64_t ldh, const void* wg, const void* wu, const void* meta,
                             const void* order, void* act, int E, int maxt, int top, int F, int K, float limit,
                             float alpha, hipStream_t st) {
  if (maxt <= 0) return;
  if (maxt > 65535) throw std::runtime_error("moe_gate_up: too many row tiles");
  GemmTileArgs a{};
  a.A = (const bf16_t*)h; a.B = (const bf16_t*)wg; a.B2 = (const bf16_t*)wu; a.C = act;
  a.N = F; a.K = K; a.sAm = ldh; a.sBb = (int64_t)F * K; a.sBn = K; a.sCm = F;
  a.meta = (const int*)meta; a.order = (const int*)order; a.E = E; a.maxt = maxt; a.top = top;
  a.limit = limit; a.alpha = alpha;
  dim3 g((F + GT_BN - 1) / GT_BN, maxt);
  gemm_tile_kernel<GT_GATE_UP, bf16_t><<<g, 256, 0, st>>>(a);
  HIP_CHECK_LAUNCH();
}

// y[r, n] = act[r, :] . down_e[n, :] over the tile list (fp32)
void launch_moe_down_tile(const void* act, const void* wd, const void* meta, void* y, int E, int maxt, int N, int F,
                          hipStream_t st) {
  if (maxt <= 0) return;
  if (maxt > 65535) throw std::runtime_error("moe_down: too many row tiles");
  GemmTileArgs a{};
  a.A = (const bf16_t*)act; a.B = (const bf16_t*)wd; a.C = y;
  a.N = N; a.K = F; a.sAm = F; a.sBb = (int64_t)N * F; a.sBn = F; a.sCm = N;
  a.meta = (const int*)meta; a.E = E; a.maxt = maxt; a.top = 1;
  dim3 g((N + GT_BN - 1) / GT_BN, maxt);
  gemm_tile_kernel<GT_DOWN, float><<<g, 256, 0, st>>>(a);
  HIP_CHECK_LAUNCH();
}
