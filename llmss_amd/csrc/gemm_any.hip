// Strided, batched matrix product for any shape and either storage type, fp32 accumulation on the vector ALUs:
//
//   C[b][m][n] = sum_k A[b][m][k] * B[b][n][k]
//   A(m, k) = A[b * sAb + m * sAm + k]            (k contiguous)
//   B(n, k) = B[b * sBb + n * sBn + k * sBk]      (either index may be the contiguous one)
//   C(m, n) = C[b * sCb + m * sCm + n]
//
// It serves (a) the true-fp32 execution of a model (the MFMA GEMMs of gemm.hip are bf16 / fp8 only), (b) per-head
// batched products against a slice of a weight (the absorbed projections of latent attention: B indexed k-major),
// (c) products whose output must stay fp32 (router logits) and (d) shapes the MFMA kernels refuse (K % 16,
// unaligned rows). 64x64 tile per 256-thread workgroup, 16-deep k steps through LDS, 4x4 outputs per lane; every
// load and store is bounds-checked, so no shape assumption is left to the caller.
#include "anytype.h"
#include "tile_valu.h"

struct GemmAnyArgs {
  const void* A;
  const void* B;
  void* C;
  int M, N, K;
  int64_t sAb, sAm, sBb, sBn, sBk, sCb, sCm;
};

template <typename TA, typename TB, typename TC>
__global__ __launch_bounds__(256) void gemm_any_kernel(GemmAnyArgs p) {
  __shared__ float As[TV_BK][TV_LD];
  __shared__ float Bs[TV_BK][TV_LD];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * TV_BM, n0 = blockIdx.x * TV_BN;
  const TA* A = (const TA*)p.A + (int64_t)blockIdx.z * p.sAb;
  const TB* B = (const TB*)p.B + (int64_t)blockIdx.z * p.sBb;
  TC* C = (TC*)p.C + (int64_t)blockIdx.z * p.sCb;
  float acc[4][4] = {};
  const bool b_kmajor = p.sBk != 1;  // B's contiguous index is n: let neighbouring lanes take neighbouring n
  for (int k0 = 0; k0 < p.K; k0 += TV_BK) {
    {
      const int r = tid >> 2, kk = (tid & 3) * 4;
      const int m = m0 + r;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + kk + i;
        As[kk + i][r] = (m < p.M && k < p.K) ? El<TA>::ld(A + (int64_t)m * p.sAm + k) : 0.f;
      }
    }
    if (!b_kmajor) {
      const int r = tid >> 2, kk = (tid & 3) * 4;
      const int n = n0 + r;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + kk + i;
        Bs[kk + i][r] = (n < p.N && k < p.K) ? El<TB>::ld(B + (int64_t)n * p.sBn + (int64_t)k * p.sBk) : 0.f;
      }
    } else {
      const int r = tid & 63, kk = (tid >> 6) * 4;
      const int n = n0 + r;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = k0 + kk + i;
        Bs[kk + i][r] = (n < p.N && k < p.K) ? El<TB>::ld(B + (int64_t)n * p.sBn + (int64_t)k * p.sBk) : 0.f;
      }
    }
    __syncthreads();
    tv_mac(acc, As, Bs, tid);
    __syncthreads();
  }
  const int tx = tid & 15, ty = tid >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < p.N) El<TC>::st(C + (int64_t)m * p.sCm + n, acc[i][j]);
    }
  }
}

template <typename TA, typename TB>
static void gemm_any_c(int dc, const GemmAnyArgs& a, dim3 g, hipStream_t st) {
  if (dc == 0)
    gemm_any_kernel<TA, TB, bf16_t><<<g, 256, 0, st>>>(a);
  else
    gemm_any_kernel<TA, TB, float><<<g, 256, 0, st>>>(a);
}

void launch_gemm_any(const void* A, const void* B, void* C, int M, int N, int K, int batch, int64_t sAb, int64_t sAm,
                     int64_t sBb, int64_t sBn, int64_t sBk, int64_t sCb, int64_t sCm, int da, int db, int dc,
                     hipStream_t st) {
  if (M <= 0 || N <= 0 || batch <= 0) return;
  if ((da | db | dc) & ~1) throw std::runtime_error("gemm_any: bad dtype code");
  if (batch > 65535 || (M + TV_BM - 1) / TV_BM > 65535) throw std::runtime_error("gemm_any: grid too large");
  GemmAnyArgs a{A, B, C, M, N, K, sAb, sAm, sBb, sBn, sBk, sCb, sCm};
  dim3 g((N + TV_BN - 1) / TV_BN, (M + TV_BM - 1) / TV_BM, batch);
  if (da == 0 && db == 0) gemm_any_c<bf16_t, bf16_t>(dc, a, g, st);
  else if (da == 1 && db == 0) gemm_any_c<float, bf16_t>(dc, a, g, st);
  else if (da == 0 && db == 1) gemm_any_c<bf16_t, float>(dc, a, g, st);
  else gemm_any_c<float, float>(dc, a, g, st);
  HIP_CHECK_LAUNCH();
}
