// 64x64x16 fp32 tile step on the vector ALUs, shared by gemm_any.hip and the grouped expert GEMMs of moe.hip.
// A and B tiles sit k-major in LDS as floats ([k][row], row stride padded to 68 so the float4 reads of the 16
// thread columns do not collide); lane (tx, ty) of the 16x16 thread grid owns outputs rows ty*4.., columns tx*4...
#pragma once
#include "common.h"

#define TV_BM 64
#define TV_BN 64
#define TV_BK 16
#define TV_LD 68

__device__ __forceinline__ void tv_mac(float (&acc)[4][4], const float (&As)[TV_BK][TV_LD],
                                       const float (&Bs)[TV_BK][TV_LD], int tid) {
  const int tx = tid & 15, ty = tid >> 4;
#pragma unroll
  for (int kk = 0; kk < TV_BK; ++kk) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(&As[kk][ty * 4]);
    const f32x4 b = *reinterpret_cast<const f32x4*>(&Bs[kk][tx * 4]);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
  }
}
