// A residual stream kept in fp32: scaled embedding gather and the fused "residual add + RMS norm" whose norm
// weight may be stored around zero (y = x / rms(x) * (offset + w), offset 1) or plainly (offset 0).
//
// The other families keep their residual in bf16 (norm.hip add_norm); designs that define the residual sum in
// 32-bit use these kernels instead: the stream x [T, H] is fp32 and updated in place, only the normed output that
// feeds the matrix products is rounded to the model's storage type.
#include "anytype.h"

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

// x[t] += (a[t] + b[t])   (either addend may be absent; a in the storage type, b in fp32)
// y[t]  = x[t] * rsqrt(mean(x[t]^2) + eps) * (woff + w)      (skipped when y is null)
// The sum is formed as x + (a + b): the two sublayer outputs of a parallel block are added to each other first.
template <typename T>
__global__ __launch_bounds__(256) void resid_add_norm_kernel(float* __restrict__ x, const T* __restrict__ a, int64_t lda,
                                                             const float* __restrict__ b, int64_t ldb,
                                                             const T* __restrict__ w, float woff, float eps,
                                                             T* __restrict__ y, int64_t ldy, int H) {
  __shared__ float red[16];
  const int t = blockIdx.x;
  float* xr = x + (int64_t)t * H;
  const T* ar = a ? a + (int64_t)t * lda : nullptr;
  const float* br = b ? b + (int64_t)t * ldb : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    float v = xr[c];
    if (ar || br) {
      float d = 0.f;
      if (ar) d = El<T>::ld(ar + c);
      if (br) d = ar ? d + br[c] : br[c];
      v += d;
      xr[c] = v;
    }
    ss += v * v;
  }
  if (!y) return;
  const float tot = block_sum(ss, red);
  const float r = 1.0f / sqrtf(tot / (float)H + eps);
  T* yr = y + (int64_t)t * ldy;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    // each thread re-reads the elements it wrote itself
    El<T>::st(yr + c, xr[c] * r * (woff + El<T>::ld(w + c)));
  }
}

void launch_resid_add_norm(void* x, const void* a, int64_t lda, const void* b, int64_t ldb, const void* w, float woff,
                           float eps, void* y, int64_t ldy, int T_, int H, int dt, hipStream_t st) {
  if (T_ == 0) return;
  DISPATCH_T(dt, T, (resid_add_norm_kernel<T><<<T_, 256, 0, st>>>((float*)x, (const T*)a, lda, (const float*)b, ldb,
                                                                    (const T*)w, woff, eps, (T*)y, ldy, H)));
  HIP_CHECK_LAUNCH();
}
