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
