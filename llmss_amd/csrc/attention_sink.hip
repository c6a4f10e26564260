// Softmax attention with a sink, a soft cap, partial rotary positions and head mixing, over a paged key/value cache
// whose key and value widths may differ.
//
//   s_h(i, j) = cap * tanh(scale * q_h(i) . k_g(j) / cap)          (cap 0: no cap)          g = h / (H / G)
//   p_h(i, j) = exp(s_h(i, j)) / (1 + sum_j' exp(s_h(i, j')))      j' over the causal keys: a sink of score 0
//   w_h(i, j) = sum_h' talk[h, h'] p_h'(i, j)                      (talk absent: w = p)
//   out_h(i)  = sum_j w_h(i, j) v_g(j)
//
// Mixing weights across heads commutes with the weighted sum over keys: out_h(i) = sum_h' talk[h, h'] O_h'(i)[g]
// with O_h'(i)[c] = sum_j p_h'(i, j) v_c(j) the weighted sum of head h''s weights over the values of group c. So
// the attention kernel runs an ordinary one-pass online softmax per head and accumulates against the whole value
// row of a key (all G groups side by side, as the cache stores it), and a small second kernel mixes. Without a
// talk matrix only the head's own group is accumulated.
//
// The sink enters the online softmax as its initial state: running maximum 0, running denominator 1, no value.
//
// One kernel serves portions of prompts, continued portions and single decoded tokens: a row finds its sequence and
// position through cu / ctx_lens and reads every key, those of its own step too, from the paged cache.
// Scores, softmax and sums are fp32; the cache is read in the model's storage type.
#include "anytype.h"
#include "seqrows.h"

// q (+ bias), k (+ bias) rotated on the first `rot` dimensions of each head (i paired with i + rot / 2) by the
// angle table cs [npos, rot / 2, 2] = (cos, sin) already scaled; v (+ bias) copied. q -> qout fp32 [T, H * dim];
// k, v -> the paged caches at slots[t] (slot < 0: not cached).
template <typename T>
__global__ __launch_bounds__(256) void rope_bias_cache_kernel(const T* __restrict__ proj, int64_t ldp, int off_q,
                                                              int off_k, int off_v, const T* __restrict__ bias,
                                                              const int64_t* __restrict__ positions,
                                                              const float* __restrict__ cs, int npos, int rot,
                                                              float* __restrict__ qout, T* __restrict__ kc,
                                                              T* __restrict__ vc, const int64_t* __restrict__ slots,
                                                              int H, int G, int dim, int vdim) {
  const int t = blockIdx.x;
  int64_t p = positions[t];
  p = p < 0 ? 0 : (p >= npos ? npos - 1 : p);
  const int half = rot >> 1;
  const float* tab = cs + p * (int64_t)half * 2;
  const T* row = proj + (int64_t)t * ldp;
  const int64_t slot = slots[t];
  const int nq = H * dim, nk = G * dim, nv = G * vdim;
  // bias layout: q | k | v
  for (int e = threadIdx.x; e < nq + nk; e += blockDim.x) {
    const bool isk = e >= nq;
    const int idx = isk ? e - nq : e;
    const int d = idx % dim;
    const int base = (isk ? off_k : off_q) + idx - d;
    const T* b = bias ? bias + (isk ? nq : 0) + idx - d : nullptr;
    float val = El<T>::ld(row + base + d) + (b ? El<T>::ld(b + d) : 0.f);
    if (d < rot) {
      const int i = d < half ? d : d - half;
      const int od = d < half ? d + half : d - half;
      const float other = El<T>::ld(row + base + od) + (b ? El<T>::ld(b + od) : 0.f);
      const float c = tab[2 * i], s = tab[2 * i + 1];
      val = d < half ? val * c - other * s : val * c + other * s;
    }
    if (!isk) qout[(int64_t)t * nq + idx] = val;
    else if (slot >= 0) El<T>::st(kc + slot * (int64_t)nk + idx, val);
  }
  if (slot >= 0)
    for (int e = threadIdx.x; e < nv; e += blockDim.x)
      El<T>::st(vc + slot * (int64_t)nv + e,
                El<T>::ld(row + off_v + e) + (bias ? El<T>::ld(bias + nq + nk + e) : 0.f));
}

void launch_rope_bias_cache(const void* proj, int64_t ldp, int off_q, int off_k, int off_v, const void* bias,
                            const void* positions, const void* cs, int npos, int rot, void* qout, void* kc, void* vc,
                            const void* slots, int T_, int H, int G, int dim, int vdim, int dt, hipStream_t st) {
  if (T_ == 0) return;
  if (rot < 0 || rot > dim || (rot & 1)) throw std::runtime_error("rope_bias_cache: rotary dims must be even, <= dim");
  DISPATCH_T(dt, T, (rope_bias_cache_kernel<T><<<T_, 256, 0, st>>>(
      (const T*)proj, ldp, off_q, off_k, off_v, (const T*)bias, (const int64_t*)positions, (const float*)cs, npos, rot,
      (float*)qout, (T*)kc, (T*)vc, (const int64_t*)slots, H, G, dim, vdim)));
  HIP_CHECK_LAUNCH();
}

// Workgroup: one row t, one key group g, NW of its query heads (a wave each). Grid (T, G * chunks of heads, chunks
// of value columns). A block of KB keys of group g is staged in LDS for all waves; a wave scores it with lanes over
// keys, updates its online softmax and accumulates over value columns (lanes over columns, NR registers per lane),
// reading value rows from the cache. Value columns v0 .. v0 + RV - 1 of the key's whole value row [G * vdim]
// (all = 1) or of group g's part (all = 0). out [T, H, RVtot] fp32.
template <typename T, int NR>
__global__ void sink_attn_kernel(const float* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc,
                                 const int* __restrict__ bt, int maxb, const int* __restrict__ cu,
                                 const int* __restrict__ ctx, float* __restrict__ out, int B, int H, int G, int dim,
                                 int vdim, int bs, float scale, float cap, int all, int KB, int Dp, int hchunks,
                                 int RVchunk) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int NW = blockDim.x >> 6;
  T* tile = reinterpret_cast<T*>(smem);
  float* qs = reinterpret_cast<float*>(smem + (((size_t)KB * Dp * sizeof(T) + 15) & ~(size_t)15));
  float* ps = qs + (size_t)NW * dim;
  const int t = blockIdx.x, wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int rep = H / G;
  const int g = blockIdx.y / hchunks;
  const int hl = (blockIdx.y % hchunks) * NW + wv;
  const bool live = hl < rep;
  const int h = g * rep + hl;
  const int RVtot = all ? G * vdim : vdim;
  const int v0 = blockIdx.z * RVchunk;
  const int RV = min(RVchunk, RVtot - v0);
  const int64_t vrow = (int64_t)G * vdim;
  const int voff = (all ? 0 : g * vdim) + v0;
  const RowSeq r = row_seq(cu, ctx, B, t);
  float* o = out + ((int64_t)t * H + h) * RVtot + v0;
  if (r.pos < 0) {
    if (live)
      for (int i = lane; i < RV; i += 64) o[i] = 0.f;
    return;
  }
  float* qw = qs + (size_t)wv * dim;
  float* p = ps + (size_t)wv * KB;
  if (live) {
    const float* qsrc = q + ((int64_t)t * H + h) * dim;
    for (int d = lane; d < dim; d += 64) qw[d] = qsrc[d] * scale;
  }
  float acc[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) acc[i] = 0.f;
  float m = 0.f, l = 1.f;  // the sink: score 0, weight exp(0 - m), no value
  const float icap = cap > 0.f ? 1.0f / cap : 0.f;
  const int* btr = bt + (int64_t)r.b * maxb;
  for (int j0 = 0; j0 <= r.pos; j0 += KB) {
    const int nk = min(KB, r.pos - j0 + 1);
    __syncthreads();
    for (int kk = wv; kk < nk; kk += NW) {
      const int j = j0 + kk;
      const int64_t slot = (int64_t)btr[j / bs] * bs + j % bs;
      const T* src = kc + (slot * G + g) * dim;
      T* dst = tile + (size_t)kk * Dp;
      for (int d = lane; d < dim; d += 64) dst[d] = src[d];
    }
    __syncthreads();
    if (live) {
      float s = -INFINITY;
      if (lane < nk) {
        const T* row = tile + (size_t)lane * Dp;
        float d_ = 0.f;
        for (int d = 0; d < dim; ++d) d_ = fmaf(qw[d], El<T>::ld(row + d), d_);
        s = cap > 0.f ? cap * tanhf(d_ * icap) : d_;
      }
      const float m_new = fmaxf(m, warp_max(s));
      const float alpha = expf(m - m_new);
      const float pj = lane < nk ? expf(s - m_new) : 0.f;
      l = l * alpha + warp_sum(pj);
      m = m_new;
      if (lane < KB) p[lane] = pj;
#pragma unroll
      for (int i = 0; i < NR; ++i) acc[i] *= alpha;
    }
    __syncthreads();
    if (live) {
      for (int kk = 0; kk < nk; ++kk) {
        const float pj = p[kk];
        const int j = j0 + kk;
        const int64_t slot = (int64_t)btr[j / bs] * bs + j % bs;
        const T* row = vc + slot * vrow + voff;
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const int c = lane + 64 * i;
          if (c < RV) acc[i] = fmaf(pj, El<T>::ld(row + c), acc[i]);
        }
      }
    }
  }
  if (live) {
    const float inv = 1.0f / l;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int c = lane + 64 * i;
      if (c < RV) o[c] = acc[i] * inv;
    }
  }
}

template <typename T>
static void sink_attn_t(const void* q, const void* kc, const void* vc, const void* bt, int maxb, const void* cu,
                        const void* ctx, void* out, int T_, int B, int H, int G, int dim, int vdim, int bs,
                        float scale, float cap, int all, hipStream_t st) {
  const int rep = H / G;
  const int NW = std::min(rep, 8);
  const int hchunks = (rep + NW - 1) / NW;
  int Dp;  // key row stride in LDS: an odd number of 4-byte words (lanes score neighbouring keys)
  if (sizeof(T) == 2) {
    Dp = (dim + 1) & ~1;
    if (((Dp / 2) & 1) == 0) Dp += 2;
  } else {
    Dp = dim | 1;
  }
  int KB = 64;
  auto bytes = [&](int kb) { return (((size_t)kb * Dp * sizeof(T) + 15) & ~(size_t)15) + (size_t)NW * (dim + kb) * 4; };
  while (KB > 4 && bytes(KB) > 60 * 1024) KB >>= 1;
  if (bytes(KB) > 60 * 1024) throw std::runtime_error("sink attention: head dimension too large for LDS");
  const int RVtot = all ? G * vdim : vdim;
  const int RVchunk = std::min(RVtot, 512);
  const int zch = (RVtot + RVchunk - 1) / RVchunk;
  if (G * hchunks > 65535 || zch > 65535) throw std::runtime_error("sink attention: too many heads");
  dim3 g(T_, G * hchunks, zch);
  const int nr = (RVchunk + 63) / 64;
#define LAUNCH_SA(NR_)                                                                                              \
  sink_attn_kernel<T, NR_><<<g, NW * 64, bytes(KB), st>>>((const float*)q, (const T*)kc, (const T*)vc,              \
                                                          (const int*)bt, maxb, (const int*)cu, (const int*)ctx,    \
                                                          (float*)out, B, H, G, dim, vdim, bs, scale, cap, all, KB, \
                                                          Dp, hchunks, RVchunk)
  if (nr <= 1) LAUNCH_SA(1);
  else if (nr <= 2) LAUNCH_SA(2);
  else if (nr <= 4) LAUNCH_SA(4);
  else LAUNCH_SA(8);
#undef LAUNCH_SA
}

void launch_sink_attn(const void* q, const void* kc, const void* vc, const void* bt, int maxb, const void* cu,
                      const void* ctx, void* out, int T_, int B, int H, int G, int dim, int vdim, int bs, float scale,
                      float cap, int all, int dt, hipStream_t st) {
  if (T_ == 0 || B == 0) return;
  if (G < 1 || H % G) throw std::runtime_error("sink attention: heads must be a multiple of the key/value heads");
  DISPATCH_T(dt, T, (sink_attn_t<T>(q, kc, vc, bt, maxb, cu, ctx, out, T_, B, H, G, dim, vdim, bs, scale, cap, all,
                                    st)));
  HIP_CHECK_LAUNCH();
}

// y[t, h * vdim + v] = c * sum_h' talk[h, h'] O[t, h', g(h) * vdim + v]     (talk null: y = c * O[t, h, v])
template <typename T>
__global__ __launch_bounds__(256) void talk_mix_kernel(const float* __restrict__ O, const float* __restrict__ talk,
                                                       float c, T* __restrict__ y, int64_t ldy, int H, int G,
                                                       int vdim) {
  const int t = blockIdx.x;
  const int rep = H / G;
  const int RVtot = talk ? G * vdim : vdim;
  const float* Ot = O + (int64_t)t * H * RVtot;
  for (int e = threadIdx.x; e < H * vdim; e += blockDim.x) {
    const int h = e / vdim, v = e % vdim;
    float a;
    if (talk) {
      a = 0.f;
      const int col = (h / rep) * vdim + v;
      for (int hh = 0; hh < H; ++hh) a = fmaf(talk[h * H + hh], Ot[(int64_t)hh * RVtot + col], a);
    } else {
      a = Ot[(int64_t)h * RVtot + v];
    }
    El<T>::st(y + (int64_t)t * ldy + e, a * c);
  }
}

void launch_talk_mix(const void* O, const void* talk, float c, void* y, int64_t ldy, int T_, int H, int G, int vdim,
                     int dt, hipStream_t st) {
  if (T_ == 0) return;
  DISPATCH_T(dt, T, (talk_mix_kernel<T><<<T_, 256, 0, st>>>((const float*)O, (const float*)talk, c, (T*)y, ldy, H, G,
                                                            vdim)));
  HIP_CHECK_LAUNCH();
}
