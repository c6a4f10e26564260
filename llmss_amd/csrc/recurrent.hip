// Linear recurrences over a matrix state per head, carried from token to token in fp32.
//
// Every head keeps a state S [dim, vdim]. Per token, with key k and query q [dim] and value v [vdim]:
//
//   decay (MODE 0):  S <- a S + k v^T                          o = S^T q     a = decay[head], a constant
//   delta (MODE 1):  S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q
//                    k <- k / sqrt(|k|^2 + 1e-6), q <- q / sqrt(|q|^2 + 1e-6) / sqrt(dim)
//                    beta = sigmoid(b), g = exp(-exp(A_log[head]) softplus(a + dt_bias[head]))
//
// Both updates act on the columns of S independently: column c needs only v[c] and the whole k and q. So a thread
// owns one column (dim <= 128 values in registers; larger dims are split over 2 or 4 neighbouring lanes that
// reduce with shuffles), and a workgroup owns (sequence, head, block of columns). Tokens are walked in order; the
// rows of CT tokens at a time are staged in LDS by the whole workgroup (activation and the per-token scalars are
// applied there). The state is read from the sequence's slot unless the portion starts at position 0 (then it is
// zero, whatever the slot held) and written back at the end. Rows of a padded sequence (no slot) are zeroed.
#include "anytype.h"
#include "seqrows.h"

#define REC_CT 8

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
};

// TQ: storage of q / k / v; TP: storage of a / b. R: state values per lane, P lanes per column.
template <typename TQ, typename TP, int R, int MODE>
__global__ __launch_bounds__(256) void recurrence_kernel(RecArgs A, int P, int cols) {
  extern __shared__ float sm[];
  const int b = blockIdx.x, h = blockIdx.y;
  const int dim = A.dim, vdim = A.vdim;
  const int g = h / (A.H / A.G);
  const int qlen = A.cu[b + 1] - A.cu[b];
  if (qlen <= 0) return;
  const int t0 = A.cu[b], n = A.ctx[b], slot = A.sslots[b];
  const int col = blockIdx.z * cols + threadIdx.x / P, part = threadIdx.x % P;
  const bool live = col < vdim && threadIdx.x / P < cols;
  if (slot < 0 || n <= 0) {
    if (live && part == 0)
      for (int j = 0; j < qlen; ++j) A.out[(int64_t)(t0 + j) * A.ldo + (int64_t)h * vdim + col] = 0.f;
    return;
  }
  const int p0 = n - qlen;
  const int d0 = part * R;  // this lane's rows of the column: d0 .. d0 + R - 1
  float S[R];
  float* sp = A.state + (((int64_t)slot * A.H + h) * dim) * vdim;
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = (live && p0 > 0 && d0 + i < dim) ? sp[(int64_t)(d0 + i) * vdim + col] : 0.f;
  // LDS per staged token: k [dim], q [dim], v [cols], 2 scalars
  const int per = 2 * dim + cols + 2;
  float a_const = 0.f, dtb = 0.f;
  if (MODE == 0) a_const = A.decay[h];
  else {
    a_const = expf(A.decay[h]);
    dtb = A.dt_bias[h];
  }
  const float qmul = MODE == 1 ? 1.0f / sqrtf((float)dim) : 1.0f;
  for (int j0 = 0; j0 < qlen; j0 += REC_CT) {
    const int nt = min(REC_CT, qlen - j0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < nt * per; idx += blockDim.x) {
      const int jj = idx / per, e = idx % per;
      const int64_t t = t0 + j0 + jj;
      float val;
      if (e < 2 * dim) {
        const bool isq = e >= dim;
        const int d = isq ? e - dim : e;
        const TQ* src = isq ? (const TQ*)A.q + t * A.ldq : (const TQ*)A.k + t * A.ldk;
        val = El<TQ>::ld(src + (int64_t)g * dim + d);
        if (A.silu_in) val = val / (1.0f + expf(-val));
      } else if (e < 2 * dim + cols) {
        const int c = blockIdx.z * cols + (e - 2 * dim);
        val = c < vdim ? El<TQ>::ld((const TQ*)A.v + t * A.ldv + (int64_t)h * vdim + c) : 0.f;
        if (A.silu_in) val = val / (1.0f + expf(-val));
      } else if (MODE == 1) {
        const TP* ab = (const TP*)A.ab + t * A.ldab;
        if (e == 2 * dim + cols) {  // beta
          val = 1.0f / (1.0f + expf(-El<TP>::ld(ab + A.off_b + h)));
        } else {  // g
          const float z = El<TP>::ld(ab + A.off_a + h) + dtb;
          const float sp_ = z > 20.f ? z : log1pf(expf(z));
          val = expf(-a_const * sp_);
        }
      } else {
        val = 0.f;
      }
      sm[idx] = val;
    }
    __syncthreads();
    for (int jj = 0; jj < nt; ++jj) {
      const float* ks = sm + jj * per;
      const float* qs = ks + dim;
      const float vv = ks[2 * dim + min((int)threadIdx.x / P, cols - 1)];
      float o = 0.f;
      if (MODE == 0) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
          if (d0 + i < dim) {
            S[i] = fmaf(a_const, S[i], ks[d0 + i] * vv);
            o = fmaf(S[i], qs[d0 + i], o);
          }
        }
        for (int m = 1; m < P; m <<= 1) o += __shfl_xor(o, m, 64);
      } else {
        const float beta = ks[2 * dim + cols], gg = ks[2 * dim + cols + 1];
        float kk = 0.f, qq = 0.f, sk = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
          if (d0 + i < dim) {
            const float kd = ks[d0 + i], qd = qs[d0 + i];
            kk = fmaf(kd, kd, kk);
            qq = fmaf(qd, qd, qq);
            S[i] *= gg;
            sk = fmaf(S[i], kd, sk);
          }
        }
        for (int m = 1; m < P; m <<= 1) {
          kk += __shfl_xor(kk, m, 64);
          qq += __shfl_xor(qq, m, 64);
          sk += __shfl_xor(sk, m, 64);
        }
        const float kn = 1.0f / sqrtf(kk + 1e-6f), qn = qmul / sqrtf(qq + 1e-6f);
        const float u = beta * (vv - sk * kn);
#pragma unroll
        for (int i = 0; i < R; ++i) {
          if (d0 + i < dim) {
            S[i] = fmaf(ks[d0 + i] * kn, u, S[i]);
            o = fmaf(S[i], qs[d0 + i], o);
          }
        }
        for (int m = 1; m < P; m <<= 1) o += __shfl_xor(o, m, 64);
        o *= qn;
      }
      if (live && part == 0) A.out[(int64_t)(t0 + j0 + jj) * A.ldo + (int64_t)h * vdim + col] = o;
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (d0 + i < dim) sp[(int64_t)(d0 + i) * vdim + col] = S[i];
  }
}

template <typename TQ, typename TP, int MODE>
static void recurrence_t(const RecArgs& A, int B, hipStream_t st) {
  const int dim = A.dim, vdim = A.vdim;
  int P = 1;
  while (P < 4 && dim > 128 * P) P <<= 1;
  if (dim > 128 * P) throw std::runtime_error("recurrence: key dimension above 512");
  const int per_lane = (dim + P - 1) / P;
  const int R = per_lane <= 32 ? 32 : (per_lane <= 64 ? 64 : 128);
  const int cols = std::min(vdim, 64 / P);  // one wave per workgroup: many small workgroups fill the chip
  const int threads = ((cols * P + 63) / 64) * 64;
  dim3 g(B, A.H, (vdim + cols - 1) / cols);
  if (A.H > 65535 || g.z > 65535) throw std::runtime_error("recurrence: too many heads or columns");
  const size_t lds = (size_t)REC_CT * (2 * dim + cols + 2) * 4;
  if (R == 32) recurrence_kernel<TQ, TP, 32, MODE><<<g, threads, lds, st>>>(A, P, cols);
  else if (R == 64) recurrence_kernel<TQ, TP, 64, MODE><<<g, threads, lds, st>>>(A, P, cols);
  else recurrence_kernel<TQ, TP, 128, MODE><<<g, threads, lds, st>>>(A, P, cols);
}

void launch_recurrence(int mode, const void* q, const void* k, const void* v, int64_t ldq, int64_t ldk, int64_t ldv,
                       const void* ab, int64_t ldab, int off_a, int off_b, const void* decay, const void* dt_bias,
                       void* state, const void* cu, const void* ctx, const void* sslots, void* out, int64_t ldo, int B,
                       int H, int G, int dim, int vdim, int silu_in, int dq, int dp, hipStream_t st) {
  if (B == 0) return;
  if (G < 1 || H % G) throw std::runtime_error("recurrence: heads must be a multiple of the key heads");
  RecArgs A{q, k, v, ldq, ldk, ldv, ab, ldab, off_a, off_b, (const float*)decay, (const float*)dt_bias, (float*)state,
            (const int*)cu, (const int*)ctx, (const int*)sslots, (float*)out, ldo, H, G, dim, vdim, silu_in};
  if (mode == 0) DISPATCH_T(dq, TQ, (recurrence_t<TQ, float, 0>(A, B, st)));
  else DISPATCH_T(dq, TQ, DISPATCH_T(dp, TP, (recurrence_t<TQ, TP, 1>(A, B, st))));
  HIP_CHECK_LAUNCH();
}
