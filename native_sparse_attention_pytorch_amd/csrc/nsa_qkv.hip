// Epilogue of the fused qkv projection (NSA.py:583-614, 643) as one kernel per direction.
//
// The projection's output row of a token, 'b n ((hq + 2 hk) d)', is read once.  From it the forward
// writes everything the three attention branches consume: the head-split rotated queries and keys
// (selection and sliding branches), the overlapping compression windows of the un-rotated keys and
// values with the intra-window positions added, in the 'b h w (cbs d)' layout the compression GEMM
// reads, and - for an fp32 projection - the bf16 head-split copies of the un-rotated queries and
// of the values (a bf16 projection is consumed in place through strided views).  The backward is
// the mirror image: one pass over the tokens that sums, per head, the inverse rotation of the
// rotated gradient, the direct gradient and the <= ceil(cbs/stride) window slots that hold the
// token (gather form: no atomics, fixed order) and writes the gradient of the projection's output
// row directly - no per-tensor rotation, overlap-add, head merge and concatenation kernels.
//
// A thread owns 8 consecutive features of one token and walks the heads, so the rotation angles of
// its four feature pairs are computed once per token instead of once per head.  HBM-bound: every
// input and output element moves once.
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

struct QkvArgs {
  int b, n, hq, hk, cbs, st, w, offset;
  long s_batch, s_tok;          // element strides of the projection output (and of its gradient)
};

template <typename T>
__device__ __forceinline__ void load_f8(const T* p, float (&x)[8]);
template <>
__device__ __forceinline__ void load_f8<__bf16>(const __bf16* p, float (&x)[8]) {
  const bf16x8 v = load8(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = (float)v[e];
}
template <>
__device__ __forceinline__ void load_f8<float>(const float* p, float (&x)[8]) {
  const floatx4 a = *reinterpret_cast<const floatx4*>(p), c = *reinterpret_cast<const floatx4*>(p + 4);
#pragma unroll
  for (int e = 0; e < 4; ++e) { x[e] = a[e]; x[4 + e] = c[e]; }
}

template <typename T>
__device__ __forceinline__ void store_f8(T* p, const float (&x)[8]);
template <>
__device__ __forceinline__ void store_f8<__bf16>(__bf16* p, const float (&x)[8]) {
  bf16x8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (__bf16)x[e];
  *reinterpret_cast<bf16x8*>(p) = v;
}
template <>
__device__ __forceinline__ void store_f8<float>(float* p, const float (&x)[8]) {
  floatx4 a, c;
#pragma unroll
  for (int e = 0; e < 4; ++e) { a[e] = x[e]; c[e] = x[4 + e]; }
  *reinterpret_cast<floatx4*>(p) = a;
  *reinterpret_cast<floatx4*>(p + 4) = c;
}

// pairs (2p, 2p+1) rotated by the angle whose sine / cosine are sn[p] / cs[p]
__device__ __forceinline__ void rotate8(const float (&x)[8], const float (&sn)[4], const float (&cs)[4], float (&r)[8]) {
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    r[2 * p] = x[2 * p] * cs[p] - x[2 * p + 1] * sn[p];
    r[2 * p + 1] = x[2 * p + 1] * cs[p] + x[2 * p] * sn[p];
  }
}

// Window slots (ww, j) that hold token `tok` (which may be one of the cbs - st virtual zero tokens
// left of token 0): ww*st + j - (cbs - st) == tok, 0 <= j < cbs, 0 <= ww < w.
__device__ __forceinline__ void window_range(const QkvArgs& A, int tok, int& a, int& w_lo, int& w_hi) {
  a = tok + A.cbs - A.st;
  w_hi = min(a / A.st, A.w - 1);
  w_lo = (a - A.cbs + 1 <= 0) ? 0 : (a - A.cbs + A.st) / A.st;       // ceil((a - cbs + 1) / st)
}

template <int D, typename T, typename TR>
__global__ __launch_bounds__(256) void qkv_prep_fwd_kernel(const QkvArgs A, const T* __restrict__ qkv, const float* __restrict__ freqs,
                                                           const T* __restrict__ kpos, const T* __restrict__ vpos,
                                                           __bf16* __restrict__ q16, TR* __restrict__ rq, TR* __restrict__ rk,
                                                           __bf16* __restrict__ v16, T* __restrict__ kw, T* __restrict__ vw) {
  constexpr int CPR = D / 8, TPB = 256 / CPR;
  const int lead = A.cbs > 0 ? A.cbs - A.st : 0;
  const int tok = (int)blockIdx.x * TPB + (int)threadIdx.x / CPR - lead;
  const int c = threadIdx.x % CPR, bb = blockIdx.y;
  if (tok >= A.n) return;
  const bool real = tok >= 0;
  float sn[4], cs[4];
  if (real) {
    const float pos = (float)(tok + A.offset);
#pragma unroll
    for (int p = 0; p < 4; ++p) sincosf(pos * freqs[4 * c + p], &sn[p], &cs[p]);
  }
  const T* row = qkv + bb * A.s_batch + (long)max(tok, 0) * A.s_tok + 8 * c;
  if (real) {
#pragma unroll 4
    for (int h = 0; h < A.hq; ++h) {
      float x[8], r[8];
      load_f8<T>(row + (long)h * D, x);
      const long at = (((long)bb * A.hq + h) * A.n + tok) * D + 8 * c;
      if (q16 != nullptr) store_f8<__bf16>(q16 + at, x);
      rotate8(x, sn, cs, r);
      store_f8<TR>(rq + at, r);
    }
  }
  int a = 0, w_lo = 0, w_hi = -1;
  if (A.cbs > 0 && A.w > 0) window_range(A, tok, a, w_lo, w_hi);
  const T* krow = row + (long)A.hq * D;
  const T* vrow = krow + (long)A.hk * D;
#pragma unroll 2
  for (int h = 0; h < A.hk; ++h) {
    float xk[8], xv[8];
    if (real) {
      load_f8<T>(krow + (long)h * D, xk);
      load_f8<T>(vrow + (long)h * D, xv);
      const long at = (((long)bb * A.hk + h) * A.n + tok) * D + 8 * c;
      float r[8];
      rotate8(xk, sn, cs, r);
      store_f8<TR>(rk + at, r);
      if (v16 != nullptr) store_f8<__bf16>(v16 + at, xv);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) { xk[e] = 0.f; xv[e] = 0.f; }
    }
    for (int ww = w_lo; ww <= w_hi; ++ww) {
      const int j = a - ww * A.st;
      float pk[8], pv[8], ok[8], ov[8];
      load_f8<T>(kpos + ((long)h * A.cbs + j) * D + 8 * c, pk);
      load_f8<T>(vpos + ((long)h * A.cbs + j) * D + 8 * c, pv);
#pragma unroll
      for (int e = 0; e < 8; ++e) { ok[e] = xk[e] + pk[e]; ov[e] = xv[e] + pv[e]; }
      const long slot = ((((long)bb * A.hk + h) * A.w + ww) * A.cbs + j) * D + 8 * c;
      store_f8<T>(kw + slot, ok);
      store_f8<T>(vw + slot, ov);
    }
  }
}

template <int D, typename T>
__global__ __launch_bounds__(256) void qkv_prep_bwd_kernel(const QkvArgs A, const __bf16* __restrict__ dq16, const __bf16* __restrict__ drq,
                                                           const __bf16* __restrict__ drk, const __bf16* __restrict__ dv16,
                                                           const T* __restrict__ dkw, const T* __restrict__ dvw,
                                                           const float* __restrict__ freqs, T* __restrict__ dqkv) {
  constexpr int CPR = D / 8, TPB = 256 / CPR;
  const int tok = (int)blockIdx.x * TPB + (int)threadIdx.x / CPR;
  const int c = threadIdx.x % CPR, bb = blockIdx.y;
  if (tok >= A.n) return;
  float sn[4], cs[4];
  {
    const float pos = (float)(tok + A.offset);
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      sincosf(pos * freqs[4 * c + p], &sn[p], &cs[p]);
      sn[p] = -sn[p];                                   // the transpose of a rotation is the rotation by the negative angle
    }
  }
  T* row = dqkv + bb * A.s_batch + (long)tok * A.s_tok + 8 * c;
#pragma unroll 4
  for (int h = 0; h < A.hq; ++h) {
    const long at = (((long)bb * A.hq + h) * A.n + tok) * D + 8 * c;
    float g[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] = 0.f;
    if (drq != nullptr) {
      float x[8];
      load_f8<__bf16>(drq + at, x);
      rotate8(x, sn, cs, g);
    }
    if (dq16 != nullptr) {
      float x[8];
      load_f8<__bf16>(dq16 + at, x);
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] += x[e];
    }
    store_f8<T>(row + (long)h * D, g);
  }
  int a = 0, w_lo = 0, w_hi = -1;
  if (A.cbs > 0 && A.w > 0) window_range(A, tok, a, w_lo, w_hi);
  T* krow = row + (long)A.hq * D;
  T* vrow = krow + (long)A.hk * D;
#pragma unroll 2
  for (int h = 0; h < A.hk; ++h) {
    const long at = (((long)bb * A.hk + h) * A.n + tok) * D + 8 * c;
    float gk[8], gv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) { gk[e] = 0.f; gv[e] = 0.f; }
    if (drk != nullptr) {
      float x[8];
      load_f8<__bf16>(drk + at, x);
      rotate8(x, sn, cs, gk);
    }
    if (dv16 != nullptr) load_f8<__bf16>(dv16 + at, gv);
    for (int ww = w_lo; ww <= w_hi; ++ww) {
      const int j = a - ww * A.st;
      const long slot = ((((long)bb * A.hk + h) * A.w + ww) * A.cbs + j) * D + 8 * c;
      if (dkw != nullptr) {
        float x[8];
        load_f8<T>(dkw + slot, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) gk[e] += x[e];
      }
      if (dvw != nullptr) {
        float x[8];
        load_f8<T>(dvw + slot, x);
#pragma unroll
        for (int e = 0; e < 8; ++e) gv[e] += x[e];
      }
    }
    store_f8<T>(krow + (long)h * D, gk);
    store_f8<T>(vrow + (long)h * D, gv);
  }
}

static int qkv_args(const nsa_qkv_desc* d, QkvArgs& A) {
  if (!d) return NSA_E_ARG;
  if (d->batch <= 0 || d->seq <= 0 || d->heads <= 0 || d->kv_heads <= 0 || d->batch > 65535) return NSA_E_ARG;
  if (d->dim_head != 64 && d->dim_head != 128) return NSA_E_UNSUPPORTED;
  if (d->block < 0 || (d->block > 0 && (d->stride <= 0 || d->block < d->stride))) return NSA_E_ARG;
  const long width = (long)(d->heads + 2 * d->kv_heads) * d->dim_head;
  if (d->qkv_stride[1] < width || (d->qkv_stride[0] | d->qkv_stride[1]) & 7) return NSA_E_ARG;
  A.b = d->batch; A.n = d->seq; A.hq = d->heads; A.hk = d->kv_heads;
  A.cbs = d->block; A.st = d->block > 0 ? d->stride : 1;
  A.w = d->block > 0 ? d->seq / d->stride : 0;
  A.offset = d->offset;
  A.s_batch = d->qkv_stride[0]; A.s_tok = d->qkv_stride[1];
  return 0;
}

}  // namespace nsa

using namespace nsa;

template <int D, typename T, typename TR = __bf16>
static int qkv_fwd_launch(const QkvArgs& A, const void* qkv, const float* freqs, const void* kpos, const void* vpos, void* q16, void* rq,
                          void* rk, void* v16, void* kw, void* vw, hipStream_t st) {
  constexpr int TPB = 256 / (D / 8);
  const int lead = A.cbs > 0 ? A.cbs - A.st : 0;
  hipLaunchKernelGGL((qkv_prep_fwd_kernel<D, T, TR>), dim3((unsigned)((A.n + lead + TPB - 1) / TPB), A.b), dim3(256), 0, st, A, (const T*)qkv, freqs,
                     (const T*)kpos, (const T*)vpos, (__bf16*)q16, (TR*)rq, (TR*)rk, (__bf16*)v16, (T*)kw, (T*)vw);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

template <int D, typename T>
static int qkv_bwd_launch(const QkvArgs& A, const void* dq16, const void* drq, const void* drk, const void* dv16, const void* dkw,
                          const void* dvw, const float* freqs, void* dqkv, hipStream_t st) {
  constexpr int TPB = 256 / (D / 8);
  hipLaunchKernelGGL((qkv_prep_bwd_kernel<D, T>), dim3((unsigned)((A.n + TPB - 1) / TPB), A.b), dim3(256), 0, st, A, (const __bf16*)dq16,
                     (const __bf16*)drq, (const __bf16*)drk, (const __bf16*)dv16, (const T*)dkw, (const T*)dvw, freqs, (T*)dqkv);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

extern "C" int nsa_qkv_prep_fwd(const nsa_qkv_desc* d, const void* qkv, const float* freqs, const void* k_pos, const void* v_pos,
                                void* q16, void* rq, void* rk, void* v16, void* k_windows, void* v_windows, void* stream) {
  QkvArgs A;
  const int rc = qkv_args(d, A);
  if (rc) return rc;
  if (!qkv || !freqs || !rq || !rk) return NSA_E_ARG;
  if (A.w > 0 && (!k_pos || !v_pos || !k_windows || !v_windows)) return NSA_E_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (d->fp32 == 2) {      // fp32 in, fp32 rotated outputs (the fp32 forward kernels read q and v from the projection itself)
    if (d->dim_head == 64) return qkv_fwd_launch<64, float, float>(A, qkv, freqs, k_pos, v_pos, nullptr, rq, rk, nullptr, k_windows, v_windows, st);
    return qkv_fwd_launch<128, float, float>(A, qkv, freqs, k_pos, v_pos, nullptr, rq, rk, nullptr, k_windows, v_windows, st);
  }
  if (d->fp32) {
    if (d->dim_head == 64) return qkv_fwd_launch<64, float>(A, qkv, freqs, k_pos, v_pos, q16, rq, rk, v16, k_windows, v_windows, st);
    return qkv_fwd_launch<128, float>(A, qkv, freqs, k_pos, v_pos, q16, rq, rk, v16, k_windows, v_windows, st);
  }
  if (d->dim_head == 64) return qkv_fwd_launch<64, __bf16>(A, qkv, freqs, k_pos, v_pos, q16, rq, rk, v16, k_windows, v_windows, st);
  return qkv_fwd_launch<128, __bf16>(A, qkv, freqs, k_pos, v_pos, q16, rq, rk, v16, k_windows, v_windows, st);
}

extern "C" int nsa_qkv_prep_bwd(const nsa_qkv_desc* d, const void* d_q16, const void* d_rq, const void* d_rk, const void* d_v16,
                                const void* d_k_windows, const void* d_v_windows, const float* freqs, void* d_qkv, void* stream) {
  QkvArgs A;
  const int rc = qkv_args(d, A);
  if (rc) return rc;
  if (!freqs || !d_qkv) return NSA_E_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (d->fp32) {
    if (d->dim_head == 64) return qkv_bwd_launch<64, float>(A, d_q16, d_rq, d_rk, d_v16, d_k_windows, d_v_windows, freqs, d_qkv, st);
    return qkv_bwd_launch<128, float>(A, d_q16, d_rq, d_rk, d_v16, d_k_windows, d_v_windows, freqs, d_qkv, st);
  }
  if (d->dim_head == 64) return qkv_bwd_launch<64, __bf16>(A, d_q16, d_rq, d_rk, d_v16, d_k_windows, d_v_windows, freqs, d_qkv, st);
  return qkv_bwd_launch<128, __bf16>(A, d_q16, d_rq, d_rk, d_v16, d_k_windows, d_v_windows, freqs, d_qkv, st);
}
