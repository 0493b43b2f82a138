// fp32 forward kernels: the attention branches evaluated entirely in fp32 (products, softmax,
// accumulation), for fp32 modules that are run for inference and must agree with the reference's
// fp32 torch path to its own test tolerance (1e-5, tests/test_sparse_attn.py:86).  The bf16 MFMA
// kernels cannot give that; these do, at VALU speed.  They follow the same contracts as
// nsa_select_fwd (NSA.py:741-819) and nsa_dense_fwd (NSA.py:153-184, 632-639, 841-850).
//
// One wavefront serves one (batch, kv head, query): the G query heads of the group are taken GT at a
// time; a segment of up to 64 key rows is staged in LDS (row stride d + 1: conflict-free when lane
// = key walks a column), logits are computed with lane = key, the softmax runs online (running
// maximum / sum per head, wave reductions), and P V is accumulated with lane = feature from
// coalesced value rows.  Any head dimension <= 128 that is a multiple of 4, any group size, any
// block size.
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

constexpr int kF32MaxD = 128;
constexpr int kF32GT = 4;          // query heads per pass

struct F32Args {
  int b, hk, g, n, nk, d;          // n: number of queries (rows of q / out); nk: key rows after the memory slots
  int qoff;                       // query row i sits at sequence position i + qoff
  float scale;
  long sq[3], sk[3], sv[3];
  // dense
  int mode, causal, wb, wf, st, mem;
  // selection
  int S, B, W, idx64;
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

struct F32State {
  float m[kF32GT], l[kF32GT], acc[kF32GT][2];
};

// One segment of `cnt` <= 64 consecutive key rows starting at `row0` of this (batch, kv head)'s k / v.
// Rows at or beyond `rows_valid` read as zero keys and zero values (a selected block's padding past
// the sequence end counts with logit 0, NSA.py:744-752).  Lane `key` is masked when key > limit.
__device__ __forceinline__ void f32_segment(const F32Args& A, const float* __restrict__ q_s, float* __restrict__ k_s, float* __restrict__ p_s,
                                            const float* __restrict__ kb, const float* __restrict__ vb, int row0, int cnt, int rows_valid, int limit,
                                            int gn, F32State& S, int lane) {
  const int d = A.d, RS = d + 1, d4 = d >> 2;
  // stage the key rows (coalesced 16-byte loads, scalar LDS stores into the padded rows)
  for (int e = lane; e < cnt * d4; e += 64) {
    const int r = e / d4, c = e % d4;
    floatx4 x = {0.f, 0.f, 0.f, 0.f};
    if (row0 + r < rows_valid) x = *reinterpret_cast<const floatx4*>(kb + (long)(row0 + r) * A.sk[2] + 4 * c);
#pragma unroll
    for (int t = 0; t < 4; ++t) k_s[r * RS + 4 * c + t] = x[t];
  }
  __builtin_amdgcn_wave_barrier();          // one wave per work-group: its LDS operations execute in order
  float s[kF32GT];
#pragma unroll
  for (int g = 0; g < kF32GT; ++g) s[g] = 0.f;
  if (lane < cnt) {
    const float* kr = k_s + lane * RS;
    for (int dd = 0; dd < d; ++dd) {
      const float kv = kr[dd];
#pragma unroll
      for (int g = 0; g < kF32GT; ++g) s[g] = __builtin_fmaf(q_s[g * kF32MaxD + dd], kv, s[g]);
    }
  }
  const bool live = lane < cnt && lane <= limit;
#pragma unroll
  for (int g = 0; g < kF32GT; ++g) {
    const float sv = live ? s[g] * A.scale : -INFINITY;
    const float tmax = wave_max(sv);
    const float mn = fmaxf(S.m[g], tmax);
    const float mref = (mn == -INFINITY) ? 0.f : mn;
    const float alpha = expf(S.m[g] - mref);            // m = -inf: 0
    const float p = expf(sv - mref);
    S.l[g] = S.l[g] * alpha + wave_sum(p);
    S.m[g] = mn;
    S.acc[g][0] *= alpha;
    S.acc[g][1] *= alpha;
    p_s[g * 64 + lane] = p;
  }
  __builtin_amdgcn_wave_barrier();
  const int nrow = min(cnt, max(0, rows_valid - row0));      // zero value rows add nothing
  for (int r = 0; r < nrow; ++r) {
    const float* vr = vb + (long)(row0 + r) * A.sv[2];
    const float v0 = lane < d ? vr[lane] : 0.f;
    const float v1 = lane + 64 < d ? vr[lane + 64] : 0.f;
#pragma unroll
    for (int g = 0; g < kF32GT; ++g) {
      const float p = p_s[g * 64 + r];
      S.acc[g][0] = __builtin_fmaf(p, v0, S.acc[g][0]);
      S.acc[g][1] = __builtin_fmaf(p, v1, S.acc[g][1]);
    }
  }
  __builtin_amdgcn_wave_barrier();
  (void)gn;
}

__device__ __forceinline__ void f32_load_q(const F32Args& A, const float* __restrict__ q, int b, int hk, int i, int g0, float* q_s, int lane) {
  for (int e = lane; e < kF32GT * A.d; e += 64) {
    const int g = e / A.d, dd = e % A.d;
    q_s[g * kF32MaxD + dd] = (g0 + g < A.g) ? q[b * A.sq[0] + (long)(hk * A.g + g0 + g) * A.sq[1] + (long)i * A.sq[2] + dd] : 0.f;
  }
  __builtin_amdgcn_wave_barrier();
}

__device__ __forceinline__ void f32_store(const F32Args& A, const F32State& S, int b, int hk, int i, int g0, float* __restrict__ out,
                                          float* __restrict__ lse, int lane) {
#pragma unroll
  for (int g = 0; g < kF32GT; ++g) {
    if (g0 + g >= A.g) continue;
    const long hq = (long)hk * A.g + g0 + g;
    const float inv = S.l[g] > 0.f ? 1.0f / S.l[g] : 0.f;
    float* o = out + (((long)b * A.hk * A.g + hq) * A.n + i) * A.d;
    if (lane < A.d) o[lane] = S.acc[g][0] * inv;
    if (lane + 64 < A.d) o[lane + 64] = S.acc[g][1] * inv;
    if (lane == 0 && lse != nullptr) lse[((long)b * A.hk * A.g + hq) * A.n + i] = S.l[g] > 0.f ? S.m[g] + logf(S.l[g]) : -INFINITY;
  }
}

__device__ __forceinline__ void f32_reset(F32State& S) {
#pragma unroll
  for (int g = 0; g < kF32GT; ++g) { S.m[g] = -INFINITY; S.l[g] = 0.f; S.acc[g][0] = 0.f; S.acc[g][1] = 0.f; }
}

// interval-masked attention: band (mode 0) or memory slots + strided prefix (mode 1)
__global__ __launch_bounds__(64) void f32_dense_fwd_kernel(const F32Args A, const float* __restrict__ q, const float* __restrict__ k,
                                                           const float* __restrict__ v, float* __restrict__ out, float* __restrict__ lse) {
  __shared__ float q_s[kF32GT * kF32MaxD];
  __shared__ float k_s[64 * (kF32MaxD + 1)];
  __shared__ float p_s[kF32GT * 64];
  const int lane = threadIdx.x, i = blockIdx.x, bh = blockIdx.y, b = bh / A.hk, hk = bh % A.hk;
  const float* kb = k + b * A.sk[0] + hk * A.sk[1];
  const float* vb = v + b * A.sv[0] + hk * A.sv[1];
  const int pos = i + A.qoff;
  int lo, hi;
  if (A.mode == 0) { lo = max(0, pos - A.wb); hi = min(A.nk - 1, pos + A.wf); }
  else { lo = 0; hi = A.causal ? min(A.nk - 1, pos / A.st - 1) : A.nk - 1; }
  for (int g0 = 0; g0 < A.g; g0 += kF32GT) {
    F32State S;
    f32_reset(S);
    f32_load_q(A, q, b, hk, i, g0, q_s, lane);
    if (A.mem > 0) f32_segment(A, q_s, k_s, p_s, kb, vb, 0, A.mem, A.mem, 63, A.g - g0, S, lane);      // memory slots: always visible
    for (int r = lo; r <= hi; r += 64) {
      const int cnt = min(64, hi - r + 1);
      f32_segment(A, q_s, k_s, p_s, kb, vb, A.mem + r, cnt, A.mem + A.nk, 63, A.g - g0, S, lane);
    }
    f32_store(A, S, b, hk, i, g0, out, lse, lane);
  }
}

// block-selection attention: the live slots' blocks, then the own block up to the query
__global__ __launch_bounds__(64) void f32_select_fwd_kernel(const F32Args A, const float* __restrict__ q, const float* __restrict__ k,
                                                            const float* __restrict__ v, const void* __restrict__ idx,
                                                            const uint8_t* __restrict__ fmask, float* __restrict__ out, float* __restrict__ lse) {
  __shared__ float q_s[kF32GT * kF32MaxD];
  __shared__ float k_s[64 * (kF32MaxD + 1)];
  __shared__ float p_s[kF32GT * 64];
  const int lane = threadIdx.x, i = blockIdx.x, bh = blockIdx.y, b = bh / A.hk, hk = bh % A.hk;
  const float* kb = k + b * A.sk[0] + hk * A.sk[1];
  const float* vb = v + b * A.sv[0] + hk * A.sv[1];
  for (int g0 = 0; g0 < A.g; g0 += kF32GT) {
    F32State S;
    f32_reset(S);
    f32_load_q(A, q, b, hk, i, g0, q_s, lane);
    for (int s = 0; s < A.S; ++s) {
      const size_t pos = ((size_t)bh * A.n + i) * A.S + s;
      if (!fmask[pos]) continue;                         // wave-uniform
      long j = A.idx64 ? reinterpret_cast<const long long*>(idx)[pos] : (long)reinterpret_cast<const int*>(idx)[pos];
      if (j < 0 || j >= A.W) continue;
      for (int r = 0; r < A.B; r += 64)
        f32_segment(A, q_s, k_s, p_s, kb, vb, (int)j * A.B + r, min(64, A.B - r), A.nk, 63, A.g - g0, S, lane);
    }
    if (A.causal) {
      const int pos = i + A.qoff, own0 = (pos / A.B) * A.B;
      for (int r = own0; r <= pos; r += 64)
        f32_segment(A, q_s, k_s, p_s, kb, vb, r, min(64, pos - r + 1), A.nk, 63, A.g - g0, S, lane);
    }
    f32_store(A, S, b, hk, i, g0, out, lse, lane);
  }
}

static int f32_common(int batch, int kv_heads, int group, int seq, int q_offset, int dim_head, float scale, const int64_t* qs, const int64_t* ks,
                      const int64_t* vs, F32Args& A) {
  if (batch <= 0 || kv_heads <= 0 || group <= 0 || seq <= 0 || q_offset < 0) return NSA_E_ARG;
  A.qoff = q_offset;
  if (dim_head <= 0 || dim_head > kF32MaxD || (dim_head & 3)) return NSA_E_UNSUPPORTED;
  if ((long)batch * kv_heads > 65535) return NSA_E_UNSUPPORTED;
  A.b = batch; A.hk = kv_heads; A.g = group; A.n = seq; A.d = dim_head; A.scale = scale;
  for (int t = 0; t < 3; ++t) {
    A.sq[t] = qs[t]; A.sk[t] = ks[t]; A.sv[t] = vs[t];
    if ((A.sk[t] | A.sv[t]) & 3) return NSA_E_ARG;       // key / value rows are read 16 bytes at a time
  }
  return 0;
}

}  // namespace nsa

using namespace nsa;

extern "C" int nsa_dense_fwd_f32(const nsa_dense_desc* d, const float* q, const float* k, const float* v, float* out, float* lse,
                                 int32_t q_offset, void* stream) {
  if (!d || !q || !k || !v || !out) return NSA_E_ARG;
  F32Args A{};
  const int rc = f32_common(d->batch, d->kv_heads, d->group, d->seq, q_offset, d->dim_head, d->scale, d->q_stride, d->k_stride, d->v_stride, A);
  if (rc) return rc;
  if (d->num_keys < 0 || d->num_mem < 0 || d->num_mem > 64) return NSA_E_ARG;
  A.nk = d->num_keys; A.mem = d->num_mem; A.mode = d->mode; A.causal = d->causal ? 1 : 0;
  A.wb = A.wf = 0; A.st = 1;
  if (d->mode == 0) {
    if (d->window < 0 || d->num_mem != 0) return NSA_E_ARG;
    A.wb = d->window; A.wf = A.causal ? 0 : d->window;
  } else if (d->mode == 1) {
    if (d->stride <= 0) return NSA_E_ARG;
    if (A.causal && A.mem == 0) return NSA_E_ARG;
    A.st = d->stride;
  } else {
    return NSA_E_ARG;
  }
  hipLaunchKernelGGL(f32_dense_fwd_kernel, dim3(A.n, A.b * A.hk), dim3(64), 0, (hipStream_t)stream, A, q, k, v, out, lse);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

extern "C" int nsa_select_fwd_f32(const nsa_select_desc* d, const float* q, const float* k, const float* v, const void* idx,
                                  const uint8_t* fmask, float* out, float* lse, int32_t num_keys, int32_t q_offset, void* stream) {
  if (!d || !q || !k || !v || !out) return NSA_E_ARG;
  F32Args A{};
  const int rc = f32_common(d->batch, d->kv_heads, d->group, d->seq, q_offset, d->dim_head, d->scale, d->q_stride, d->k_stride, d->v_stride, A);
  if (rc) return rc;
  if (d->num_sel < 0 || d->block <= 0 || (d->num_sel > 0 && (!idx || !fmask))) return NSA_E_ARG;
  if (num_keys <= 0 || (d->causal && d->seq + q_offset > num_keys)) return NSA_E_ARG;      // a query's own position must have a key row
  A.nk = num_keys; A.S = d->num_sel; A.B = d->block; A.W = (num_keys + d->block - 1) / d->block; A.causal = d->causal ? 1 : 0;
  A.idx64 = d->idx_is_int64 ? 1 : 0;
  hipLaunchKernelGGL(f32_select_fwd_kernel, dim3(A.n, A.b * A.hk), dim3(64), 0, (hipStream_t)stream, A, q, k, v, idx, fmask, out, lse);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}
