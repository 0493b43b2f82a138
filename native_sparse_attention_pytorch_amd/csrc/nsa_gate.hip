// Fused strategy-gate combine (NSA.py:323-327, 854-860): out[b,i,h*d..] = sum_s sigmoid(logit[b,i,
// 3h+s]) * branch_s[b,h,i,:], s = compressed, selected, sliding - written directly in the merged
// 'b n (h d)' layout the output projection reads.  Pure HBM-bandwidth kernels: forward reads
// 3 branch rows + 3 logits and writes 1 row per (b,h,i); backward reads 4 rows, writes 3 rows + 3
// logit gradients.  8 bf16 (16 bytes) per lane.
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

struct GateArgs {
  int b, h, n, d;
  long sc[3], sf[3], ss[3];      // element strides {batch, head, token} of the three branches
};

__device__ __forceinline__ float sigmoidf(float x) { return 1.0f / (1.0f + __expf(-x)); }

template <int D>
__global__ __launch_bounds__(256) void gate_fwd_kernel(const GateArgs A, const __bf16* __restrict__ logits, const __bf16* __restrict__ c,
                                                       const __bf16* __restrict__ f, const __bf16* __restrict__ s, __bf16* __restrict__ out) {
  constexpr int LPR = D / 8, RPB = 256 / LPR;
  const long row = (long)blockIdx.x * RPB + threadIdx.x / LPR;          // row = (b*n + i)*h + head
  const long rows = (long)A.b * A.n * A.h;
  if (row >= rows) return;
  const int dd = (threadIdx.x % LPR) * 8;
  const long hh = row % A.h, bi = row / A.h, i = bi % A.n, b = bi / A.n;
  const __bf16* lg = logits + bi * (3 * A.h) + 3 * hh;
  const float g0 = sigmoidf((float)lg[0]), g1 = sigmoidf((float)lg[1]), g2 = sigmoidf((float)lg[2]);
  const bf16x8 x0 = load8(c + b * A.sc[0] + hh * A.sc[1] + i * A.sc[2] + dd);
  const bf16x8 x1 = load8(f + b * A.sf[0] + hh * A.sf[1] + i * A.sf[2] + dd);
  const bf16x8 x2 = load8(s + b * A.ss[0] + hh * A.ss[1] + i * A.ss[2] + dd);
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (__bf16)(g0 * (float)x0[e] + g1 * (float)x1[e] + g2 * (float)x2[e]);
  *reinterpret_cast<bf16x8*>(out + row * D + dd) = r;
}

template <int D>
__global__ __launch_bounds__(256) void gate_bwd_kernel(const GateArgs A, const __bf16* __restrict__ logits, const __bf16* __restrict__ c,
                                                       const __bf16* __restrict__ f, const __bf16* __restrict__ s, const __bf16* __restrict__ dout,
                                                       __bf16* __restrict__ dlogits, __bf16* __restrict__ dc, __bf16* __restrict__ df, __bf16* __restrict__ ds) {
  constexpr int LPR = D / 8, RPB = 256 / LPR;
  const long row = (long)blockIdx.x * RPB + threadIdx.x / LPR;
  const long rows = (long)A.b * A.n * A.h;
  const bool ok = row < rows;
  const long rowc = ok ? row : 0;
  const int dd = (threadIdx.x % LPR) * 8;
  const long hh = rowc % A.h, bi = rowc / A.h, i = bi % A.n, b = bi / A.n;
  const __bf16* lg = logits + bi * (3 * A.h) + 3 * hh;
  const float g0 = sigmoidf((float)lg[0]), g1 = sigmoidf((float)lg[1]), g2 = sigmoidf((float)lg[2]);
  const bf16x8 x0 = load8(c + b * A.sc[0] + hh * A.sc[1] + i * A.sc[2] + dd);
  const bf16x8 x1 = load8(f + b * A.sf[0] + hh * A.sf[1] + i * A.sf[2] + dd);
  const bf16x8 x2 = load8(s + b * A.ss[0] + hh * A.ss[1] + i * A.ss[2] + dd);
  const bf16x8 go = load8(dout + rowc * D + dd);
  bf16x8 r0, r1, r2;
  float a0 = 0.f, a1 = 0.f, a2 = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float gv = (float)go[e];
    r0[e] = (__bf16)(g0 * gv); r1[e] = (__bf16)(g1 * gv); r2[e] = (__bf16)(g2 * gv);
    a0 += gv * (float)x0[e]; a1 += gv * (float)x1[e]; a2 += gv * (float)x2[e];
  }
#pragma unroll
  for (int mk = LPR / 2; mk >= 1; mk >>= 1) {
    a0 += __shfl_xor(a0, mk, 64); a1 += __shfl_xor(a1, mk, 64); a2 += __shfl_xor(a2, mk, 64);
  }
  if (!ok) return;
  const long orow = ((b * A.h + hh) * A.n + i) * D + dd;               // branch gradients: contiguous [b,h,n,d]
  *reinterpret_cast<bf16x8*>(dc + orow) = r0;
  *reinterpret_cast<bf16x8*>(df + orow) = r1;
  *reinterpret_cast<bf16x8*>(ds + orow) = r2;
  if ((threadIdx.x % LPR) == 0) {
    __bf16* dl = dlogits + bi * (3 * A.h) + 3 * hh;
    dl[0] = (__bf16)(a0 * g0 * (1.f - g0));
    dl[1] = (__bf16)(a1 * g1 * (1.f - g1));
    dl[2] = (__bf16)(a2 * g2 * (1.f - g2));
  }
}

}  // namespace nsa

using namespace nsa;

static int gate_args(GateArgs& A, int b, int h, int n, int d, const int64_t* sc, const int64_t* sf, const int64_t* ss) {
  if (b <= 0 || h <= 0 || n <= 0) return NSA_E_ARG;
  if (d != 64 && d != 128) return NSA_E_UNSUPPORTED;
  A.b = b; A.h = h; A.n = n; A.d = d;
  for (int t = 0; t < 3; ++t) {
    A.sc[t] = sc[t]; A.sf[t] = sf[t]; A.ss[t] = ss[t];
    if ((sc[t] | sf[t] | ss[t]) & 7) return NSA_E_ARG;
  }
  return 0;
}

extern "C" int nsa_gate_fwd(int32_t batch, int32_t heads, int32_t seq, int32_t dim_head, const void* logits,
                            const void* c, const int64_t* c_stride, const void* f, const int64_t* f_stride,
                            const void* s, const int64_t* s_stride, void* out, void* stream) {
  GateArgs A;
  if (!logits || !c || !f || !s || !out || !c_stride || !f_stride || !s_stride) return NSA_E_ARG;
  const int rc = gate_args(A, batch, heads, seq, dim_head, c_stride, f_stride, s_stride);
  if (rc) return rc;
  const long rows = (long)batch * seq * heads;
  hipStream_t st = (hipStream_t)stream;
  if (dim_head == 64) {
    hipLaunchKernelGGL((gate_fwd_kernel<64>), dim3((unsigned)((rows + 31) / 32)), dim3(256), 0, st, A, (const __bf16*)logits, (const __bf16*)c,
                       (const __bf16*)f, (const __bf16*)s, (__bf16*)out);
  } else {
    hipLaunchKernelGGL((gate_fwd_kernel<128>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st, A, (const __bf16*)logits, (const __bf16*)c,
                       (const __bf16*)f, (const __bf16*)s, (__bf16*)out);
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

extern "C" int nsa_gate_bwd(int32_t batch, int32_t heads, int32_t seq, int32_t dim_head, const void* logits,
                            const void* c, const int64_t* c_stride, const void* f, const int64_t* f_stride,
                            const void* s, const int64_t* s_stride, const void* d_out,
                            void* d_logits, void* dc, void* df, void* ds, void* stream) {
  GateArgs A;
  if (!logits || !c || !f || !s || !d_out || !d_logits || !dc || !df || !ds || !c_stride || !f_stride || !s_stride) return NSA_E_ARG;
  const int rc = gate_args(A, batch, heads, seq, dim_head, c_stride, f_stride, s_stride);
  if (rc) return rc;
  const long rows = (long)batch * seq * heads;
  hipStream_t st = (hipStream_t)stream;
  if (dim_head == 64) {
    hipLaunchKernelGGL((gate_bwd_kernel<64>), dim3((unsigned)((rows + 31) / 32)), dim3(256), 0, st, A, (const __bf16*)logits, (const __bf16*)c,
                       (const __bf16*)f, (const __bf16*)s, (const __bf16*)d_out, (__bf16*)d_logits, (__bf16*)dc, (__bf16*)df, (__bf16*)ds);
  } else {
    hipLaunchKernelGGL((gate_bwd_kernel<128>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st, A, (const __bf16*)logits, (const __bf16*)c,
                       (const __bf16*)f, (const __bf16*)s, (const __bf16*)d_out, (__bf16*)d_logits, (__bf16*)dc, (__bf16*)df, (__bf16*)ds);
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}
