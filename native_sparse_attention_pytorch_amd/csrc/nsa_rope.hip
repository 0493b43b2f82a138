// Rotary position embedding on 'b h n d' bf16 tensors (NSA.py:238, 643: queries and keys of the
// selection and sliding branches).  Feature pairs (2k, 2k+1) are rotated by pos * freqs[k]
// (angles and arithmetic in fp32, result rounded to bf16, as the torch path does).  One kernel
// replaces the dozen elementwise launches of the composed torch expression; `inverse` rotates by
// the negative angle, which is the backward.  HBM-bound: reads and writes every element once.
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

template <int D>
__global__ __launch_bounds__(256) void rope_kernel(const __bf16* __restrict__ x, long s0, long s1, long s2, int b, int h, int n,
                                                   const float* __restrict__ freqs, int offset, int inverse, __bf16* __restrict__ out,
                                                   long o0, long o1, long o2) {
  constexpr int LPR = D / 8, RPB = 256 / LPR;
  const long row = (long)blockIdx.x * RPB + threadIdx.x / LPR;       // row = (b*h + head)*n + i
  const long rows = (long)b * h * n;
  if (row >= rows) return;
  const int c = threadIdx.x % LPR;
  const long i = row % n, bhh = row / n, hh = bhh % h, bb = bhh / h;
  const bf16x8 v = load8(x + bb * s0 + hh * s1 + i * s2 + 8 * c);
  const float pos = (float)(i + offset);
  bf16x8 r;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    float sn, cs;
    sincosf(pos * freqs[4 * c + p], &sn, &cs);
    if (inverse) sn = -sn;
    const float a = (float)v[2 * p], bq = (float)v[2 * p + 1];
    r[2 * p] = (__bf16)(a * cs - bq * sn);
    r[2 * p + 1] = (__bf16)(bq * cs + a * sn);
  }
  *reinterpret_cast<bf16x8*>(out + bb * o0 + hh * o1 + i * o2 + 8 * c) = r;
}

}  // namespace nsa

extern "C" int nsa_rope(const void* x, const int64_t* x_stride, int32_t batch, int32_t heads, int32_t seq, int32_t dim_head,
                        const float* freqs, int32_t offset, int32_t inverse, void* out, const int64_t* out_stride, void* stream) {
  using namespace nsa;
  if (!x || !x_stride || !freqs || !out || batch <= 0 || heads <= 0 || seq <= 0) return NSA_E_ARG;
  if ((x_stride[0] | x_stride[1] | x_stride[2]) & 7) return NSA_E_ARG;
  long o0 = (long)heads * seq * dim_head, o1 = (long)seq * dim_head, o2 = dim_head;
  if (out_stride) {
    if ((out_stride[0] | out_stride[1] | out_stride[2]) & 7) return NSA_E_ARG;
    o0 = out_stride[0]; o1 = out_stride[1]; o2 = out_stride[2];
  }
  const long rows = (long)batch * heads * seq;
  hipStream_t st = (hipStream_t)stream;
  if (dim_head == 64) {
    hipLaunchKernelGGL((rope_kernel<64>), dim3((unsigned)((rows + 31) / 32)), dim3(256), 0, st, (const __bf16*)x, (long)x_stride[0], (long)x_stride[1],
                       (long)x_stride[2], batch, heads, seq, freqs, offset, inverse, (__bf16*)out, o0, o1, o2);
  } else if (dim_head == 128) {
    hipLaunchKernelGGL((rope_kernel<128>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st, (const __bf16*)x, (long)x_stride[0], (long)x_stride[1],
                       (long)x_stride[2], batch, heads, seq, freqs, offset, inverse, (__bf16*)out, o0, o1, o2);
  } else {
    return NSA_E_UNSUPPORTED;
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}
