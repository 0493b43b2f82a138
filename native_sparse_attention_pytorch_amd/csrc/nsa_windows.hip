// Compression windows (NSA.py:270-275, 589-603): window w of a 'b h n d' tensor holds tokens
// (w+1)*stride - cbs .. (w+1)*stride - 1 (zeros left of token 0), plus the learned intra-window
// position embedding 'h cbs d'.  The forward is a gather (+ add) that writes the windows directly
// in the 'b h w (cbs d)' layout the compression GEMM reads; the backward is the matching
// overlap-add in gather form (every token sums the <= ceil(cbs/stride) window slots that hold
// it: no atomics, fixed order).  HBM-bound: forward reads n*d and writes w*cbs*d elements per
// (b, h); one launch each instead of pad + unfold + permute + add (+ their backward kernels).
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

template <int D>
__global__ __launch_bounds__(256) void windows_fwd_kernel(const __bf16* __restrict__ x, long s0, long s1, long s2, const __bf16* __restrict__ pos,
                                                          int bh, int h, int w, int cbs, int st, __bf16* __restrict__ out) {
  constexpr int CPR = D / 8;
  const long e = (long)blockIdx.x * 256 + threadIdx.x;             // one 16-byte chunk of one window slot
  const long total = (long)bh * w * cbs * CPR;
  if (e >= total) return;
  const int c = (int)(e % CPR);
  const long slot = e / CPR;                                       // ((b*h + hh)*w + ww)*cbs + j
  const int j = (int)(slot % cbs);
  const long t1 = slot / cbs;
  const int ww = (int)(t1 % w);
  const int bhh = (int)(t1 / w), hh = bhh % h, bb = bhh / h;
  const long tok = (long)ww * st + j - (cbs - st);
  bf16x8 v = zero_frag();
  if (tok >= 0) v = load8(x + bb * s0 + hh * s1 + tok * s2 + 8 * c);
  if (pos != nullptr) {
    const bf16x8 p = load8(pos + ((long)hh * cbs + j) * D + 8 * c);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (__bf16)((float)v[i] + (float)p[i]);
  }
  *reinterpret_cast<bf16x8*>(out + slot * D + 8 * c) = v;
}

template <int D>
__global__ __launch_bounds__(256) void windows_bwd_kernel(const __bf16* __restrict__ dwin, int bh, int n, int w, int cbs, int st,
                                                          __bf16* __restrict__ dx) {
  constexpr int CPR = D / 8;
  const long e = (long)blockIdx.x * 256 + threadIdx.x;             // one 16-byte chunk of one token
  const long total = (long)bh * n * CPR;
  if (e >= total) return;
  const int c = (int)(e % CPR);
  const long row = e / CPR;
  const int tok = (int)(row % n);
  const long bhh = row / n;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  // slots (ww, j) with ww*st + j - (cbs - st) == tok, 0 <= j < cbs
  const int a = tok + cbs - st;
  int w_hi = a / st;
  if (w_hi > w - 1) w_hi = w - 1;
  int w_lo = (a - cbs + 1 + st - 1) / st;                          // ceil((a - cbs + 1) / st), a - cbs + 1 may be negative
  if (a - cbs + 1 <= 0) w_lo = 0;
  for (int ww = w_lo; ww <= w_hi; ++ww) {
    const int j = a - ww * st;
    const bf16x8 g = load8(dwin + (((long)bhh * w + ww) * cbs + j) * D + 8 * c);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += (float)g[i];
  }
  bf16x8 r;
#pragma unroll
  for (int i = 0; i < 8; ++i) r[i] = (__bf16)acc[i];
  *reinterpret_cast<bf16x8*>(dx + row * D + 8 * c) = r;
}

}  // namespace nsa

extern "C" int nsa_windows_fwd(const void* x, const int64_t* x_stride, const void* pos, int32_t batch, int32_t heads, int32_t seq,
                               int32_t dim_head, int32_t block, int32_t stride, void* out, void* stream) {
  using namespace nsa;
  if (!x || !x_stride || !out || batch <= 0 || heads <= 0 || seq < 0 || stride <= 0 || block < stride) return NSA_E_ARG;
  if ((x_stride[0] | x_stride[1] | x_stride[2]) & 7) return NSA_E_ARG;
  const int w = seq / stride;
  if (w == 0) return 0;
  const long chunks = (long)batch * heads * w * block * (dim_head / 8);
  const dim3 grid((unsigned)((chunks + 255) / 256));
  hipStream_t st = (hipStream_t)stream;
  if (dim_head == 64)
    hipLaunchKernelGGL((windows_fwd_kernel<64>), grid, dim3(256), 0, st, (const __bf16*)x, (long)x_stride[0], (long)x_stride[1], (long)x_stride[2],
                       (const __bf16*)pos, batch * heads, heads, w, block, stride, (__bf16*)out);
  else if (dim_head == 128)
    hipLaunchKernelGGL((windows_fwd_kernel<128>), grid, dim3(256), 0, st, (const __bf16*)x, (long)x_stride[0], (long)x_stride[1], (long)x_stride[2],
                       (const __bf16*)pos, batch * heads, heads, w, block, stride, (__bf16*)out);
  else
    return NSA_E_UNSUPPORTED;
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

extern "C" int nsa_windows_bwd(const void* d_windows, int32_t batch, int32_t heads, int32_t seq, int32_t dim_head, int32_t block,
                               int32_t stride, void* dx, void* stream) {
  using namespace nsa;
  if (!d_windows || !dx || batch <= 0 || heads <= 0 || seq <= 0 || stride <= 0 || block < stride) return NSA_E_ARG;
  const int w = seq / stride;
  const long chunks = (long)batch * heads * seq * (dim_head / 8);
  const dim3 grid((unsigned)((chunks + 255) / 256));
  hipStream_t st = (hipStream_t)stream;
  if (dim_head == 64)
    hipLaunchKernelGGL((windows_bwd_kernel<64>), grid, dim3(256), 0, st, (const __bf16*)d_windows, batch * heads, seq, w, block, stride, (__bf16*)dx);
  else if (dim_head == 128)
    hipLaunchKernelGGL((windows_bwd_kernel<128>), grid, dim3(256), 0, st, (const __bf16*)d_windows, batch * heads, seq, w, block, stride, (__bf16*)dx);
  else
    return NSA_E_UNSUPPORTED;
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}
