// Block-importance softmax and per-query top-k (NSA.py:693-713, 721): one wave per query row.
// Input row: nb importance logits (fp32, -inf = cannot be selected).  The row is softmaxed with
// the reference's extra -1e3 column (so a row with nothing visible becomes all zeros), then the
// k largest probabilities are extracted in descending order, ties going to the lower block
// index.  HBM-bound: reads nb*4 bytes per row, writes k*(4+4+1).
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

template <int VPL>
__global__ __launch_bounds__(256) void topk_kernel(const float* __restrict__ in, long rows, int nb, int k, int softmax,
                                                   int* __restrict__ idx, float* __restrict__ vals, uint8_t* __restrict__ fmask) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const float* src = in + row * nb;
  float x[VPL];
#pragma unroll
  for (int r = 0; r < VPL; ++r) {
    const int j = lane + 64 * r;
    x[r] = j < nb ? src[j] : -INFINITY;
  }
  if (softmax) {
    float mx = -1e3f;
#pragma unroll
    for (int r = 0; r < VPL; ++r) mx = fmaxf(mx, x[r]);
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < VPL; ++r) { x[r] = __expf(x[r] - mx); sum += x[r]; }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) sum += __shfl_xor(sum, o, 64);
    sum += __expf(-1e3f - mx);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int r = 0; r < VPL; ++r) x[r] *= inv;
  }
#pragma unroll
  for (int r = 0; r < VPL; ++r)
    if (lane + 64 * r >= nb) x[r] = -1.0f;               // padding loses against every real entry
  for (int s = 0; s < k; ++s) {
    float bv = x[0];
    int bj = lane;
#pragma unroll
    for (int r = 1; r < VPL; ++r)
      if (x[r] > bv) { bv = x[r]; bj = lane + 64 * r; }   // strict: ties keep the lower index
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oj = __shfl_xor(bj, o, 64);
      if (ov > bv || (ov == bv && oj < bj)) { bv = ov; bj = oj; }
    }
    if ((bj & 63) == lane) {
#pragma unroll
      for (int r = 0; r < VPL; ++r)
        if ((bj >> 6) == r) x[r] = -2.0f;                 // taken
    }
    if (lane == 0) {
      idx[row * k + s] = bj;
      vals[row * k + s] = bv;
      fmask[row * k + s] = bv > 1e-10f ? 1 : 0;
    }
  }
}

}  // namespace nsa

extern "C" int nsa_topk(const float* scores, int64_t rows, int32_t nb, int32_t k, int32_t apply_softmax,
                        int32_t* idx, float* vals, uint8_t* fmask, void* stream) {
  using namespace nsa;
  if (!scores || !idx || !vals || !fmask || rows <= 0 || nb <= 0 || k <= 0 || k > nb) return NSA_E_ARG;
  if (nb > 64 * 32) return NSA_E_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  const int vpl = (nb + 63) / 64;
#define NSA_TOPK(V) hipLaunchKernelGGL((topk_kernel<V>), grid, block, 0, st, scores, (long)rows, nb, k, apply_softmax, idx, vals, fmask)
  if (vpl <= 1) NSA_TOPK(1);
  else if (vpl <= 2) NSA_TOPK(2);
  else if (vpl <= 4) NSA_TOPK(4);
  else if (vpl <= 8) NSA_TOPK(8);
  else if (vpl <= 16) NSA_TOPK(16);
  else NSA_TOPK(32);
#undef NSA_TOPK
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}
