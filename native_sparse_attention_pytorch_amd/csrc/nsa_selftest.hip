// Hardware self-test of the register layouts every NSA kernel relies on (see mfma32 and
// make_ident in nsa_common.hpp).  One wave multiplies A[32x16] by B[16x32] (row-major bf16 in
// memory) into C[32x32] fp32 and also writes T = transpose-by-identity of X[32x32] bf16.
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

__global__ __launch_bounds__(64) void selftest_kernel(const __bf16* A, const __bf16* B, float* Cm, const __bf16* X, float* T) {
  const int lane = threadIdx.x, n = lane & 31, h = lane >> 5;
  bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a[e] = A[n * 16 + 8 * h + e];          // A: row n, k = 8h+e
    b[e] = B[(8 * h + e) * 32 + n];        // B: k = 8h+e, col n
  }
  floatx16 c = mfma32(a, b, zero_acc());
#pragma unroll
  for (int i = 0; i < 16; ++i) Cm[(8 * (i >> 2) + 4 * h + (i & 3)) * 32 + n] = c[i];

  bf16x8 ilo, ihi, xlo, xhi;
  make_ident(lane, ilo, ihi);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    xlo[e] = X[n * 32 + 8 * h + e];
    xhi[e] = X[n * 32 + 16 + 8 * h + e];
  }
  floatx16 t = mfma32(xlo, ilo, zero_acc());
  t = mfma32(xhi, ihi, t);
  // expected: lane <-> column n of X, register i <-> row 8*(i/4)+4h+(i%4)
#pragma unroll
  for (int i = 0; i < 16; ++i) T[(8 * (i >> 2) + 4 * h + (i & 3)) * 32 + n] = t[i];
}

}  // namespace nsa

extern "C" int nsa_selftest_mfma(const void* A, const void* B, float* Cm, const void* X, float* T, void* stream) {
  if (!A || !B || !Cm || !X || !T) return NSA_E_ARG;
  hipLaunchKernelGGL(nsa::selftest_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (const __bf16*)A, (const __bf16*)B, Cm, (const __bf16*)X, T);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

// ---------------------------------------------------------------------------- memory probe
// What the memory system gives the access pattern of the block-selection walks: every wavefront
// repeats { gather `reads` groups of four 1 KB rows from pseudo-random rows of src, scatter `writes`
// groups of four 1 KB rows to pseudo-random rows of dst } with the loads of a round in flight
// together.  With src small it measures the L2 / memory-side cache, with both large the HBM under
// mixed read / write traffic - the ceiling the walks' achieved GB/s should be compared with.
namespace nsa {

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

__global__ __launch_bounds__(64) void row_traffic_kernel(const floatx4* __restrict__ src, unsigned src_rows, floatx4* __restrict__ dst,
                                                         unsigned dst_rows, int reads, int writes, int iters, int nontemporal, unsigned seed) {
  const unsigned w = blockIdx.x, lane = threadIdx.x;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
    const unsigned base = seed + (w * (unsigned)iters + it) * 64u;
    for (int r = 0; r < reads; ++r) {
      floatx4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = src[(size_t)(probe_hash(base + 4 * r + u) % src_rows) * 64 + lane];
#pragma unroll
      for (int u = 0; u < 4; ++u) acc += v[u];
    }
    for (int r = 0; r < writes; ++r) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        floatx4* p = &dst[(size_t)(probe_hash(base + 32 + 4 * r + u) % dst_rows) * 64 + lane];
        if (nontemporal) __builtin_nontemporal_store(acc, p);
        else *p = acc;
      }
    }
  }
  // keep the loads alive when nothing is written
  if (writes == 0 && acc[0] == 12345.678f) dst[lane] = acc;
}

}  // namespace nsa

extern "C" int nsa_probe_row_traffic(const void* src, size_t src_rows, void* dst, size_t dst_rows, int32_t reads, int32_t writes,
                                     int32_t iters, int32_t waves, int32_t nontemporal, uint32_t seed, void* stream) {
  if (!src || !dst || src_rows == 0 || dst_rows == 0 || src_rows > 0xffffffffu || dst_rows > 0xffffffffu) return NSA_E_ARG;
  if (reads < 0 || writes < 0 || reads > 8 || writes > 8 || iters <= 0 || waves <= 0) return NSA_E_ARG;
  hipLaunchKernelGGL(nsa::row_traffic_kernel, dim3(waves), dim3(64), 0, (hipStream_t)stream, (const nsa::floatx4*)src, (unsigned)src_rows,
                     (nsa::floatx4*)dst, (unsigned)dst_rows, reads, writes, iters, nontemporal, seed);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}
