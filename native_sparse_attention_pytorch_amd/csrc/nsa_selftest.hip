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
