// Shared device helpers for the gfx950 (CDNA4, wave64) NSA kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nsa {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(8 * sizeof(float)))) float floatx8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t uintx4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t uintx2;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// D(32x32) += A(32x16) * B(16x32), bf16 inputs, fp32 accumulate.
// Register layout (lane l, half h = l / 32):
//   A: row m = l % 32, k = 8h .. 8h+7          (8 bf16 per lane)
//   B: col n = l % 32, k = 8h .. 8h+7          (8 bf16 per lane)
//   D: col n = l % 32, reg i (0..15) holds row m = 8*(i/4) + 4h + (i%4)
__device__ __forceinline__ floatx16 mfma32(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 zero_frag() {
  uintx4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}

__device__ __forceinline__ floatx16 zero_acc() {
  floatx16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.f;
  return z;
}

// 16-byte global load of 8 consecutive bf16 (address must be 16-byte aligned).
__device__ __forceinline__ bf16x8 load8(const __bf16* p) {
  return *reinterpret_cast<const bf16x8*>(p);
}

// Pack 8 consecutive accumulator registers (first .. first+7) into one bf16 operand.
__device__ __forceinline__ bf16x8 pack8(const floatx16& acc, int first) {
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (__bf16)acc[first + e];
  return r;
}

// Constant B operands that turn an MFMA into a register transpose:
//   ident_lo: B[k][n] = (n == k),      ident_hi: B[k][n] = (n == k + 16)
// mfma32(X_lo, ident_lo, 0) + mfma32(X_hi, ident_hi, .) gives D[m][n] = X[m][n] for a
// 32x32 bf16 tile X held as two A operands (columns 0..15 and 16..31); D then has
// lane <-> column, registers <-> rows, which is the operand layout for a contraction
// over the rows of X.  Products with 0/1 are exact, so the transpose is lossless.
__device__ __forceinline__ void make_ident(int lane, bf16x8& lo, bf16x8& hi) {
  const int n = lane & 31, h = lane >> 5;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    lo[e] = (__bf16)((n == 8 * h + e) ? 1.0f : 0.0f);
    hi[e] = (__bf16)((n == 16 + 8 * h + e) ? 1.0f : 0.0f);
  }
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

// store 4 floats as 4 bf16 (8 bytes)
__device__ __forceinline__ void store4_bf16(__bf16* p, float a, float b, float c, float d) {
  bf16x4 r;
  r[0] = (__bf16)a; r[1] = (__bf16)b; r[2] = (__bf16)c; r[3] = (__bf16)d;
  *reinterpret_cast<bf16x4*>(p) = r;
}

}  // namespace nsa
