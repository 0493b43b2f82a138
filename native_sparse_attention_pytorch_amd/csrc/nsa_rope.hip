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

// Run-time addressing of a decode step replayed from a graph: state[0] = rows already cached = the new token's position;
// the *_row strides turn the cache / ring base addresses into the row's address.
struct DecodeDyn {
  const int* state;
  long kc_row, vc_row, krun_row, vrun_row;
  int ring, last_pos;                // last_pos: the last row the caches have
};

// Decode step: the new token's query heads rotated to position pos (-> rq), its key heads
// rotated and written into row pos of the key cache, its value heads copied into row pos of
// the value cache (NSA.py:384-393) - one launch instead of two rotations and a copy.
template <int D>
__global__ __launch_bounds__(256) void decode_prep_kernel(const __bf16* __restrict__ q, long q0, long q1, const __bf16* __restrict__ k, long k0, long k1,
                                                          const __bf16* __restrict__ v, long v0, long v1, int b, int hq, int hk,
                                                          const float* __restrict__ freqs, int pos, __bf16* __restrict__ rq,
                                                          __bf16* __restrict__ krow, long kr0, long kr1, __bf16* __restrict__ vrow, long vr0, long vr1,
                                                          __bf16* __restrict__ krun, long ku0, long ku1, __bf16* __restrict__ vrun, long vu0, long vu1,
                                                          DecodeDyn dyn) {
  constexpr int LPR = D / 8, RPB = 256 / LPR;
  if (dyn.state != nullptr) {
    // position read at run time (the launch is replayed from a graph): row pos of the caches, row pos % ring of the window rings
    pos = dyn.state[0];
    if (pos < 0 || pos > dyn.last_pos) return;       // replayed past the caches' capacity: write nothing
    krow += (long)pos * dyn.kc_row;
    vrow += (long)pos * dyn.vc_row;
    if (krun != nullptr) {
      const int slot = pos % dyn.ring;
      krun += (long)slot * dyn.krun_row;
      vrun += (long)slot * dyn.vrun_row;
    }
  }
  const int per = hq + 2 * hk;
  const long row = (long)blockIdx.x * RPB + threadIdx.x / LPR;
  if (row >= (long)b * per) return;
  const int c = threadIdx.x % LPR;
  const int bb = (int)(row / per), r = (int)(row % per);
  const __bf16* src;
  __bf16* dst;
  bool rot = true;
  if (r < hq) { src = q + bb * q0 + r * q1; dst = rq + ((long)bb * hq + r) * D; }
  else if (r < hq + hk) { src = k + bb * k0 + (r - hq) * k1; dst = krow + bb * kr0 + (r - hq) * kr1; }
  else { src = v + bb * v0 + (r - hq - hk) * v1; dst = vrow + bb * vr0 + (r - hq - hk) * vr1; rot = false; }
  const bf16x8 x = load8(src + 8 * c);
  // the un-rotated key / value also go into the open compression window (NSA.py:377-380)
  if (krun != nullptr && r >= hq) {
    __bf16* run = r < hq + hk ? krun + bb * ku0 + (r - hq) * ku1 : vrun + bb * vu0 + (r - hq - hk) * vu1;
    *reinterpret_cast<bf16x8*>(run + 8 * c) = x;
  }
  bf16x8 o = x;
  if (rot) {
    const float p = (float)pos;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float sn, cs;
      sincosf(p * freqs[4 * c + e], &sn, &cs);
      const float a = (float)x[2 * e], bq = (float)x[2 * e + 1];
      o[2 * e] = (__bf16)(a * cs - bq * sn);
      o[2 * e + 1] = (__bf16)(bq * cs + a * sn);
    }
  }
  *reinterpret_cast<bf16x8*>(dst + 8 * c) = o;
}

}  // namespace nsa

namespace nsa {
int decode_prep_launch(const void* q, const int64_t* q_stride, const void* k, const int64_t* k_stride, const void* v,
                       const int64_t* v_stride, int32_t batch, int32_t heads, int32_t kv_heads, int32_t dim_head,
                       const float* freqs, int32_t pos, void* rq, void* k_row, const int64_t* k_row_stride, void* v_row,
                       const int64_t* v_row_stride, void* k_run_row, const int64_t* k_run_stride, void* v_run_row,
                       const int64_t* v_run_stride, const DecodeDyn& dyn, void* stream) {
  if (!q || !k || !v || !q_stride || !k_stride || !v_stride || !freqs || !rq || !k_row || !v_row || !k_row_stride || !v_row_stride)
    return NSA_E_ARG;
  if (batch <= 0 || heads <= 0 || kv_heads <= 0 || pos < 0) return NSA_E_ARG;
  if ((q_stride[0] | q_stride[1] | k_stride[0] | k_stride[1] | v_stride[0] | v_stride[1] | k_row_stride[0] | k_row_stride[1] |
       v_row_stride[0] | v_row_stride[1]) & 7)
    return NSA_E_ARG;
  long ku[2] = {0, 0}, vu[2] = {0, 0};
  if (k_run_row || v_run_row) {
    if (!k_run_row || !v_run_row || !k_run_stride || !v_run_stride) return NSA_E_ARG;
    if ((k_run_stride[0] | k_run_stride[1] | v_run_stride[0] | v_run_stride[1]) & 7) return NSA_E_ARG;
    ku[0] = k_run_stride[0]; ku[1] = k_run_stride[1]; vu[0] = v_run_stride[0]; vu[1] = v_run_stride[1];
  }
  const long rows = (long)batch * (heads + 2 * kv_heads);
  hipStream_t st = (hipStream_t)stream;
  if (dim_head == 64) {
    hipLaunchKernelGGL((decode_prep_kernel<64>), dim3((unsigned)((rows + 31) / 32)), dim3(256), 0, st, (const __bf16*)q, (long)q_stride[0],
                       (long)q_stride[1], (const __bf16*)k, (long)k_stride[0], (long)k_stride[1], (const __bf16*)v, (long)v_stride[0],
                       (long)v_stride[1], batch, heads, kv_heads, freqs, pos, (__bf16*)rq, (__bf16*)k_row, (long)k_row_stride[0],
                       (long)k_row_stride[1], (__bf16*)v_row, (long)v_row_stride[0], (long)v_row_stride[1], (__bf16*)k_run_row, ku[0], ku[1],
                       (__bf16*)v_run_row, vu[0], vu[1], dyn);
  } else if (dim_head == 128) {
    hipLaunchKernelGGL((decode_prep_kernel<128>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st, (const __bf16*)q, (long)q_stride[0],
                       (long)q_stride[1], (const __bf16*)k, (long)k_stride[0], (long)k_stride[1], (const __bf16*)v, (long)v_stride[0],
                       (long)v_stride[1], batch, heads, kv_heads, freqs, pos, (__bf16*)rq, (__bf16*)k_row, (long)k_row_stride[0],
                       (long)k_row_stride[1], (__bf16*)v_row, (long)v_row_stride[0], (long)v_row_stride[1], (__bf16*)k_run_row, ku[0], ku[1],
                       (__bf16*)v_run_row, vu[0], vu[1], dyn);
  } else {
    return NSA_E_UNSUPPORTED;
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

int decode_prep_dyn(const void* q, const int64_t* q_stride, const void* k, const int64_t* k_stride, const void* v, const int64_t* v_stride,
                    int32_t batch, int32_t heads, int32_t kv_heads, int32_t dim_head, const float* freqs, void* rq, void* k_cache,
                    const int64_t* kc_stride, void* v_cache, const int64_t* vc_stride, void* k_run, const int64_t* krun_stride, void* v_run,
                    const int64_t* vrun_stride, int32_t ring, int32_t last_pos, const int32_t* state, void* stream) {
  if (!state || !kc_stride || !vc_stride || ((kc_stride[2] | vc_stride[2]) & 7)) return NSA_E_ARG;
  DecodeDyn dyn{state, (long)kc_stride[2], (long)vc_stride[2], 0, 0, 1, last_pos};
  if (k_run || v_run) {
    if (!krun_stride || !vrun_stride || ring <= 0 || ((krun_stride[2] | vrun_stride[2]) & 7)) return NSA_E_ARG;
    dyn.krun_row = krun_stride[2]; dyn.vrun_row = vrun_stride[2]; dyn.ring = ring;
  }
  return decode_prep_launch(q, q_stride, k, k_stride, v, v_stride, batch, heads, kv_heads, dim_head, freqs, 0, rq, k_cache, kc_stride, v_cache,
                            vc_stride, k_run, krun_stride, v_run, vrun_stride, dyn, stream);
}
}  // namespace nsa

extern "C" int nsa_decode_prep(const void* q, const int64_t* q_stride, const void* k, const int64_t* k_stride, const void* v,
                               const int64_t* v_stride, int32_t batch, int32_t heads, int32_t kv_heads, int32_t dim_head,
                               const float* freqs, int32_t pos, void* rq, void* k_row, const int64_t* k_row_stride, void* v_row,
                               const int64_t* v_row_stride, void* k_run_row, const int64_t* k_run_stride, void* v_run_row,
                               const int64_t* v_run_stride, void* stream) {
  return nsa::decode_prep_launch(q, q_stride, k, k_stride, v, v_stride, batch, heads, kv_heads, dim_head, freqs, pos, rq, k_row, k_row_stride,
                                 v_row, v_row_stride, k_run_row, k_run_stride, v_run_row, v_run_stride, nsa::DecodeDyn{nullptr, 0, 0, 0, 0, 1, 0}, stream);
}

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
