// The module's RMS norm (NSA.py:230, 579: nn.RMSNorm over the model dimension) and the column sums of its backward pass
// (bias gradients of the projections NSA.py:853, the intra-window position gradients of NSA.py:599-600).  Byte work bound
// by HBM: a wave owns a row, a lane 16-byte pieces of it, so every load instruction of a wave covers 1 KB of one row.
//   forward : reads x, writes y and the row's 1/rms                        (2 rows of bytes per row)
//   backward: reads x, dy, writes dx                                       (3 rows of bytes per row)
//             + the weight gradient as per-work-group partial column sums, added up by colsum_reduce_kernel
//   colsum  : reads the matrix once, same partials + reduce
// The order of every sum is fixed by the launch shape: results do not change from run to run.
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int mk = 32; mk >= 1; mk >>= 1) v += __shfl_xor(v, mk, 64);
  return v;
}

// y = x * rsqrt(mean(x^2) + eps) * w, fp32 arithmetic, one rounding to bf16
template <int NV>
__global__ __launch_bounds__(256) void rmsnorm_fwd_kernel(long rows, int dim, long xs, const __bf16* __restrict__ x,
                                                          const __bf16* __restrict__ w, float eps, __bf16* __restrict__ y,
                                                          float* __restrict__ rstd) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float wf[NV][8];
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int col = (v * 64 + lane) * 8;
    const bf16x8 t = col < dim ? load8(w + col) : zero_frag();
#pragma unroll
    for (int e = 0; e < 8; ++e) wf[v][e] = (float)t[e];
  }
  const float inv_dim = 1.0f / (float)dim;
  for (long row = (long)blockIdx.x * 4 + wave; row < rows; row += (long)gridDim.x * 4) {
    bf16x8 xv[NV];
    float ss = 0.f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int col = (v * 64 + lane) * 8;
      xv[v] = col < dim ? load8(x + row * xs + col) : zero_frag();
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += (float)xv[v][e] * (float)xv[v][e];
    }
    const float r = rsqrtf(wave_sum(ss) * inv_dim + eps);
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int col = (v * 64 + lane) * 8;
      bf16x8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (__bf16)((float)xv[v][e] * r * wf[v][e]);
      if (col < dim) *reinterpret_cast<bf16x8*>(y + row * (long)dim + col) = o;
    }
    if (lane == 0) rstd[row] = r;
  }
}

// dx = r * (g - x * r^2 * mean(g * x)), g = dy * w;  dw[col] = sum over rows of dy * x * r (partial: this work-group's rows)
template <int NV>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(long rows, int dim, long xs, const __bf16* __restrict__ x,
                                                          const __bf16* __restrict__ w, const float* __restrict__ rstd,
                                                          const __bf16* __restrict__ dy, __bf16* __restrict__ dx,
                                                          float* __restrict__ partial) {
  extern __shared__ float red[];                     // [4][dim]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float wf[NV][8], dw[NV][8];
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int col = (v * 64 + lane) * 8;
    const bf16x8 t = col < dim ? load8(w + col) : zero_frag();
#pragma unroll
    for (int e = 0; e < 8; ++e) { wf[v][e] = (float)t[e]; dw[v][e] = 0.f; }
  }
  const float inv_dim = 1.0f / (float)dim;
  for (long row = (long)blockIdx.x * 4 + wave; row < rows; row += (long)gridDim.x * 4) {
    bf16x8 xv[NV];
    float gv[NV][8];
    float c = 0.f;
    const float r = rstd[row];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int col = (v * 64 + lane) * 8;
      const bool in = col < dim;
      xv[v] = in ? load8(x + row * xs + col) : zero_frag();
      const bf16x8 a = in ? load8(dy + row * (long)dim + col) : zero_frag();
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float d = (float)a[e], xe = (float)xv[v][e];
        dw[v][e] += d * xe * r;
        gv[v][e] = d * wf[v][e];
        c += gv[v][e] * xe;
      }
    }
    const float coef = wave_sum(c) * inv_dim * r * r * r;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      const int col = (v * 64 + lane) * 8;
      bf16x8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (__bf16)(r * gv[v][e] - (float)xv[v][e] * coef);
      if (col < dim) *reinterpret_cast<bf16x8*>(dx + row * (long)dim + col) = o;
    }
  }
  if (!partial) return;
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    const int col = (v * 64 + lane) * 8;
    if (col < dim) {
#pragma unroll
      for (int e = 0; e < 8; ++e) red[wave * dim + col + e] = dw[v][e];
    }
  }
  __syncthreads();
  for (int col = threadIdx.x; col < dim; col += 256)
    partial[(long)blockIdx.x * dim + col] = (red[col] + red[dim + col]) + (red[2 * dim + col] + red[3 * dim + col]);
}

struct ColsumArgs {
  long r1, s0, s1, sg;        // row r = (r / r1) * s0 + (r % r1) * s1, group g at g * sg (elements)
  long rows;
  int cols, lpr, chunk;       // lpr lanes a row (power of two), chunk rows a work-group
};

// partial[g][blockIdx.x][cols] = sum of this work-group's rows of group g
__global__ __launch_bounds__(256) void colsum_kernel(const ColsumArgs A, const __bf16* __restrict__ x, float* __restrict__ partial) {
  __shared__ float red[8][256];
  const int cl = threadIdx.x % A.lpr, rl = threadIdx.x / A.lpr, rpi = 256 / A.lpr;
  const int col = (blockIdx.y * A.lpr + cl) * 8;
  const bool in = col < A.cols;
  const long first = (long)blockIdx.x * A.chunk + rl, last = min((long)blockIdx.x * A.chunk + A.chunk, A.rows);
  const __bf16* base = x + blockIdx.z * A.sg + col;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (in && first < last) {
    // rows are walked as (outer, inner) pairs: one division up front, none in the loop
    long o = first / A.r1, i = first - o * A.r1;
    const int count = (int)((last - first + rpi - 1) / rpi);
#pragma unroll 4
    for (int it = 0; it < count; ++it) {
      const bf16x8 t = load8(base + o * A.s0 + i * A.s1);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += (float)t[e];
      i += rpi;
      while (i >= A.r1) { i -= A.r1; ++o; }
    }
  }
  float* out = partial + ((long)blockIdx.z * gridDim.x + blockIdx.x) * A.cols + col;
  if (rpi == 1) {
    if (in) {
#pragma unroll
      for (int e = 0; e < 8; ++e) out[e] = acc[e];
    }
    return;
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[e][threadIdx.x] = acc[e];
  for (int half = rpi / 2; half >= 1; half /= 2) {               // rows rl and rl + half of the same columns
    __syncthreads();
    if (rl < half) {
#pragma unroll
      for (int e = 0; e < 8; ++e) red[e][threadIdx.x] += red[e][threadIdx.x + half * A.lpr];
    }
  }
  if (rl == 0 && in) {
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = red[e][threadIdx.x];
  }
}

// out[i] = sum over p < parts of slices[p][i], four entries a thread (the split weight-gradient GEMM's partial products)
template <class OT>
__global__ __launch_bounds__(256) void sum_slices_kernel(const float* __restrict__ slices, int parts, long n, OT* __restrict__ out) {
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= n) return;
  float4 a = *reinterpret_cast<const float4*>(slices + i);
  int p = 1;
  for (; p + 3 < parts; p += 4) {
    float4 t[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) t[j] = *reinterpret_cast<const float4*>(slices + (long)(p + j) * n + i);
#pragma unroll
    for (int j = 0; j < 4; ++j) { a.x += t[j].x; a.y += t[j].y; a.z += t[j].z; a.w += t[j].w; }
  }
  for (; p < parts; ++p) {
    const float4 t = *reinterpret_cast<const float4*>(slices + (long)p * n + i);
    a.x += t.x; a.y += t.y; a.z += t.z; a.w += t.w;
  }
  out[i] = (OT)a.x; out[i + 1] = (OT)a.y; out[i + 2] = (OT)a.z; out[i + 3] = (OT)a.w;
}

// out[g][col] = sum over p of partial[g][p][col]; 32 columns x 32 slices of p a work-group, 8 loads in flight a thread
template <class OT>
__global__ __launch_bounds__(1024) void colsum_reduce_kernel(const float* __restrict__ partial, int parts, int cols, OT* __restrict__ out) {
  __shared__ float red[32][33];
  const int cl = threadIdx.x & 31, pl = threadIdx.x >> 5;
  const int col = blockIdx.x * 32 + cl;
  const float* base = partial + (long)blockIdx.y * parts * cols + col;
  float s = 0.f;
  if (col < cols) {
    int p = pl;
    for (; p + 7 * 32 < parts; p += 8 * 32) {
      float t[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) t[j] = base[(long)(p + j * 32) * cols];
      s += ((t[0] + t[1]) + (t[2] + t[3])) + ((t[4] + t[5]) + (t[6] + t[7]));
    }
    for (; p < parts; p += 32) s += base[(long)p * cols];
  }
  red[pl][cl] = s;
  __syncthreads();
  if (pl == 0 && col < cols) {
    float t = 0.f;
#pragma unroll
    for (int j = 0; j < 32; ++j) t += red[j][cl];
    out[(long)blockIdx.y * cols + col] = (OT)t;
  }
}

static int reduce_launch(const float* partial, int groups, int parts, int cols, void* out, int out_fp32, hipStream_t st) {
  const dim3 grid((cols + 31) / 32, groups);
  if (out_fp32) colsum_reduce_kernel<float><<<grid, 1024, 0, st>>>(partial, parts, cols, (float*)out);
  else colsum_reduce_kernel<__bf16><<<grid, 1024, 0, st>>>(partial, parts, cols, (__bf16*)out);
  return (int)hipGetLastError();
}

static int norm_chunks(int dim) {                   // 16-byte pieces a lane: a wave covers 512 columns a piece
  for (int nv = 1; nv <= 8; nv *= 2)
    if (dim <= 512 * nv) return nv;
  return 0;
}

static int norm_groups(long rows) { return (int)std::min<long>((rows + 3) / 4, 512); }   // 2 work-groups a CU; one partial each

}  // namespace nsa

using namespace nsa;

extern "C" int nsa_rmsnorm_partials(int64_t rows) { return rows > 0 ? norm_groups(rows) : 0; }

extern "C" int nsa_rmsnorm_fwd(int64_t rows, int32_t dim, const void* x, int64_t x_row_stride, const void* weight, float eps,
                               void* y, float* rstd, void* stream) {
  if (rows < 0 || dim <= 0) return NSA_E_ARG;
  if (rows == 0) return 0;
  if (!x || !weight || !y || !rstd) return NSA_E_ARG;
  const int nv = norm_chunks(dim);
  if (!nv || dim % 8 || x_row_stride % 8 || x_row_stride < dim || ((uintptr_t)x | (uintptr_t)weight | (uintptr_t)y) % 16)
    return NSA_E_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const int grid = (int)std::min<long>((rows + 3) / 4, 2048);
#define NSA_FWD(NV) rmsnorm_fwd_kernel<NV><<<grid, 256, 0, st>>>(rows, dim, x_row_stride, (const __bf16*)x, (const __bf16*)weight, eps, (__bf16*)y, rstd)
  switch (nv) { case 1: NSA_FWD(1); break; case 2: NSA_FWD(2); break; case 4: NSA_FWD(4); break; default: NSA_FWD(8); }
#undef NSA_FWD
  return (int)hipGetLastError();
}

extern "C" int nsa_rmsnorm_bwd(int64_t rows, int32_t dim, const void* x, int64_t x_row_stride, const void* weight, const float* rstd,
                               const void* dy, void* dx, void* dweight, int32_t dweight_fp32, float* partials,
                               void* stream) {
  if (rows < 0 || dim <= 0) return NSA_E_ARG;
  if (rows == 0) return 0;
  if (!x || !weight || !rstd || !dy || !dx || (dweight && !partials)) return NSA_E_ARG;
  const int nv = norm_chunks(dim);
  if (!nv || dim % 8 || x_row_stride % 8 || x_row_stride < dim ||
      ((uintptr_t)x | (uintptr_t)weight | (uintptr_t)dy | (uintptr_t)dx) % 16)
    return NSA_E_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const int grid = norm_groups(rows);
  float* part = dweight ? partials : nullptr;
  const size_t lds = dweight ? (size_t)4 * dim * sizeof(float) : 0;
#define NSA_BWD(NV) rmsnorm_bwd_kernel<NV><<<grid, 256, lds, st>>>(rows, dim, x_row_stride, (const __bf16*)x, (const __bf16*)weight, rstd, \
                                                                   (const __bf16*)dy, (__bf16*)dx, part)
  switch (nv) { case 1: NSA_BWD(1); break; case 2: NSA_BWD(2); break; case 4: NSA_BWD(4); break; default: NSA_BWD(8); }
#undef NSA_BWD
  if (hipError_t e = hipGetLastError()) return (int)e;
  return dweight ? reduce_launch(partials, 1, grid, dim, dweight, dweight_fp32, st) : 0;
}

namespace {
struct ColsumShape { int lpr, colblocks, parts, chunk; };
ColsumShape colsum_shape(int64_t rows, int32_t cols, int32_t groups) {
  ColsumShape s;
  const int pieces = (cols + 7) / 8;
  s.lpr = 1;
  while (s.lpr < pieces && s.lpr < 256) s.lpr *= 2;
  s.colblocks = (pieces + s.lpr - 1) / s.lpr;
  const int rpi = 256 / s.lpr;
  // about two work-groups a CU over all groups and column blocks, at least 4 sweeps of rows each, at most 256 partials
  long parts = std::min<long>(std::min<long>(512 / ((long)s.colblocks * groups), 256), rows / ((long)rpi * 4));
  parts = std::max<long>(parts, 1);
  s.chunk = (int)((rows + parts - 1) / parts);
  s.parts = (int)((rows + s.chunk - 1) / s.chunk);
  return s;
}
}  // namespace

extern "C" int64_t nsa_colsum_workspace(int64_t rows, int32_t cols, int32_t groups) {
  if (rows <= 0 || cols <= 0 || groups <= 0) return 0;
  return (int64_t)colsum_shape(rows, cols, groups).parts * groups * cols * (int64_t)sizeof(float);
}

extern "C" int nsa_colsum(const void* x, int32_t groups, int64_t group_stride, int64_t outer, int64_t outer_stride, int64_t inner,
                          int64_t inner_stride, int32_t cols, void* out, int32_t out_fp32, float* workspace, void* stream) {
  if (groups <= 0 || outer < 0 || inner < 0 || cols <= 0 || !out) return NSA_E_ARG;
  const int64_t rows = outer * inner;
  hipStream_t st = (hipStream_t)stream;
  if (rows == 0) return reduce_launch(nullptr, groups, 0, cols, out, out_fp32, st);      // zeros
  if (!x || !workspace) return NSA_E_ARG;
  if (cols % 8 || group_stride % 8 || outer_stride % 8 || inner_stride % 8 || (uintptr_t)x % 16 || groups > 65535)
    return NSA_E_UNSUPPORTED;
  const ColsumShape s = colsum_shape(rows, cols, groups);
  ColsumArgs A;
  A.r1 = inner; A.s0 = outer_stride; A.s1 = inner_stride; A.sg = group_stride; A.rows = rows;
  A.cols = cols; A.lpr = s.lpr; A.chunk = s.chunk;
  colsum_kernel<<<dim3(s.parts, s.colblocks, groups), 256, 0, st>>>(A, (const __bf16*)x, workspace);
  if (hipError_t e = hipGetLastError()) return (int)e;
  return reduce_launch(workspace, groups, s.parts, cols, out, out_fp32, st);
}

extern "C" int nsa_sum_slices(const float* slices, int32_t parts, int64_t n, void* out, int32_t out_fp32, void* stream) {
  if (parts <= 0 || n < 0) return NSA_E_ARG;
  if (n == 0) return 0;
  if (!slices || !out) return NSA_E_ARG;
  if (n % 4 || (uintptr_t)slices % 16 || (uintptr_t)out % 8 || n > ((int64_t)1 << 40)) return NSA_E_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const unsigned grid = (unsigned)((n / 4 + 255) / 256);
  if (out_fp32) sum_slices_kernel<float><<<grid, 256, 0, st>>>(slices, parts, n, (float*)out);
  else sum_slices_kernel<__bf16><<<grid, 256, 0, st>>>(slices, parts, n, (__bf16*)out);
  return (int)hipGetLastError();
}
