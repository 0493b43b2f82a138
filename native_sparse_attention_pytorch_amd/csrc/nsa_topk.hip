// Block-importance softmax and per-query top-k (NSA.py:693-713, 721): one wave per query row.
// Input row: nb importance logits (fp32, -inf = cannot be selected).  The row is softmaxed with
// the reference's extra -1e3 column (so a row with nothing visible becomes all zeros), then the
// k (<= 64) largest probabilities are extracted in descending order, ties going to the lower
// block index.  HBM-bound nominally: reads nb*4 bytes per row, writes k*(4+4+1).
#include <type_traits>
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

// max over the 64 lanes: DPP butterflies inside every row of 16 lanes (VALU speed, no LDS round
// trips), then the four row maxima through readlane
__device__ __forceinline__ float wave_max(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xF, 0xF, false));
  };
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0xB1>{}));     // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x4E>{}));     // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x141>{}));    // row_half_mirror: quads of a half row
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x140>{}));    // row_mirror: the two half rows
  const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
  const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
  const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
  const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
  return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

// Lane l holds the VPL consecutive entries l*VPL .. l*VPL+VPL-1 and, across rounds, its own best
// remaining entry; a round is a value-only wave maximum, a ballot of the lanes that hold it (the
// lowest lane holds the lowest index, and inside a lane the scan keeps the lower one: ties go to the
// lower block index), and a re-scan in the winning lane.  Result s stays in lane s until the end,
// so the outputs leave in one coalesced store each.
// Pooling of raw decode logits in front of the top-k (NSA.py:448-476): row (b, u) of the top-k is the mean of
// logits[b, u*pg + g, j*npf + c] over g < pg heads and c < npf compressed keys (row stride nc).
struct PoolArgs { int pg, npf, nc, units; };
// Run-time row length for a decode step replayed from a graph: state[1] compressed keys are cached, so a row has
// nb = state[1] / per_block entries and min(k, nb) of them are selected; the outputs keep the row stride kstride.
struct TopkDyn { const int* state; int per_block; };

template <int VPL, bool POOL>
__global__ __launch_bounds__(256) void topk_kernel(const float* __restrict__ in, long rows, int nb, int k, int softmax, int vec4, PoolArgs pool,
                                                   int* __restrict__ idx, float* __restrict__ vals, uint8_t* __restrict__ fmask, int kstride, TopkDyn dyn,
                                                   int pseq, int pblk) {
  const int lane = threadIdx.x & 63;
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  // pseq > 0: row r belongs to query r % pseq, and only its columns below floor(query / pblk) are defined (the blocks that
  // lie completely before the query); the rest counts as -inf and is not read
  const int lim = pseq > 0 ? min(nb, (int)(row % pseq) / pblk) : nb;
  if (dyn.state != nullptr) {
    nb = min(nb, dyn.state[1] / dyn.per_block);
    k = min(k, nb);
    if (k <= 0) return;
  }
  const float* src = in + row * nb;
  float x[VPL];
  bool loaded = false;
  if constexpr (POOL) {
    __shared__ float row_s[4][64 * VPL];
    float* rs = row_s[threadIdx.x >> 6];
    const long b = row / pool.units, u = row % pool.units;
    const float* base = in + (b * pool.units * pool.pg + u * pool.pg) * (long)pool.nc;
    const float norm = 1.0f / (float)(pool.pg * pool.npf);
    if (pool.npf == 4 && (pool.nc & 3) == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0) {
      // a block's four logits are one 16-byte load; consecutive lanes take consecutive blocks (whole cache lines per
      // instruction, all loads of a head independent), the sums go through LDS into the per-lane contiguous layout
      float acc[VPL];
#pragma unroll
      for (int r = 0; r < VPL; ++r) acc[r] = 0.f;
      constexpr int GU = VPL <= 4 ? 4 : (VPL <= 16 ? 2 : 1);      // heads whose loads are issued together
#pragma unroll GU
      for (int g = 0; g < pool.pg; ++g) {
        floatx4 t[VPL];
#pragma unroll
        for (int r = 0; r < VPL; ++r) {
          const int j = r * 64 + lane;
          t[r] = j < nb ? *reinterpret_cast<const floatx4*>(base + (long)g * pool.nc + 4L * j) : floatx4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int r = 0; r < VPL; ++r) acc[r] += (t[r][0] + t[r][1]) + (t[r][2] + t[r][3]);
      }
#pragma unroll
      for (int r = 0; r < VPL; ++r) rs[r * 64 + lane] = acc[r];
    } else {
      for (int j = lane; j < nb; j += 64) {
        float a = 0.f;
        for (int g = 0; g < pool.pg; ++g)
          for (int c = 0; c < pool.npf; ++c) a += base[(long)g * pool.nc + (long)j * pool.npf + c];
        rs[j] = a;
      }
    }
    __builtin_amdgcn_wave_barrier();                     // LDS operations of one wave execute in order
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
      const int j = lane * VPL + r;
      x[r] = j < nb ? rs[j] * norm : -INFINITY;
    }
    loaded = true;
  }
  if constexpr (VPL % 4 == 0) {
    if (vec4 && !loaded) {                               // rows are 16-byte aligned and nb % 4 == 0
#pragma unroll
      for (int r4 = 0; r4 < VPL / 4; ++r4) {
        const int j = lane * VPL + 4 * r4;
        floatx4 t = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        if (j < lim) t = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(src + j));      // read once
#pragma unroll
        for (int e = 0; e < 4; ++e) x[4 * r4 + e] = (j + e < lim) ? t[e] : -INFINITY;
      }
      loaded = true;
    }
  }
  if (!loaded) {
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
      const int j = lane * VPL + r;
      x[r] = j < lim ? src[j] : -INFINITY;
    }
  }
  if (softmax) {
    float mx = -1e3f;
#pragma unroll
    for (int r = 0; r < VPL; ++r) mx = fmaxf(mx, x[r]);
    mx = wave_max(mx);
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
  for (int r = 0; r < VPL; ++r) {
    // NaN (a diverged row): ordered first, like torch.topk, so every comparison below stays defined; padding loses against
    // every real entry.  Selects, not branches: as `if / else if` the same lines made the sibling kernel six times slower.
    float xr = x[r];
    xr = (xr == xr) ? xr : INFINITY;
    x[r] = (lane * VPL + r >= nb) ? -1.0f : xr;
  }

  float bv;
  int br;
  auto rescan = [&]() {
    bv = x[0]; br = 0;
#pragma unroll
    for (int r = 1; r < VPL; ++r)
      if (x[r] > bv) { bv = x[r]; br = r; }               // strict: ties keep the lower index
  };
  rescan();
  float res_v = 0.f;
  int res_j = 0;
  for (int s = 0; s < k; ++s) {
    const float m = wave_max(bv);
    const unsigned long long holders = __ballot(bv == m);
    const int w = __builtin_ctzll(holders);               // lowest lane = lowest index among equals
    const int jw = __builtin_amdgcn_readlane(lane * VPL + br, w);
    if (lane == s) { res_v = m; res_j = jw; }
    if (lane == w) {
#pragma unroll
      for (int r = 0; r < VPL; ++r)
        if (r == br) x[r] = -2.0f;                        // taken
      rescan();
    }
  }
  if (lane < k) {
    idx[row * kstride + lane] = res_j;
    const bool finite = res_v < INFINITY;                 // a NaN or +inf score comes out as NaN with a dead slot
    vals[row * kstride + lane] = finite ? res_v : NAN;
    fmask[row * kstride + lane] = (finite && res_v > 1e-10f) ? 1 : 0;
  }
}

// Four rows per wave, 16 lanes per row: for rows of up to 512 entries and k <= 16.  A round of the kernel above costs
// the same ~60 instructions whether a wave serves one row or four, and most of them are the winning lane's re-scan of
// its VPL entries, which every lane of the wave pays for.  Here a lane's entries live in LDS (its own segment: no
// lane ever reads another's), cut into groups of eight whose maxima stay in registers; the winner marks its entry
// taken, re-reads that one group and refreshes one maximum.  Row maxima are DPP butterflies inside a row of 16 lanes
// (no readlane), the winner is the lowest set bit of the row's 16 bits of the ballot.  Order of equal values: lower
// lane first, inside a lane lower group first, inside a group lower entry first - lower block index, as above.
__device__ __forceinline__ float row16_max(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xF, 0xF, false));
  };
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0xB1>{}));
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x4E>{}));
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x141>{}));
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x140>{}));
  return v;
}
__device__ __forceinline__ float row16_sum(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xF, 0xF, false));
  };
  v += dpp(v, std::integral_constant<int, 0xB1>{});
  v += dpp(v, std::integral_constant<int, 0x4E>{});
  v += dpp(v, std::integral_constant<int, 0x141>{});
  v += dpp(v, std::integral_constant<int, 0x140>{});
  return v;
}

template <int VPL>
__global__ __launch_bounds__(256) void topk_rows4_kernel(const float* __restrict__ in, long rows, int nb, int k, int softmax, int vec4,
                                                         int* __restrict__ idx, float* __restrict__ vals, uint8_t* __restrict__ fmask,
                                                         int pseq, int pblk) {
  constexpr int GS = VPL < 8 ? VPL : 8, NG = VPL / GS;
  constexpr int SEG = VPL + 4;                            // a lane's segment, padded: 16-byte reads of 16 lanes hit 64 distinct banks
  __shared__ __align__(16) float xs[16][16 * SEG];        // [row of the work-group][lane `sub`][entries sub*VPL ..]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = lane & 15, rs = lane >> 4;
  const long row = (long)blockIdx.x * 16 + wave * 4 + rs;
  const bool live = row < rows;                             // a dead row group works on the last row and stores nothing
  const float* src = in + (live ? row : rows - 1) * nb;
  const int lim = pseq > 0 ? min(nb, (int)((live ? row : rows - 1) % pseq) / pblk) : nb;      // see topk_kernel
  float* row_s = xs[wave * 4 + rs];
  float* mine_s = row_s + sub * SEG;
  float x[VPL];
  // with 16-byte aligned rows the loads are coalesced (consecutive lanes, consecutive 16 bytes) and the entries reach
  // their owners through LDS after the softmax, which does not care about the order; otherwise a lane loads its own
  const bool spread = vec4 != 0;
  if (spread) {
#pragma unroll
    for (int r4 = 0; r4 < VPL / 4; ++r4) {
      const int j = 4 * (sub + 16 * r4);
      floatx4 t = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      if (j < lim) t = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(src + j));      // read once
#pragma unroll
      for (int e = 0; e < 4; ++e) x[4 * r4 + e] = (j + e < lim) ? t[e] : -INFINITY;
    }
  } else {
#pragma unroll
    for (int r = 0; r < VPL; ++r) {
      const int j = sub * VPL + r;
      x[r] = j < lim ? src[j] : -INFINITY;
    }
  }
  if (softmax) {
    float mx = -1e3f;
#pragma unroll
    for (int r = 0; r < VPL; ++r) mx = fmaxf(mx, x[r]);
    mx = row16_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < VPL; ++r) { x[r] = __expf(x[r] - mx); sum += x[r]; }
    sum = row16_sum(sum) + __expf(-1e3f - mx);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int r = 0; r < VPL; ++r) x[r] *= inv;
  }
  if (spread) {
#pragma unroll
    for (int r4 = 0; r4 < VPL / 4; ++r4) {
      const int j = 4 * (sub + 16 * r4);                    // entries j .. j+3 belong to lane j / VPL
      *reinterpret_cast<floatx4*>(row_s + (j / VPL) * SEG + j % VPL) = floatx4{x[4 * r4], x[4 * r4 + 1], x[4 * r4 + 2], x[4 * r4 + 3]};
    }
    __builtin_amdgcn_wave_barrier();                        // LDS operations of one wave execute in order
#pragma unroll
    for (int r4 = 0; r4 < VPL / 4; ++r4) {
      const floatx4 t = *reinterpret_cast<const floatx4*>(mine_s + 4 * r4);
#pragma unroll
      for (int e = 0; e < 4; ++e) x[4 * r4 + e] = t[e];
    }
  }
  float gm[NG];
  int ga[NG];
#pragma unroll
  for (int g = 0; g < NG; ++g) {
#pragma unroll
    for (int t = 0; t < GS; ++t) {
      const int r = g * GS + t;
      float xr = x[r];
      xr = (xr == xr) ? xr : INFINITY;                      // NaN: ordered first (see topk_kernel); selects, not branches
      xr = (sub * VPL + r >= nb) ? -1.0f : xr;              // padding loses against every real entry
      x[r] = xr;
      if (t == 0 || xr > gm[g]) { gm[g] = xr; ga[g] = r; }  // strict: ties keep the lower index
    }
  }
#pragma unroll
  for (int r4 = 0; r4 < VPL / 4; ++r4)
    *reinterpret_cast<floatx4*>(mine_s + 4 * r4) = floatx4{x[4 * r4], x[4 * r4 + 1], x[4 * r4 + 2], x[4 * r4 + 3]};

  float res_v = 0.f;
  int res_j = 0;
  for (int s = 0; s < k; ++s) {
    float bv = gm[0];
    int ba = ga[0];
#pragma unroll
    for (int g = 1; g < NG; ++g)
      if (gm[g] > bv) { bv = gm[g]; ba = ga[g]; }
    const float m = row16_max(bv);
    const unsigned long long holders = __ballot(bv == m);
    const unsigned row_bits = (unsigned)(holders >> (lane & 48)) & 0xffffu;       // never 0: one of the row's lanes holds m (NaN was mapped to +inf above)
    const int w = __builtin_ctz(row_bits);                                        // lowest lane = lowest index among equals
    const int jw = __shfl(sub * VPL + ba, (lane & 48) + w, 64);
    if (sub == s) { res_v = m; res_j = jw; }
    if (sub == w) {
      mine_s[ba] = -2.0f;                                   // taken
      const int g0 = ba & ~(GS - 1);                        // first entry of the group that held it
      float y[GS];
#pragma unroll
      for (int t4 = 0; t4 < GS / 4; ++t4) {
        const floatx4 t = *reinterpret_cast<const floatx4*>(mine_s + g0 + 4 * t4);
#pragma unroll
        for (int e = 0; e < 4; ++e) y[4 * t4 + e] = t[e];
      }
      float ngm = y[0];
      int nga = g0;
#pragma unroll
      for (int t = 1; t < GS; ++t)
        if (y[t] > ngm) { ngm = y[t]; nga = g0 + t; }
#pragma unroll
      for (int g = 0; g < NG; ++g)
        if (g * GS == g0) { gm[g] = ngm; ga[g] = nga; }
    }
  }
  if (live && sub < k) {
    idx[row * k + sub] = res_j;
    const bool finite = res_v < INFINITY;
    vals[row * k + sub] = finite ? res_v : NAN;
    fmask[row * k + sub] = (finite && res_v > 1e-10f) ? 1 : 0;
  }
}

}  // namespace nsa

#define NSA_TOPK_POOL false
static int topk_launch(const float* scores, int64_t rows, int32_t nb, int32_t k, int32_t apply_softmax, int32_t pseq, int32_t pblk,
                       int32_t* idx, float* vals, uint8_t* fmask, void* stream) {
  using namespace nsa;
  if (!scores || !idx || !vals || !fmask || rows <= 0 || nb <= 0 || k <= 0 || k > nb) return NSA_E_ARG;
  if (nb > 64 * 32 || k > 64) return NSA_E_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  const int vpl = (nb + 63) / 64;
  const int vec4 = (nb % 4 == 0) && ((reinterpret_cast<uintptr_t>(scores) & 15) == 0);
  if (k <= 16 && nb <= 512) {          // four rows per wave
    const dim3 grid4((unsigned)((rows + 15) / 16));
#define NSA_TOPK4(V) hipLaunchKernelGGL((topk_rows4_kernel<V>), grid4, block, 0, st, scores, (long)rows, nb, k, apply_softmax, vec4, idx, vals, fmask, pseq, pblk)
    if (nb <= 64) NSA_TOPK4(4);
    else if (nb <= 128) NSA_TOPK4(8);
    else if (nb <= 256) NSA_TOPK4(16);
    else NSA_TOPK4(32);
#undef NSA_TOPK4
    hipError_t e4 = hipGetLastError();
    return e4 == hipSuccess ? 0 : (int)e4;
  }
  const PoolArgs pool{0, 1, 0, 1};
  const TopkDyn dyn{nullptr, 1};
#define NSA_TOPK(V) hipLaunchKernelGGL((topk_kernel<V, NSA_TOPK_POOL>), grid, block, 0, st, scores, (long)rows, nb, k, apply_softmax, vec4, pool, idx, vals, fmask, k, dyn, pseq, pblk)
#define NSA_TOPK_DISPATCH()            \
  if (vpl <= 1) NSA_TOPK(1);           \
  else if (vpl <= 2) NSA_TOPK(2);      \
  else if (vpl <= 4) NSA_TOPK(4);      \
  else if (vpl <= 8) NSA_TOPK(8);      \
  else if (vpl <= 16) NSA_TOPK(16);    \
  else NSA_TOPK(32)
  NSA_TOPK_DISPATCH();
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

extern "C" int nsa_topk(const float* scores, int64_t rows, int32_t nb, int32_t k, int32_t apply_softmax,
                        int32_t* idx, float* vals, uint8_t* fmask, void* stream) {
  return topk_launch(scores, rows, nb, k, apply_softmax, 0, 1, idx, vals, fmask, stream);
}

extern "C" int nsa_topk_prefix(const float* scores, int64_t rows, int32_t nb, int32_t k, int32_t apply_softmax, int32_t seq, int32_t block,
                               int32_t* idx, float* vals, uint8_t* fmask, void* stream) {
  if (seq <= 0 || block <= 0 || rows % seq != 0) return NSA_E_ARG;
  return topk_launch(scores, rows, nb, k, apply_softmax, seq, block, idx, vals, fmask, stream);
}

#undef NSA_TOPK_POOL
#define NSA_TOPK_POOL true
namespace nsa {
// state == nullptr: num_compressed keys are cached; otherwise num_compressed is the capacity (row stride of the logits, upper bound of the
// row length) and the count is read from state[1] when the kernel runs
int decode_topk_launch(const float* logits, int32_t batch, int32_t kv_heads, int32_t group, int32_t num_compressed,
                       int32_t per_block, int32_t share, int32_t k, int32_t* idx, float* vals, uint8_t* fmask, const int32_t* state, void* stream) {
  using namespace nsa;
  if (!logits || !idx || !vals || !fmask || batch <= 0 || kv_heads <= 0 || group <= 0 || per_block <= 0 || num_compressed <= 0) return NSA_E_ARG;
  const int nb = num_compressed / per_block;
  if (k <= 0 || k > nb) return NSA_E_ARG;
  if (nb > 64 * 32 || k > 64) return NSA_E_UNSUPPORTED;
  const int units = share ? kv_heads : kv_heads * group;
  const long rows = (long)batch * units;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  const int vpl = (nb + 63) / 64;
  const int vec4 = 0, apply_softmax = 1;
  const float* scores = logits;
  const PoolArgs pool{share ? group : 1, per_block, num_compressed, units};
  const TopkDyn dyn{state, per_block};
  const int pseq = 0, pblk = 1;
  NSA_TOPK_DISPATCH();
#undef NSA_TOPK_DISPATCH
#undef NSA_TOPK
#undef NSA_TOPK_POOL
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}
}  // namespace nsa

extern "C" int nsa_decode_topk(const float* logits, int32_t batch, int32_t kv_heads, int32_t group, int32_t num_compressed,
                               int32_t per_block, int32_t share, int32_t k, int32_t* idx, float* vals, uint8_t* fmask, void* stream) {
  return nsa::decode_topk_launch(logits, batch, kv_heads, group, num_compressed, per_block, share, k, idx, vals, fmask, nullptr, stream);
}
