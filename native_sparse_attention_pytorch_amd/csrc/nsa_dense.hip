// Interval-masked GQA flash attention for gfx950: the sliding-window branch (band mask,
// NSA.py:48-56, 841-850) and the compressed branch (stride mask, NSA.py:632-639) share one set
// of kernels.  Query (b, head, i) sees key kk iff lo(i) <= kk <= hi(i):
//   band   : lo = i - wb, hi = i + wf                    (wf = 0 when causal)
//   stride : lo = 0,      hi = floor(i / st) - 1          (all keys when not causal)
// In stride mode the first `mem` rows of k/v are memory slots every query sees
// (NSA.py:621-626); kk counts the compressed keys after them.  The compressed forward can also
// emit the block-importance logits of NSA.py:652-691 (mean over the G heads of a group and over
// the npf = B/st compressed keys of a fine block; -inf where the reference's fill values make
// the softmax term vanish), which feed the top-k kernel.
//
// All operands live in registers (no LDS staging); V^T / K^T / Q^T / dO^T operands are made
// with identity-MFMA transposes (nsa_common.hpp).  One wave = one 32-row tile (32/G queries x G
// heads) in the query-stationary kernels, one 32-key tile in the key-stationary dK/dV kernel.
#include "nsa_common.hpp"
#include "nsa_dense_plan.hpp"

namespace nsa {

struct Interval { int lo, hi; };

__device__ __forceinline__ Interval visible_range(const DensePlan& P, int i) {
  Interval r;
  if (P.mode == 0) {
    r.lo = max(0, i - P.wb);
    r.hi = min(P.nkeys - 1, i + P.wf);
  } else {
    r.lo = 0;
    r.hi = P.causal ? min(P.nkeys - 1, i / P.st - 1) : P.nkeys - 1;
  }
  return r;
}

// ------------------------------------------------------------------------------- forward
template <int D>
__global__ __launch_bounds__(64) void dense_fwd_kernel(const DensePlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                       const __bf16* __restrict__ v, __bf16* __restrict__ out, float* __restrict__ lse,
                                                       float* __restrict__ pooled) {
  constexpr int KS = D / 16, DT = D / 32;
  const int lane = threadIdx.x, n_ = lane & 31, h = lane >> 5;
  const int bh = blockIdx.y, b = bh / P.hkv, hk = bh % P.hkv;
  const int ppt = 32 >> P.lg;
  const int i0 = blockIdx.x * ppt;
  const int pq = n_ >> P.lg, g = n_ & (P.g - 1);
  const bool valid = i0 + pq < P.n;
  const int i = valid ? i0 + pq : P.n - 1;
  const int ilast = min(P.n - 1, i0 + ppt - 1);
  const int hq = hk * P.g + g;

  bf16x8 Qf[KS], ilo, ihi;
  make_ident(lane, ilo, ihi);
  {
    const __bf16* qp = q + b * P.sq[0] + (long)hq * P.sq[1] + (long)i * P.sq[2] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) Qf[ks] = load8(qp + 16 * ks);
  }
  const Interval me = visible_range(P, i);
  const int tile_lo = visible_range(P, i0).lo, tile_hi = visible_range(P, ilast).hi;
  const float sc = P.scale * kLog2e;

  float m = -INFINITY, l = 0.f;
  floatx16 Oa[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) Oa[dt] = zero_acc();

  const __bf16* kbase = k + b * P.sk[0] + hk * P.sk[1] + 8 * h;
  const __bf16* vbase = v + b * P.sv[0] + hk * P.sv[1] + 8 * h;
  const int t_first = (P.mem > 0) ? -1 : (tile_lo >> 5);
  const int t_last = tile_hi >> 5;                       // tile_hi may be -1 -> t_last = -1

  for (int t = t_first; t <= t_last; ++t) {
    if (t == 0 && t_first == -1) t = tile_lo >> 5;       // after the memory tile jump to the first visible tile
    const bool memtile = t < 0;
    // keys of this tile: memory rows 0..mem-1, or compressed / token keys 32t .. 32t+31
    const int kk = memtile ? n_ : 32 * t + n_;
    const bool kok = memtile ? (n_ < P.mem) : (kk < P.nkeys);
    const long krow = kok ? (memtile ? kk : kk + P.mem) : 0;
    bf16x8 Kf[KS], Vv[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Kf[ks] = kok ? load8(kbase + krow * P.sk[2] + 16 * ks) : zero_frag();
      Vv[ks] = kok ? load8(vbase + krow * P.sv[2] + 16 * ks) : zero_frag();
    }
    floatx16 Sa = zero_acc();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) Sa = mfma32(Kf[ks], Qf[ks], Sa);

    // visibility of the 16 keys this lane holds for its row
    const int klo = memtile ? 0 : me.lo, khi = memtile ? P.mem - 1 : me.hi;
    const int kb0 = memtile ? 0 : 32 * t;
    float tmax = -INFINITY;
#pragma unroll
    for (int i2 = 0; i2 < 16; ++i2) {
      const int key = kb0 + 8 * (i2 >> 2) + 4 * h + (i2 & 3);
      const float s = (key >= klo && key <= khi) ? Sa[i2] * sc : -INFINITY;
      Sa[i2] = s;
      tmax = fmaxf(tmax, s);
    }

    if (P.pool && !memtile) {
      // block-importance logits: groups of npf consecutive keys, then the G heads of the group
      const float to_nat = kLn2;                         // scores are in log2 units here
      const int npf = P.npf;
      float grp[4];                                      // one value per register quartet (a)
#pragma unroll
      for (int a = 0; a < 4; ++a) grp[a] = 0.f;
      if (npf >= 4) {
#pragma unroll
        for (int a = 0; a < 4; ++a) grp[a] = (Sa[4 * a] + Sa[4 * a + 1]) + (Sa[4 * a + 2] + Sa[4 * a + 3]);
        if (npf >= 8) {
#pragma unroll
          for (int a = 0; a < 4; ++a) grp[a] += xor32(grp[a]);
        }
        if (npf == 16) { grp[0] += grp[1]; grp[2] += grp[3]; }
        if (npf == 32) { grp[0] = (grp[0] + grp[1]) + (grp[2] + grp[3]); }
      }
      // number of values this lane holds and their first key offsets inside the tile
#pragma unroll
      for (int i2 = 0; i2 < 16; ++i2) {
        float val; int koff; bool mine;
        if (npf == 1) { val = Sa[i2]; koff = 8 * (i2 >> 2) + 4 * h + (i2 & 3); mine = true; }
        else if (npf == 2) { val = Sa[i2 & ~1] + Sa[i2 | 1]; koff = 8 * (i2 >> 2) + 4 * h + (i2 & 2); mine = (i2 & 1) == 0; }
        else if (npf == 4) { val = grp[i2 >> 2]; koff = 8 * (i2 >> 2) + 4 * h; mine = (i2 & 3) == 0; }
        else if (npf == 8) { val = grp[i2 >> 2]; koff = 8 * (i2 >> 2); mine = (i2 & 3) == 0 && h == 0; }
        else if (npf == 16) { val = grp[(i2 >> 3) * 2]; koff = 16 * (i2 >> 3); mine = (i2 & 7) == 0 && h == 0; }
        else { val = grp[0]; koff = 0; mine = i2 == 0 && h == 0; }
        if (P.share) {
          for (int mk = 1; mk < P.g; mk <<= 1) val += __shfl_xor(val, mk, 64);
        }
        const int jblk = (kb0 + koff) / npf;
        const bool writer = mine && valid && jblk < P.nb && (!P.share || g == 0);
        if (writer) {
          float Lv = val * to_nat / (float)(npf * (P.share ? P.g : 1));
          if (P.mask_own && jblk == i / P.B) Lv = -INFINITY;
          const long prow = P.share ? ((long)bh * P.n + i) : (((long)b * P.hkv * P.g + hq) * P.n + i);
          pooled[prow * P.nb + jblk] = Lv;
        }
      }
    }

    tmax = fmaxf(tmax, xor32(tmax));
    const float mnew = fmaxf(m, tmax);
    const float mref = (mnew == -INFINITY) ? 0.f : mnew;
    const float alpha = fast_exp2(m - mref);
    float rs = 0.f;
#pragma unroll
    for (int i2 = 0; i2 < 16; ++i2) {
      const float p = fast_exp2(Sa[i2] - mref);
      Sa[i2] = p;
      rs += p;
    }
    rs += xor32(rs);
    l = l * alpha + rs;
    m = mnew;
    const bf16x8 Pf0 = pack8(Sa, 0), Pf1 = pack8(Sa, 8);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      floatx16 tv = mfma32(Vv[2 * dt], ilo, zero_acc());
      tv = mfma32(Vv[2 * dt + 1], ihi, tv);
#pragma unroll
      for (int e = 0; e < 16; ++e) Oa[dt][e] *= alpha;
      Oa[dt] = mfma32(pack8(tv, 0), Pf0, Oa[dt]);
      Oa[dt] = mfma32(pack8(tv, 8), Pf1, Oa[dt]);
    }
  }

  if (P.pool) {
    // fine blocks whose compressed keys no query of this tile can see were never visited
    const int jstart = min(P.nb, (32 * (t_last + 1)) / P.npf);
    const int cntj = P.nb - jstart;
    const int rows_here = min(ppt, P.n - i0) * (P.share ? 1 : P.g);
    for (int e = lane; e < rows_here * cntj; e += 64) {
      const int rr = e / cntj, jj = jstart + e % cntj;
      const int qi = i0 + (P.share ? rr : rr / P.g);
      const long prow = P.share ? ((long)bh * P.n + qi) : (((long)b * P.hkv * P.g + hk * P.g + rr % P.g) * P.n + qi);
      pooled[prow * P.nb + jj] = -INFINITY;
    }
  }

  if (valid) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    __bf16* op = out + b * P.so[0] + (long)hq * P.so[1] + (long)i * P.so[2] + 4 * h;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a)
        store4_bf16(op + 32 * dt + 8 * a, Oa[dt][4 * a] * inv, Oa[dt][4 * a + 1] * inv, Oa[dt][4 * a + 2] * inv, Oa[dt][4 * a + 3] * inv);
    if (h == 0) lse[((long)b * P.hkv * P.g + hq) * P.n + i] = (m + fast_log2(l)) * kLn2;
  }
}

// ------------------------------------------------------------------------------ backward
// delta[b,hq,i] = sum_d out * d_out
template <int D>
__global__ __launch_bounds__(256) void dense_delta_kernel(const DensePlan P, const __bf16* __restrict__ out, const __bf16* __restrict__ dout, float* __restrict__ delta) {
  constexpr int LPR = D / 8, RPB = 256 / LPR;
  const int tid = threadIdx.x;
  const long row = (long)blockIdx.x * RPB + tid / LPR;
  const long rows = (long)P.bh * P.g * P.n;
  const int dd = (tid % LPR) * 8;
  float s = 0.f;
  if (row < rows) {
    const long i = row % P.n, bhq = row / P.n;
    const long b = bhq / (P.hkv * P.g), hq = bhq % (P.hkv * P.g);
    const bf16x8 o = load8(out + b * P.so[0] + hq * P.so[1] + i * P.so[2] + dd);
    const bf16x8 d = load8(dout + b * P.sdo[0] + hq * P.sdo[1] + i * P.sdo[2] + dd);
#pragma unroll
    for (int e = 0; e < 8; ++e) s += (float)o[e] * (float)d[e];
  }
#pragma unroll
  for (int mk = LPR / 2; mk >= 1; mk >>= 1) s += __shfl_xor(s, mk, 64);
  if (row < rows && (tid % LPR) == 0) delta[row] = s;
}

// dQ, query-stationary (same walk as the forward)
template <int D>
__global__ __launch_bounds__(64) void dense_bwd_dq_kernel(const DensePlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                          const __bf16* __restrict__ v, const __bf16* __restrict__ dout,
                                                          const float* __restrict__ lse, const float* __restrict__ delta, __bf16* __restrict__ dq) {
  constexpr int KS = D / 16, DT = D / 32;
  const int lane = threadIdx.x, n_ = lane & 31, h = lane >> 5;
  const int bh = blockIdx.y, b = bh / P.hkv, hk = bh % P.hkv;
  const int ppt = 32 >> P.lg;
  const int i0 = blockIdx.x * ppt;
  const int pq = n_ >> P.lg, g = n_ & (P.g - 1);
  const bool valid = i0 + pq < P.n;
  const int i = valid ? i0 + pq : P.n - 1;
  const int ilast = min(P.n - 1, i0 + ppt - 1);
  const int hq = hk * P.g + g;

  bf16x8 Qf[KS], Gf[KS], ilo, ihi;
  make_ident(lane, ilo, ihi);
  {
    const __bf16* qp = q + b * P.sq[0] + (long)hq * P.sq[1] + (long)i * P.sq[2] + 8 * h;
    const __bf16* gp = dout + b * P.sdo[0] + (long)hq * P.sdo[1] + (long)i * P.sdo[2] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) { Qf[ks] = load8(qp + 16 * ks); Gf[ks] = load8(gp + 16 * ks); }
  }
  const long srow = ((long)b * P.hkv * P.g + hq) * P.n + i;
  const float lse_r = lse[srow] * kLog2e, del_r = delta[srow];
  const Interval me = visible_range(P, i);
  const int tile_lo = visible_range(P, i0).lo, tile_hi = visible_range(P, ilast).hi;
  const float sc = P.scale * kLog2e;
  floatx16 Qa[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) Qa[dt] = zero_acc();
  const __bf16* kbase = k + b * P.sk[0] + hk * P.sk[1] + 8 * h;
  const __bf16* vbase = v + b * P.sv[0] + hk * P.sv[1] + 8 * h;
  const int t_first = (P.mem > 0) ? -1 : (tile_lo >> 5);
  const int t_last = tile_hi >> 5;

  for (int t = t_first; t <= t_last; ++t) {
    if (t == 0 && t_first == -1) t = tile_lo >> 5;
    const bool memtile = t < 0;
    const int kk = memtile ? n_ : 32 * t + n_;
    const bool kok = memtile ? (n_ < P.mem) : (kk < P.nkeys);
    const long krow = kok ? (memtile ? kk : kk + P.mem) : 0;
    bf16x8 Kf[KS], Vf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Kf[ks] = kok ? load8(kbase + krow * P.sk[2] + 16 * ks) : zero_frag();
      Vf[ks] = kok ? load8(vbase + krow * P.sv[2] + 16 * ks) : zero_frag();
    }
    floatx16 Sa = zero_acc(), Pa = zero_acc();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Sa = mfma32(Kf[ks], Qf[ks], Sa);
      Pa = mfma32(Vf[ks], Gf[ks], Pa);
    }
    const int klo = memtile ? 0 : me.lo, khi = memtile ? P.mem - 1 : me.hi;
    const int kb0 = memtile ? 0 : 32 * t;
#pragma unroll
    for (int i2 = 0; i2 < 16; ++i2) {
      const int key = kb0 + 8 * (i2 >> 2) + 4 * h + (i2 & 3);
      const float p = (key >= klo && key <= khi) ? fast_exp2(Sa[i2] * sc - lse_r) : 0.f;
      Sa[i2] = p * (Pa[i2] - del_r);
    }
    const bf16x8 Sf0 = pack8(Sa, 0), Sf1 = pack8(Sa, 8);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      floatx16 tk = mfma32(Kf[2 * dt], ilo, zero_acc());
      tk = mfma32(Kf[2 * dt + 1], ihi, tk);
      Qa[dt] = mfma32(pack8(tk, 0), Sf0, Qa[dt]);
      Qa[dt] = mfma32(pack8(tk, 8), Sf1, Qa[dt]);
    }
  }
  if (valid) {
    __bf16* op = dq + srow * D + 4 * h;
    const float s = P.scale;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a)
        store4_bf16(op + 32 * dt + 8 * a, Qa[dt][4 * a] * s, Qa[dt][4 * a + 1] * s, Qa[dt][4 * a + 2] * s, Qa[dt][4 * a + 3] * s);
  }
}

// Query range [qlo, qhi) that can see any key of key tile t (t = -1: the memory tile).
__device__ __forceinline__ void tile_query_range(const DensePlan& P, int t, int& qlo, int& qhi) {
  if (t < 0) { qlo = 0; qhi = P.n; return; }
  if (P.mode == 0) {
    qlo = max(0, 32 * t - P.wf);
    qhi = min(P.n, 32 * t + 31 + P.wb + 1);
  } else {
    qlo = P.causal ? min(P.n, (32 * t + 1) * P.st) : 0;      // key kk visible iff i >= (kk+1)*st
    qhi = P.n;
  }
}

// dK/dV of one 32-key tile over one chunk of the queries that can see it (key-stationary);
// same register scheme as sel_bwd_dkv_kernel.
template <int D>
__global__ __launch_bounds__(64) void dense_bwd_dkv_kernel(const DensePlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                           const __bf16* __restrict__ v, const __bf16* __restrict__ dout,
                                                           const float* __restrict__ lse, const float* __restrict__ delta, float* __restrict__ part) {
  constexpr int KS = D / 16, DT = D / 32;
  __shared__ __align__(16) float lse_s[32];
  __shared__ __align__(16) float del_s[32];
  __shared__ __align__(16) int lo_s[32];
  __shared__ __align__(16) int hi_s[32];
  const int lane = threadIdx.x, n_ = lane & 31, h = lane >> 5;
  const int bh = blockIdx.y, b = bh / P.hkv, hk = bh % P.hkv;
  const int tix = blockIdx.x / P.chunks, c = blockIdx.x % P.chunks;
  const int t = tix - (P.mem > 0 ? 1 : 0);
  const bool memtile = t < 0;
  int qlo, qhi;
  tile_query_range(P, t, qlo, qhi);
  const int c0 = qlo + c * P.chunk_q, c1 = min(qhi, c0 + P.chunk_q);
  if (c0 >= c1) return;

  const int kk = memtile ? n_ : 32 * t + n_;              // this lane's key (index space of the mask)
  const bool kok = memtile ? (n_ < P.mem) : (kk < P.nkeys);
  bf16x8 Kf[KS], Vf[KS], ilo, ihi;
  make_ident(lane, ilo, ihi);
  {
    const long krow = kok ? (memtile ? kk : kk + P.mem) : 0;
    const __bf16* kp = k + b * P.sk[0] + hk * P.sk[1] + krow * P.sk[2] + 8 * h;
    const __bf16* vp = v + b * P.sv[0] + hk * P.sv[1] + krow * P.sv[2] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Kf[ks] = kok ? load8(kp + 16 * ks) : zero_frag();
      Vf[ks] = kok ? load8(vp + 16 * ks) : zero_frag();
    }
  }
  floatx16 dKa[DT], dVa[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) { dKa[dt] = zero_acc(); dVa[dt] = zero_acc(); }
  const float sc = P.scale * kLog2e;
  const int ppt = 32 >> P.lg;
  const int pq = n_ >> P.lg, g = n_ & (P.g - 1);
  const int hq = hk * P.g + g;

  for (int i0 = c0; i0 < c1; i0 += ppt) {
    const bool valid = i0 + pq < c1;
    const int i = valid ? i0 + pq : i0;
    const __bf16* qp = q + b * P.sq[0] + (long)hq * P.sq[1] + (long)i * P.sq[2] + 8 * h;
    const __bf16* gp = dout + b * P.sdo[0] + (long)hq * P.sdo[1] + (long)i * P.sdo[2] + 8 * h;
    bf16x8 Qf[KS], Gf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) { Qf[ks] = load8(qp + 16 * ks); Gf[ks] = load8(gp + 16 * ks); }
    if (h == 0) {
      const long srow = ((long)b * P.hkv * P.g + hq) * P.n + i;
      lse_s[n_] = valid ? lse[srow] * kLog2e : INFINITY;
      del_s[n_] = delta[srow];
      const Interval me = visible_range(P, i);
      lo_s[n_] = memtile ? 0 : me.lo;
      hi_s[n_] = memtile ? P.mem - 1 : me.hi;
    }
    __syncthreads();
    floatx16 Sa = zero_acc(), Pa = zero_acc();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Sa = mfma32(Qf[ks], Kf[ks], Sa);
      Pa = mfma32(Gf[ks], Vf[ks], Pa);
    }
    floatx16 dSa;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const floatx4 l4 = *reinterpret_cast<const floatx4*>(&lse_s[8 * a + 4 * h]);
      const floatx4 d4 = *reinterpret_cast<const floatx4*>(&del_s[8 * a + 4 * h]);
      const int* lo4 = &lo_s[8 * a + 4 * h];
      const int* hi4 = &hi_s[8 * a + 4 * h];
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) {
        const int i2 = 4 * a + bb;
        const float p = (kk >= lo4[bb] && kk <= hi4[bb]) ? fast_exp2(Sa[i2] * sc - l4[bb]) : 0.f;
        Sa[i2] = p;
        dSa[i2] = p * (Pa[i2] - d4[bb]);
      }
    }
    const bf16x8 Pf0 = pack8(Sa, 0), Pf1 = pack8(Sa, 8);
    const bf16x8 Sf0 = pack8(dSa, 0), Sf1 = pack8(dSa, 8);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      floatx16 tt = mfma32(Gf[2 * dt], ilo, zero_acc());
      tt = mfma32(Gf[2 * dt + 1], ihi, tt);
      dVa[dt] = mfma32(pack8(tt, 0), Pf0, dVa[dt]);
      dVa[dt] = mfma32(pack8(tt, 8), Pf1, dVa[dt]);
      tt = mfma32(Qf[2 * dt], ilo, zero_acc());
      tt = mfma32(Qf[2 * dt + 1], ihi, tt);
      dKa[dt] = mfma32(pack8(tt, 0), Sf0, dKa[dt]);
      dKa[dt] = mfma32(pack8(tt, 8), Sf1, dKa[dt]);
    }
    __syncthreads();
  }
  float* pk = part + (((size_t)bh * P.key_tiles + tix) * P.chunks + c) * (2 * 32 * D) + (size_t)n_ * D + 4 * h;
  float* pv = pk + 32 * D;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      floatx4 x, y;
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) { x[bb] = dKa[dt][4 * a + bb]; y[bb] = dVa[dt][4 * a + bb]; }
      *reinterpret_cast<floatx4*>(pk + 32 * dt + 8 * a) = x;
      *reinterpret_cast<floatx4*>(pv + 32 * dt + 8 * a) = y;
    }
}

template <int D>
__global__ __launch_bounds__(256) void dense_bwd_dkv_reduce_kernel(const DensePlan P, const float* __restrict__ part, __bf16* __restrict__ dk, __bf16* __restrict__ dv) {
  const int tix = blockIdx.x, bh = blockIdx.y;
  const int t = tix - (P.mem > 0 ? 1 : 0);
  int qlo, qhi;
  tile_query_range(P, t, qlo, qhi);
  const int live = qhi > qlo ? (qhi - qlo + P.chunk_q - 1) / P.chunk_q : 0;
  const int keys = t < 0 ? P.mem : min(32, P.nkeys - 32 * t);
  const long row0 = t < 0 ? 0 : (long)P.mem + 32 * t;
  const float* base = part + ((size_t)bh * P.key_tiles + tix) * P.chunks * (2 * 32 * D);
  constexpr int CPR = D / 4;
  for (int e = threadIdx.x; e < 2 * keys * CPR; e += 256) {
    const int which = e / (keys * CPR), rem = e % (keys * CPR);
    const int key = rem / CPR, dd = (rem % CPR) * 4;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int c = 0; c < live; ++c)
      acc += *reinterpret_cast<const floatx4*>(base + (size_t)c * (2 * 32 * D) + (size_t)which * 32 * D + (size_t)key * D + dd);
    const float s = which == 0 ? P.scale : 1.0f;
    __bf16* dst = (which == 0 ? dk : dv) + ((size_t)bh * P.krows + row0 + key) * D + dd;
    store4_bf16(dst, acc[0] * s, acc[1] * s, acc[2] * s, acc[3] * s);
  }
}

}  // namespace nsa

using namespace nsa;

#define NSA_LAUNCH_CHECK()                         \
  do {                                             \
    hipError_t e_ = hipGetLastError();             \
    if (e_ != hipSuccess) return (int)e_;          \
  } while (0)

extern "C" int nsa_dense_workspace_bytes(const nsa_dense_desc* d, size_t* bwd_bytes) {
  DensePlan P;
  const int rc = make_dense_plan(d, P);
  if (rc) return rc;
  if (bwd_bytes) *bwd_bytes = P.bwd_total;
  return 0;
}

template <int D>
static int dense_fwd_launch(const DensePlan& P, const void* q, const void* k, const void* v, void* out, float* lse, float* pooled, hipStream_t st) {
  const int ppt = 32 >> P.lg;
  hipLaunchKernelGGL((dense_fwd_kernel<D>), dim3((P.n + ppt - 1) / ppt, P.bh), dim3(64), 0, st, P, (const __bf16*)q, (const __bf16*)k,
                     (const __bf16*)v, (__bf16*)out, lse, pooled);
  NSA_LAUNCH_CHECK();
  return 0;
}

extern "C" int nsa_dense_fwd(const nsa_dense_desc* d, const void* q, const void* k, const void* v, void* out, float* lse, float* pooled, void* stream) {
  DensePlan P;
  const int rc = make_dense_plan(d, P);
  if (rc) return rc;
  if (!q || !k || !v || !out || !lse || (P.pool && !pooled)) return NSA_E_ARG;
  if (P.D == 64) return dense_fwd_launch<64>(P, q, k, v, out, lse, pooled, (hipStream_t)stream);
  if (P.D == 128) return dense_fwd_launch<128>(P, q, k, v, out, lse, pooled, (hipStream_t)stream);
  return NSA_E_UNSUPPORTED;
}

template <int D>
static int dense_bwd_launch(const DensePlan& P, const void* q, const void* k, const void* v, const void* out, const void* dout, const float* lse,
                            void* ws, void* dq, void* dk, void* dv, hipStream_t st) {
  float* delta = reinterpret_cast<float*>((char*)ws + P.off_delta);
  float* part = reinterpret_cast<float*>((char*)ws + P.off_part);
  const long rows = (long)P.bh * P.g * P.n;
  constexpr int RPB = 256 / (D / 8);
  hipLaunchKernelGGL((dense_delta_kernel<D>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, st, P, (const __bf16*)out, (const __bf16*)dout, delta);
  NSA_LAUNCH_CHECK();
  const int ppt = 32 >> P.lg;
  hipLaunchKernelGGL((dense_bwd_dq_kernel<D>), dim3((P.n + ppt - 1) / ppt, P.bh), dim3(64), 0, st, P, (const __bf16*)q, (const __bf16*)k,
                     (const __bf16*)v, (const __bf16*)dout, lse, delta, (__bf16*)dq);
  NSA_LAUNCH_CHECK();
  hipLaunchKernelGGL((dense_bwd_dkv_kernel<D>), dim3(P.key_tiles * P.chunks, P.bh), dim3(64), 0, st, P, (const __bf16*)q, (const __bf16*)k,
                     (const __bf16*)v, (const __bf16*)dout, lse, delta, part);
  NSA_LAUNCH_CHECK();
  hipLaunchKernelGGL((dense_bwd_dkv_reduce_kernel<D>), dim3(P.key_tiles, P.bh), dim3(256), 0, st, P, part, (__bf16*)dk, (__bf16*)dv);
  NSA_LAUNCH_CHECK();
  return 0;
}

extern "C" int nsa_dense_bwd(const nsa_dense_desc* d, const void* q, const void* k, const void* v, const void* out, const void* d_out,
                             const float* lse, void* bwd_ws, size_t bwd_bytes, void* dq, void* dk, void* dv, void* stream) {
  DensePlan P;
  const int rc = make_dense_plan(d, P);
  if (rc) return rc;
  if (bwd_bytes < P.bwd_total) return NSA_E_WORKSPACE;
  if (!q || !k || !v || !out || !d_out || !lse || !bwd_ws || !dq || !dk || !dv) return NSA_E_ARG;
  if (P.D == 64) return dense_bwd_launch<64>(P, q, k, v, out, d_out, lse, bwd_ws, dq, dk, dv, (hipStream_t)stream);
  if (P.D == 128) return dense_bwd_launch<128>(P, q, k, v, out, d_out, lse, bwd_ws, dq, dk, dv, (hipStream_t)stream);
  return NSA_E_UNSUPPORTED;
}
