// Single-token decode attention over the key / value caches (NSA.py:338-547): the G query
// heads of one kv head attend either to a contiguous key range (compressed branch, with the
// memory slots as extra keys and the scaled logits written out for the importance scores;
// sliding branch) or to the selected blocks plus the query's own block (selection branch).
//
// HBM-bound: every cached key / value row a query attends is read once.  The keys of a unit
// (batch, kv head) are cut into 32-key tiles that are dealt round-robin to the waves of
// `nsplit` work-groups (split-K), so that a single long sequence still fills the chip; every
// wave keeps a running (max, sum, O) and writes one fp32 partial, and a second kernel merges the
// partials of a head.  Scores are computed transposed, S^T = K Q^T on the 32x32x16 MFMA with the
// query heads as (zero-padded) columns: a lane then owns one head, the softmax statistics are
// per-lane scalars and the rescaling of O^T = V^T P needs no cross-lane traffic.
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

namespace nsa {

struct DecodePlan {
  int b, hk, g, d;
  int units;         // per batch: hk (shared selection / ranges) or hk*g (per-head selection)
  int gc;            // query heads per unit
  int mode, start, count, mem;
  int B, S, kv_len, tps;
  int tiles, nsplit, nparts, rec;    // rec: floats per partial record: [gc][d] O, [gc] max, [gc] sum, padded to 16 bytes
  int idx64;
  float scale;
  long sq[2], sk[3], sv[3];
};

template <int D>
__global__ __launch_bounds__(256) void decode_attend_kernel(const DecodePlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                            const __bf16* __restrict__ v, const __bf16* __restrict__ mem_k,
                                                            const __bf16* __restrict__ mem_v, const void* __restrict__ idx,
                                                            const unsigned char* __restrict__ fmask, float* __restrict__ part,
                                                            float* __restrict__ logits) {
  constexpr int KS = D / 16, DT = D / 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_ = lane & 31, h = lane >> 5;
  const int ug = blockIdx.y, b = ug / P.units, u = ug % P.units;
  const int hk = (P.units == P.hk) ? u : u / P.g;
  const int head0 = (P.units == P.hk) ? u * P.g : u;
  const int wid = blockIdx.x * 4 + wave, nw = P.nsplit * 4;

  bf16x8 Qf[KS];
  {
    const bool okq = n_ < P.gc;
    const __bf16* qp = q + b * P.sq[0] + (long)(head0 + (okq ? n_ : 0)) * P.sq[1] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) Qf[ks] = okq ? load8(qp + 16 * ks) : zero_frag();
  }
  bf16x8 ilo, ihi;
  make_ident(lane, ilo, ihi);
  const float sc = P.scale * kLog2e;
  const int mem_tiles = (P.mem + 31) >> 5;

  float m = -INFINITY, l = 0.f;
  floatx16 Oa[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) Oa[dt] = zero_acc();

  for (int t = wid; t < P.tiles; t += nw) {
    // tile -> rows of (kb, vb) with row stride (ks_, vs_), first row key0, nvalid rows
    const __bf16 *kb, *vb;
    long ks_, vs_, key0;
    int nvalid, lcol = -1;           // lcol: column of the tile's first key in the logits row
    if (P.mode == 0) {
      if (t < mem_tiles) {
        kb = mem_k + (long)hk * P.mem * D; vb = mem_v + (long)hk * P.mem * D;
        ks_ = vs_ = D; key0 = 32 * t; nvalid = min(32, P.mem - 32 * t);
      } else {
        const int tt = t - mem_tiles;
        kb = k + b * P.sk[0] + hk * P.sk[1]; vb = v + b * P.sv[0] + hk * P.sv[1];
        ks_ = P.sk[2]; vs_ = P.sv[2]; key0 = P.start + 32 * tt; nvalid = min(32, P.count - 32 * tt);
        lcol = 32 * tt;
      }
    } else {
      const int slot = t / P.tps, sub = t % P.tps;
      kb = k + b * P.sk[0] + hk * P.sk[1]; vb = v + b * P.sv[0] + hk * P.sv[1];
      ks_ = P.sk[2]; vs_ = P.sv[2];
      long blk;
      bool live = true;
      if (slot < P.S) {
        const long e = (long)ug * P.S + slot;
        blk = P.idx64 ? reinterpret_cast<const long*>(idx)[e] : (long)reinterpret_cast<const int*>(idx)[e];
        live = fmask[e] != 0 && blk >= 0 && blk * P.B < P.kv_len;
      } else {
        blk = (P.kv_len - 1) / P.B;                   // the query's own block, up to itself
      }
      key0 = blk * P.B + 32 * sub;
      nvalid = live ? (int)min((long)32, min((long)P.B - 32 * sub, (long)P.kv_len - key0)) : 0;
    }
    if (nvalid <= 0) continue;                        // wave-uniform

    const bool okr = n_ < nvalid;
    const __bf16* kp = kb + (key0 + (okr ? n_ : 0)) * ks_ + 8 * h;
    const __bf16* vp = vb + (key0 + (okr ? n_ : 0)) * vs_ + 8 * h;
    floatx16 Sa = zero_acc();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) Sa = mfma32(okr ? load8(kp + 16 * ks) : zero_frag(), Qf[ks], Sa);
    bf16x8 VT[DT][2];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const bf16x8 va = okr ? load8(vp + 32 * dt) : zero_frag();
      const bf16x8 vb2 = okr ? load8(vp + 32 * dt + 16) : zero_frag();
      floatx16 tr = mfma32(va, ilo, zero_acc());
      tr = mfma32(vb2, ihi, tr);
      VT[dt][0] = pack8(tr, 0);
      VT[dt][1] = pack8(tr, 8);
    }

    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int kl = 8 * (i >> 2) + 4 * h + (i & 3);
      if (logits != nullptr && lcol >= 0 && n_ < P.gc && kl < nvalid)
        logits[((long)b * P.hk * P.g + head0 + n_) * P.count + lcol + kl] = Sa[i] * P.scale;
      const float s = kl < nvalid ? Sa[i] * sc : -INFINITY;
      Sa[i] = s;
      mx = fmaxf(mx, s);
    }
    mx = fmaxf(mx, xor32(mx));
    const float mn = fmaxf(m, mx);
    const float alpha = fast_exp2(m - mn);
    float ls = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float p = fast_exp2(Sa[i] - mn);
      Sa[i] = p;
      ls += p;
    }
    l = l * alpha + ls;
    m = mn;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) Oa[dt][i] *= alpha;
#pragma unroll
      for (int u2 = 0; u2 < 2; ++u2) Oa[dt] = mfma32(VT[dt][u2], pack8(Sa, 8 * u2), Oa[dt]);
    }
  }
  l += xor32(l);

  // partial record of this wave: [gc][D] O, [gc] max, [gc] sum
  if (n_ < P.gc) {
    float* rec = part + ((long)ug * P.nparts + wid) * P.rec;
    if (h == 0) { rec[P.gc * D + n_] = m; rec[P.gc * D + P.gc + n_] = l; }
    float* o = rec + n_ * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        floatx4 w = {Oa[dt][4 * i4], Oa[dt][4 * i4 + 1], Oa[dt][4 * i4 + 2], Oa[dt][4 * i4 + 3]};
        *reinterpret_cast<floatx4*>(o + 32 * dt + 8 * i4 + 4 * h) = w;
      }
  }
}

// one work-group per query head, one thread per feature: streaming merge of the head's partials
template <int D>
__global__ __launch_bounds__(D) void decode_merge_kernel(const DecodePlan P, const float* __restrict__ part, __bf16* __restrict__ out) {
  const int hq = P.hk * P.g;
  const int bh = blockIdx.x, b = bh / hq, head = bh % hq;
  const int u = (P.units == P.hk) ? head / P.g : head, gi = (P.units == P.hk) ? head % P.g : 0;
  const float* base = part + (long)(b * P.units + u) * P.nparts * P.rec;
  float M = -INFINITY;
  const int om = P.gc * D + gi, ol = om + P.gc;
  for (int p = 0; p < P.nparts; ++p) M = fmaxf(M, base[(long)p * P.rec + om]);
  float acc = 0.f, L = 0.f;
  if (M > -INFINITY) {
    for (int p = 0; p < P.nparts; ++p) {
      const float* rec = base + (long)p * P.rec;
      const float w = fast_exp2(rec[om] - M);          // exp2(-inf) = 0 for waves that saw no key
      L += w * rec[ol];
      acc += w * rec[gi * D + threadIdx.x];
    }
  }
  out[(long)bh * D + threadIdx.x] = (__bf16)(L > 0.f ? acc / L : 0.f);
}

static int make_decode_plan(const nsa_decode_desc* dsc, DecodePlan& P) {
  if (!dsc) return NSA_E_ARG;
  P = DecodePlan{};
  P.b = dsc->batch; P.hk = dsc->kv_heads; P.g = dsc->group; P.d = dsc->dim_head;
  if (P.b <= 0 || P.hk <= 0 || P.g <= 0) return NSA_E_ARG;
  if (P.d != 64 && P.d != 128) return NSA_E_UNSUPPORTED;
  if (P.g > 32) return NSA_E_UNSUPPORTED;
  P.mode = dsc->mode;
  P.scale = dsc->scale;
  P.idx64 = dsc->idx_is_int64;
  for (int i = 0; i < 2; ++i) P.sq[i] = dsc->q_stride[i];
  for (int i = 0; i < 3; ++i) { P.sk[i] = dsc->k_stride[i]; P.sv[i] = dsc->v_stride[i]; }
  if ((P.sq[0] | P.sq[1] | P.sk[0] | P.sk[1] | P.sk[2] | P.sv[0] | P.sv[1] | P.sv[2]) & 7) return NSA_E_ARG;
  if (P.mode == 0) {
    P.start = dsc->start; P.count = dsc->count; P.mem = dsc->num_mem;
    if (P.start < 0 || P.count < 0 || P.mem < 0) return NSA_E_ARG;
    P.units = P.hk; P.gc = P.g;
    P.tiles = (P.mem + 31) / 32 + (P.count + 31) / 32;
  } else if (P.mode == 1) {
    P.B = dsc->block; P.S = dsc->num_sel; P.kv_len = dsc->kv_len;
    if (P.B < 1 || P.S < 0 || P.kv_len < 1) return NSA_E_ARG;
    const bool per_head = dsc->per_head_sel != 0;
    P.units = per_head ? P.hk * P.g : P.hk;
    P.gc = per_head ? 1 : P.g;
    P.tps = (P.B + 31) / 32;
    P.tiles = (P.S + 1) * P.tps;
  } else {
    return NSA_E_ARG;
  }
  const long units = (long)P.b * P.units;
  if (units > 65535) return NSA_E_UNSUPPORTED;
  int ns = (P.tiles + 3) / 4;
  const long cap = units >= 1024 ? 1 : 1024 / units;
  if (ns > cap) ns = (int)cap;
  if (ns > 64) ns = 64;
  if (ns < 1) ns = 1;
  P.nsplit = ns; P.nparts = ns * 4;
  P.rec = P.gc * P.d + ((2 * P.gc + 3) & ~3);
  return 0;
}

}  // namespace nsa

extern "C" int nsa_decode_workspace_bytes(const nsa_decode_desc* dsc, size_t* bytes) {
  nsa::DecodePlan P;
  if (int e = nsa::make_decode_plan(dsc, P)) return e;
  if (!bytes) return NSA_E_ARG;
  *bytes = (size_t)P.b * P.units * P.nparts * P.rec * sizeof(float);
  return 0;
}

extern "C" int nsa_decode_attend(const nsa_decode_desc* dsc, const void* q, const void* k, const void* v, const void* mem_k,
                                 const void* mem_v, const void* idx, const uint8_t* fmask, void* ws, size_t ws_bytes, void* out,
                                 float* logits, void* stream) {
  using namespace nsa;
  DecodePlan P;
  if (int e = make_decode_plan(dsc, P)) return e;
  if (!q || !out || !ws) return NSA_E_ARG;
  if (P.mode == 0 && ((P.count > 0 && (!k || !v)) || (P.mem > 0 && (!mem_k || !mem_v)))) return NSA_E_ARG;
  if (P.mode == 1 && (!k || !v || (P.S > 0 && (!idx || !fmask)))) return NSA_E_ARG;
  if (ws_bytes < (size_t)P.b * P.units * P.nparts * P.rec * sizeof(float)) return NSA_E_WORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(P.nsplit, P.b * P.units);
  const int heads = P.b * P.hk * P.g;
  if (P.d == 64) {
    hipLaunchKernelGGL((decode_attend_kernel<64>), grid, dim3(256), 0, st, P, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v,
                       (const __bf16*)mem_k, (const __bf16*)mem_v, idx, fmask, (float*)ws, logits);
    hipLaunchKernelGGL((decode_merge_kernel<64>), dim3(heads), dim3(64), 0, st, P, (const float*)ws, (__bf16*)out);
  } else {
    hipLaunchKernelGGL((decode_attend_kernel<128>), grid, dim3(256), 0, st, P, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v,
                       (const __bf16*)mem_k, (const __bf16*)mem_v, idx, fmask, (float*)ws, logits);
    hipLaunchKernelGGL((decode_merge_kernel<128>), dim3(heads), dim3(128), 0, st, P, (const float*)ws, (__bf16*)out);
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}
