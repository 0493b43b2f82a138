// Host-side launch plan of the interval-masked (sliding / compressed) attention kernels.
#pragma once
#include <stddef.h>
#include <stdint.h>
#include <algorithm>
#include "../../include/nsa_hip.h"

namespace nsa {

struct DensePlan {
  int b, hkv, g, lg, n, nkeys, mem, krows, D, bh;
  int mode, causal, wb, wf, st;
  int st_sh;                 // log2(st) when the stride is a power of two (the division becomes a shift), else -1
  int pool, npf, nb, B, share, mask_own, nofill;
  int topk;                  // > 0: the forward selects this many blocks per query itself instead of writing the logits
  int dkv_fp32;              // dk / dv leave the reduce kernel as fp32 instead of bf16
  float scale;
  int key_tiles, chunks, chunk_q;
  long sq[3], sk[3], sv[3], so[3], sdo[3];
  size_t off_delta, off_part, bwd_total;
};

static inline size_t dense_align_up(size_t x) { return (x + 255) & ~(size_t)255; }

static inline int make_dense_plan(const nsa_dense_desc* d, DensePlan& P) {
  if (!d) return NSA_E_ARG;
  if (d->batch <= 0 || d->kv_heads <= 0 || d->group <= 0 || d->seq <= 0 || d->num_keys < 0 || d->num_mem < 0) return NSA_E_ARG;
  if (d->dim_head != 64 && d->dim_head != 128) return NSA_E_UNSUPPORTED;
  if (d->group > 32 || (d->group & (d->group - 1))) return NSA_E_UNSUPPORTED;
  if (d->mode != 0 && d->mode != 1) return NSA_E_ARG;
  P.b = d->batch; P.hkv = d->kv_heads; P.g = d->group; P.n = d->seq; P.nkeys = d->num_keys; P.mem = d->num_mem;
  P.krows = P.nkeys + P.mem; P.D = d->dim_head; P.mode = d->mode; P.causal = d->causal ? 1 : 0; P.scale = d->scale;
  P.dkv_fp32 = d->dkv_fp32 ? 1 : 0;
  P.lg = 0;
  while ((1 << P.lg) < P.g) ++P.lg;
  const long bh = (long)P.b * P.hkv;
  if (bh > 65535) return NSA_E_UNSUPPORTED;
  P.bh = (int)bh;
  P.topk = 0;
  P.wb = P.wf = 0; P.st = 1; P.pool = 0; P.npf = 1; P.nb = 0; P.B = 1; P.share = 1; P.mask_own = 0; P.nofill = 0;
  if (P.mode == 0) {
    if (d->window < 0 || P.mem != 0 || P.nkeys != P.n) return NSA_E_ARG;
    P.wb = d->window; P.wf = P.causal ? 0 : d->window;
  } else {
    if (d->stride <= 0 || P.mem > 32 || P.krows <= 0) return NSA_E_ARG;
    if (P.causal && P.mem == 0) return NSA_E_ARG;             // early queries would see nothing
    P.st = d->stride;
    if (d->pool) {
      if (d->sel_block <= 0 || d->sel_block % d->stride) return NSA_E_ARG;
      P.npf = d->sel_block / d->stride;
      if (P.npf > 32 || (P.npf & (P.npf - 1))) return NSA_E_UNSUPPORTED;
      P.pool = 1; P.B = d->sel_block; P.share = d->share ? 1 : 0;
      P.nofill = (d->pool == 2 && d->causal) ? 1 : 0;      // the caller reads row i only below column floor(i / B)
      P.mask_own = d->stride != d->sel_block;
      P.nb = P.nkeys / P.npf;
      if (P.nb == 0) P.pool = 0;
    }
  }
  P.st_sh = -1;
  if (P.st > 0 && !(P.st & (P.st - 1))) { P.st_sh = 0; while ((1 << P.st_sh) < P.st) ++P.st_sh; }
  for (int t = 0; t < 3; ++t) {
    P.sq[t] = d->q_stride[t]; P.sk[t] = d->k_stride[t]; P.sv[t] = d->v_stride[t]; P.so[t] = d->o_stride[t]; P.sdo[t] = d->do_stride[t];
    if ((P.sq[t] | P.sk[t] | P.sv[t] | P.so[t] | P.sdo[t]) & 7) return NSA_E_ARG;
    if (t > 0 && ((P.sq[t] | P.sdo[t]) < 0 || ((P.sq[t] | P.sdo[t]) >> 32))) return NSA_E_UNSUPPORTED;      // 32-bit stride arithmetic in the dK/dV gathers
  }
  // the K / V tile copies address a lane's row as a 32-bit byte offset (up to 15 rows) from a scalar base
  if (P.sk[2] < 0 || P.sv[2] < 0 || (P.sk[2] >> 26) || (P.sv[2] >> 26)) return NSA_E_UNSUPPORTED;
  // dK/dV walk: 64-row tiles of k/v (memory slots included), the queries that can see a tile
  // are cut into chunks of chunk_q; smaller chunks when there would be too few work-groups
  P.key_tiles = (P.krows + 63) / 64;
  const long span = P.mode == 0 ? ((long)64 + P.wb + P.wf < P.n ? (long)64 + P.wb + P.wf : P.n) : P.n;
#ifndef NSA_DKV_MIN_WGS
#define NSA_DKV_MIN_WGS 2048
#endif
  if (P.mode == 0) {
    // band: a tile's visible queries (64 + window of them) in equal chunks, as few as give the chip NSA_DKV_MIN_WGS work-groups
    // (a chunk of 512 beside one of 64 is a work-group that runs eight times longer than its neighbour)
    long want = (NSA_DKV_MIN_WGS + bh * P.key_tiles - 1) / (bh * P.key_tiles);
    want = std::max<long>(1, std::min<long>(want, (span + 127) / 128));
    P.chunk_q = (int)(((span + want - 1) / want + 31) / 32 * 32);
  } else {
    P.chunk_q = 1024;
    while (P.chunk_q > 128 && bh * P.key_tiles * ((span + P.chunk_q - 1) / P.chunk_q) < 2048) P.chunk_q /= 2;
  }
  P.chunks = (int)((span + P.chunk_q - 1) / P.chunk_q);
  size_t o = 0;
  P.off_delta = o; o = dense_align_up(o + (size_t)bh * P.g * P.n * 4);
  P.off_part = o;  o = dense_align_up(o + (size_t)bh * P.key_tiles * P.chunks * 2 * 64 * P.D * 4);
  P.bwd_total = o;
  return 0;
}

}  // namespace nsa
