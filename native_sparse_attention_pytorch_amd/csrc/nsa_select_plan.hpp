// Host-side launch plan of the block-selection kernels: validated dimensions, work-unit sizes
// and the byte layout of the three caller-owned workspaces.  Recomputed from the descriptor on
// every call (pure function, a few dozen integer operations), passed to kernels by value.
#pragma once
#include <stddef.h>
#include <stdint.h>
#include "../../include/nsa_hip.h"

#ifndef NSA_PHASE_BYTES
#define NSA_PHASE_BYTES (1L << 22)
#endif

#ifndef NSA_DKV_UNITS_WANTED
#define NSA_DKV_UNITS_WANTED 4096
#endif
#ifndef NSA_DKV_CHUNK_FIXED
#define NSA_DKV_CHUNK_FIXED 0      // a power of two to override the choice (experiments)
#endif

namespace nsa {

struct SelPlan {
  int b, hkv, g, lg, n, S, SP, B, D, causal, W, nch, bh, idx64;
  float scale;
  // Work-unit tables.  A unit = up to `chunk` consecutive pairs of one (query phase, block)
  // cell; cells are ordered phase-major so that units running at the same time gather Q rows of
  // the same query range (L2 reuse).  Table t: 0 = forward walk, 1 = dQ walk, 2 = dK/dV walk
  // (a single phase: the whole sequence, so a wave keeps its dK/dV accumulators as long as
  // possible).
  int chunk[3], phase[3], np[3], ub[3];
  size_t off_unit[3];
  size_t off_urec[3];        // per (batch*kv head, unit) a record of 8 ints: block, own, list start, v0, v1
  int ub_kv;                 // = ub[2]
  long list_cap;             // inverse-index entries reserved per (batch, kv head)
  size_t prow;               // number of partial rows; row `prow` is a spare that padding rows write to
  long sq[3], sk[3], sv[3], so[3];
  // index workspace
  size_t off_cnt, off_blk, off_list, index_total;
  // forward workspace
  size_t off_opart, off_lsepart, fwd_total;
  // backward workspace
  size_t off_delta, off_dqpart, off_dkvpart, bwd_total;
};

static inline size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }

static inline int make_plan(const nsa_select_desc* d, SelPlan& P) {
  if (!d) return NSA_E_ARG;
  if (d->batch <= 0 || d->kv_heads <= 0 || d->group <= 0 || d->seq <= 0 || d->num_sel < 0 || d->block <= 0) return NSA_E_ARG;
  if (d->dim_head != 64 && d->dim_head != 128) return NSA_E_UNSUPPORTED;
  if (d->block > 64) return NSA_E_UNSUPPORTED;                 // a block is one or two 32-key register tiles; keys past the block are masked
  if (d->group > 32 || (d->group & (d->group - 1))) return NSA_E_UNSUPPORTED;
  if (d->num_sel > 62) return NSA_E_UNSUPPORTED;
  if (!d->causal && d->num_sel == 0) return NSA_E_ARG;
  P.b = d->batch; P.hkv = d->kv_heads; P.g = d->group; P.n = d->seq; P.S = d->num_sel; P.SP = d->num_sel + 1;
  P.B = d->block; P.D = d->dim_head; P.causal = d->causal ? 1 : 0; P.idx64 = d->idx_is_int64 ? 1 : 0;
  P.scale = d->scale;
  P.lg = 0;
  while ((1 << P.lg) < P.g) ++P.lg;
  P.W = (P.n + P.B - 1) / P.B;
  if (P.W > 16384) return NSA_E_UNSUPPORTED;
  if ((long)P.n * P.SP >= 0x7fffffffL) return NSA_E_UNSUPPORTED;
  P.nch = (P.n + 255) / 256;
  const long bh = (long)P.b * P.hkv;
  if (bh > 65535) return NSA_E_UNSUPPORTED;
  P.bh = (int)bh;
  for (int t = 0; t < 3; ++t) { P.sq[t] = d->q_stride[t]; P.sk[t] = d->k_stride[t]; P.sv[t] = d->v_stride[t]; P.so[t] = d->o_stride[t]; }
  for (int t = 0; t < 3; ++t)
    if ((P.sq[t] | P.sk[t] | P.sv[t] | P.so[t]) & 7) return NSA_E_ARG;      // rows must start 16-byte aligned
  for (int t = 1; t < 3; ++t)                                               // head and token strides: 32-bit arithmetic in the gathers
    if ((P.sq[t] | P.so[t]) < 0 || ((P.sq[t] | P.so[t]) >> 32)) return NSA_E_UNSUPPORTED;
  const long pairs = (long)P.n * (P.S + P.causal);
  // phase length: the Q rows (forward) / Q and dO rows (dQ walk) of one phase are about the size
  // of one XCD's 4 MB L2 (measured best on MI355X among 0.5 .. 64 MB; shorter phases make the
  // work units too small, longer ones lose the L2 reuse of the gathered rows)
  const long row_bytes = (long)P.g * P.D * 2;
  long ph = 256;
  while (ph * 2 * row_bytes <= (long)NSA_PHASE_BYTES && ph < (1L << 20)) ph *= 2;
  P.chunk[0] = 256;  P.phase[0] = (int)ph;
  P.chunk[1] = 256;  P.phase[1] = (int)(ph > 256 ? ph / 2 : ph);
  // dK/dV walk: a unit keeps its accumulators for `chunk` pairs and leaves a 2 x 32KT x D fp32 partial behind, so long units
  // are cheaper per pair - but the chip holds 512 to 1024 work-groups of this kernel at a time, and a launch with fewer
  // units than a few rounds of that runs as long as its longest units whatever the rest does (seq 8k, 4 kv heads: 512 units
  // of 1024 pairs occupy half of the SIMDs for the whole launch).  Shorter units when the launch would have under ~4096.
  {
    const long want = bh * pairs / NSA_DKV_UNITS_WANTED;
    P.chunk[2] = NSA_DKV_CHUNK_FIXED ? NSA_DKV_CHUNK_FIXED : (want >= 1024 ? 1024 : want >= 512 ? 512 : 256);
  }
  P.phase[2] = ((P.n + 255) / 256) * 256;
  for (int t = 0; t < 3; ++t) {
    P.np[t] = (P.n + P.phase[t] - 1) / P.phase[t];
    const long cells = (long)P.np[t] * P.W;
    const long ub = cells + (pairs + P.chunk[t] - 1) / P.chunk[t];
    if (ub > 0x3fffffffL) return NSA_E_UNSUPPORTED;
    P.ub[t] = (int)ub;
  }
  P.ub_kv = P.ub[2];
  P.list_cap = (long)P.n * (P.S > 0 ? P.S : 1);

  size_t o = 0;
  P.off_cnt = o;    o = align_up(o + (size_t)bh * P.nch * P.W * 4);
  P.off_blk = o;    o = align_up(o + (size_t)bh * (P.W + 1) * 4);
  for (int t = 0; t < 3; ++t) { P.off_unit[t] = o; o = align_up(o + (size_t)bh * ((size_t)P.np[t] * P.W + 1) * 4); }
  for (int t = 0; t < 3; ++t) { P.off_urec[t] = o; o = align_up(o + (size_t)bh * (size_t)P.ub[t] * 32); }
  P.off_list = o;   o = align_up(o + (size_t)bh * P.list_cap * 4);
  P.index_total = o;

  const size_t prow = (size_t)bh * P.n * P.SP * P.g;      // partial rows: (query, slot, head)
  P.prow = prow;
  o = 0;
  P.off_opart = o;   o = align_up(o + (prow + 1) * P.D * 2);
  P.off_lsepart = o; o = align_up(o + (prow + 1) * 4);
  P.fwd_total = o;

  const int KT = (P.B + 31) / 32;
  o = 0;
  P.off_delta = o;   o = align_up(o + (size_t)bh * P.g * P.n * 4);
  P.off_dqpart = o;  o = align_up(o + (prow + 1) * P.D * 2);
  P.off_dkvpart = o; o = align_up(o + (size_t)bh * P.ub_kv * 2 * 32 * KT * P.D * 4);
  P.bwd_total = o;
  return 0;
}

}  // namespace nsa
