// Single-token decode attention over the key / value caches (NSA.py:338-547): the G query
// heads of one kv head attend either to a contiguous key range (compressed branch, with the
// memory slots as extra keys and the scaled logits written out for the importance scores;
// sliding branch) or to the selected blocks plus the query's own block (selection branch).
//
// HBM-bound: every cached key / value row a query attends is read once.  The keys of a unit
// (batch, kv head) are cut into 32-key tiles that are dealt round-robin to the waves of
// `nsplit` work-groups (split-K), so that a single long sequence still fills the chip; every
// wave keeps a running (max, sum, O) and writes one fp32 partial, and a second kernel merges the
// partials of a head.  Rows are fetched one tile ahead with whole-row coalesced loads and become
// MFMA operands through a per-wave LDS tile (row operand for K, transposing LDS load for V^T):
// reading each row in 32-byte pieces straight into the operand layout touches every cache line
// from several instructions and re-fetches it from L2 once the L1 thrashes.  Scores are computed transposed, S^T = K Q^T on the 32x32x16 MFMA with the
// query heads as (zero-padded) columns: a lane then owns one head, the softmax statistics are
// per-lane scalars and the rescaling of O^T = V^T P needs no cross-lane traffic.
#include "nsa_common.hpp"
#include "../../include/nsa_hip.h"

#ifndef NSA_DECODE_TILES_PER_WAVE
#define NSA_DECODE_TILES_PER_WAVE 2     // measured at 32k context: 1 tile per wave 197 us (batch 32), 4 tiles 96 us (batch 1) against 187 / 90 us
#endif
#ifndef NSA_DECODE_WG_TARGET
#define NSA_DECODE_WG_TARGET 4096     // work-groups of one attend launch beyond which the key range is not split further (batch 32, 32k context: 2048 -> 197 us per step, 4096 and more -> 187 us)
#endif

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
  int sstride, lstride;              // row strides of the selection (idx / fmask) and of the logits output
  // Lengths read at run time, for a step replayed from a captured graph: dyn[0] = rows in the key / value caches before
  // this token, dyn[1] = compressed keys cached.  The fields above then hold capacities (the grid and the partial
  // records are sized for them) and resolve() replaces them inside the kernel.
  const int* dyn;
  int dyn_kind;                      // 1 compressed range, 2 selected blocks, 3 sliding window
  int window, per_block, smax;
  int cap_len, cap_nc;               // rows the key / value caches and the compressed caches hold: the counters are clamped to them
};

__device__ __forceinline__ void resolve(DecodePlan& P) {
  if (P.dyn == nullptr) return;
  // a caller that replays the step more often than the caches have rows must not make the kernels read or write past them
  const int kv_len = min(max(P.dyn[0], 0) + 1, P.cap_len), nc = min(max(P.dyn[1], 0), P.cap_nc);
  if (P.dyn_kind == 1) {
    P.count = nc;
    if (nc == 0) P.mem = 0;                            // no compressed key yet: the branch contributes nothing (NSA.py:401)
    P.tiles = ((P.mem + 31) >> 5) + ((nc + 31) >> 5);
  } else if (P.dyn_kind == 2) {
    P.kv_len = kv_len;
    P.S = min(P.smax, nc / P.per_block);
    P.tiles = (P.S + 1) * P.tps;
  } else {
    const int w = min(kv_len, P.window + 1);
    P.start = kv_len - w;
    P.count = w;
    P.tiles = (w + 31) >> 5;
  }
}

constexpr int kDecodeWaves = 2;      // waves per work-group; each stages its own K / V tile in LDS

struct DecodeTile {
  const __bf16 *kb, *vb;             // row 0 of the tile
  long ks, vs;                       // row strides
  int nvalid, lcol;                  // rows in use; column of row 0 in the logits row (-1: not written)
};

// tile t of unit (b, hk, ug) -> its rows; nvalid <= 0 for tiles with nothing to attend
__device__ __forceinline__ DecodeTile decode_tile(const DecodePlan& P, int D, int t, int b, int hk, int ug, const __bf16* k, const __bf16* v,
                                                  const __bf16* mem_k, const __bf16* mem_v, const void* idx, const unsigned char* fmask) {
  DecodeTile T;
  T.lcol = -1;
  if (P.mode == 0) {
    const int mem_tiles = (P.mem + 31) >> 5;
    if (t < mem_tiles) {
      T.kb = mem_k + ((long)hk * P.mem + 32 * t) * D;
      T.vb = mem_v + ((long)hk * P.mem + 32 * t) * D;
      T.ks = T.vs = D;
      T.nvalid = min(32, P.mem - 32 * t);
    } else {
      const int tt = t - mem_tiles;
      T.kb = k + b * P.sk[0] + hk * P.sk[1] + (long)(P.start + 32 * tt) * P.sk[2];
      T.vb = v + b * P.sv[0] + hk * P.sv[1] + (long)(P.start + 32 * tt) * P.sv[2];
      T.ks = P.sk[2]; T.vs = P.sv[2];
      T.nvalid = min(32, P.count - 32 * tt);
      T.lcol = 32 * tt;
    }
  } else {
    const int slot = t / P.tps, sub = t % P.tps;
    long blk;
    bool live = true;
    if (slot < P.S) {
      const long e = (long)ug * P.sstride + slot;
      const unsigned char fm = fmask[e];              // requested together with the index: one round trip, not two
      blk = P.idx64 ? reinterpret_cast<const long*>(idx)[e] : (long)reinterpret_cast<const int*>(idx)[e];
      live = (fm != 0) & (blk >= 0) & (blk * P.B < P.kv_len);
      if (!live) blk = 0;
    } else {
      blk = (P.kv_len - 1) / P.B;                     // the query's own block, up to itself
    }
    const long key0 = blk * P.B + 32 * sub;
    T.kb = k + b * P.sk[0] + hk * P.sk[1] + key0 * P.sk[2];
    T.vb = v + b * P.sv[0] + hk * P.sv[1] + key0 * P.sv[2];
    T.ks = P.sk[2]; T.vs = P.sv[2];
    T.nvalid = live ? (int)min((long)32, min((long)P.B - 32 * sub, (long)P.kv_len - key0)) : 0;
  }
  return T;
}

// One branch of a decode step: what a launch needs besides the grid.
struct AttendArgs {
  DecodePlan P;
  const __bf16 *q, *k, *v, *mem_k, *mem_v;
  const void* idx;
  const unsigned char* fmask;
  float* part;
  float* logits;
};

// Work-group (bx, blockIdx.y) of a branch: bx = index among the branch's split-K work-groups.
template <int D>
__device__ __forceinline__ void decode_attend_body(const AttendArgs& A, const int bx) {
  constexpr int KS = D / 16, DT = D / 32, RS = D + 8, RSV = D + 16;   // row reads want 4 banks per row, transpose loads 8
  constexpr int LPR = D / 8, RPI = 64 / LPR, NI = 32 / RPI;      // lanes per row, rows per load instruction, instructions per tile
  DecodePlan P = A.P;
  resolve(P);
  const __bf16* __restrict__ q = A.q;
  const __bf16* __restrict__ k = A.k;
  const __bf16* __restrict__ v = A.v;
  const __bf16* __restrict__ mem_k = A.mem_k;
  const __bf16* __restrict__ mem_v = A.mem_v;
  const void* __restrict__ idx = A.idx;
  const unsigned char* __restrict__ fmask = A.fmask;
  float* __restrict__ part = A.part;
  float* __restrict__ logits = A.logits;
  __shared__ __align__(16) __bf16 kv_s[kDecodeWaves][2][32 * RSV];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_ = lane & 31, h = lane >> 5;
  const int lr = lane / LPR, lc = lane % LPR;
  __bf16* k_s = kv_s[wave][0];
  __bf16* v_s = kv_s[wave][1];
  const int ug = blockIdx.y, b = ug / P.units, u = ug % P.units;
  const int hk = (P.units == P.hk) ? u : u / P.g;
  const int head0 = (P.units == P.hk) ? u * P.g : u;
  const int wid = bx * kDecodeWaves + wave, nw = P.nsplit * kDecodeWaves;

  bf16x8 Qf[KS];
  {
    const bool okq = n_ < P.gc;
    const __bf16* qp = q + b * P.sq[0] + (long)(head0 + (okq ? n_ : 0)) * P.sq[1] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) Qf[ks] = okq ? load8(qp + 16 * ks) : zero_frag();
  }
  const float sc = P.scale * kLog2e;

  float m = -INFINITY, l = 0.f;
  floatx16 Oa[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) Oa[dt] = zero_acc();

  // rows are fetched with whole-row coalesced loads (LPR lanes per row) one tile ahead of the
  // arithmetic, and turned into MFMA operands through the wave's private LDS tiles
  bf16x8 kr[NI], vr[NI];
  auto issue = [&](const DecodeTile& T) {
#pragma unroll
    for (int r = 0; r < NI; ++r) {
      const int row = RPI * r + lr;
      const long rc = row < T.nvalid ? row : 0;
      kr[r] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(T.kb + rc * T.ks + 8 * lc));      // every cached row is read once per step
      vr[r] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(T.vb + rc * T.vs + 8 * lc));
    }
  };
  auto next_tile = [&](int t, DecodeTile& T) {
    for (; t < P.tiles; t += nw) {
      T = decode_tile(P, D, t, b, hk, ug, k, v, mem_k, mem_v, idx, fmask);
      if (T.nvalid > 0) break;
    }
    return t;
  };

  DecodeTile T, Tn;
  int t = next_tile(wid, T);
  if (t < P.tiles) issue(T);
  while (t < P.tiles) {
#pragma unroll
    for (int r = 0; r < NI; ++r) {
      *reinterpret_cast<bf16x8*>(k_s + (RPI * r + lr) * RS + 8 * lc) = kr[r];
      *reinterpret_cast<bf16x8*>(v_s + (RPI * r + lr) * RSV + 8 * lc) = vr[r];
    }
    const int tn = next_tile(t + nw, Tn);
    if (tn < P.tiles) issue(Tn);
    __builtin_amdgcn_sched_barrier(0);

    floatx16 Sa = zero_acc();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) Sa = mfma32(lds_row_operand(k_s, RS, ks, lane), Qf[ks], Sa);

    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int kl = 8 * (i >> 2) + 4 * h + (i & 3);
      if (logits != nullptr && T.lcol >= 0 && n_ < P.gc && kl < T.nvalid)
        logits[((long)b * P.hk * P.g + head0 + n_) * P.lstride + T.lcol + kl] = Sa[i] * P.scale;
      const float s = kl < T.nvalid ? Sa[i] * sc : -INFINITY;
      Sa[i] = s;
      mx = fmaxf(mx, s);
    }
    mx = halves_max(mx);
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
      for (int u2 = 0; u2 < 2; ++u2)
        Oa[dt] = mfma32(lds_transposed_operand(v_s, RSV, 16 * u2, 32 * dt, lane), pack8(Sa, 8 * u2), Oa[dt]);
    }
    t = tn;
    T = Tn;
  }
  l = halves_sum(l);

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

template <int D>
__global__ __launch_bounds__(64 * kDecodeWaves) __attribute__((amdgpu_waves_per_eu(2))) void decode_attend_kernel(const AttendArgs A) {
  decode_attend_body<D>(A, blockIdx.x);
}

// Two independent branches of a step (the compressed keys and the sliding window) in one launch: the work-groups of the
// second follow those of the first along x, so the short branch fills the chip while the long one drains.
template <int D>
__global__ __launch_bounds__(64 * kDecodeWaves) __attribute__((amdgpu_waves_per_eu(2))) void decode_attend_pair_kernel(const AttendArgs A, const AttendArgs B) {
  if ((int)blockIdx.x < A.P.nsplit) decode_attend_body<D>(A, blockIdx.x);
  else decode_attend_body<D>(B, blockIdx.x - A.P.nsplit);
}

// Log-sum-exp merge of the split-K partials of head (b, head) of one branch by a work-group of D threads: the
// partials' maxima and sums are read by one thread each and reduced through LDS, then thread f accumulates
// feature f over the partials that carry weight (loads independent of each other, so they overlap).
constexpr int kMaxParts = 64 * kDecodeWaves;

template <int D>
__device__ __forceinline__ float merge_head_partials(const DecodePlan& P, const float* __restrict__ part, int b, int head, int f,
                                                     float* w_s, float* red_s) {
  const int u = (P.units == P.hk) ? head / P.g : head, gi = (P.units == P.hk) ? head % P.g : 0;
  const float* base = part + (long)(b * P.units + u) * P.nparts * P.rec;
  const int om = P.gc * D + gi, ol = om + P.gc;
  constexpr int PT = (kMaxParts + D - 1) / D;          // partials per thread
  float mp[PT], lp[PT];
  float M = -INFINITY;
#pragma unroll
  for (int r = 0; r < PT; ++r) {
    const int p = f + r * D;
    mp[r] = p < P.nparts ? base[(long)p * P.rec + om] : -INFINITY;
    lp[r] = p < P.nparts ? base[(long)p * P.rec + ol] : 0.f;
    M = fmaxf(M, mp[r]);
  }
  auto block_reduce = [&](float v, bool is_max) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float t = __shfl_xor(v, o, 64);
      v = is_max ? fmaxf(v, t) : v + t;
    }
    if (D > 64) {
      __syncthreads();
      if ((f & 63) == 0) red_s[f >> 6] = v;
      __syncthreads();
      v = red_s[0];
#pragma unroll
      for (int w = 1; w < D / 64; ++w) v = is_max ? fmaxf(v, red_s[w]) : v + red_s[w];
    }
    return v;
  };
  M = block_reduce(M, true);
  const bool any = M > -INFINITY;                      // false: no wave saw a key
  float L = 0.f;
  __syncthreads();                                     // w_s may still be read for the previous branch
#pragma unroll
  for (int r = 0; r < PT; ++r) {
    const int p = f + r * D;
    const float w = any ? fast_exp2(mp[r] - M) : 0.f;  // exp2(-inf) = 0 for waves that saw no key
    if (p < P.nparts) w_s[p] = w;
    L += w * lp[r];
  }
  L = block_reduce(L, false);
  __syncthreads();
  float acc = 0.f;
  // every wave wrote a finite record (zeros when it saw no key), so the loads need no guard and overlap
#pragma unroll 8
  for (int p = 0; p < P.nparts; ++p) acc += w_s[p] * base[(long)p * P.rec + gi * D + f];
  return L > 0.f ? acc / L : 0.f;
}

// one work-group per query head, one thread per feature
template <int D>
__global__ __launch_bounds__(D) void decode_merge_kernel(const DecodePlan P, const float* __restrict__ part, __bf16* __restrict__ out) {
  __shared__ float w_s[kMaxParts], red_s[4];
  const int hq = P.hk * P.g;
  const int bh = blockIdx.x, b = bh / hq, head = bh % hq;
  out[(long)bh * D + threadIdx.x] = (__bf16)merge_head_partials<D>(P, part, b, head, threadIdx.x, w_s, red_s);
}

// Merge of the three branches' partials, sigmoid strategy gate and head merge in one pass
// (NSA.py:534-545): out[b, head*D + f] = sum_s sigmoid(logit[b, 3*head + s]) * branch_s.
// A branch without a workspace (no compressed key cached yet) contributes zero.  `advance` (optional): the step's
// position counter, incremented here once every attention kernel of the step has run.
struct CombineArgs {
  DecodePlan P[3];
  const float* part[3];
  int* advance;
  long gate_row;                 // elements between the gate logits of consecutive batch rows
  const __bf16* gate_bias;       // optional [3 * heads], added to the logits (a projection computed without its bias)
};

template <int D>
__global__ __launch_bounds__(D) void decode_combine_kernel(const CombineArgs A, const __bf16* __restrict__ gate_logits, __bf16* __restrict__ out) {
  __shared__ float w_s[kMaxParts], red_s[4];
  const int hq = A.P[0].hk * A.P[0].g;
  const int bh = blockIdx.x, b = bh / hq, head = bh % hq;
  float res = 0.f;
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    if (A.part[s] == nullptr) continue;
    // branch outputs are rounded to bf16 as when each is merged on its own
    const float o = (float)(__bf16)merge_head_partials<D>(A.P[s], A.part[s], b, head, threadIdx.x, w_s, red_s);
    float gl = (float)gate_logits[(long)b * A.gate_row + head * 3 + s];
    if (A.gate_bias != nullptr) gl += (float)A.gate_bias[head * 3 + s];
    res += o / (1.f + __expf(-gl));
  }
  out[(long)bh * D + threadIdx.x] = (__bf16)res;
  if (A.advance != nullptr && blockIdx.x == 0 && threadIdx.x == 0) A.advance[0] += 1;
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
  // split-K: about two tiles per wave, but no more work-groups than a few per CU
  int ns = (P.tiles + NSA_DECODE_TILES_PER_WAVE * kDecodeWaves - 1) / (NSA_DECODE_TILES_PER_WAVE * kDecodeWaves);
  const long cap = units >= NSA_DECODE_WG_TARGET ? 1 : NSA_DECODE_WG_TARGET / units;
  if (ns > cap) ns = (int)cap;
  if (ns > 64) ns = 64;
  if (ns < 1) ns = 1;
  P.nsplit = ns; P.nparts = ns * kDecodeWaves;
  P.rec = P.gc * P.d + ((2 * P.gc + 3) & ~3);
  P.sstride = P.S; P.lstride = P.count;
  return 0;
}

static int check_attend(const DecodePlan& P, const void* q, const void* k, const void* v, const void* mem_k, const void* mem_v,
                        const void* idx, const uint8_t* fmask, void* ws, size_t ws_bytes) {
  if (!q || !ws) return NSA_E_ARG;
  if (P.mode == 0 && ((P.count > 0 && (!k || !v)) || (P.mem > 0 && (!mem_k || !mem_v)))) return NSA_E_ARG;
  if (P.mode == 1 && (!k || !v || (P.S > 0 && (!idx || !fmask)))) return NSA_E_ARG;
  if (ws_bytes < (size_t)P.b * P.units * P.nparts * P.rec * sizeof(float)) return NSA_E_WORKSPACE;
  return 0;
}

static AttendArgs attend_args(const DecodePlan& P, const void* q, const void* k, const void* v, const void* mem_k, const void* mem_v,
                              const void* idx, const uint8_t* fmask, void* ws, float* logits) {
  return AttendArgs{P, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v, (const __bf16*)mem_k, (const __bf16*)mem_v, idx, fmask, (float*)ws, logits};
}

static int launch_attend(const DecodePlan& P, const void* q, const void* k, const void* v, const void* mem_k, const void* mem_v, const void* idx,
                         const uint8_t* fmask, void* ws, size_t ws_bytes, void* out, float* logits, void* stream) {
  if (int e = check_attend(P, q, k, v, mem_k, mem_v, idx, fmask, ws, ws_bytes)) return e;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(P.nsplit, P.b * P.units);
  const int heads = P.b * P.hk * P.g;
  const AttendArgs A = attend_args(P, q, k, v, mem_k, mem_v, idx, fmask, ws, logits);
  if (P.d == 64) {
    hipLaunchKernelGGL((decode_attend_kernel<64>), grid, dim3(64 * kDecodeWaves), 0, st, A);
    if (out) hipLaunchKernelGGL((decode_merge_kernel<64>), dim3(heads), dim3(64), 0, st, P, (const float*)ws, (__bf16*)out);
  } else {
    hipLaunchKernelGGL((decode_attend_kernel<128>), grid, dim3(64 * kDecodeWaves), 0, st, A);
    if (out) hipLaunchKernelGGL((decode_merge_kernel<128>), dim3(heads), dim3(128), 0, st, P, (const float*)ws, (__bf16*)out);
  }
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

// two range branches over the same (batch, kv head) units in one launch; partials only (merged later by the combine kernel)
static int launch_attend_pair(const AttendArgs& A, size_t wsa_bytes, const AttendArgs& B, size_t wsb_bytes, void* stream) {
  if (int e = check_attend(A.P, A.q, A.k, A.v, A.mem_k, A.mem_v, A.idx, A.fmask, A.part, wsa_bytes)) return e;
  if (int e = check_attend(B.P, B.q, B.k, B.v, B.mem_k, B.mem_v, B.idx, B.fmask, B.part, wsb_bytes)) return e;
  if (A.P.b * A.P.units != B.P.b * B.P.units || A.P.d != B.P.d) return NSA_E_ARG;
  const dim3 grid(A.P.nsplit + B.P.nsplit, A.P.b * A.P.units);
  hipStream_t st = (hipStream_t)stream;
  if (A.P.d == 64) hipLaunchKernelGGL((decode_attend_pair_kernel<64>), grid, dim3(64 * kDecodeWaves), 0, st, A, B);
  else hipLaunchKernelGGL((decode_attend_pair_kernel<128>), grid, dim3(64 * kDecodeWaves), 0, st, A, B);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

static int launch_combine(const DecodePlan* plans[3], const void* const ws[3], const void* gate_logits, int64_t gate_row, const void* gate_bias,
                          void* out, int* advance, void* stream) {
  if (!gate_logits || !out) return NSA_E_ARG;
  CombineArgs A;
  A.advance = advance;
  int ref = -1;
  for (int s = 0; s < 3; ++s) {
    A.part[s] = nullptr;
    A.P[s] = DecodePlan{};
    if (!ws[s]) continue;
    A.P[s] = *plans[s];
    A.part[s] = (const float*)ws[s];
    if (ref < 0) ref = s;
    else if (A.P[s].b != A.P[ref].b || A.P[s].hk != A.P[ref].hk || A.P[s].g != A.P[ref].g || A.P[s].d != A.P[ref].d) return NSA_E_ARG;
  }
  if (ref < 0) return NSA_E_ARG;
  if (ref != 0) A.P[0] = A.P[ref];         // the kernel reads the head counts from slot 0
  A.gate_row = gate_row > 0 ? (long)gate_row : 3L * A.P[ref].hk * A.P[ref].g;
  A.gate_bias = (const __bf16*)gate_bias;
  const int heads = A.P[ref].b * A.P[ref].hk * A.P[ref].g;
  hipStream_t st = (hipStream_t)stream;
  if (A.P[ref].d == 64)
    hipLaunchKernelGGL((decode_combine_kernel<64>), dim3(heads), dim3(64), 0, st, A, (const __bf16*)gate_logits, (__bf16*)out);
  else
    hipLaunchKernelGGL((decode_combine_kernel<128>), dim3(heads), dim3(128), 0, st, A, (const __bf16*)gate_logits, (__bf16*)out);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
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
  return launch_attend(P, q, k, v, mem_k, mem_v, idx, fmask, ws, ws_bytes, out, logits, stream);
}

// ------------------------------------------------------------------------------------------------------------
// nsa_decode_attend for callers that cannot allocate (a stream under graph capture, a serving loop that forbids
// hipMalloc): the split-K partials go to a fixed device array of this library instead of a caller workspace.
// Every GPU the library runs on holds its own copy of the array, at its own address, until the process ends; in
// host code the array's name is only a handle, so the address is looked up once per device with
// hipGetSymbolAddress and that pointer is what the kernels receive.  All calls on a GPU share the array: calls
// that overlap on one GPU (two streams, two threads) race.  Nothing has to be cleared between calls: every wave
// of the attend kernel writes its partial record (a neutral one when it has no tile) before the merge reads it.
#include <mutex>

namespace nsa {
constexpr size_t kNoAllocScratchBytes = NSA_DECODE_NOALLOC_SCRATCH_BYTES;
constexpr int kNoAllocMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
static void* g_scratch_ptr[kNoAllocMaxDevices];       // per device: device address of `scratch`
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kNoAllocMaxDevices) return NSA_E_UNSUPPORTED;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return NSA_E_ARG;
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}
}  // namespace nsa

extern "C" int nsa_decode_attend_noalloc(const nsa_decode_desc* dsc, const void* q, const void* k, const void* v, const void* mem_k,
                                         const void* mem_v, const void* idx, const uint8_t* fmask, void* out, float* logits, void* stream) {
  using namespace nsa;
  DecodePlan P;
  if (int e = make_decode_plan(dsc, P)) return e;
  if (!out) return NSA_E_ARG;                          // the partials are private to the library: the merged output is the result
  const size_t need = (size_t)P.b * P.units * P.nparts * P.rec * sizeof(float);
  if (need > kNoAllocScratchBytes) return NSA_E_WORKSPACE;
  void* ws = nullptr;
  if (int e = scratch_of_current_device(&ws)) return e;
  return launch_attend(P, q, k, v, mem_k, mem_v, idx, fmask, ws, kNoAllocScratchBytes, out, logits, stream);
}

extern "C" int nsa_decode_combine(const nsa_decode_desc* compressed, const void* ws_compressed, const nsa_decode_desc* selected,
                                  const void* ws_selected, const nsa_decode_desc* sliding, const void* ws_sliding,
                                  const void* gate_logits, void* out, void* stream) {
  using namespace nsa;
  const nsa_decode_desc* dsc[3] = {compressed, selected, sliding};
  const void* ws[3] = {ws_compressed, ws_selected, ws_sliding};
  DecodePlan P[3];
  const DecodePlan* pp[3] = {&P[0], &P[1], &P[2]};
  for (int s = 0; s < 3; ++s)
    if (ws[s])
      if (int e = make_decode_plan(dsc[s], P[s])) return e;
  return launch_combine(pp, ws, gate_logits, 0, nullptr, out, nullptr, stream);
}

// ---------------------------------------------------------------------------- whole step
// The attention part of one decode step as a single host call: prep, compressed branch, block
// selection, selected-block branch, sliding branch, merge + gate.  The launches are the same as
// through the separate entry points; what goes away is the host-side work between them, which
// at small batch is most of a step's time.

namespace nsa {

struct StepLayout {
  nsa_decode_desc c, f, s;
  int nb, k;                       // selection blocks available / selected this step
  int sel_units;                   // rows of idx per batch element
  size_t off_rq, off_wsc, off_wsf, off_wss, off_logits, off_idx, off_vals, off_fm, total;
  size_t wsc, wsf, wss;
};

static size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

static int make_step_layout(const nsa_decode_step_desc* d, StepLayout& L) {
  if (!d) return NSA_E_ARG;
  if (d->batch <= 0 || d->heads <= 0 || d->kv_heads <= 0 || d->heads % d->kv_heads) return NSA_E_ARG;
  if (d->pos < 0 || d->num_compressed < 0 || d->num_mem < 0 || d->per_block <= 0 || d->block <= 0 || d->num_sel < 0 || d->window < 0)
    return NSA_E_ARG;
  const int g = d->heads / d->kv_heads, kv_len = d->pos + 1;
  auto common = [&](nsa_decode_desc& x) {
    x = nsa_decode_desc{};
    x.batch = d->batch; x.kv_heads = d->kv_heads; x.group = g; x.dim_head = d->dim_head; x.scale = d->scale;
  };
  // compressed branch reads the un-rotated projection, the other two the rotated queries in the workspace
  common(L.c);
  L.c.mode = 0; L.c.start = 0; L.c.count = d->num_compressed; L.c.num_mem = d->num_compressed > 0 ? d->num_mem : 0;
  L.c.q_stride[0] = d->q_stride[0]; L.c.q_stride[1] = d->q_stride[1];
  for (int i = 0; i < 3; ++i) { L.c.k_stride[i] = d->ck_stride[i]; L.c.v_stride[i] = d->cv_stride[i]; }
  L.nb = d->num_compressed / d->per_block;
  L.k = d->num_sel < L.nb ? d->num_sel : L.nb;
  L.sel_units = d->share ? d->kv_heads : d->heads;
  common(L.f);
  L.f.mode = 1; L.f.block = d->block; L.f.num_sel = L.k; L.f.kv_len = kv_len; L.f.per_head_sel = (!d->share && g > 1) ? 1 : 0;
  L.f.idx_is_int64 = 0;
  common(L.s);
  L.s.mode = 0;
  const int w = kv_len < d->window + 1 ? kv_len : d->window + 1;
  L.s.start = kv_len - w; L.s.count = w; L.s.num_mem = 0;
  for (nsa_decode_desc* x : {&L.f, &L.s}) {
    x->q_stride[0] = (int64_t)d->heads * d->dim_head; x->q_stride[1] = d->dim_head;
    for (int i = 0; i < 3; ++i) { x->k_stride[i] = d->kc_stride[i]; x->v_stride[i] = d->vc_stride[i]; }
  }
  if (d->num_compressed > 0)
    if (int e = nsa_decode_workspace_bytes(&L.c, &L.wsc)) return e;
  if (d->num_compressed <= 0) L.wsc = 0;
  if (int e = nsa_decode_workspace_bytes(&L.f, &L.wsf)) return e;
  if (int e = nsa_decode_workspace_bytes(&L.s, &L.wss)) return e;
  size_t o = 0;
  L.off_rq = o;     o = up256(o + (size_t)d->batch * d->heads * d->dim_head * 2);
  L.off_wsc = o;    o = up256(o + L.wsc);
  L.off_wsf = o;    o = up256(o + L.wsf);
  L.off_wss = o;    o = up256(o + L.wss);
  L.off_logits = o; o = up256(o + (size_t)d->batch * d->heads * (d->num_compressed > 0 ? d->num_compressed : 1) * 4);
  const size_t sel = (size_t)d->batch * L.sel_units * (L.k > 0 ? L.k : 1);
  L.off_idx = o;    o = up256(o + sel * 4);
  L.off_vals = o;   o = up256(o + sel * 4);
  L.off_fm = o;     o = up256(o + sel);
  L.total = o;
  return 0;
}

}  // namespace nsa

extern "C" int nsa_decode_step_workspace_bytes(const nsa_decode_step_desc* desc, size_t* bytes, size_t* idx_offset, size_t* fmask_offset,
                                               int32_t* num_selected) {
  nsa::StepLayout L;
  if (int e = nsa::make_step_layout(desc, L)) return e;
  if (!bytes) return NSA_E_ARG;
  *bytes = L.total;
  if (idx_offset) *idx_offset = L.off_idx;
  if (fmask_offset) *fmask_offset = L.off_fm;
  if (num_selected) *num_selected = L.k;
  return 0;
}

extern "C" int nsa_decode_step(const nsa_decode_step_desc* d, const void* q, const void* k, const void* v, const float* freqs,
                               void* k_cache, void* v_cache, const void* ck_cache, const void* cv_cache, const void* mem_k,
                               const void* mem_v, void* k_run_row, void* v_run_row, const void* gate_logits, void* ws, size_t ws_bytes,
                               void* out, void* stream) {
  using namespace nsa;
  StepLayout L;
  if (int e = make_step_layout(d, L)) return e;
  if (!q || !k || !v || !freqs || !k_cache || !v_cache || !gate_logits || !ws || !out) return NSA_E_ARG;
  if (ws_bytes < L.total) return NSA_E_WORKSPACE;
  if (d->num_compressed > 0 && (!ck_cache || !cv_cache)) return NSA_E_ARG;
  char* w = (char*)ws;
  void* rq = w + L.off_rq;
  // row `pos` of the caches
  const int64_t krs[2] = {d->kc_stride[0], d->kc_stride[1]}, vrs[2] = {d->vc_stride[0], d->vc_stride[1]};
  __bf16* k_row = (__bf16*)k_cache + (int64_t)d->pos * d->kc_stride[2];
  __bf16* v_row = (__bf16*)v_cache + (int64_t)d->pos * d->vc_stride[2];
  if (int e = nsa_decode_prep(q, d->q_stride, k, d->k_stride, v, d->v_stride, d->batch, d->heads, d->kv_heads, d->dim_head, freqs, d->pos, rq,
                              k_row, krs, v_row, vrs, k_run_row, k_run_row ? d->krun_stride : nullptr, v_run_row,
                              v_run_row ? d->vrun_stride : nullptr, stream))
    return e;
  const bool has_c = d->num_compressed > 0;
  float* logits = (float*)(w + L.off_logits);
  // the compressed range and the sliding window are independent of each other: one launch for both
  DecodePlan Pc_{}, Ps_;
  if (int e = make_decode_plan(&L.s, Ps_)) return e;
  if (has_c) {
    if (int e = make_decode_plan(&L.c, Pc_)) return e;
    if (int e = launch_attend_pair(attend_args(Pc_, q, ck_cache, cv_cache, mem_k, mem_v, nullptr, nullptr, w + L.off_wsc, logits), L.wsc,
                                   attend_args(Ps_, rq, k_cache, v_cache, nullptr, nullptr, nullptr, nullptr, w + L.off_wss, nullptr), L.wss, stream))
      return e;
  } else if (int e = launch_attend(Ps_, rq, k_cache, v_cache, nullptr, nullptr, nullptr, nullptr, w + L.off_wss, L.wss, nullptr, nullptr, stream)) {
    return e;
  }
  int32_t* idx = (int32_t*)(w + L.off_idx);
  uint8_t* fm = (uint8_t*)(w + L.off_fm);
  if (L.k > 0)
    if (int e = nsa_decode_topk(logits, d->batch, d->kv_heads, d->heads / d->kv_heads, d->num_compressed, d->per_block, d->share, L.k, idx,
                                (float*)(w + L.off_vals), fm, stream))
      return e;
  if (int e = nsa_decode_attend(&L.f, rq, k_cache, v_cache, nullptr, nullptr, L.k > 0 ? idx : nullptr, L.k > 0 ? fm : nullptr, w + L.off_wsf,
                                L.wsf, nullptr, nullptr, stream))
    return e;
  return nsa_decode_combine(has_c ? &L.c : nullptr, has_c ? w + L.off_wsc : nullptr, &L.f, w + L.off_wsf, &L.s, w + L.off_wss, gate_logits, out,
                            stream);
}

// Declared in nsa_rope.hip / nsa_topk.hip: the prep and top-k launches with lengths read from device memory.
namespace nsa {
int decode_prep_dyn(const void* q, const int64_t* q_stride, const void* k, const int64_t* k_stride, const void* v, const int64_t* v_stride,
                    int32_t batch, int32_t heads, int32_t kv_heads, int32_t dim_head, const float* freqs, void* rq, void* k_cache,
                    const int64_t* kc_stride, void* v_cache, const int64_t* vc_stride, void* k_run, const int64_t* krun_stride, void* v_run,
                    const int64_t* vrun_stride, int32_t ring, int32_t last_pos, const int32_t* state, void* stream);
int decode_topk_launch(const float* logits, int32_t batch, int32_t kv_heads, int32_t group, int32_t num_compressed, int32_t per_block,
                       int32_t share, int32_t k, int32_t* idx, float* vals, uint8_t* fmask, const int32_t* state, void* stream);
}  // namespace nsa

extern "C" int nsa_decode_step_dyn(const nsa_decode_step_desc* cap, int32_t* state, const void* q, const void* k, const void* v,
                                   const float* freqs, void* k_cache, void* v_cache, const void* ck_cache, const void* cv_cache,
                                   const void* mem_k, const void* mem_v, void* k_run, void* v_run, int64_t krun_row_stride,
                                   int64_t vrun_row_stride, int32_t run_ring, const void* gate_logits, int64_t gate_row_stride,
                                   const void* gate_bias, void* ws, size_t ws_bytes, void* out, int32_t advance, void* stream) {
  using namespace nsa;
  StepLayout L;
  if (int e = make_step_layout(cap, L)) return e;
  if (!state || !q || !k || !v || !freqs || !k_cache || !v_cache || !gate_logits || !ws || !out) return NSA_E_ARG;
  if (ws_bytes < L.total) return NSA_E_WORKSPACE;
  const bool has_c = cap->num_compressed > 0;
  if (has_c && (!ck_cache || !cv_cache)) return NSA_E_ARG;
  DecodePlan Pc{}, Pf, Ps;
  if (has_c)
    if (int e = make_decode_plan(&L.c, Pc)) return e;
  if (int e = make_decode_plan(&L.f, Pf)) return e;
  if (int e = make_decode_plan(&L.s, Ps)) return e;
  int kind = 1;
  for (DecodePlan* P : {&Pc, &Pf, &Ps}) {
    P->dyn = state; P->dyn_kind = kind++;
    P->window = cap->window; P->per_block = cap->per_block; P->smax = L.k;
    P->cap_len = cap->pos + 1; P->cap_nc = cap->num_compressed;
  }
  Pc.lstride = cap->num_compressed;
  Pf.sstride = L.k;

  char* w = (char*)ws;
  void* rq = w + L.off_rq;
  const int64_t krun_s[3] = {cap->krun_stride[0], cap->krun_stride[1], krun_row_stride};
  const int64_t vrun_s[3] = {cap->vrun_stride[0], cap->vrun_stride[1], vrun_row_stride};
  if (int e = decode_prep_dyn(q, cap->q_stride, k, cap->k_stride, v, cap->v_stride, cap->batch, cap->heads, cap->kv_heads, cap->dim_head, freqs, rq,
                              k_cache, cap->kc_stride, v_cache, cap->vc_stride, k_run, krun_s, v_run, vrun_s, run_ring, cap->pos, state, stream))
    return e;
  float* logits = (float*)(w + L.off_logits);
  if (has_c) {
    if (int e = launch_attend_pair(attend_args(Pc, q, ck_cache, cv_cache, mem_k, mem_v, nullptr, nullptr, w + L.off_wsc, logits), L.wsc,
                                   attend_args(Ps, rq, k_cache, v_cache, nullptr, nullptr, nullptr, nullptr, w + L.off_wss, nullptr), L.wss, stream))
      return e;
  } else if (int e = launch_attend(Ps, rq, k_cache, v_cache, nullptr, nullptr, nullptr, nullptr, w + L.off_wss, L.wss, nullptr, nullptr, stream)) {
    return e;
  }
  int32_t* idx = (int32_t*)(w + L.off_idx);
  uint8_t* fm = (uint8_t*)(w + L.off_fm);
  if (L.k > 0)
    if (int e = decode_topk_launch(logits, cap->batch, cap->kv_heads, cap->heads / cap->kv_heads, cap->num_compressed, cap->per_block, cap->share,
                                   L.k, idx, (float*)(w + L.off_vals), fm, state, stream))
      return e;
  if (int e = launch_attend(Pf, rq, k_cache, v_cache, nullptr, nullptr, L.k > 0 ? idx : nullptr, L.k > 0 ? fm : nullptr, w + L.off_wsf, L.wsf,
                            nullptr, nullptr, stream))
    return e;
  const DecodePlan* pp[3] = {&Pc, &Pf, &Ps};
  const void* wsp[3] = {has_c ? w + L.off_wsc : nullptr, w + L.off_wsf, w + L.off_wss};
  if (int e = launch_combine(pp, wsp, gate_logits, gate_row_stride, gate_bias, out, advance ? state : nullptr, stream)) return e;
  return 0;
}
