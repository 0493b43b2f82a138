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
// Forward and dQ are query-stationary: a work-group of 4 waves owns 128 rows (128/G consecutive
// queries x the G heads of one kv group, so the group shares every K/V tile), each wave 32 rows.
// 64-key K/V tiles are copied straight from global memory into swizzled LDS tiles one tile ahead
// (global_load_lds_dwordx4: no staging registers, two buffers, one barrier per tile) and read
// back as MFMA operands: row operands with 16-byte LDS reads, transposed operands (V^T, K^T)
// with the gfx950 LDS transpose load.  dK/dV is key-stationary: two waves own a 64-key tile
// (32 keys each) and stream the query rows that can see it through registers and padded LDS
// tiles, like the dK/dV walk of the block-selection kernels.
#include <type_traits>
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
    r.hi = P.causal ? min(P.nkeys - 1, (P.st_sh >= 0 ? (i >> P.st_sh) : i / P.st) - 1) : P.nkeys - 1;
  }
  return r;
}

constexpr int kBK = 64;          // keys per K/V tile

// maximum / sum over the 16 lanes of a DPP row, left in every lane of the row
__device__ __forceinline__ float row16_bcast_max(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xF, 0xF, false));
  };
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0xB1>{}));     // quad_perm [1,0,3,2]
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x4E>{}));     // quad_perm [2,3,0,1]
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x141>{}));    // row_half_mirror
  v = fmaxf(v, dpp(v, std::integral_constant<int, 0x140>{}));    // row_mirror
  return v;
}
__device__ __forceinline__ float row16_bcast_sum(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xF, 0xF, false));
  };
  v += dpp(v, std::integral_constant<int, 0xB1>{});
  v += dpp(v, std::integral_constant<int, 0x4E>{});
  v += dpp(v, std::integral_constant<int, 0x141>{});
  v += dpp(v, std::integral_constant<int, 0x140>{});
  return v;
}

// Work-group ids go round-robin over the 8 XCDs, each with its own L2.  Work items that re-read each other's rows
// (neighbouring query tiles of a sliding window, neighbouring key tiles of its backward, the key tiles of one query
// chunk) must therefore not be neighbours in work-group id: item v = (x % 8) * ceil(count / 8) + x / 8 gives every
// XCD one contiguous range of items, walked in order.  Measured on the sliding-window kernels at seq 32k (window 512):
// with ids taken as they come every tile fetched its rows from HBM (forward 2.6 GB for 0.4 GB of operands).
__device__ __forceinline__ int xcd_contiguous(int x, int count) {
  const int per = (count + 7) >> 3;
  return (x & 7) * per + (x >> 3);
}
static inline unsigned xcd_grid_for(int count) { return 8u * (unsigned)((count + 7) >> 3); }

// Key tiles walked by a query tile: t = -1 is the memory tile (stride mode), then 64-key tiles
// t_lo .. t_hi of the interval union.
struct TileWalk {
  int t_first, t_lo, t_hi;
  __device__ __forceinline__ int next(int t) const { return t < 0 ? t_lo : t + 1; }
};

__device__ __forceinline__ TileWalk make_walk(const DensePlan& P, int i_first, int i_last) {
  TileWalk w;
  const int lo = visible_range(P, i_first).lo, hi = visible_range(P, i_last).hi;
  w.t_lo = lo / kBK;
  w.t_hi = hi >= 0 ? hi / kBK : -1;
  w.t_first = P.mem > 0 ? -1 : w.t_lo;
  return w;
}

#ifndef NSA_DQ_AHK
#define NSA_DQ_AHK 3
#endif
#ifndef NSA_DQ_AHT
#define NSA_DQ_AHT 1
#endif
#ifndef NSA_FWD_AHK
#define NSA_FWD_AHK 3
#endif
#ifndef NSA_FWD_AHV
#define NSA_FWD_AHV 2
#endif
// ------------------------------------------------------------------------------- forward
// One candidate inserted into the running selections of the four queries a wave serves at a time (16 lanes per query, lane s
// of a group holds the s-th best block so far: logit L, block I; descending, equal logits in the order they came, i.e. lower
// block first).  c is the candidate's logit for the lane's query, ci its block.  Entries at least as large stay, the first
// smaller one takes the candidate, the rest move one lane up (DPP row shift inside the 16 lanes); a candidate no larger
// than the last entry changes nothing.
__device__ __forceinline__ void topk_insert(float& L, int& I, float c, int ci) {
  const float Lp = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0x7f800000, __builtin_bit_cast(int, L), 0x111, 0xF, 0xF, false));   // row_shr:1, lane 0: +inf
  const int Ip = __builtin_amdgcn_update_dpp(0, I, 0x111, 0xF, 0xF, false);
  const bool keep = L >= c, keepp = Lp >= c;
  L = keep ? L : (keepp ? c : Lp);
  I = keep ? I : (keepp ? ci : Ip);
}

// NPF = selection block / compress stride when the importance logits are wanted, 0 otherwise.
// TK: the block selection itself is made here (NSA.py:693-721 on the logits of NSA.py:652-691): instead of writing the
// logits out, every query keeps the P.topk <= 16 best blocks seen so far while the key tiles stream by, and the kernel ends
// by writing their indices (descending logit, ties to the lower block) and the slot mask `probability > 1e-10`.
template <int D, int NPF, bool TK = false>
__global__ __launch_bounds__(256, 2) void dense_fwd_kernel(const DensePlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                        const __bf16* __restrict__ v, __bf16* __restrict__ out, float* __restrict__ lse,
                                                        float* __restrict__ pooled, int* __restrict__ tk_idx, uint8_t* __restrict__ tk_mask) {
  constexpr int KS = D / 16, DT = D / 32, TILE = kBK * D;
  constexpr int TKP = TK ? 4 : 1;              // up to 16 queries per wave, four at a time
  float tkL[TKP];
  int tkI[TKP];
#pragma unroll
  for (int p2 = 0; p2 < TKP; ++p2) { tkL[p2] = -INFINITY; tkI[p2] = threadIdx.x & 15; }
  // two swizzled tiles each for K and V, filled by asynchronous copies: tile t+1 lands while tile t is being used
  __shared__ __align__(1024) __bf16 k_s[2 * TILE];
  __shared__ __align__(1024) __bf16 v_s[2 * TILE];
  constexpr bool POOL = NPF > 0;
  constexpr int NBT = POOL ? kBK / (POOL ? NPF : 1) : 1;        // fine blocks per key tile
  __shared__ __align__(16) float pool_s[POOL ? 4 * 32 * NBT : 1];   // per wave: [rows or queries of the tile][fine blocks of the key tile]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n_ = lane & 31, h = lane >> 5;
  const int bh = blockIdx.y, b = bh / P.hkv, hk = bh % P.hkv;
  const int ppt = 32 >> P.lg;                       // queries per wave tile
  // band mode: equal work per tile, neighbouring tiles share most of their window -> one XCD per contiguous range of tiles;
  // stride mode keeps the round-robin order (the compressed keys fit every L2), causal from the last tile down: work grows
  // with the position, and the longest work-groups should not be the last to start
  const int qtiles = (P.n + 4 * ppt - 1) / (4 * ppt);
  const int xt = P.mode == 0 ? xcd_contiguous(blockIdx.x, qtiles) : (P.causal ? qtiles - 1 - (int)blockIdx.x : (int)blockIdx.x);
  if (xt >= qtiles) return;
  const int q0 = xt * 4 * ppt;                      // first query of the work-group
  const int i0 = q0 + wave * ppt;
  const int pq = n_ >> P.lg, g = n_ & (P.g - 1);
  const bool valid = i0 + pq < P.n;
  const int i = min(i0 + pq, P.n - 1);
  const int hq = hk * P.g + g;

  bf16x8 Qf[KS];
  {
    const __bf16* qp = q + b * P.sq[0] + (long)hq * P.sq[1] + (long)i * P.sq[2] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) Qf[ks] = load8(qp + 16 * ks);
  }
  const Interval me = visible_range(P, i);
  const TileWalk walk = make_walk(P, q0, min(P.n - 1, q0 + 4 * ppt - 1));
  // this wave's own reach (its tiles are a subset of the work-group's)
  const int my_hi = visible_range(P, min(P.n - 1, i0 + ppt - 1)).hi, my_lo = visible_range(P, min(i0, P.n - 1)).lo;
  // keys in [all_lo, all_hi] are visible to every row of this wave: tiles inside need no per-element mask
  const int all_hi = visible_range(P, min(i0, P.n - 1)).hi, all_lo = visible_range(P, min(P.n - 1, i0 + ppt - 1)).lo;
  const float sc = P.scale * kLog2e;

  float m = -INFINITY, l = 0.f;
  floatx16 Oa[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) Oa[dt] = zero_acc();

  const __bf16* kbase = k + b * P.sk[0] + hk * P.sk[1];
  const __bf16* vbase = v + b * P.sv[0] + hk * P.sv[1];
  TileDma<D, 256> kdma, vdma;
  kdma.init(tid, P.sk[2], k_s);
  vdma.init(tid, P.sv[2], v_s);
  auto load_tile = [&](int t, int into) {
    const long first = t < 0 ? 0 : (long)P.mem + (long)t * kBK;
    const long limit = t < 0 ? P.mem : (long)P.mem + P.nkeys;
    kdma.issue(kbase, first, limit, into * TILE * 2);
    vdma.issue(vbase, first, limit, into * TILE * 2);
  };
  int t = walk.t_first, buf = 0;
  if (t <= walk.t_hi || t < 0) load_tile(t, 0);      // (a memory tile is always walked: every copy issued is waited for)

  for (; t <= walk.t_hi; t = walk.next(t), buf ^= 1) {
    // one barrier per tile: behind it this wave's and every other wave's part of tile t has landed, and all waves are done
    // with tile t-1, whose buffer the copy of tile t+1 may now overwrite
    wait_all_loads();
    __syncthreads();
    const int tn = walk.next(t);
    // The copy of the next tile: between the MFMAs of this tile's scores where it can be (a copy instruction holds the
    // wave's issue for about as long as two MFMAs run), up front for a tile that needs the clamped path or a wave with no
    // scores to compute
    const long nfirst = (long)P.mem + (long)tn * kBK;                    // (the memory tile is never a next tile)
    const bool more = tn <= walk.t_hi, spread = more && nfirst + kBK <= (long)P.mem + P.nkeys;
    const __bf16* ktb = kbase + nfirst * P.sk[2];
    const __bf16* vtb = vbase + nfirst * P.sv[2];
    const unsigned noff = (buf ^ 1) * TILE * 2;
    const __bf16* kt_s = k_s + buf * TILE;
    const __bf16* vt_s = v_s + buf * TILE;
    const bool memtile = t < 0;
    const int kb0 = memtile ? 0 : t * kBK;
    // skip tiles outside this wave's reach (the barriers below are still executed)
    const bool active = memtile || (kb0 <= my_hi && kb0 + kBK - 1 >= my_lo);
    if (!active || !spread) {
      if (more) load_tile(tn, buf ^ 1);
    }
    if (active) {
      floatx16 Sa[2];
      Sa[0] = zero_acc();
      Sa[1] = zero_acc();
      auto scores = [&](auto copying) {
        constexpr int RN = TileDma<D, 256>::ROUNDS;
        static_assert(2 * RN <= KS, "one copy round after every second MFMA");
        operands_ahead<2 * KS, NSA_FWD_AHK>([&](int i2) { return lds_row_operand_swz<D>(kt_s + 32 * (i2 / KS) * D, i2 % KS, lane); },
                                            [&](int i2, bf16x8 a) {
                                              Sa[i2 / KS] = mfma32(a, Qf[i2 % KS], Sa[i2 / KS]);
                                              if (decltype(copying)::value && (i2 & 1) && (i2 >> 1) < 2 * RN) {
                                                if ((i2 >> 1) < RN) kdma.round_full(ktb, noff, i2 >> 1);
                                                else vdma.round_full(vtb, noff, (i2 >> 1) - RN);
                                              }
                                            });
      };
      // (two copies of the score products rather than copies under an execution mask: measured faster where the registers allow it)
      if (spread) scores(std::true_type{});
      else scores(std::false_type{});
      const int klo = memtile ? 0 : me.lo, khi = memtile ? P.mem - 1 : me.hi;
      floatx16 Sraw[2];
      if (POOL) { Sraw[0] = Sa[0]; Sraw[1] = Sa[1]; }
      float tmax = -INFINITY;
      auto scale_scores = [&](auto masked) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i2 = 0; i2 < 16; ++i2) {
            const int key = kb0 + 32 * kt + 8 * (i2 >> 2) + 4 * h + (i2 & 3);
            // raw scores: the (positive) scale is folded into the exponent's multiply-add below, the maximum is taken raw
            const float s = (!decltype(masked)::value || ((key >= klo) & (key <= khi))) ? Sa[kt][i2] : -INFINITY;
            Sa[kt][i2] = s;
            tmax = fmaxf(tmax, s);
          }
      };
      const bool plain = !memtile && kb0 >= all_lo && kb0 + kBK - 1 <= all_hi;      // wave-uniform
      if (plain) scale_scores(std::false_type{});
      else scale_scores(std::true_type{});

      if (POOL && !memtile) {
        // Block-importance logits of this 64-key tile: sum the raw logits over the npf keys of a fine block (in registers /
        // one exchange between the lane halves) and over the G heads of the group (adjacent lanes: DPP quad permutes for
        // G <= 4), stage the sums in LDS and write them with coalesced stores; visibility is index arithmetic at store time.
        // One straight-line variant per way of summing heads, chosen by one wave-uniform switch per tile: with the choice
        // made value by value inside, the compiler threaded a dozen scalar branches through every half tile.
        // HS = 0: one row per head (no sharing, or groups of one head); 2 / 4: shared, group of 2 / 4; 1: shared, any other
        auto pool = [&](auto hs) {
          constexpr int HS = decltype(hs)::value;
          constexpr bool SH = HS != 0;
          constexpr int npf = POOL ? NPF : 1, nbt = NBT;
          float* pw = pool_s + wave * (32 * nbt);
          const int prow_local = SH ? pq : n_;           // query inside the wave tile (shared) or row of the wave tile (per head)
          const bool mine = (npf < 8 || h == 0) && (!SH || g == 0);
#pragma unroll
          for (int kt = 0; kt < 2; ++kt) {
            float grp[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) grp[a] = 0.f;
            if (npf >= 4) {
#pragma unroll
              for (int a = 0; a < 4; ++a) grp[a] = (Sraw[kt][4 * a] + Sraw[kt][4 * a + 1]) + (Sraw[kt][4 * a + 2] + Sraw[kt][4 * a + 3]);
              if (npf >= 8) {
#pragma unroll
                for (int a = 0; a < 4; ++a) grp[a] = halves_sum(grp[a]);
              }
              if (npf == 16) { grp[0] += grp[1]; grp[2] += grp[3]; }
              if (npf == 32) { grp[0] = (grp[0] + grp[1]) + (grp[2] + grp[3]); }
            }
            // the distinct sums of this 32-key half
            constexpr int NV = npf == 1 ? 16 : npf == 2 ? 8 : npf <= 8 ? 4 : npf == 16 ? 2 : 1;
            float val[NV];
            int koff[NV];
#pragma unroll
            for (int vi = 0; vi < NV; ++vi) {
              if (npf == 1) { val[vi] = Sraw[kt][vi]; koff[vi] = 8 * (vi >> 2) + 4 * h + (vi & 3); }
              else if (npf == 2) { val[vi] = Sraw[kt][2 * vi] + Sraw[kt][2 * vi + 1]; koff[vi] = 8 * (vi >> 1) + 4 * h + 2 * (vi & 1); }
              else if (npf == 4) { val[vi] = grp[vi]; koff[vi] = 8 * vi + 4 * h; }
              else if (npf == 8) { val[vi] = grp[vi]; koff[vi] = 8 * vi; }
              else if (npf == 16) { val[vi] = grp[2 * vi]; koff[vi] = 16 * vi; }
              else { val[vi] = grp[0]; koff[vi] = 0; }
            }
            if (HS == 2 || HS == 4) {
#pragma unroll
              for (int vi = 0; vi < NV; ++vi) val[vi] += dpp_quad_xor1(val[vi]);
            }
            if (HS == 4) {
#pragma unroll
              for (int vi = 0; vi < NV; ++vi) val[vi] += dpp_quad_xor2(val[vi]);
            }
            if (HS == 1) {
              for (int mk = 1; mk < P.g; mk <<= 1) {
#pragma unroll
                for (int vi = 0; vi < NV; ++vi) val[vi] += __shfl_xor(val[vi], mk, 64);
              }
            }
            if (TK) {
              // the staged values are the final logits: scaled, -inf where the block cannot be selected
              const float norm_t = P.scale / (float)(npf * (SH ? P.g : 1));
              const int jbt = kb0 / npf, qi_t = i0 + prow_local;
              const bool all_vis = P.causal && plain && i0 + ppt <= P.n && jbt + nbt <= P.nb;      // wave-uniform, as `direct` below
#pragma unroll
              for (int vi = 0; vi < NV; ++vi) {
                float x = val[vi] * norm_t;            // (a NaN logit never compares greater: it is not selected)
                if (!all_vis) {
                  const int jblk = jbt + (32 * kt + koff[vi]) / npf;
                  const int blo = jblk * P.B, bhi = blo + P.B;
                  const bool own = (blo <= qi_t) & (qi_t < bhi);
                  const bool vis = (!P.causal | (bhi <= qi_t)) & !(P.mask_own & own) & (jblk < P.nb) & (qi_t < P.n);
                  x = vis ? x : -INFINITY;
                }
                val[vi] = x;
              }
            }
            if (mine) {
#pragma unroll
              for (int vi = 0; vi < NV; ++vi) pw[prow_local * nbt + (32 * kt + koff[vi]) / npf] = val[vi];
            }
          }
          __builtin_amdgcn_wave_barrier();
          const int rows_here = SH ? ppt : 32;
          const float norm = P.scale / (float)(npf * (SH ? P.g : 1));
          const int jb0 = kb0 / npf;
          if (TK) {
            // Four queries at a time, 16 lanes each.  A lane reads all candidates of its query (broadcast reads) into
            // registers; one of them is its own to test against the query's current last entry (read from the group's lane
            // 15: a lower bound of the threshold once inserts have happened, which only lets a no-op insert through), the
            // ballot says which candidate positions have a taker in any of the four queries, and only those run the insert.
            constexpr int CAND = nbt < 16 ? nbt : 16, RDS = nbt / CAND;
            const int sub = lane & 15, rgrp = lane >> 4;
            // (the reads of all groups of four first, then the tests, then the inserts: one LDS round trip for the lot)
            float own_c[TKP][RDS], thr[TKP];
            const float* prow[TKP];
#pragma unroll
            for (int p2 = 0; p2 < TKP; ++p2) {
              prow[p2] = pw + min(4 * p2 + rgrp, rows_here - 1) * nbt;
              if (4 * p2 < rows_here) {
#pragma unroll
                for (int rd = 0; rd < RDS; ++rd) own_c[p2][rd] = prow[p2][rd * CAND + (sub < CAND ? sub : 0)];
                // the group's last entry, from its lane 15 (swizzle inside 32 lanes: source lane = (lane & 16) | 15)
                thr[p2] = __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, tkL[p2]), 0x1F0));
              }
            }
#pragma unroll
            for (int p2 = 0; p2 < TKP; ++p2) {
              if (4 * p2 < rows_here) {
                const bool rlive = 4 * p2 + rgrp < rows_here;
#pragma unroll
                for (int rd = 0; rd < RDS; ++rd) {
                  // (with several rounds per tile the threshold of the first serves them all: a lower bound lets no-ops through)
                  const unsigned long long pend = __ballot(rlive & (sub < CAND) & (own_c[p2][rd] > thr[p2]));
                  const unsigned m16 = (unsigned)(pend | (pend >> 16) | (pend >> 32) | (pend >> 48)) & 0xffffu;
                  if (m16) {
                    float c[CAND];
                    if (CAND >= 4) {
#pragma unroll
                      for (int j4 = 0; j4 < CAND / 4; ++j4) {
                        const floatx4 t4 = *reinterpret_cast<const floatx4*>(prow[p2] + rd * CAND + 4 * j4);
#pragma unroll
                        for (int e = 0; e < 4; ++e) c[4 * j4 + e] = t4[e];
                      }
                    } else {
#pragma unroll
                      for (int j = 0; j < CAND; ++j) c[j] = prow[p2][rd * CAND + j];
                    }
                    // positions four at a time: late in a walk most groups of four have no taker
#pragma unroll
                    for (int j4 = 0; j4 < (CAND + 3) / 4; ++j4) {
                      if (m16 & (0xfu << (4 * j4))) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                          const int j = 4 * j4 + e;
                          if (j < CAND && (m16 & (1u << j))) topk_insert(tkL[p2], tkI[p2], c[j], jb0 + rd * CAND + j);
                        }
                      }
                    }
                  }
                }
              }
            }
            __builtin_amdgcn_wave_barrier();
            return;
          }
          // The bulk of the tiles under a causal mask: every row of the wave sees every key of the tile, so every block of
          // the tile is complete, visible and not the row's own, and (checked here) rows and blocks all exist.  Then a value's
          // address is one wave-uniform base per tile plus a per-lane offset that does not depend on the tile.
          const bool direct = P.causal && plain && i0 + ppt <= P.n && jb0 + nbt <= P.nb && (long)P.g * P.n * P.nb < (1l << 30);
          if (direct) {
            float* tbase = pooled + ((long)(SH ? bh : bh * P.g) * P.n + i0) * P.nb + jb0;
            for (int e = lane; e < rows_here * nbt; e += 64) {
              const int rr = e / nbt, jj = e % nbt;
              const unsigned off = SH ? (unsigned)(rr * P.nb + jj) : (unsigned)(((rr & (P.g - 1)) * P.n + (rr >> P.lg)) * P.nb + jj);
              tbase[off] = pw[e] * norm;
            }
          } else
          for (int e = lane; e < rows_here * nbt; e += 64) {
            const int rr = e / nbt, jj = e % nbt;
            const int qi = i0 + (SH ? rr : (rr >> P.lg));
            const int jblk = jb0 + jj;
            const float sum = pw[e];
            // all npf keys of the block visible: (jblk+1)*npf - 1 <= qi/st - 1  <=>  (jblk+1)*B <= qi
            const int blo = jblk * P.B, bhi = blo + P.B;
            const bool own = (blo <= qi) & (qi < bhi);
            const bool vis = (!P.causal | (bhi <= qi)) & !(P.mask_own & own);
            const long head = SH ? (long)bh : (long)bh * P.g + (rr & (P.g - 1));
            if ((qi < P.n) & (jblk < P.nb)) pooled[(head * P.n + qi) * P.nb + jblk] = vis ? sum * norm : -INFINITY;
          }
          __builtin_amdgcn_wave_barrier();
        };
        if (!P.share || P.g == 1) pool(std::integral_constant<int, 0>{});
        else if (P.g == 4) pool(std::integral_constant<int, 4>{});
        else if (P.g == 2) pool(std::integral_constant<int, 2>{});
        else pool(std::integral_constant<int, 1>{});
      }

      tmax = halves_max(tmax);
      // The reference maximum m of a row (raw units) follows the running maximum only when that has grown by more than
      // kSlack in the exponent's units: until then the probabilities are taken against the stale reference (at most
      // 2^kSlack, exact in fp32 and with the same relative rounding in bf16) and nothing needs rescaling.  Softmax is
      // invariant to the reference, so the result is the same function; what goes away is the multiplication of the
      // whole accumulator tile by factors that are 1 or close to it in nearly every tile.  One wave-uniform test.
      // (m = -inf, tmax finite: the difference is +inf and the row moves; both -inf: NaN compares false, nothing to do)
      constexpr float kSlack = 8.f;
      if (__any((tmax - m) * sc > kSlack)) {
        const float mnew = fmaxf(m, tmax);
        const float alpha = fast_exp2((mnew == -INFINITY) ? 0.f : (m - mnew) * sc);
        m = mnew;
        l *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int e = 0; e < 16; ++e) Oa[dt][e] *= alpha;
      }
      const float mref = (m == -INFINITY) ? 0.f : m * sc;
      float rs = 0.f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i2 = 0; i2 < 16; ++i2) {
          const float p = fast_exp2(__builtin_fmaf(Sa[kt][i2], sc, -mref));
          Sa[kt][i2] = p;
          rs += p;
        }
      l += rs;                  // this lane's half of the keys: the halves are added once, after the walk
      bf16x8 Pf[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) Pf[c] = pack8(Sa[c >> 1], 8 * (c & 1));
      operands_ahead<4 * DT, NSA_FWD_AHV>([&](int i2) { return lds_transposed_operand_swz<D>(vt_s, 16 * (i2 / DT), 32 * (i2 % DT), lane); },
                                          [&](int i2, bf16x8 a) { Oa[i2 % DT] = mfma32(a, Pf[i2 / DT], Oa[i2 % DT]); });
    }
  }

  if (TK) {
    // A query's selections: lane s of its group holds the s-th.  Their probabilities under the padded softmax of NSA.py:693-695
    // follow from the entries alone wherever the mask can depend on them: every logit outside the list is at most the
    // list's smallest, so leaving them out of the normaliser moves a probability near the 1e-10 threshold by less than its
    // fp32 rounding (nb * 1e-10 relative).
    const int sub = lane & 15, rgrp = lane >> 4;
    const int rows_here = max(0, min(ppt, P.n - i0));
#pragma unroll
    for (int p2 = 0; p2 < TKP; ++p2) {
      if (4 * p2 < rows_here) {
        const float L = tkL[p2];
        const float mx = fmaxf(-1e3f, row16_bcast_max(L));
        const float e = __expf(L - mx);
        const float sum = row16_bcast_sum(e) + __expf(-1e3f - mx);
        const float pr = e * (1.0f / sum);
        const int rr = 4 * p2 + rgrp;
        if (rr < rows_here && sub < P.topk) {
          const long at = ((long)bh * P.n + i0 + rr) * P.topk + sub;
          tk_idx[at] = tkI[p2];
          tk_mask[at] = (pr < INFINITY && pr > 1e-10f) ? 1 : 0;
        }
      }
    }
  }
  if (POOL && !TK && !P.nofill) {
    // fine blocks whose compressed keys no query of this wave's tile can see were never visited
    const int last_visited = my_hi >= 0 ? min(walk.t_hi, my_hi / kBK) : -1;
    const int jstart = min(P.nb, (kBK * (last_visited + 1)) / (POOL ? NPF : 1));
    const int cntj = P.nb - jstart;
    const int rows_here = max(0, min(ppt, P.n - i0)) * (P.share ? 1 : P.g);
    // row by row (no division by the run-time count), 16 bytes per lane where the rows allow it
    const bool vec = cntj > 0 && !(P.nb & 3) && !(jstart & 3);
    for (int rr = 0; rr < rows_here; ++rr) {
      const int qi = i0 + (P.share ? rr : (rr >> P.lg));
      const long prow = P.share ? ((long)bh * P.n + qi) : (((long)b * P.hkv * P.g + hk * P.g + (rr & (P.g - 1))) * P.n + qi);
      float* dst = pooled + prow * P.nb;
      if (vec) {
        const floatx4 ninf = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        for (int jj = jstart + 4 * lane; jj < P.nb; jj += 256) *reinterpret_cast<floatx4*>(dst + jj) = ninf;
      } else {
        for (int jj = jstart + lane; jj < P.nb; jj += 64) dst[jj] = -INFINITY;
      }
    }
  }

  l = halves_sum(l);
  if (valid) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    __bf16* op = out + b * P.so[0] + (long)hq * P.so[1] + (long)i * P.so[2] + 4 * h;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int a = 0; a < 4; ++a)
        store4_bf16(op + 32 * dt + 8 * a, Oa[dt][4 * a] * inv, Oa[dt][4 * a + 1] * inv, Oa[dt][4 * a + 2] * inv, Oa[dt][4 * a + 3] * inv);
    if (h == 0) lse[((long)b * P.hkv * P.g + hq) * P.n + i] = (m * sc + fast_log2(l)) * kLn2;
  }
}

// ------------------------------------------------------------------------------ backward
// dQ, query-stationary (same tile walk as the forward): dS^T = P^T o (V dO^T - delta),
// dQ^T += K^T dS^T with K^T read through the LDS transpose load.
template <int D>
__global__ __launch_bounds__(256, 2) void dense_bwd_dq_kernel(const DensePlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                           const __bf16* __restrict__ v, const __bf16* __restrict__ out,
                                                           const __bf16* __restrict__ dout, const float* __restrict__ lse,
                                                           float* __restrict__ delta, __bf16* __restrict__ dq) {
  constexpr int KS = D / 16, DT = D / 32, TILE = kBK * D;
  // as in the forward kernel: two swizzled tiles each for K and V, filled by asynchronous copies, one barrier per tile
  __shared__ __align__(1024) __bf16 k_s[2 * TILE];
  __shared__ __align__(1024) __bf16 v_s[2 * TILE];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n_ = lane & 31, h = lane >> 5;
  const int bh = blockIdx.y, b = bh / P.hkv, hk = bh % P.hkv;
  const int ppt = 32 >> P.lg;
  const int qtiles = (P.n + 4 * ppt - 1) / (4 * ppt);
  const int xt = P.mode == 0 ? xcd_contiguous(blockIdx.x, qtiles) : (int)blockIdx.x;      // see the forward kernel
  if (xt >= qtiles) return;
  const int q0 = xt * 4 * ppt;
  const int i0 = q0 + wave * ppt;
  const int pq = n_ >> P.lg, g = n_ & (P.g - 1);
  const bool valid = i0 + pq < P.n;
  const int i = min(i0 + pq, P.n - 1);
  const int hq = hk * P.g + g;

  bf16x8 Qf[KS], Gf[KS];
  {
    const __bf16* qp = q + b * P.sq[0] + (long)hq * P.sq[1] + (long)i * P.sq[2] + 8 * h;
    const __bf16* gp = dout + b * P.sdo[0] + (long)hq * P.sdo[1] + (long)i * P.sdo[2] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) { Qf[ks] = load8(qp + 16 * ks); Gf[ks] = load8(gp + 16 * ks); }
  }
  const long srow = ((long)b * P.hkv * P.g + hq) * P.n + i;
  const float lse_r = lse[srow] * kLog2e;
  // delta = sum_d out * d_out of this lane's row: this kernel holds the row's d_out anyway, reads the row of out beside it
  // and leaves the sums for the dK/dV kernel that follows on the stream (a pass of its own over out and d_out before)
  float del_r = 0.f;
  {
    const __bf16* op = out + b * P.so[0] + (long)hq * P.so[1] + (long)i * P.so[2] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 o8 = load8(op + 16 * ks);
#pragma unroll
      for (int e = 0; e < 8; ++e) del_r = __builtin_fmaf((float)o8[e], (float)Gf[ks][e], del_r);
    }
    del_r = halves_sum(del_r);
    if (valid && h == 0) delta[srow] = del_r;
  }
  const Interval me = visible_range(P, i);
  const TileWalk walk = make_walk(P, q0, min(P.n - 1, q0 + 4 * ppt - 1));
  const int my_hi = visible_range(P, min(P.n - 1, i0 + ppt - 1)).hi, my_lo = visible_range(P, min(i0, P.n - 1)).lo;
  const int all_hi = visible_range(P, min(i0, P.n - 1)).hi, all_lo = visible_range(P, min(P.n - 1, i0 + ppt - 1)).lo;
  const float sc = P.scale * kLog2e;
  floatx16 Qa[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) Qa[dt] = zero_acc();

  const __bf16* kbase = k + b * P.sk[0] + hk * P.sk[1];
  const __bf16* vbase = v + b * P.sv[0] + hk * P.sv[1];
  TileDma<D, 256> kdma, vdma;
  kdma.init(tid, P.sk[2], k_s);
  vdma.init(tid, P.sv[2], v_s);
  auto load_tile = [&](int t, int into) {
    const long first = t < 0 ? 0 : (long)P.mem + (long)t * kBK;
    const long limit = t < 0 ? P.mem : (long)P.mem + P.nkeys;
    kdma.issue(kbase, first, limit, into * TILE * 2);
    vdma.issue(vbase, first, limit, into * TILE * 2);
  };
  int t = walk.t_first, buf = 0;
  if (t <= walk.t_hi || t < 0) load_tile(t, 0);

  for (; t <= walk.t_hi; t = walk.next(t), buf ^= 1) {
    wait_all_loads();
    __syncthreads();
    const int tn = walk.next(t);
    // the copy of the next tile goes between the S / dP MFMAs where it can (see the forward kernel)
    const long nfirst = (long)P.mem + (long)tn * kBK;
    const bool more = tn <= walk.t_hi, spread = more && nfirst + kBK <= (long)P.mem + P.nkeys;
    const __bf16* ktb = kbase + nfirst * P.sk[2];
    const __bf16* vtb = vbase + nfirst * P.sv[2];
    const unsigned noff = (buf ^ 1) * TILE * 2;
    const __bf16* kt_s = k_s + buf * TILE;
    const __bf16* vt_s = v_s + buf * TILE;
    const bool memtile = t < 0;
    const int kb0 = memtile ? 0 : t * kBK;
    const bool active = memtile || (kb0 <= my_hi && kb0 + kBK - 1 >= my_lo);
    if (!active || !spread) {
      if (more) load_tile(tn, buf ^ 1);
    }
    const unsigned lanes = spread ? ~0u : 0u;
    auto tile_math = [&](auto masked) {
      constexpr int RN = TileDma<D, 256>::ROUNDS;
      static_assert(2 * RN <= KS, "one copy round after every fourth MFMA");
      // one 32-key half at a time: S and dP (2 KS MFMAs), then dS of that half on the VALU - independent of the other
      // half's MFMAs, which the scheduler may run beside it - and 8 registers of packed dS instead of 32 of S and dP
      const int klo = memtile ? 0 : me.lo, khi = memtile ? P.mem - 1 : me.hi;
      bf16x8 Sf[4];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        floatx16 Sa = zero_acc(), Pa = zero_acc();
        // operand i: k-step i / 2, even i from K (scores), odd i from V (dP)
        operands_ahead<2 * KS, NSA_DQ_AHK>(
            [&](int i2) { return lds_row_operand_swz<D>(((i2 & 1) ? vt_s : kt_s) + 32 * kt * D, i2 >> 1, lane); },
            [&](int i2, bf16x8 a) {
              if (i2 & 1) Pa = mfma32(a, Gf[i2 >> 1], Pa);
              else Sa = mfma32(a, Qf[i2 >> 1], Sa);
              const int c = (kt * 2 * KS + i2) >> 2;      // a copy round after every fourth MFMA of the tile
              if ((i2 & 3) == 3 && c < 2 * RN) {
                if (c < RN) kdma.round_full_if(lanes, ktb, noff, c);
                else vdma.round_full_if(lanes, vtb, noff, c - RN);
              }
            });
#pragma unroll
        for (int i2 = 0; i2 < 16; ++i2) {
          const int key = kb0 + 32 * kt + 8 * (i2 >> 2) + 4 * h + (i2 & 3);
          // the mask goes into the exponent (exp2(-inf) = 0, '&' instead of '&&'): a select around the exponential is compiled
          // as a branch per element
          float x = __builtin_fmaf(Sa[i2], sc, -lse_r);
          if (decltype(masked)::value) x = ((key >= klo) & (key <= khi)) ? x : -INFINITY;
          const float p = fast_exp2(x);
          Sa[i2] = p * (Pa[i2] - del_r);
        }
        Sf[2 * kt] = pack8(Sa, 0);
        Sf[2 * kt + 1] = pack8(Sa, 8);
      }
      operands_ahead<4 * DT, NSA_DQ_AHT>([&](int i2) { return lds_transposed_operand_swz<D>(kt_s, 16 * (i2 / DT), 32 * (i2 % DT), lane); },
                                         [&](int i2, bf16x8 a) { Qa[i2 % DT] = mfma32(a, Sf[i2 / DT], Qa[i2 % DT]); });
    };
    if (active) {
      // a tile every row of the wave sees completely needs no per-element mask (wave-uniform); each
      // variant is one straight-line block so that VALU work and MFMAs can be interleaved
      if (!memtile && kb0 >= all_lo && kb0 + kBK - 1 <= all_hi) tile_math(std::false_type{});
      else tile_math(std::true_type{});
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

// Query range [qlo, qhi) that can see any key of the 64-row tile T of k/v (rows counted from the
// start of the arrays, memory slots included).
__device__ __forceinline__ void tile_query_range(const DensePlan& P, int T, int& qlo, int& qhi) {
  qhi = P.n;
  if (P.mode == 0) {
    qlo = max(0, kBK * T - P.wf);
    qhi = min(P.n, kBK * T + kBK - 1 + P.wb + 1);
  } else if (!P.causal || kBK * T < P.mem) {
    qlo = 0;
  } else {
    qlo = (int)min((long)P.n, ((long)kBK * T - P.mem + 1) * P.st);      // compressed key c is visible iff i >= (c+1)*st
  }
}

__device__ __forceinline__ void chunk_range(const DensePlan& P, int T, int c, int& qlo, int& qhi, int& c0, int& c1) {
  tile_query_range(P, T, qlo, qhi);
  if (P.mode == 0) {
    c0 = qlo + c * P.chunk_q;
    c1 = min(qhi, c0 + P.chunk_q);
  } else {
    c0 = max(qlo, c * P.chunk_q);
    c1 = min(qhi, (c + 1) * P.chunk_q);
  }
}

// Work-group x of the dK/dV walk -> (key tile T, query chunk c); false for the padding ids of the grid.  Band mode:
// tile-major, one contiguous range of key tiles per XCD (neighbouring tiles see almost the same queries).  Stride mode:
// all key tiles of a query chunk on one XCD (they stream the same Q / dO rows), chunks dealt to the XCDs in a zig-zag
// (rounds of 8 chunks, every other round reversed) because under the causal mask a later chunk sees more key tiles.
__device__ __forceinline__ bool chunk_of(const DensePlan& P, int x, int& T, int& c, int& qlo, int& qhi, int& c0, int& c1) {
  if (P.mode == 0) {
    const int v = xcd_contiguous(x, P.key_tiles * P.chunks);
    if (v >= P.key_tiles * P.chunks) return false;
    T = v / P.chunks; c = v % P.chunks;
  } else {
    const int xc = x & 7, idx = x >> 3, round = idx / P.key_tiles;
    T = idx % P.key_tiles;
    c = 8 * round + ((round & 1) ? 7 - xc : xc);
    if (c >= P.chunks) return false;
  }
  chunk_range(P, T, c, qlo, qhi, c0, c1);
  return true;
}
static inline unsigned dkv_grid(const DensePlan& P) {
  return P.mode == 0 ? xcd_grid_for(P.key_tiles * P.chunks) : 8u * (unsigned)(((P.chunks + 7) / 8) * P.key_tiles);
}

#ifndef NSA_DKV_AHEAD
#define NSA_DKV_AHEAD 3
#endif
#ifndef NSA_DKV_PIPE_MIN_D
#define NSA_DKV_PIPE_MIN_D 128    // head dimensions from here on take dense_bwd_dkv_pipe_kernel (one wave per SIMD)
#endif
#ifndef NSA_DKV_STAGES
#define NSA_DKV_STAGES 1      // measured on MI355X (compressed branch, seq 32k, d 128): 1, 2 or 3 tiles ahead all 4.7 ms
#endif

// dK/dV of one 64-row tile of k/v over one chunk of the queries that can see it (key-stationary);
// wave kt owns rows 32kt .. 32kt+31 of the tile.  Rows are indexed from the start of the arrays,
// so in stride mode row r is visible to query i iff r <= hi(i) + mem.
template <int D>
__global__ __launch_bounds__(128) void dense_bwd_dkv_kernel(const DensePlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                            const __bf16* __restrict__ v, const __bf16* __restrict__ dout,
                                                            const float* __restrict__ lse, const float* __restrict__ delta, float* __restrict__ part) {
  constexpr int KS = D / 16, DT = D / 32, RS = D + 8;
  __shared__ __align__(16) float lse_s[32];
  __shared__ __align__(16) float del_s[32];
  __shared__ __align__(16) int lo_s[32];
  __shared__ __align__(16) int hi_s[32];
  __shared__ __align__(16) __bf16 xq_s[32 * RS];
  __shared__ __align__(16) __bf16 xg_s[32 * RS];
  const int kt = threadIdx.x >> 6, lane = threadIdx.x & 63, n_ = lane & 31, h = lane >> 5;
  const int bh = blockIdx.y, b = bh / P.hkv, hk = bh % P.hkv;
  // band mode: chunks are counted from the tile's first visible query, tile-major order (adjacent
  // tiles see almost the same queries).  Stride mode: chunks are absolute query ranges in
  // chunk-major order, so that work-groups running together read the same Q/dO chunk (L2 reuse
  // across the key tiles) instead of each streaming its own.
  int T, c, qlo, qhi, c0, c1;
  if (!chunk_of(P, blockIdx.x, T, c, qlo, qhi, c0, c1)) return;
  if (c0 >= c1) return;

  const int kr_ = kBK * T + 32 * kt + n_;                // this lane's row of k/v
  const bool kok = kr_ < P.krows;
  bf16x8 Kf[KS], Vf[KS];
  {
    const long krow = kok ? kr_ : 0;
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
  const __bf16* qbase = q + b * P.sq[0] + (long)(hk * P.g) * P.sq[1];
  const __bf16* gbase = dout + b * P.sdo[0] + (long)(hk * P.g) * P.sdo[1];
  constexpr int CPR = D / 8, RPI = 64 / CPR, NT = 32 / RPI;

  // wave 0 gathers the tile's Q rows, wave 1 its dO rows (coalesced), NSA_DKV_STAGES tiles ahead: at
  // one wave per SIMD the depth of this pipeline is the only latency hiding there is
  struct Stage { bf16x8 raw[NT]; float lse_r, del_r; };
  auto issue = [&](Stage& st, int i0) {
    const __bf16* base = kt == 0 ? qbase : gbase;
    const long sh = kt == 0 ? P.sq[1] : P.sdo[1], sn = kt == 0 ? P.sq[2] : P.sdo[2];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int rr = t * RPI + lane / CPR;
      const int qi = min(i0 + (rr >> P.lg), P.n - 1);
      // head and token strides are below 2^32 (checked when the plan is made): 32 x 32 -> 64-bit multiply-adds
      const unsigned long off = (unsigned long)(unsigned)(rr & (P.g - 1)) * (unsigned)sh + (unsigned long)(unsigned)qi * (unsigned)sn;
      st.raw[t] = load8(base + off + 8 * (lane % CPR));
    }
    const int qi = min(i0 + pq, P.n - 1);
    const long srow = ((long)b * P.hkv * P.g + hq) * P.n + qi;
    st.lse_r = lse[srow]; st.del_r = delta[srow];        // scaled where it is used: arithmetic here would wait for the loads
  };
  constexpr int NS = NSA_DKV_STAGES;
  Stage stg[NS];
#pragma unroll
  for (int s2 = 0; s2 < NS; ++s2) issue(stg[s2], c0 + s2 * ppt);
  wait_all_loads();
  auto step = [&](int i0, Stage& cur) {
    const bool valid = i0 + pq < c1;
    const int i = min(i0 + pq, P.n - 1);
    {
      __bf16* dst = kt == 0 ? xq_s : xg_s;
#pragma unroll
      for (int t = 0; t < NT; ++t) *reinterpret_cast<bf16x8*>(dst + (t * RPI + lane / CPR) * RS + 8 * (lane % CPR)) = cur.raw[t];
    }
    if (kt == 0 && h == 0) {
      lse_s[n_] = valid ? cur.lse_r * kLog2e : INFINITY;   // +inf: a padding row gets p = 0
      del_s[n_] = cur.del_r;
      const Interval me = visible_range(P, i);
      lo_s[n_] = P.mode == 0 ? me.lo : 0;
      hi_s[n_] = P.mode == 0 ? me.hi : me.hi + P.mem;
    }
    __syncthreads();
    issue(cur, i0 + NS * ppt);                             // the freed stage takes the tile NS steps ahead
    __builtin_amdgcn_sched_barrier(0);

    // the whole tile's arithmetic as one straight-line block per variant (masked / unmasked), so that
    // the scheduler can overlap the softmax VALU work with the MFMAs on either side of it
    auto tile_math = [&](auto masked) {
    floatx16 Sa = zero_acc(), Pa = zero_acc();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Sa = mfma32(lds_row_operand(xq_s, RS, ks, lane), Kf[ks], Sa);     // [row][key]: lane <-> key, registers <-> rows
      Pa = mfma32(lds_row_operand(xg_s, RS, ks, lane), Vf[ks], Pa);
    }
    floatx16 dSa;
    {
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const floatx4 l4 = *reinterpret_cast<const floatx4*>(&lse_s[8 * a + 4 * h]);
        const floatx4 d4 = *reinterpret_cast<const floatx4*>(&del_s[8 * a + 4 * h]);
        const int* lo4 = &lo_s[8 * a + 4 * h];
        const int* hi4 = &hi_s[8 * a + 4 * h];
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          const int i2 = 4 * a + bb;
          float x = __builtin_fmaf(Sa[i2], sc, -l4[bb]);      // mask in the exponent: see the dQ kernel
          if (decltype(masked)::value) x = ((kr_ >= lo4[bb]) & (kr_ <= hi4[bb])) ? x : -INFINITY;
          const float p = fast_exp2(x);
          Sa[i2] = p;
          dSa[i2] = p * (Pa[i2] - d4[bb]);
        }
      }
    }
    const bf16x8 Pf0 = pack8(Sa, 0), Pf1 = pack8(Sa, 8);
    const bf16x8 Sf0 = pack8(dSa, 0), Sf1 = pack8(dSa, 8);
    // dV^T += dO^T P, dK^T += Q^T dS: 4 * DT MFMAs whose LDS operands are read NSA_DKV_AHEAD MFMAs ahead (the
    // compiler keeps transpose loads in source order; read right before their MFMA, LDS latency paces the phase)
    operands_ahead<4 * DT, NSA_DKV_AHEAD>(
        [&](int i) { return lds_transposed_operand((i & 2) ? xq_s : xg_s, RS, 16 * (i & 1), 32 * (i >> 2), lane); },
        [&](int i, const bf16x8& a) {
          const int dt = i >> 2, w = i & 3;
          if (w == 0) dVa[dt] = mfma32(a, Pf0, dVa[dt]);
          else if (w == 1) dVa[dt] = mfma32(a, Pf1, dVa[dt]);
          else if (w == 2) dKa[dt] = mfma32(a, Sf0, dKa[dt]);
          else dKa[dt] = mfma32(a, Sf1, dKa[dt]);
        });
    };
    {
      // rows of this wave are visible to every query of the tile iff they lie between the largest lower
      // and the smallest upper bound, which consecutive queries take at the tile's ends (wave-uniform)
      const Interval vf = visible_range(P, min(i0, P.n - 1)), vl = visible_range(P, min(i0 + ppt - 1, P.n - 1));
      const int all_lo = P.mode == 0 ? vl.lo : 0, all_hi = P.mode == 0 ? vf.hi : vf.hi + P.mem;
      const int r0 = kBK * T + 32 * kt;
      if (r0 >= all_lo && r0 + 31 <= all_hi) tile_math(std::false_type{});
      else tile_math(std::true_type{});
    }
    __syncthreads();
  };
  // whole rounds of NS tiles first: a round's steps are unconditional, so the wait before each step's
  // commit counts exactly the loads issued after that stage's
  int i0 = c0;
  if (i0 + (NS - 1) * ppt < c1) {
    wait_all_loads();      // again: the compiler sinks the later stages' first loads to here, past the wait above
    do {
#pragma unroll
      for (int s2 = 0; s2 < NS; ++s2) step(i0 + s2 * ppt, stg[s2]);
      i0 += NS * ppt;
    } while (i0 + (NS - 1) * ppt < c1);
  }
#pragma unroll
  for (int s2 = 0; s2 < NS - 1; ++s2)
    if (i0 + s2 * ppt < c1) step(i0 + s2 * ppt, stg[s2]);
  // partial [bh][tile][chunk][2][64][D] fp32; dKa/dVa hold [feature 32dt + 8a + 4h + bb][row 32kt + n_]
  float* pk = part + (((size_t)bh * P.key_tiles + T) * P.chunks + c) * (2 * kBK * D) + (size_t)(32 * kt + n_) * D + 4 * h;
  float* pv = pk + kBK * D;
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

// The same walk for head dimensions whose accumulators leave room for one wave per SIMD only (d = 128: 128 registers of dK / dV
// accumulators, 64 of K / V operands).  With one wave per SIMD nothing overlaps a wave's MFMAs but its own instruction order,
// so the step is laid out by hand and fenced (cycle stamps of the kernel above at d = 128: 23 % of a step in the tile's LDS
// write, 11 % in two barriers, 6 % issuing loads, and the softmax entirely outside the MFMA runs):
//   * the tile's arithmetic is six runs of MFMAs in dependency order - S = Q K^T, dP = dO V^T, dV from rows 0-15, dV from rows
//     16-31, dK from rows 0-15, dK from rows 16-31 - and the softmax is dealt out in slices beside the MFMAs of the run
//     before the one that needs the slice's result (p of rows 0-15 beside dP, p of rows 16-31 beside the first dV run, ...);
//   * the Q / dO tile is double-buffered in LDS: the next tile goes from its staging registers to the other buffer beside the
//     S MFMAs, each row's staging register is reloaded with the tile after that right behind its store, and one barrier per
//     step is left, which stands before the last run (see the loop).
template <int D>
__global__ __launch_bounds__(128) void dense_bwd_dkv_pipe_kernel(const DensePlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                                 const __bf16* __restrict__ v, const __bf16* __restrict__ dout,
                                                                 const float* __restrict__ lse, const float* __restrict__ delta,
                                                                 float* __restrict__ part) {
  constexpr int KS = D / 16, DT = D / 32, RS = D + 8;
  __shared__ __align__(16) float lse_s[2][32];
  __shared__ __align__(16) float del_s[2][32];
  __shared__ __align__(16) int lo_s[2][32];
  __shared__ __align__(16) int hi_s[2][32];
  __shared__ __align__(16) __bf16 tile_s[2][2][32 * RS];        // [buffer][Q rows | dO rows]: one array, so that a read's address
                                                                 // is one lane-dependent base per buffer + an immediate
  const int kt = threadIdx.x >> 6, lane = threadIdx.x & 63, n_ = lane & 31, h = lane >> 5;
  const int bh = blockIdx.y, b = bh / P.hkv, hk = bh % P.hkv;
  int T, c, qlo, qhi, c0, c1;
  if (!chunk_of(P, blockIdx.x, T, c, qlo, qhi, c0, c1)) return;
  if (c0 >= c1) return;

  const int kr_ = kBK * T + 32 * kt + n_;                // this lane's row of k/v
  const bool kok = kr_ < P.krows;
  bf16x8 Kf[KS], Vf[KS];
  {
    const long krow = kok ? kr_ : 0;
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
  constexpr int CPR = D / 8, RPI = 64 / CPR, NT = 32 / RPI;
  static_assert(NT == KS, "one staged row group beside every S MFMA");

  // wave 0 stages the tile's Q rows, wave 1 its dO rows, through buffer loads: the descriptor starts at the tile's first
  // query of this kv head's query heads and ends with the last row of the last of them, so a lane's offset is the same in
  // every step (no address arithmetic in the loop) and no row index needs a clamp (the launcher checks that the heads of a
  // group span less than 2^31 elements).  What a row past the end of the sequence reads depends on the head: in the group's
  // last head it lies beyond the descriptor and reads as zeros; in an earlier head of a contiguous 'h n d' array it lands on
  // the leading rows of the next head (and its lse / delta likewise).  Either way such a row is neutralised by its
  // log-sum-exp, which store_smalls replaces by +inf for every row at or beyond c1: p = exp2(finite - inf) = 0 and
  // dS = 0 * (finite) = 0, so finite values of any size in the aliased rows add nothing to dK / dV.
  const int ktu = __builtin_amdgcn_readfirstlane(kt);
  const __bf16* slab = ktu == 0 ? q + b * P.sq[0] + (long)(hk * P.g) * P.sq[1] : dout + b * P.sdo[0] + (long)(hk * P.g) * P.sdo[1];
  const long sh = ktu == 0 ? P.sq[1] : P.sdo[1], sn = ktu == 0 ? P.sq[2] : P.sdo[2];
  const long extent = (long)(P.g - 1) * sh + (long)(P.n - 1) * sn + D;            // elements from slab to the end of its last row
  const long srow0 = ((long)b * P.hkv * P.g + hq) * P.n;
  unsigned voff[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int rr = t * RPI + lane / CPR;
    voff[t] = 2u * (unsigned)((long)(rr & (P.g - 1)) * sh + (long)(rr >> P.lg) * sn + 8 * (lane % CPR));
  }
  bf16x8 raw[NT];
  float lse_r, del_r;
  __amdgpu_buffer_rsrc_t rows_of_tile;
  auto aim_rows = [&](int i0) {
    const long first = min((long)i0 * sn, extent);
    rows_of_tile = __builtin_amdgcn_make_buffer_rsrc((void*)(slab + first), 0, (int)(2 * (extent - first)), 0x00020000);
  };
  auto load_rows = [&](int t) {
    raw[t] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(rows_of_tile, (int)voff[t], 0, 0));
  };
  // Per-row scalars of a tile: wave 0 stages log-sum-exp and delta (buffer loads again: one descriptor per array, moved along
  // with the tile), wave 1 the bounds of the rows' visible ranges - and those only for tiles that are not visible as a whole
  // to all 64 key rows, the others never read them.  Split like this the two waves carry about the same number of
  // instructions per step, which at one wave per SIMD is what a step costs.
  const float* lse_slab = lse + ((long)b * P.hkv + hk) * P.g * (long)P.n;
  const float* del_slab = delta + ((long)b * P.hkv + hk) * P.g * (long)P.n;
  const long rows_slab = (long)P.g * P.n;
  const int soff = 4 * (g * P.n + pq);
  __amdgpu_buffer_rsrc_t lse_of_tile, del_of_tile;
  auto load_smalls = [&](int i0) {
    if (ktu == 0) {
      const long first = min((long)i0, rows_slab);
      lse_of_tile = __builtin_amdgcn_make_buffer_rsrc((void*)(lse_slab + first), 0, (int)(4 * (rows_slab - first)), 0x00020000);
      del_of_tile = __builtin_amdgcn_make_buffer_rsrc((void*)(del_slab + first), 0, (int)(4 * (rows_slab - first)), 0x00020000);
      lse_r = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(lse_of_tile, soff, 0, 0));
      del_r = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(del_of_tile, soff, 0, 0));
    }
  };
  const int t0 = kBK * T;
  auto whole_tile_visible = [&](int i0) {
    const Interval vf = visible_range(P, min(i0, P.n - 1)), vl = visible_range(P, min(i0 + ppt - 1, P.n - 1));
    const int all_lo = P.mode == 0 ? vl.lo : 0, all_hi = P.mode == 0 ? vf.hi : vf.hi + P.mem;
    return t0 >= all_lo && t0 + kBK - 1 <= all_hi;
  };
  auto store_rows = [&](int t, int buf) {
    __bf16* dst = tile_s[buf][kt];
    *reinterpret_cast<bf16x8*>(dst + (t * RPI + lane / CPR) * RS + 8 * (lane % CPR)) = raw[t];
  };
  auto store_smalls = [&](int i0, int buf) {
    if (ktu == 0) {
      if (h == 0) {
        lse_s[buf][n_] = i0 + pq < c1 ? lse_r * kLog2e : INFINITY;   // +inf: a padding row gets p = 0
        del_s[buf][n_] = del_r;
      }
    } else if (!whole_tile_visible(i0)) {
      if (h == 0) {
        const Interval me = visible_range(P, min(i0 + pq, P.n - 1));
        lo_s[buf][n_] = P.mode == 0 ? me.lo : 0;
        hi_s[buf][n_] = P.mode == 0 ? me.hi : me.hi + P.mem;
      }
    }
  };
  // tile c0 into buffer 0, tile c0 + ppt into the staging registers
  aim_rows(c0);
#pragma unroll
  for (int t = 0; t < NT; ++t) load_rows(t);
  load_smalls(c0);
#pragma unroll
  for (int t = 0; t < NT; ++t) store_rows(t, 0);
  store_smalls(c0, 0);
  aim_rows(c0 + ppt);
#pragma unroll
  for (int t = 0; t < NT; ++t) load_rows(t);
  load_smalls(c0 + ppt);
  __syncthreads();

  // The step's barrier stands before the tile's last run of MFMAs (dK from rows 16-31), not behind it: that run's operands
  // are read from LDS before the barrier and the run itself is carried into the next step, where its MFMAs cover the round
  // trips of the next tile's first LDS reads (cycle stamps: 490 of 2650 ticks of a step passed between the barrier and the
  // first MFMA).  Carried across: the run's B operand Sf1c, its A operands opc[], and whether the next tile needs the mask.
  bf16x8 Sf1c = zero_frag(), opc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) opc[dt] = zero_frag();
  const int r0 = kBK * T + 32 * __builtin_amdgcn_readfirstlane(kt);
  auto unmasked_at = [&](int i0) {
    // rows of this wave are visible to every query of the tile iff they lie between the largest lower
    // and the smallest upper bound, which consecutive queries take at the tile's ends (wave-uniform)
    const Interval vf = visible_range(P, min(i0, P.n - 1)), vl = visible_range(P, min(i0 + ppt - 1, P.n - 1));
    const int all_lo = P.mode == 0 ? vl.lo : 0, all_hi = P.mode == 0 ? vf.hi : vf.hi + P.mem;
    return r0 >= all_lo && r0 + 31 <= all_hi;
  };
  bool unmasked = unmasked_at(c0);
  int buf = 0;
  for (int i0 = c0; i0 < c1; i0 += ppt, buf ^= 1) {
    const __bf16* xq = tile_s[buf][0];
    const __bf16* xg = tile_s[buf][1];
    aim_rows(i0 + 2 * ppt);
    {
      constexpr int N = 2 * KS + 3 * DT, AH = NSA_DKV_AHEAD;
      auto rd = [&](int i) {
        if (i < KS) return lds_row_operand(xq, RS, i, lane);
        if (i < 2 * KS) return lds_row_operand(xg, RS, i - KS, lane);
        const int j = i - 2 * KS, run = j / DT, dt = j % DT;
        return lds_transposed_operand(run < 2 ? xg : xq, RS, 16 * (run & 1), 32 * dt, lane);
      };
      // this tile's first reads, then the carried run
      bf16x8 ring[AH + 1];
#pragma unroll
      for (int i = 0; i < AH; ++i) ring[i] = rd(i);
      floatx4 l4[4], d4[4];
#pragma unroll
      for (int a = 0; a < 4; ++a) l4[a] = *reinterpret_cast<const floatx4*>(&lse_s[buf][8 * a + 4 * h]);
      // One copy of the step for all tiles (two copies, with and without the mask, cost the register allocator 150 registers).
      // The mask costs the arithmetic nothing: a row that must not see this lane's key gets +inf for its log-sum-exp, so its
      // exponent is -inf and p = 0; only tiles at an edge of the visible range read the bounds and patch l4.
      if (!unmasked) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const intx4 lo = *reinterpret_cast<const intx4*>(&lo_s[buf][8 * a + 4 * h]);
          const intx4 hi = *reinterpret_cast<const intx4*>(&hi_s[buf][8 * a + 4 * h]);
#pragma unroll
          for (int bb = 0; bb < 4; ++bb) l4[a][bb] = ((kr_ >= lo[bb]) & (kr_ <= hi[bb])) ? l4[a][bb] : INFINITY;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        dKa[dt] = mfma32(opc[dt], Sf1c, dKa[dt]);
        __builtin_amdgcn_sched_barrier(0);
      }
      floatx16 Sa = zero_acc(), Pa = zero_acc();
      bf16x8 Pf0, Pf1, Sf0, Sf1;
      // softmax slices: p (from S) for this lane's rows first .. first + count - 1, then dS (from p and dP, in dP's place)
      auto soft1 = [&](int first, int count) {
#pragma unroll
        for (int e = 0; e < count; ++e) {
          const int i2 = first + e, a = i2 >> 2, bb = i2 & 3;
          Sa[i2] = fast_exp2(__builtin_fmaf(Sa[i2], sc, -l4[a][bb]));
        }
        if (first + count == 8) Pf0 = pack8(Sa, 0);
        if (first + count == 16) Pf1 = pack8(Sa, 8);
      };
      auto soft2 = [&](int first, int count) {
#pragma unroll
        for (int e = 0; e < count; ++e) {
          const int i2 = first + e, a = i2 >> 2, bb = i2 & 3;
          Pa[i2] = Sa[i2] * (Pa[i2] - d4[a][bb]);
        }
        if (first + count == 8) Sf0 = pack8(Pa, 0);
        if (first + count == 16) Sf1 = pack8(Pa, 8);
      };
      constexpr int EA = 8 / KS, EB = 8 / DT;
#pragma unroll
      for (int i = 0; i < N; ++i) {
        if (i + AH < N) ring[(i + AH) % (AH + 1)] = rd(i + AH);
        const bf16x8 a = ring[i % (AH + 1)];
        if (i < KS) {
          Sa = mfma32(a, Kf[i], Sa);                                  // [row][key]: lane <-> key, registers <-> rows
          store_rows(i, buf ^ 1);                                     // next tile: registers -> the other buffer,
          load_rows(i);                                               // the tile after it -> the freed registers
        } else if (i < 2 * KS) {
          Pa = mfma32(a, Vf[i - KS], Pa);
          soft1(EA * (i - KS), EA);
        } else {
          const int j = i - 2 * KS, run = j / DT, dt = j % DT;
          if (run == 0) {
            dVa[dt] = mfma32(a, Pf0, dVa[dt]);
            soft1(8 + EB * dt, EB);
            if (dt == 0) {
#pragma unroll
              for (int a2 = 0; a2 < 4; ++a2) d4[a2] = *reinterpret_cast<const floatx4*>(&del_s[buf][8 * a2 + 4 * h]);
            }
          }
          else if (run == 1) { dVa[dt] = mfma32(a, Pf1, dVa[dt]); soft2(EB * dt, EB); }
          else {
            dKa[dt] = mfma32(a, Sf0, dKa[dt]);
            soft2(8 + EB * dt, EB);
            opc[dt] = lds_transposed_operand(xq, RS, 16, 32 * dt, lane);       // the carried run's operands
            if (dt == 0) { store_smalls(i0 + ppt, buf ^ 1); load_smalls(i0 + 2 * ppt); }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      Sf1c = Sf1;
    }
    unmasked = unmasked_at(i0 + ppt);
    __syncthreads();
  }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) dKa[dt] = mfma32(opc[dt], Sf1c, dKa[dt]);
  // partial [bh][tile][chunk][2][64][D] fp32; dKa/dVa hold [feature 32dt + 8a + 4h + bb][row 32kt + n_]
  float* pk = part + (((size_t)bh * P.key_tiles + T) * P.chunks + c) * (2 * kBK * D) + (size_t)(32 * kt + n_) * D + 4 * h;
  float* pv = pk + kBK * D;
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
__global__ __launch_bounds__(256) void dense_bwd_dkv_reduce_kernel(const DensePlan P, const float* __restrict__ part, void* __restrict__ dk, void* __restrict__ dv) {
  const int T = blockIdx.x, bh = blockIdx.y;
  const int keys = min(kBK, P.krows - kBK * T);
  const float* base = part + ((size_t)bh * P.key_tiles + T) * P.chunks * (2 * kBK * D);
  constexpr int CPR = D / 4;
  // the chunks that hold queries for this tile are consecutive; only those were written
  int clo = P.chunks, chi = 0;
  for (int c = 0; c < P.chunks; ++c) {
    int qlo, qhi, c0, c1;
    chunk_range(P, T, c, qlo, qhi, c0, c1);
    if (c0 < c1) { clo = min(clo, c); chi = c + 1; }
  }
  for (int e = threadIdx.x; e < 2 * keys * CPR; e += 256) {
    const int which = e / (keys * CPR), rem = e % (keys * CPR);
    const int key = rem / CPR, dd = (rem % CPR) * 4;
    floatx4 acc = {0.f, 0.f, 0.f, 0.f};
    const float* src = base + (size_t)which * kBK * D + (size_t)key * D + dd;
#pragma unroll 8
    for (int c = clo; c < chi; ++c) acc += __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(src + (size_t)c * (2 * kBK * D)));
    const float s = which == 0 ? P.scale : 1.0f;
    const size_t at = ((size_t)bh * P.krows + (size_t)kBK * T + key) * D + dd;
    if (P.dkv_fp32) *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(which == 0 ? dk : dv) + at) = acc * s;
    else store4_bf16(reinterpret_cast<__bf16*>(which == 0 ? dk : dv) + at, acc[0] * s, acc[1] * s, acc[2] * s, acc[3] * s);
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

template <int D, int NPF, bool TK>
static int dense_fwd_launch2(const DensePlan& P, const void* q, const void* k, const void* v, void* out, float* lse, float* pooled, int* tk_idx,
                             uint8_t* tk_mask, hipStream_t st) {
  const int qpw = 4 * (32 >> P.lg);                 // queries per work-group
  hipLaunchKernelGGL((dense_fwd_kernel<D, NPF, TK>), dim3(P.mode == 0 ? xcd_grid_for((P.n + qpw - 1) / qpw) : (unsigned)((P.n + qpw - 1) / qpw), P.bh), dim3(256), 0, st, P, (const __bf16*)q, (const __bf16*)k,
                     (const __bf16*)v, (__bf16*)out, lse, pooled, tk_idx, tk_mask);
  NSA_LAUNCH_CHECK();
  return 0;
}

template <int D, bool TK>
static int dense_fwd_launch(const DensePlan& P, const void* q, const void* k, const void* v, void* out, float* lse, float* pooled, int* tk_idx,
                            uint8_t* tk_mask, hipStream_t st) {
  switch (P.pool ? P.npf : 0) {
    case 0: if (!TK) return dense_fwd_launch2<D, 0, false>(P, q, k, v, out, lse, pooled, tk_idx, tk_mask, st); break;
    case 1: return dense_fwd_launch2<D, 1, TK>(P, q, k, v, out, lse, pooled, tk_idx, tk_mask, st);
    case 2: return dense_fwd_launch2<D, 2, TK>(P, q, k, v, out, lse, pooled, tk_idx, tk_mask, st);
    case 4: return dense_fwd_launch2<D, 4, TK>(P, q, k, v, out, lse, pooled, tk_idx, tk_mask, st);
    case 8: return dense_fwd_launch2<D, 8, TK>(P, q, k, v, out, lse, pooled, tk_idx, tk_mask, st);
    case 16: return dense_fwd_launch2<D, 16, TK>(P, q, k, v, out, lse, pooled, tk_idx, tk_mask, st);
    case 32: return dense_fwd_launch2<D, 32, TK>(P, q, k, v, out, lse, pooled, tk_idx, tk_mask, st);
  }
  return NSA_E_UNSUPPORTED;
}

extern "C" int nsa_dense_fwd(const nsa_dense_desc* d, const void* q, const void* k, const void* v, void* out, float* lse, float* pooled, void* stream) {
  DensePlan P;
  const int rc = make_dense_plan(d, P);
  if (rc) return rc;
  if (!q || !k || !v || !out || !lse || (P.pool && !pooled)) return NSA_E_ARG;
  if (P.D == 64) return dense_fwd_launch<64, false>(P, q, k, v, out, lse, pooled, nullptr, nullptr, (hipStream_t)stream);
  if (P.D == 128) return dense_fwd_launch<128, false>(P, q, k, v, out, lse, pooled, nullptr, nullptr, (hipStream_t)stream);
  return NSA_E_UNSUPPORTED;
}

extern "C" int nsa_compress_topk_supported(const nsa_dense_desc* d, int32_t num_selected) {
  DensePlan P;
  if (make_dense_plan(d, P)) return 0;
  // a wave serves its (at most 16) queries four at a time with 16 lanes each: selections shared by a group of >= 2 heads, <= 16 of them
  return P.mode == 1 && P.pool && P.share && P.g >= 2 && num_selected >= 1 && num_selected <= 16 && num_selected <= P.nb;
}

extern "C" int nsa_compress_topk_fwd(const nsa_dense_desc* d, const void* q, const void* k, const void* v, void* out, float* lse,
                                     int32_t num_selected, int32_t* idx, uint8_t* fmask, void* stream) {
  DensePlan P;
  const int rc = make_dense_plan(d, P);
  if (rc) return rc;
  if (!q || !k || !v || !out || !lse || !idx || !fmask) return NSA_E_ARG;
  if (!nsa_compress_topk_supported(d, num_selected)) return NSA_E_UNSUPPORTED;
  P.topk = num_selected;
  P.nofill = 1;
  if (P.D == 64) return dense_fwd_launch<64, true>(P, q, k, v, out, lse, nullptr, idx, fmask, (hipStream_t)stream);
  if (P.D == 128) return dense_fwd_launch<128, true>(P, q, k, v, out, lse, nullptr, idx, fmask, (hipStream_t)stream);
  return NSA_E_UNSUPPORTED;
}

template <int D>
static int dense_bwd_launch(const DensePlan& P, const void* q, const void* k, const void* v, const void* out, const void* dout, const float* lse,
                            void* ws, void* dq, void* dk, void* dv, hipStream_t st) {
  float* delta = reinterpret_cast<float*>((char*)ws + P.off_delta);
  float* part = reinterpret_cast<float*>((char*)ws + P.off_part);
  const int qpw = 4 * (32 >> P.lg);
  hipLaunchKernelGGL((dense_bwd_dq_kernel<D>), dim3(P.mode == 0 ? xcd_grid_for((P.n + qpw - 1) / qpw) : (unsigned)((P.n + qpw - 1) / qpw), P.bh), dim3(256), 0, st, P, (const __bf16*)q, (const __bf16*)k,
                     (const __bf16*)v, (const __bf16*)out, (const __bf16*)dout, lse, delta, (__bf16*)dq);      // also writes delta
  NSA_LAUNCH_CHECK();
  const auto group_span = [&](const long* st) { return (long)(P.g - 1) * st[1] + (long)(P.n - 1) * st[2] + D; };
  // the pipelined kernel's buffer loads take 32-bit byte offsets within one kv head's query heads (rows) and their lse / delta
  if (D >= NSA_DKV_PIPE_MIN_D && group_span(P.sq) < (1l << 30) && group_span(P.sdo) < (1l << 30) && (long)P.g * P.n < (1l << 29))
    hipLaunchKernelGGL((dense_bwd_dkv_pipe_kernel<D>), dim3(dkv_grid(P), P.bh), dim3(128), 0, st, P, (const __bf16*)q, (const __bf16*)k,
                       (const __bf16*)v, (const __bf16*)dout, lse, delta, part);
  else
    hipLaunchKernelGGL((dense_bwd_dkv_kernel<D>), dim3(dkv_grid(P), P.bh), dim3(128), 0, st, P, (const __bf16*)q, (const __bf16*)k,
                       (const __bf16*)v, (const __bf16*)dout, lse, delta, part);
  NSA_LAUNCH_CHECK();
  hipLaunchKernelGGL((dense_bwd_dkv_reduce_kernel<D>), dim3(P.key_tiles, P.bh), dim3(256), 0, st, P, part, dk, dv);
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
