// Block-selection attention for gfx950, walked KV-block by KV-block.
//
// The reference kernel (TRI.py:73-484) is query-centric: every 16-query tile re-gathers the
// S selected K/V blocks of each of its queries, so a K/V block is fetched once per (query,
// slot) pair and only the G heads of one query share a fetched key (arithmetic intensity ~G
// flop/byte).  Here the (query, slot) pairs are first counting-sorted by block (the "inverse
// index"); one wavefront then keeps a 64-key K/V block resident in registers as MFMA operands
// and streams through it the queries that selected it, 32 rows (= 32/G pairs x G heads) at a
// time.  Per pair the kernel moves G*d*2 bytes of Q in and a G*d partial result out instead of
// 2*B*d*2 bytes of K/V.  Each pair gets its own locally normalised softmax partial; a second,
// bandwidth-bound kernel merges a query's partials (log-sum-exp merge).  The backward uses the
// same walk: dK/dV of a block accumulate on chip in the wave that owns the block (no atomics),
// dQ partials are merged per query like the forward partials.
//
// The resident K/V block lives in registers as MFMA operands (its transposed form made once per
// work unit with an MFMA against a constant identity operand, make_ident in nsa_common.hpp); the
// streamed Q / dO rows are gathered with coalesced 16-byte loads, staged in row-major LDS tiles
// and read back as row operands or through the LDS transpose load.
#include "nsa_common.hpp"
#include "nsa_select_plan.hpp"

namespace nsa {

// ------------------------------------------------------------------------------- index build

constexpr int kCountChunk = 256;   // queries per counting chunk

__device__ __forceinline__ int read_idx(const void* idx, int is64, size_t pos) {
  if (is64) {
    long long v = reinterpret_cast<const long long*>(idx)[pos];
    return (v < 0 || v > 0x7fffffffLL) ? -1 : (int)v;
  }
  return reinterpret_cast<const int*>(idx)[pos];
}

// cnt[bh][chunk][j] = number of live slots of the chunk's queries that name block j.  Consecutive lanes take consecutive
// entries of the chunk's [query][slot] run (coalesced), sixteen rounds' loads in flight before the first is used: with up
// to 16 slots per query the whole chunk is one memory round trip.
__global__ __launch_bounds__(256) void sel_count_kernel(const SelPlan P, const void* idx, const uint8_t* fmask, char* iws) {
  extern __shared__ int hist[];
  const int c = blockIdx.x, bh = blockIdx.y, tid = threadIdx.x;
  const int q0 = c * kCountChunk;
  const int total = min(kCountChunk, P.n - q0) * P.S;
  const size_t base = ((size_t)bh * P.n + q0) * P.S;
  constexpr int RK = 16;
  int live[RK], j[RK];
  auto load = [&](int e0) {
#pragma unroll
    for (int r = 0; r < RK; ++r) {
      const int e = e0 + r * 256 + tid, ec = max(0, min(e, total - 1));
      live[r] = e < total ? fmask[base + ec] : 0;
      j[r] = e < total ? read_idx(idx, P.idx64, base + ec) : -1;
    }
  };
  if (total > 0) load(0);
  for (int jj = tid; jj < P.W; jj += 256) hist[jj] = 0;
  __syncthreads();
  for (int e0 = 0; e0 < total; e0 += RK * 256) {
    if (e0 > 0) load(e0);
#pragma unroll
    for (int r = 0; r < RK; ++r)
      if (live[r] && j[r] >= 0 && j[r] < P.W) atomicAdd(&hist[j[r]], 1);     // integer LDS counter: order-independent
  }
  __syncthreads();
  int* cnt = reinterpret_cast<int*>(iws + P.off_cnt) + ((size_t)bh * P.nch + c) * P.W;
  for (int jj = tid; jj < P.W; jj += 256) cnt[jj] = hist[jj];
}

// exclusive scan over the counting chunks of every block (in place in cnt) and over blocks
// (blk_off)
__global__ __launch_bounds__(256) void sel_scan_kernel(const SelPlan P, char* iws) {
  extern __shared__ int tot[];
  const int bh = blockIdx.x, tid = threadIdx.x;
  int* cnt = reinterpret_cast<int*>(iws + P.off_cnt) + (size_t)bh * P.nch * P.W;
  for (int j = tid; j < P.W; j += 256) {
    int run = 0;
    // chunks in batches of 16 whose loads are independent (one memory round trip per batch, not per chunk)
    for (int c0 = 0; c0 < P.nch; c0 += 16) {
      int t[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) t[u] = (c0 + u < P.nch) ? cnt[(size_t)(c0 + u) * P.W + j] : 0;
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        if (c0 + u < P.nch) cnt[(size_t)(c0 + u) * P.W + j] = run;
        run += t[u];
      }
    }
    tot[j] = run;
  }
  __syncthreads();
  // exclusive scan of tot[] over the blocks: per-thread serial over a contiguous slice, then the slice sums
  __shared__ int slice[256];
  const int per = (P.W + 255) / 256;
  const int lo = min(P.W, tid * per), hi = min(P.W, lo + per);
  int sum = 0;
  for (int j = lo; j < hi; ++j) sum += tot[j];
  slice[tid] = sum;
  __syncthreads();
  if (tid == 0) {
    int acc = 0;
    for (int k = 0; k < 256; ++k) { const int v = slice[k]; slice[k] = acc; acc += v; }
  }
  __syncthreads();
  int* blk = reinterpret_cast<int*>(iws + P.off_blk) + (size_t)bh * (P.W + 1);
  int acc = slice[tid];
  for (int j = lo; j < hi; ++j) { blk[j] = acc; acc += tot[j]; }
  if (hi == P.W && lo < hi) blk[P.W] = acc;
  if (P.W == 0 && tid == 0) blk[0] = 0;
}

// pairs of cell (phase p, block j) of table t: own queries (if the block lies in the phase and
// the call is causal) followed by the block's list entries whose query is in the phase
struct CellInfo { int own, first, count; };

__device__ __forceinline__ CellInfo cell_info(const SelPlan& P, const char* iws, int bh, int t, int p, int j) {
  const int* cnt = reinterpret_cast<const int*>(iws + P.off_cnt) + (size_t)bh * P.nch * P.W;
  const int* blk = reinterpret_cast<const int*>(iws + P.off_blk) + (size_t)bh * (P.W + 1);
  const int totj = blk[j + 1] - blk[j];
  const int cpp = P.phase[t] / kCountChunk;                 // counting chunks per phase
  const int c0 = p * cpp, c1 = c0 + cpp;
  const int s0 = c0 < P.nch ? cnt[(size_t)c0 * P.W + j] : totj;
  const int s1 = c1 < P.nch ? cnt[(size_t)c1 * P.W + j] : totj;
  CellInfo ci;
  ci.first = blk[j] + s0;
  ci.count = s1 - s0;
  const long k0 = (long)j * P.B, ph0 = (long)p * P.phase[t];
  ci.own = (P.causal && k0 >= ph0 && k0 < ph0 + P.phase[t]) ? min(P.B, P.n - j * P.B) : 0;
  return ci;
}

// unit_off[t][bh][cell] = exclusive prefix sum of ceil(pairs(cell) / chunk[t]), cells phase-major
__global__ __launch_bounds__(1024) void sel_units_kernel(const SelPlan P, char* iws) {
  __shared__ int wave_tot[16];
  __shared__ int total_s;
  const int bh = blockIdx.x, t = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cells = P.np[t] * P.W;
  int* uo = reinterpret_cast<int*>(iws + P.off_unit[t]) + (size_t)bh * (cells + 1);
  const int per = (cells + 1023) / 1024;
  const int lo = min(cells, tid * per), hi = min(cells, lo + per);
  // (phase, block) of a cell are carried along instead of divided out; chunk[] is a power of two.  The kernel is a handful
  // of waves and a chain of dependent loads: the cell records of a thread's first cells are kept for the second pass
  // instead of fetched again.
  const int csh = 31 - __clz(P.chunk[t]);
  constexpr int KEEP = 8;
  CellInfo kept[KEEP];
  int sum = 0;
  {
    int pp = lo / P.W, j = lo % P.W;
#pragma unroll
    for (int u = 0; u < KEEP; ++u) {
      kept[u] = CellInfo{0, 0, 0};
      if (lo + u < hi) {
        kept[u] = cell_info(P, iws, bh, t, pp, j);
        sum += (kept[u].own + kept[u].count + P.chunk[t] - 1) >> csh;
        if (++j == P.W) { j = 0; ++pp; }
      }
    }
    for (int c = lo + KEEP; c < hi; ++c) {
      const CellInfo ci = cell_info(P, iws, bh, t, pp, j);
      sum += (ci.own + ci.count + P.chunk[t] - 1) >> csh;
      if (++j == P.W) { j = 0; ++pp; }
    }
  }
  // exclusive scan of the threads' sums over the work-group: inside a wave by shuffles, then the 16 wave totals
  int incl = sum;
  for (int dlt = 1; dlt < 64; dlt <<= 1) {
    const int y = __shfl_up(incl, dlt, 64);
    if (lane >= dlt) incl += y;
  }
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  if (wave == 0) {
    const int tw = lane < 16 ? wave_tot[lane] : 0;
    int xs = tw;
    for (int dlt = 1; dlt < 16; dlt <<= 1) {
      const int y = __shfl_up(xs, dlt, 64);
      if (lane >= dlt) xs += y;
    }
    if (lane < 16) wave_tot[lane] = xs - tw;
    if (lane == 15) { total_s = xs; uo[cells] = xs; }
  }
  __syncthreads();
  // besides the prefix sums, one record per unit: a walk's work-group then finds its unit with one
  // load instead of a binary search over the prefix sums (a dozen dependent loads at one wave per SIMD)
  int4* rec = reinterpret_cast<int4*>(iws + P.off_urec[t]) + (size_t)bh * P.ub[t] * 2;
  int acc = incl - sum + wave_tot[wave];
  {
    int pp = lo / P.W, j = lo % P.W;
    auto emit = [&](int c, const CellInfo& ci) {
      uo[c] = acc;
      const int L = ci.own + ci.count, nu = (L + P.chunk[t] - 1) >> csh;
      for (int k = 0; k < nu; ++k) {
        rec[2 * (acc + k)] = int4{j, ci.own, ci.first, k << csh};
        rec[2 * (acc + k) + 1] = int4{min(L, (k + 1) << csh), 0, 0, 0};
      }
      acc += nu;
      if (++j == P.W) { j = 0; ++pp; }
    };
#pragma unroll
    for (int u = 0; u < KEEP; ++u)
      if (lo + u < hi) emit(lo + u, kept[u]);
    for (int c = lo + KEEP; c < hi; ++c) emit(c, cell_info(P, iws, bh, t, pp, j));
  }
  for (int u = total_s + tid; u < P.ub[t]; u += 1024) {       // padding units: empty range
    rec[2 * u] = int4{0, 0, 0, 0};
    rec[2 * u + 1] = int4{0, 0, 0, 0};
  }
}

// NW waves per work-group, each with a quarter (NW = 4) of the chunk's queries: a wave's entries are ranked 64 at a time, one
// dependent round per 64 entries, so the rounds of a chunk run four abreast.  The waves' starting positions inside a block's
// run of the chunk come from a count of each wave's entries first (integer LDS counters again); the lists are the same as
// one wave walking the whole chunk would write.  NW = 1 where 5 W counters do not fit the 64 KB of LDS a launch may ask for.
template <int NW>
__global__ __launch_bounds__(64 * NW) void sel_fill_kernel(const SelPlan P, const void* idx, const uint8_t* fmask, char* iws) {
  extern __shared__ int base_all[];              // [NW][W]: where wave w's next entry of block j goes
  const int c = blockIdx.x, bh = blockIdx.y, lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int* cnt = reinterpret_cast<const int*>(iws + P.off_cnt) + ((size_t)bh * P.nch + c) * P.W;
  const int* blk = reinterpret_cast<const int*>(iws + P.off_blk) + (size_t)bh * (P.W + 1);
  int* list = reinterpret_cast<int*>(iws + P.off_list) + (size_t)bh * P.list_cap;
  int* base = base_all + w * P.W;
  const int q0c = c * kCountChunk;
  const int nqc = min(kCountChunk, P.n - q0c);
  constexpr int QW = kCountChunk / NW;           // queries per wave
  const int q0 = q0c + w * QW;
  const int nq = max(0, min(QW, q0c + nqc - q0));
  const int total = nq * P.S;
  const size_t pos0 = ((size_t)bh * P.n + q0) * P.S;
  // The wave's first RK rounds of entries (all of them with up to 16 slots per query and four waves) are fetched at once and
  // stay in registers: one memory round trip for the count and the ranking together, instead of one per round.
  constexpr int RK = 16;
  int live[RK], jv[RK];
#pragma unroll
  for (int r = 0; r < RK; ++r) {
    const int e = r * 64 + lane, ec = max(0, min(e, total - 1));
    live[r] = e < total ? fmask[pos0 + ec] : 0;
    jv[r] = e < total ? read_idx(idx, P.idx64, pos0 + ec) : -1;
    if (jv[r] >= P.W) jv[r] = -1;
  }
  if (NW > 1) {
    for (int j = threadIdx.x; j < NW * P.W; j += 64 * NW) base_all[j] = 0;
    __syncthreads();
#pragma unroll
    for (int r = 0; r < RK; ++r)
      if (live[r] && jv[r] >= 0) atomicAdd(&base[jv[r]], 1);
    for (int e0 = RK * 64; e0 < total; e0 += 64) {
      const int e = e0 + lane;
      if (e < total && fmask[pos0 + e]) {
        const int j = read_idx(idx, P.idx64, pos0 + e);
        if (j >= 0 && j < P.W) atomicAdd(&base[j], 1);
      }
    }
    __syncthreads();
    // counts -> starting positions: the block's run, the chunk's offset in it, the waves before this one
    for (int j = threadIdx.x; j < P.W; j += 64 * NW) {
      int run = blk[j] + cnt[j];
#pragma unroll
      for (int w2 = 0; w2 < NW; ++w2) { const int v = base_all[w2 * P.W + j]; base_all[w2 * P.W + j] = run; run += v; }
    }
    __syncthreads();
  } else {
    for (int j = lane; j < P.W; j += 64) base[j] = blk[j] + cnt[j];
    __syncthreads();
  }
  if (total <= 0) return;
  // (from here on a wave is on its own - the waves of a partial chunk have different numbers of rounds - and touches only its
  // own row of counters.  A wave's LDS operations execute in the order they were issued, so all that has to be kept is the
  // compiler's order of them; a fence would also wait for the list stores in flight, one memory round trip per round.)
  auto wave_sync = [] { asm volatile("" ::: "memory"); };
  const int nbits = 32 - __builtin_clz((unsigned)max(P.W - 1, 1));      // bits of a block index
  // one round: the 64 entries e0 + lane; j = the lane's block (-1: no entry, dead slot or block out of range)
  auto round = [&](int e0, int j) {
    const int e = e0 + lane;
    const int entry = (q0 + e / P.S) * P.SP + e % P.S;
    // lanes of this pass that name the same block: intersect, bit by bit of the block index, the ballots of the lanes
    // that agree with this lane (about 10 ballots instead of 64 lane reads); dead lanes are masked out
    unsigned long long same_m = __ballot(j >= 0);
    for (int bit = 0; bit < nbits; ++bit) {
      const bool one = (j >> bit) & 1;
      const unsigned long long bal = __ballot(one);
      same_m &= one ? bal : ~bal;
    }
    const int rank = __popcll(same_m & ((1ull << lane) - 1ull));
    const int same = __popcll(same_m);
    if (j >= 0) list[base[j] + rank] = entry;
    wave_sync();
    if (j >= 0 && rank == same - 1) base[j] += same;
    wave_sync();
  };
#pragma unroll
  for (int r = 0; r < RK; ++r)
    if (r * 64 < total) round(r * 64, live[r] ? jv[r] : -1);
  // what does not fit the registers (more than 16 slots per query, or one wave for the whole chunk): fetched two rounds
  // ahead of their use (branch-free, from a clamped position) - a round is otherwise one dependent global load long
  if (total > RK * 64) {
    struct Fetched { int live, j; };
    auto fetch = [&](int e0) {
      const int e = min(e0 + lane, total - 1);
      Fetched f;
      f.live = fmask[pos0 + e];
      f.j = read_idx(idx, P.idx64, pos0 + e);
      return f;
    };
    Fetched f0 = fetch(RK * 64), f1 = fetch(RK * 64 + 64);
    for (int e0 = RK * 64; e0 < total; e0 += 64) {
      const Fetched cur = f0;
      f0 = f1;
      f1 = fetch(e0 + 128);
      int j = -1;
      if (e0 + lane < total && cur.live) j = cur.j >= P.W ? -1 : cur.j;
      round(e0, j);
    }
  }
}

// --------------------------------------------------------------------------- shared pieces

struct UnitInfo {
  int j, own, lst0, v0, v1;
};

// unit u of table t -> (block j, range [v0, v1) of the cell's virtual list: `own` own-block
// positions first, then list[lst0 ...]).  Returns false for padding units.
__device__ __forceinline__ bool locate_unit(const SelPlan& P, const char* iws, int t, int bh, int u, UnitInfo& ui) {
  const int4* rec = reinterpret_cast<const int4*>(iws + P.off_urec[t]) + ((size_t)bh * P.ub[t] + u) * 2;
  const int4 r0 = rec[0], r1 = rec[1];
  ui.j = r0.x;
  ui.own = r0.y;
  ui.lst0 = r0.z;                         // index into the per-(batch, head) list
  ui.v0 = r0.w;
  ui.v1 = r1.x;
  return ui.v0 < ui.v1;
}

// the dK/dV walk's table has one phase: unit_off[bh][j] .. unit_off[bh][j + 1] are block j's units
__device__ __forceinline__ bool block_has_one_unit(const SelPlan& P, const char* iws, int bh, int j) {
  const int* unit_off = reinterpret_cast<const int*>(iws + P.off_unit[2]) + (size_t)bh * (P.W + 1);
  return unit_off[j + 1] - unit_off[j] == 1;
}

// Work-group id -> (batch*kv head, unit) such that all units of one head run, in table order,
// on as few XCDs as possible (consecutive work-group ids go round-robin over the 8 XCDs), so
// that the Q rows of a query phase are fetched into one L2 only.
__device__ __forceinline__ bool xcd_map(const SelPlan& P, int t, int& bh, int& u) {
  const int w = blockIdx.x, x = w & 7, tt = w >> 3;
  if (P.bh >= 8) {
    bh = x + 8 * (tt / P.ub[t]);
    u = tt % P.ub[t];
    return bh < P.bh;
  }
  bh = x % P.bh;
  const int sub = x / P.bh, nsub = (8 - bh + P.bh - 1) / P.bh;
  u = tt * nsub + sub;
  return u < P.ub[t];
}

static inline unsigned xcd_grid(const SelPlan& P, int t) {
  if (P.bh >= 8) return 8u * (unsigned)P.ub[t] * (unsigned)((P.bh + 7) / 8);
  const int nsub_min = 8 / P.bh;
  return 8u * (unsigned)((P.ub[t] + nsub_min - 1) / nsub_min);
}

struct RowInfo {
  int i, slot, lim, g;
  bool valid;
};

// Row `nrow` (0..31) of the 32-row tile starting at virtual position vt, in two stages so that
// the list entry (a dependent global load) is fetched tiles ahead of its use.  The fetch is
// branch-free (it always loads, from a clamped index) so that no wait is forced at a join.
struct RawEntry {
  int raw, pvc;
  bool valid;
};

__device__ __forceinline__ RawEntry fetch_entry(const SelPlan& P, const int* list, const UnitInfo& ui, int vt, int nrow) {
  RawEntry e;
  const int pv = vt + (nrow >> P.lg);
  e.valid = pv < ui.v1;
  e.pvc = min(pv, ui.v1 - 1);
  long li = (long)ui.lst0 + max(e.pvc - ui.own, 0);
  li = li < P.list_cap ? li : P.list_cap - 1;
  e.raw = list[li];
  return e;
}

__device__ __forceinline__ RowInfo decode_entry(const SelPlan& P, const UnitInfo& ui, const RawEntry& e, int nrow) {
  RowInfo r;
  r.valid = e.valid;
  r.g = nrow & (P.g - 1);
  const bool own = e.pvc < ui.own;
  const int qi = e.raw / P.SP;
  r.i = own ? ui.j * P.B + e.pvc : qi;
  r.slot = own ? P.S : e.raw - qi * P.SP;
  r.lim = own ? e.pvc : P.B - 1;
  return r;
}

// Coalesced gather of a 32-row tile: row rr = (pair rr >> lg of the tile, head rr & (G-1)).
// Each load instruction covers 64 / (D/8) whole rows (16 bytes per lane, consecutive lanes
// consecutive addresses), which the texture path handles several times faster than 32 rows x
// 32 bytes.  `my_i` is the query index of row (lane % 32); `base` points at the first head of
// the kv group.  The data goes to registers first (so that it can be in flight during the
// previous tile's compute) and is committed to a row-major LDS tile later.
template <int D>
__device__ __forceinline__ void issue_tile_loads(bf16x8 (&raw)[D / 16], const __bf16* __restrict__ base, long s_head, long s_tok, int my_i,
                                                 int gmask, int lane) {
  constexpr int CPR = D / 8, RPI = 64 / CPR, NT = 32 / RPI;
  static_assert(NT == D / 16, "tile load count");
  // all lane exchanges first, then all loads: taken in turn, every load would wait for its own exchange
  int qi[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) qi[t] = __shfl(my_i, t * RPI + lane / CPR, 64);
  // the head and token strides are below 2^32 (checked when the plan is made): 32 x 32 -> 64-bit multiply-adds
  const unsigned sh32 = (unsigned)s_head, st32 = (unsigned)s_tok;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int rr = t * RPI + lane / CPR, c = lane % CPR;
    const unsigned long off = (unsigned long)(unsigned)(rr & gmask) * sh32 + (unsigned long)(unsigned)qi[t] * st32;
    raw[t] = load8(base + off + 8 * c);
  }
}

template <int D>
__device__ __forceinline__ void commit_tile(const bf16x8 (&raw)[D / 16], __bf16* tile_s, int RS, int lane) {
  constexpr int CPR = D / 8, RPI = 64 / CPR, NT = 32 / RPI;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int rr = t * RPI + lane / CPR, c = lane % CPR;
    *reinterpret_cast<bf16x8*>(tile_s + rr * RS + 8 * c) = raw[t];
  }
}

// the same into a swizzled tile (lds_swz_off: conflict-free for row reads and for the transpose load)
template <int D>
__device__ __forceinline__ void commit_tile_swz(const bf16x8 (&raw)[D / 16], __bf16* tile_s, int lane) {
  constexpr int CPR = D / 8, RPI = 64 / CPR, NT = 32 / RPI;
#pragma unroll
  for (int t = 0; t < NT; ++t) *reinterpret_cast<bf16x8*>(tile_s + lds_swz_off<D>(t * RPI + lane / CPR, lane % CPR)) = raw[t];
}

// Write a wave's 32-row x D accumulator tile (transposed MFMA layout: lane <-> row n_,
// register (dt, a, b) <-> feature 32dt + 8a + 4h + b) as bf16 rows through LDS, so that every
// global store instruction covers whole 2*D-byte rows (16 bytes per lane, consecutive lanes
// consecutive addresses) instead of 8-byte pieces of 32 different rows.  `row` is this lane's
// destination row index into dst (rows of D elements); `scale` multiplies the values.
// One wave per work-group: LDS operations of a wave execute in order, the barriers only keep the
// compiler from reordering.
template <int D>
__device__ __forceinline__ void store_tile_rows(const floatx16 (&acc)[D / 32], float scale, size_t row, __bf16* __restrict__ dst,
                                                __bf16* tile_s, size_t* row_s, int lane) {
  constexpr int DT = D / 32, RS = D + 8;          // padded LDS row stride in elements
  constexpr int CPR = D / 8, RPI = 64 / CPR;      // 16-byte chunks per row, rows per store instruction
  const int n_ = lane & 31, h = lane >> 5;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      bf16x4 r;
#pragma unroll
      for (int bb = 0; bb < 4; ++bb) r[bb] = (__bf16)(acc[dt][4 * a + bb] * scale);
      *reinterpret_cast<bf16x4*>(tile_s + n_ * RS + 32 * dt + 8 * a + 4 * h) = r;
    }
  if (h == 0) row_s[n_] = row;
  __syncthreads();
  // all LDS reads first, then all stores: taken in turn, every store would wait for its own read
  bf16x8 v[32 / RPI];
  size_t rw[32 / RPI];
#pragma unroll
  for (int t = 0; t < 32 / RPI; ++t) {
    const int rr = t * RPI + lane / CPR, c = lane % CPR;
    v[t] = *reinterpret_cast<const bf16x8*>(tile_s + rr * RS + 8 * c);
    rw[t] = row_s[rr];
  }
#pragma unroll
  for (int t = 0; t < 32 / RPI; ++t)
    __builtin_nontemporal_store(v[t], reinterpret_cast<bf16x8*>(dst + rw[t] * D + 8 * (lane % CPR)));
  __syncthreads();
}

// ------------------------------------------------------------------------------- forward

#ifndef NSA_FWD_STAGES
#define NSA_FWD_STAGES 2      // measured on MI355X (seq 32k, d 128): 1 stage 1.47 ms, 2 stages 1.445 ms
#endif
template <int D, int KT>
__global__ __launch_bounds__(64) void sel_fwd_kernel(const SelPlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                     const __bf16* __restrict__ v, const char* __restrict__ iws, char* __restrict__ fws) {
  constexpr int KS = D / 16, DT = D / 32, TBL = 0;
  constexpr int RS = D + 8;
  __shared__ __align__(16) __bf16 tile_s[32 * RS];    // output staging
  __shared__ __align__(16) __bf16 xq_s[32 * RS];      // the tile's Q rows
  __shared__ size_t row_s[32];
  const int lane = threadIdx.x, n_ = lane & 31, h = lane >> 5;
  int bh, u;
  if (!xcd_map(P, TBL, bh, u)) return;
  const int b = bh / P.hkv, hk = bh % P.hkv;
  UnitInfo ui;
  if (!locate_unit(P, iws, TBL, bh, u, ui)) return;
  const int* list = reinterpret_cast<const int*>(iws + P.off_list) + (size_t)bh * P.list_cap;

  // Set-up in three memory round trips: (1) the unit record above, (2) the first list entries, the
  // block's K rows and its V rows, all requested before anything waits, (3) the first Q gathers,
  // requested as soon as the entries are there and in flight while V is transposed.  At one wave
  // per SIMD every dependent load here is exposed latency, and a unit is only a few dozen tiles.
  const int ppt = 32 >> P.lg;
  constexpr int NS = NSA_FWD_STAGES;
  RawEntry e0[NS];
#pragma unroll
  for (int s2 = 0; s2 < NS; ++s2) e0[s2] = fetch_entry(P, list, ui, ui.v0 + s2 * ppt, n_);
  RawEntry e_n = fetch_entry(P, list, ui, ui.v0 + NS * ppt, n_);
  __builtin_amdgcn_sched_barrier(0);

  bf16x8 Kf[KT][KS];
  bf16x8 Vraw[KT][DT][2];
#pragma unroll
  for (int kt = 0; kt < KT; ++kt) {
    const int kl = 32 * kt + n_;
    const long key = (long)ui.j * P.B + kl;
    const bool ok = kl < P.B && key < P.n;
    const long keyc = ok ? key : 0;
    const __bf16* kp = k + b * P.sk[0] + hk * P.sk[1] + keyc * P.sk[2] + 8 * h;
    const __bf16* vp = v + b * P.sv[0] + hk * P.sv[1] + keyc * P.sv[2] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) Kf[kt][ks] = ok ? load8(kp + 16 * ks) : zero_frag();
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      Vraw[kt][dt][0] = ok ? load8(vp + 32 * dt) : zero_frag();
      Vraw[kt][dt][1] = ok ? load8(vp + 32 * dt + 16) : zero_frag();
    }
  }
  __builtin_amdgcn_sched_barrier(0);

  __bf16* opart = reinterpret_cast<__bf16*>(fws + P.off_opart);
  float* lsepart = reinterpret_cast<float*>(fws + P.off_lsepart);
  const float sc = P.scale * kLog2e;

  // software pipeline: NS tiles of Q rows (coalesced gathers) in flight, list entries one more tile
  // ahead; a stage's registers take the loads of the tile NS steps ahead once it is committed to LDS
  const __bf16* qbase = q + b * P.sq[0] + (long)(hk * P.g) * P.sq[1];
  struct Stage {
    RowInfo r;
    bf16x8 raw[KS];
  };
  Stage stg[NS];
#pragma unroll
  for (int s2 = 0; s2 < NS; ++s2) {
    stg[s2].r = decode_entry(P, ui, e0[s2], n_);
    issue_tile_loads<D>(stg[s2].raw, qbase, P.sq[1], P.sq[2], stg[s2].r.i, P.g - 1, lane);
  }
  __builtin_amdgcn_sched_barrier(0);

  bf16x8 VT[DT][KT][2];
  {
    bf16x8 ilo, ihi;
    make_ident(lane, ilo, ihi);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        floatx16 t = mfma32(Vraw[kt][dt][0], ilo, zero_acc());
        t = mfma32(Vraw[kt][dt][1], ihi, t);
        VT[dt][kt][0] = pack8(t, 0);
        VT[dt][kt][1] = pack8(t, 8);
      }
  }

  wait_all_loads();        // enter the loop with nothing pending, so the loop itself only waits for what it needs
  auto step = [&](int vt, Stage& cur) {
    const RowInfo r = cur.r;
    commit_tile<D>(cur.raw, xq_s, RS, lane);
    __syncthreads();
    // the list entry is fetched before the row gathers that follow it: the wait for an entry (memory
    // operations retire in order) then never covers the gathers issued in the same step
    cur.r = decode_entry(P, ui, e_n, n_);
    e_n = fetch_entry(P, list, ui, vt + (NS + 1) * ppt, n_);
    __builtin_amdgcn_sched_barrier(0);
    issue_tile_loads<D>(cur.raw, qbase, P.sq[1], P.sq[2], cur.r.i, P.g - 1, lane);
    __builtin_amdgcn_sched_barrier(0);

    bf16x8 Qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) Qf[ks] = lds_row_operand(xq_s, RS, ks, lane);
    floatx16 Sa[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      Sa[kt] = zero_acc();
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) Sa[kt] = mfma32(Kf[kt][ks], Qf[ks], Sa[kt]);
    }
    // local softmax over the block's keys; this lane holds 16*KT keys of row n_, lane^32 the rest.  The maximum is
    // taken over the raw scores (the scale is positive) and the scale folded into the exponent's multiply-add; a tile
    // whose rows all see the whole block (every tile but the own-block ones) skips the key mask (wave-uniform)
    const bool whole = __all(r.lim >= 32 * KT - 1);
    float mx = -INFINITY;
    if (!whole) {
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i2 = 0; i2 < 16; ++i2) {
          const int kl = 32 * kt + 8 * (i2 >> 2) + 4 * h + (i2 & 3);
          if (kl > r.lim) Sa[kt][i2] = -INFINITY;
        }
    }
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i2 = 0; i2 < 16; ++i2) mx = fmaxf(mx, Sa[kt][i2]);
    mx = halves_max(mx);
    const float mxs = mx * sc;                       // the row maximum in the exponent's units (log2)
    float l = 0.f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i2 = 0; i2 < 16; ++i2) {
        const float p = fast_exp2(__builtin_fmaf(Sa[kt][i2], sc, -mxs));
        Sa[kt][i2] = p;
        l += p;
      }
    l = halves_sum(l);
    // normalise the probabilities (32 values) rather than the output tile (64)
    const float inv = 1.0f / l;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i2 = 0; i2 < 16; ++i2) Sa[kt][i2] *= inv;

    floatx16 Oa[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) Oa[dt] = zero_acc();
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int u2 = 0; u2 < 2; ++u2) {
        const bf16x8 Pf = pack8(Sa[kt], 8 * u2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) Oa[dt] = mfma32(VT[dt][kt][u2], Pf, Oa[dt]);
      }

    {
      // padding rows write to a spare row at the end of the buffers: the stores stay
      // unconditional, so the wait for the next tile's loads never has to cover them
      const size_t row = r.valid ? (((size_t)bh * P.n + r.i) * P.SP + r.slot) * P.g + r.g : P.prow;
      store_tile_rows<D>(Oa, 1.0f, row, opart, tile_s, row_s, lane);
      if (h == 0) lsepart[row] = (mxs + fast_log2(l)) * kLn2;
    }
  };
  // whole rounds of NS tiles first: their steps are unconditional, so each wait counts exactly the
  // memory operations issued after the loads it needs
  int vt = ui.v0;
  if (vt + (NS - 1) * ppt < ui.v1) {
    wait_all_loads();      // again: the compiler sinks the later stages' first loads to here, past the wait above
    do {
#pragma unroll
      for (int s2 = 0; s2 < NS; ++s2) step(vt + s2 * ppt, stg[s2]);
      vt += NS * ppt;
    } while (vt + (NS - 1) * ppt < ui.v1);
  }
#pragma unroll
  for (int s2 = 0; s2 < NS - 1; ++s2)
    if (vt + s2 * ppt < ui.v1) step(vt + s2 * ppt, stg[s2]);
}

// live-slot bitmask of query (bh, i): bit s < S = selected slot s, bit S = own block.  `sub` is the lane's index inside the
// group of lanes that serves the query (the whole wave, or one half of it when two queries share a wave: half = 0 / 1)
__device__ __forceinline__ unsigned long long live_slots(const SelPlan& P, const void* idx, const uint8_t* fmask, int bh, int i, int sub, int half, bool two) {
  bool ok = false;
  if (sub < P.S) {
    const size_t pos = ((size_t)bh * P.n + i) * P.S + sub;
    if (fmask[pos]) {
      const int j = read_idx(idx, P.idx64, pos);
      ok = j >= 0 && j < P.W;
    }
  } else if (sub == P.S) {
    ok = P.causal != 0;
  }
  const unsigned long long bal = __ballot(ok);
  return two ? ((bal >> (32 * half)) & 0xffffffffull) : bal;
}

// Queries per wave of the merge kernels: a query's partial row is G * D / 8 chunks of 16 bytes, one per lane; when that is
// at most half a wave (d = 64 with G <= 4) and the slots fit 32 mask bits, two queries share a wave instead of idling half of it.
__host__ __device__ __forceinline__ bool merge_two_per_wave(const SelPlan& P, int cpr) { return P.g * cpr <= 32 && P.SP <= 32; }

// slots whose loads a merge round issues together (measured at seq 32k, d 128, 16 slots: forward merge 0.819 / 0.825 / 0.790 /
// 0.815 ms for 1 / 2 / 4 / 8, dQ merge 0.757 / 0.783 / 0.794 / 0.801 ms: the merges stream at what the memory gives
// non-temporal reads, about 6 TB/s, and more rows in flight per wave only help the one that also has exponentials to hide)
#ifndef NSA_MERGE_BATCH
#define NSA_MERGE_BATCH 4
#endif
#ifndef NSA_MERGE_BATCH_BWD
#define NSA_MERGE_BATCH_BWD 1
#endif
// merge the per-slot partials of one query: out = sum_s exp(lse_s - LSE) * o_s
template <int D>
__global__ __launch_bounds__(256) void sel_fwd_combine_kernel(const SelPlan P, const void* idx, const uint8_t* fmask, const char* __restrict__ fws,
                                                             __bf16* __restrict__ out, float* __restrict__ lse) {
  constexpr int CPR = D / 8;                    // 16-byte chunks per row
  const bool two = merge_two_per_wave(P, CPR);
  const int lane = threadIdx.x & 63, half = two ? lane >> 5 : 0, sub = two ? lane & 31 : lane, width = two ? 32 : 64;
  const long qi = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * (two ? 2 : 1) + half;
  if (qi >= (long)P.bh * P.n) return;
  const int bh = (int)(qi / P.n), i = (int)(qi % P.n);
  const int b = bh / P.hkv, hk = bh % P.hkv;
  const unsigned long long live = live_slots(P, idx, fmask, bh, i, sub, half, two);
  const __bf16* opart = reinterpret_cast<const __bf16*>(fws + P.off_opart);
  const float* lsepart = reinterpret_cast<const float*>(fws + P.off_lsepart);
  for (int c = sub; c < P.g * CPR; c += width) {
    const int g = c / CPR, dd = (c % CPR) * 8;
    const size_t row0 = ((size_t)bh * P.n + i) * P.SP * P.g + g;
    // one pass, streaming log-sum-exp merge: acc = sum_s exp(lse_s - m) * o_s, rescaled as m grows
    float mx = -INFINITY, sum = 0.f;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    // NSA_MERGE_BATCH slots per round, their loads issued together: one row in flight per wave leaves the memory system
    // waiting for the waves (a round is then one memory latency long).  A round's spare entries repeat its last live slot
    // with weight zero.
    for (unsigned long long m = live; m;) {
      size_t row[NSA_MERGE_BATCH];
      bool ok[NSA_MERGE_BATCH];
#pragma unroll
      for (int j = 0; j < NSA_MERGE_BATCH; ++j) {
        ok[j] = m != 0;
        if (ok[j]) { row[j] = row0 + (size_t)__builtin_ctzll(m) * P.g; m &= m - 1; }
        else row[j] = row[j > 0 ? j - 1 : 0];
      }
      float ls[NSA_MERGE_BATCH];
      bf16x8 o[NSA_MERGE_BATCH];
#pragma unroll
      for (int j = 0; j < NSA_MERGE_BATCH; ++j) {
        ls[j] = __builtin_nontemporal_load(lsepart + row[j]);
        o[j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(opart + row[j] * D + dd));
      }
#pragma unroll
      for (int j = 0; j < NSA_MERGE_BATCH; ++j) {
        const float lj = ok[j] ? ls[j] : -INFINITY;
        const float mn = fmaxf(mx, lj);
        const float a = __expf(mx - mn), w = __expf(lj - mn);      // first slot: mx = -inf -> a = 0; spare entry: w = 0
        sum = sum * a + w;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = acc[e] * a + w * (float)o[j][e];
        mx = mn;
      }
    }
    const float L = live ? mx + __logf(sum) : -INFINITY;
    const float inv = live ? 1.0f / sum : 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= inv;
    const int hq = hk * P.g + g;
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (__bf16)acc[e];
    *reinterpret_cast<bf16x8*>(out + b * P.so[0] + (long)hq * P.so[1] + (long)i * P.so[2] + dd) = r;
    if (dd == 0) lse[((size_t)b * P.hkv * P.g + hq) * P.n + i] = L;
  }
}

// ------------------------------------------------------------------------------ backward

// delta[b,hq,i] = sum_d out * d_out   (TRI.py:696-756), less the gradient of the row's log-sum-exp when the caller has one:
// d loss / d logit_j = p_j (dP_j - sum_k p_k dP_k) + d_lse p_j = p_j (dP_j - (delta - d_lse))
template <int D>
__global__ __launch_bounds__(256) void sel_delta_kernel(const SelPlan P, const __bf16* __restrict__ out, const __bf16* __restrict__ dout,
                                                        const float* __restrict__ dlse, float* __restrict__ delta) {
  constexpr int LPR = D / 8;                   // lanes per row
  constexpr int RPB = 256 / LPR;               // rows per block
  const int tid = threadIdx.x;
  const long row = (long)blockIdx.x * RPB + tid / LPR;
  const long rows = (long)P.bh * P.g * P.n;
  const int dd = (tid % LPR) * 8;
  float s = 0.f;
  if (row < rows) {
    const long i = row % P.n, bhq = row / P.n;
    const long b = bhq / (P.hkv * P.g), hq = bhq % (P.hkv * P.g);
    const long off = b * P.so[0] + hq * P.so[1] + i * P.so[2] + dd;
    // (both rows are read once here and nothing of them is worth a cache line afterwards - the walk that follows gathers its
    // d_out rows in its own order: non-temporal loads, 0.116 -> 0.088 ms at seq 32k, the walk unchanged)
    const bf16x8 o = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(out + off));
    const bf16x8 d = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(dout + off));
#pragma unroll
    for (int e = 0; e < 8; ++e) s += (float)o[e] * (float)d[e];
  }
#pragma unroll
  for (int m = LPR / 2; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
  if (row < rows && (tid % LPR) == 0) delta[row] = dlse ? s - dlse[row] : s;
}

// dQ partial of every (query, slot) pair; same walk and register layout as the forward
// With GATE the kernel also writes sel_grads[b,h,i,slot] = sum over the group's heads and the
// slot's keys of dS * (scaled logit): the gradient of a multiplier of 1 applied to the slot's
// keys (the straight-through top-k gates of NSA.py:715, 793-797; TRI.py:1061-1080).
template <int D, int KT, bool GATE>
__global__ __launch_bounds__(64) void sel_bwd_dq_kernel(const SelPlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                        const __bf16* __restrict__ v, const __bf16* __restrict__ dout,
                                                        const float* __restrict__ lse, const float* __restrict__ delta,
                                                        const char* __restrict__ iws, char* __restrict__ bws, float* __restrict__ sel_grads) {
  constexpr int KS = D / 16, DT = D / 32, TBL = 1;
  constexpr int RS = D + 8;
  __shared__ __align__(16) __bf16 tile_s[32 * RS];    // output staging
  __shared__ __align__(16) __bf16 xq_s[32 * RS];      // the tile's Q rows
  __shared__ __align__(16) __bf16 xg_s[32 * RS];      // the tile's dO rows
  __shared__ size_t row_s[32];
  const int lane = threadIdx.x, n_ = lane & 31, h = lane >> 5;
  int bh, u;
  if (!xcd_map(P, TBL, bh, u)) return;
  const int b = bh / P.hkv, hk = bh % P.hkv;
  UnitInfo ui;
  if (!locate_unit(P, iws, TBL, bh, u, ui)) return;
  const int* list = reinterpret_cast<const int*>(iws + P.off_list) + (size_t)bh * P.list_cap;

  bf16x8 Kf[KT][KS], Vf[KT][KS];
  bf16x8 KTf[DT][KT][2];
  {
    bf16x8 ilo, ihi;
    make_ident(lane, ilo, ihi);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      const int kl = 32 * kt + n_;
      const long key = (long)ui.j * P.B + kl;
      const bool ok = kl < P.B && key < P.n;
      const long keyc = ok ? key : 0;
      const __bf16* kp = k + b * P.sk[0] + hk * P.sk[1] + keyc * P.sk[2] + 8 * h;
      const __bf16* vp = v + b * P.sv[0] + hk * P.sv[1] + keyc * P.sv[2] + 8 * h;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        Kf[kt][ks] = ok ? load8(kp + 16 * ks) : zero_frag();
        Vf[kt][ks] = ok ? load8(vp + 16 * ks) : zero_frag();
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        floatx16 t = mfma32(Kf[kt][2 * dt], ilo, zero_acc());
        t = mfma32(Kf[kt][2 * dt + 1], ihi, t);
        KTf[dt][kt][0] = pack8(t, 0);
        KTf[dt][kt][1] = pack8(t, 8);
      }
    }
  }

  __bf16* dqpart = reinterpret_cast<__bf16*>(bws + P.off_dqpart);
  const float sc = P.scale * kLog2e;
  const int ppt = 32 >> P.lg;
  const int HQ = P.hkv * P.g;

  const __bf16* qbase = q + b * P.sq[0] + (long)(hk * P.g) * P.sq[1];
  const __bf16* gbase = dout + b * P.so[0] + (long)(hk * P.g) * P.so[1];
  RawEntry e_n = fetch_entry(P, list, ui, ui.v0 + ppt, n_);
  RowInfo r = decode_entry(P, ui, fetch_entry(P, list, ui, ui.v0, n_), n_);
  bf16x8 rawq[KS], rawg[KS];
  float lse_r, del_r;
  {
    issue_tile_loads<D>(rawq, qbase, P.sq[1], P.sq[2], r.i, P.g - 1, lane);
    issue_tile_loads<D>(rawg, gbase, P.so[1], P.so[2], r.i, P.g - 1, lane);
    const size_t srow = ((size_t)b * HQ + hk * P.g + r.g) * P.n + r.i;
    lse_r = lse[srow] * kLog2e;
    del_r = delta[srow];
  }

  wait_all_loads();        // enter the loop with nothing pending, so the loop itself only waits for what it needs
  for (int vt = ui.v0; vt < ui.v1; vt += ppt) {
    commit_tile<D>(rawq, xq_s, RS, lane);
    commit_tile<D>(rawg, xg_s, RS, lane);
    __syncthreads();
    const RowInfo rn = decode_entry(P, ui, e_n, n_);
    issue_tile_loads<D>(rawq, qbase, P.sq[1], P.sq[2], rn.i, P.g - 1, lane);
    issue_tile_loads<D>(rawg, gbase, P.so[1], P.so[2], rn.i, P.g - 1, lane);
    float lse_n, del_n;
    {
      const size_t srown = ((size_t)b * HQ + hk * P.g + rn.g) * P.n + rn.i;
      lse_n = lse[srown] * kLog2e;
      del_n = delta[srown];
    }
    const RawEntry e_nn = fetch_entry(P, list, ui, vt + 2 * ppt, n_);
    __builtin_amdgcn_sched_barrier(0);

    bf16x8 Qf[KS], Gf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) { Qf[ks] = lds_row_operand(xq_s, RS, ks, lane); Gf[ks] = lds_row_operand(xg_s, RS, ks, lane); }
    floatx16 Sa[KT], Pa[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      Sa[kt] = zero_acc(); Pa[kt] = zero_acc();
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        Sa[kt] = mfma32(Kf[kt][ks], Qf[ks], Sa[kt]);
        Pa[kt] = mfma32(Vf[kt][ks], Gf[ks], Pa[kt]);
      }
    }
    float gs = 0.f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int i2 = 0; i2 < 16; ++i2) {
        const int kl = 32 * kt + 8 * (i2 >> 2) + 4 * h + (i2 & 3);
        const float sraw = Sa[kt][i2];
        const float p = fast_exp2((kl <= r.lim) ? __builtin_fmaf(sraw, sc, -lse_r) : -INFINITY);      // mask in the exponent: no branch around the exponential
        const float ds = p * (Pa[kt][i2] - del_r);
        Sa[kt][i2] = ds;
        if (GATE) gs += ds * sraw;
      }
    if (GATE) {
      gs = halves_sum(gs);
      for (int mk = 1; mk < P.g; mk <<= 1) gs += __shfl_xor(gs, mk, 64);      // the G heads of a pair are adjacent lanes
      if (r.valid && r.g == 0 && h == 0 && r.slot < P.S) sel_grads[((size_t)bh * P.n + r.i) * P.S + r.slot] = gs * P.scale;
    }
    floatx16 Qa[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) Qa[dt] = zero_acc();
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int u2 = 0; u2 < 2; ++u2) {
        const bf16x8 Sf = pack8(Sa[kt], 8 * u2);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) Qa[dt] = mfma32(KTf[dt][kt][u2], Sf, Qa[dt]);
      }
    {
      const size_t row = r.valid ? (((size_t)bh * P.n + r.i) * P.SP + r.slot) * P.g + r.g : P.prow;
      store_tile_rows<D>(Qa, P.scale, row, dqpart, tile_s, row_s, lane);
    }
    lse_r = lse_n; del_r = del_n;
    r = rn; e_n = e_nn;
  }
}

template <int D>
__global__ __launch_bounds__(256) void sel_bwd_dq_combine_kernel(const SelPlan P, const void* idx, const uint8_t* fmask, const char* __restrict__ bws,
                                                                __bf16* __restrict__ dq, float* __restrict__ sel_grads) {
  constexpr int CPR = D / 8;
  const bool two = merge_two_per_wave(P, CPR);
  const int lane = threadIdx.x & 63, half = two ? lane >> 5 : 0, sub = two ? lane & 31 : lane, width = two ? 32 : 64;
  const long qi = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * (two ? 2 : 1) + half;
  if (qi >= (long)P.bh * P.n) return;
  const int bh = (int)(qi / P.n), i = (int)(qi % P.n);
  const int b = bh / P.hkv, hk = bh % P.hkv;
  const unsigned long long live = live_slots(P, idx, fmask, bh, i, sub, half, two);
  // slots the walk never visited carry no gradient
  if (sel_grads && sub < P.S && !((live >> sub) & 1)) sel_grads[((size_t)bh * P.n + i) * P.S + sub] = 0.f;
  const __bf16* dqpart = reinterpret_cast<const __bf16*>(bws + P.off_dqpart);
  for (int c = sub; c < P.g * CPR; c += width) {
    const int g = c / CPR, dd = (c % CPR) * 8;
    const size_t row0 = ((size_t)bh * P.n + i) * P.SP * P.g + g;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    // (NSA_MERGE_BATCH_BWD rows in flight per round, see the forward merge)
    for (unsigned long long m = live; m;) {
      size_t row[NSA_MERGE_BATCH_BWD];
      bool ok[NSA_MERGE_BATCH_BWD];
#pragma unroll
      for (int j = 0; j < NSA_MERGE_BATCH_BWD; ++j) {
        ok[j] = m != 0;
        if (ok[j]) { row[j] = row0 + (size_t)__builtin_ctzll(m) * P.g; m &= m - 1; }
        else row[j] = row[j > 0 ? j - 1 : 0];
      }
      bf16x8 o[NSA_MERGE_BATCH_BWD];
#pragma unroll
      for (int j = 0; j < NSA_MERGE_BATCH_BWD; ++j) o[j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(dqpart + row[j] * D + dd));
#pragma unroll
      for (int j = 0; j < NSA_MERGE_BATCH_BWD; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += ok[j] ? (float)o[j][e] : 0.f;
    }
    bf16x8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (__bf16)acc[e];
    const long hq = hk * P.g + g;
    *reinterpret_cast<bf16x8*>(dq + (((long)b * P.hkv * P.g + hq) * P.n + i) * D + dd) = r;
  }
}

// dK/dV of one block, accumulated over a chunk of the block's virtual list; wave kt of the
// work-group owns keys 32kt .. 32kt+31.  The tile's Q and dO rows are gathered once per
// work-group with coalesced loads (wave 0: Q, wave 1: dO when there are two waves) into row-major
// LDS tiles.  S = Q K^T is computed with rows on the MFMA M side so that P and dS come out with
// lane <-> key and registers <-> rows, which is the B-operand layout of dV^T = dO^T P and
// dK^T = Q^T dS; dO^T and Q^T (lane <-> feature, k <-> rows) are read from the LDS tiles with
// the hardware transpose load.
//
// With FUSE_DQ the walk also produces the dQ partial of every pair (so the separate dQ walk and
// its second gather of Q and dO are not needed): each wave stores its dS (32 keys x 32 rows) as
// [key][row] in LDS; dQ^T = K^T dS^T is then formed with both operands read through the
// transpose load (K block row-major in LDS, loaded once per unit), each wave taking half of the
// features, and the finished 32 x D tile leaves through coalesced row stores.
#ifndef NSA_SEL_SWZ
#define NSA_SEL_SWZ 1      // Q / dO tiles of the backward walk in the swizzled layout (read as rows and through the transpose load)
#endif
#ifndef NSA_BWD_STAGES_D64
#define NSA_BWD_STAGES_D64 1
#endif
// waves per SIMD the d = 64 walk is compiled for: two (256 registers) ...
#ifndef NSA_BWD_D64_WAVES
#define NSA_BWD_D64_WAVES 2
#endif
// ... but only with two waves per work-group (64-key blocks).  Blocks of up to 32 keys are walked by one wave that gathers
// both tiles and holds every dQ feature tile: in 256 registers it spills, and the reloads inside the loop wait behind the
// gathers in flight (seq 16k, 32-key blocks: backward 0.515 ms with two waves per SIMD, 0.405 with one and no spills).
#ifndef NSA_BWD_D64_WAVES_MIN_KT
#define NSA_BWD_D64_WAVES_MIN_KT 2
#endif
#ifndef NSA_BWD_AHEAD_D64
#define NSA_BWD_AHEAD_D64 3
#endif
#ifndef NSA_BWD_AHEAD
#define NSA_BWD_AHEAD 3       // LDS operand reads issued this many MFMAs ahead in the backward walk
#endif
#ifndef NSA_BWD_STAGES
#define NSA_BWD_STAGES 2      // measured on MI355X (seq 32k, d 128): 1, 2 and 3 stages all 2.68-2.70 ms once the LDS operand reads run ahead
#endif
template <int D, int KT, bool FUSE_DQ>
__global__ __launch_bounds__(64 * KT) __attribute__((amdgpu_waves_per_eu(D == 64 && KT >= NSA_BWD_D64_WAVES_MIN_KT ? NSA_BWD_D64_WAVES : 1))) void sel_bwd_dkv_kernel(const SelPlan P, const __bf16* __restrict__ q, const __bf16* __restrict__ k,
                                                              const __bf16* __restrict__ v, const __bf16* __restrict__ dout,
                                                              const float* __restrict__ lse, const float* __restrict__ delta,
                                                              const char* __restrict__ iws, char* __restrict__ bws,
                                                              __bf16* __restrict__ dk, __bf16* __restrict__ dv) {
  constexpr int KS = D / 16, DT = D / 32, RS = D + 8;
  constexpr int RST = 32 + 16;                 // row stride of the [key][row] dS tile (transpose loads only: 8 banks mod 32 per row)
  constexpr int RSK = D + 16;                  // row stride of the K block copy (transpose loads only)
  constexpr int DTW = DT / KT;                 // feature tiles of dQ per wave
  constexpr int AHD = D == 64 ? NSA_BWD_AHEAD_D64 : NSA_BWD_AHEAD;      // LDS operand look-ahead
  __shared__ __align__(16) float lse_s[32];
  __shared__ __align__(16) float del_s[32];
  __shared__ __align__(16) int lim_s[32];
  __shared__ __align__(16) __bf16 xq_s[32 * RS];
  __shared__ __align__(16) __bf16 xg_s[32 * RS];
  __shared__ __align__(16) __bf16 kb_s[FUSE_DQ ? 32 * KT * RSK : 8];    // the K block, row-major
  __shared__ __align__(16) __bf16 ds_s[FUSE_DQ ? 32 * KT * RST : 8];    // dS^T: [key][row]
  __shared__ __align__(16) __bf16 dq_s[FUSE_DQ ? 32 * RS : 8];          // finished dQ tile, row-major
  __shared__ size_t row_s[32];
  const int kt = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63, n_ = lane & 31, h = lane >> 5;
  const int bh = blockIdx.y, b = bh / P.hkv, hk = bh % P.hkv;
  const int u = blockIdx.x;
  UnitInfo ui;
  if (!locate_unit(P, iws, 2, bh, u, ui)) return;
  const int* list = reinterpret_cast<const int*>(iws + P.off_list) + (size_t)bh * P.list_cap;
  const bool single_unit = dk != nullptr && block_has_one_unit(P, iws, bh, ui.j);
  const bool load_q = kt == 0;                 // with two waves: wave 0 gathers Q rows, wave 1 dO rows; one wave does both

  // the first list entries, then the block's K / V rows: all requested before anything waits
  const int ppt = 32 >> P.lg;
  // a single wave gathers both tiles: one stage (a second measured no faster where the registers allow it, d = 64 at one wave
  // per SIMD); two waves at d = 64 run two to a SIMD in 256 registers, where a second stage only adds spills (measured at
  // b4 n4096: 375 us with one stage, 460 us with two)
  constexpr int NS = KT == 1 ? 1 : (D == 64 ? NSA_BWD_STAGES_D64 : NSA_BWD_STAGES);
  RawEntry e0[NS];
#pragma unroll
  for (int s2 = 0; s2 < NS; ++s2) e0[s2] = fetch_entry(P, list, ui, ui.v0 + s2 * ppt, n_);
  RawEntry e_n = fetch_entry(P, list, ui, ui.v0 + NS * ppt, n_);
  __builtin_amdgcn_sched_barrier(0);

  bf16x8 Kf[KS], Vf[KS];
  const int kl = 32 * kt + n_;                 // this lane's key inside the block
  {
    const long key = (long)ui.j * P.B + kl;
    const bool ok = kl < P.B && key < P.n;
    const long keyc = ok ? key : 0;
    const __bf16* kp = k + b * P.sk[0] + hk * P.sk[1] + keyc * P.sk[2] + 8 * h;
    const __bf16* vp = v + b * P.sv[0] + hk * P.sv[1] + keyc * P.sv[2] + 8 * h;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      Kf[ks] = ok ? load8(kp + 16 * ks) : zero_frag();
      Vf[ks] = ok ? load8(vp + 16 * ks) : zero_frag();
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  floatx16 dKa[DT], dVa[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) { dKa[dt] = zero_acc(); dVa[dt] = zero_acc(); }

  const float sc = P.scale * kLog2e;
  const int HQ = P.hkv * P.g;
  const __bf16* qbase = q + b * P.sq[0] + (long)(hk * P.g) * P.sq[1];
  const __bf16* gbase = dout + b * P.so[0] + (long)(hk * P.g) * P.so[1];
  __bf16* dqpart = reinterpret_cast<__bf16*>(bws + P.off_dqpart);

  // software pipeline with NS tiles of rows in flight: when a stage has been committed to LDS its
  // registers take the loads of the tile NS steps ahead.  List entries run one more tile ahead.
  constexpr int NR = KT == 1 ? 2 : 1;
  struct Stage {
    RowInfo r;
    bf16x8 raw[NR][KS];      // this wave's share of the tile: Q rows (wave 0) or dO rows (wave 1); both with one wave
    float lse_r, del_r;
  };
  auto issue = [&](Stage& st, const RowInfo& rr) {
    st.r = rr;
    if (KT == 1) {
      issue_tile_loads<D>(st.raw[0], qbase, P.sq[1], P.sq[2], rr.i, P.g - 1, lane);
      issue_tile_loads<D>(st.raw[NR - 1], gbase, P.so[1], P.so[2], rr.i, P.g - 1, lane);
    } else {
      issue_tile_loads<D>(st.raw[0], load_q ? qbase : gbase, load_q ? P.sq[1] : P.so[1], load_q ? P.sq[2] : P.so[2], rr.i, P.g - 1, lane);
    }
    const size_t srow = ((size_t)b * HQ + hk * P.g + rr.g) * P.n + rr.i;
    st.lse_r = lse[srow];                                  // scaled where it is used: arithmetic here would wait for the loads
    st.del_r = delta[srow];
  };
  Stage stg[NS];
#pragma unroll
  for (int s2 = 0; s2 < NS; ++s2) issue(stg[s2], decode_entry(P, ui, e0[s2], n_));
  __builtin_amdgcn_sched_barrier(0);
  if (FUSE_DQ) {           // the row-major copy of the K block for dQ (waits for K, with the gathers already under way)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) *reinterpret_cast<bf16x8*>(kb_s + kl * RSK + 16 * ks + 8 * h) = Kf[ks];
  }

  wait_all_loads();        // enter the loop with nothing pending, so the loop itself only waits for what it needs
  auto step = [&](int vt, Stage& cur) {
    const RowInfo r = cur.r;
    // commit the current tile to LDS
    if (KT == 1) {
      NSA_SEL_SWZ ? commit_tile_swz<D>(cur.raw[0], xq_s, lane) : commit_tile<D>(cur.raw[0], xq_s, RS, lane);
      NSA_SEL_SWZ ? commit_tile_swz<D>(cur.raw[NR - 1], xg_s, lane) : commit_tile<D>(cur.raw[NR - 1], xg_s, RS, lane);
    } else {
      NSA_SEL_SWZ ? commit_tile_swz<D>(cur.raw[0], load_q ? xq_s : xg_s, lane) : commit_tile<D>(cur.raw[0], load_q ? xq_s : xg_s, RS, lane);
    }
    if (kt == 0 && h == 0) {
      lse_s[n_] = r.valid ? cur.lse_r * kLog2e : INFINITY; // +inf: a padding row gets p = 0
      del_s[n_] = cur.del_r;
      lim_s[n_] = r.lim;
      if (FUSE_DQ) row_s[n_] = r.valid ? (((size_t)bh * P.n + r.i) * P.SP + r.slot) * P.g + r.g : P.prow;
    }
    __syncthreads();

    // the freed stage takes the loads of the tile two steps ahead; fetch the entry of the tile after that
    // (the entry first, then the gathers: see the forward walk)
    const RowInfo rn = decode_entry(P, ui, e_n, n_);
    e_n = fetch_entry(P, list, ui, vt + (NS + 1) * ppt, n_);
    __builtin_amdgcn_sched_barrier(0);
    issue(cur, rn);
    __builtin_amdgcn_sched_barrier(0);

    floatx16 Sa = zero_acc(), Pa = zero_acc();              // [row][key]: lane <-> key, registers <-> rows
    operands_ahead<2 * KS, AHD>(
        [&](int i) { return NSA_SEL_SWZ ? lds_row_operand_swz<D>((i & 1) ? xg_s : xq_s, i >> 1, lane) : lds_row_operand((i & 1) ? xg_s : xq_s, RS, i >> 1, lane); },
        [&](int i, const bf16x8& a) {
          if (i & 1) Pa = mfma32(a, Vf[i >> 1], Pa);
          else Sa = mfma32(a, Kf[i >> 1], Sa);
        });
    floatx16 dSa;
    // a tile whose rows all see the whole block (every tile but the own-block ones) skips the key mask (uniform)
    const bool whole = r.lim >= 32 * KT - 1;
    if (__all(whole)) {
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const floatx4 l4 = *reinterpret_cast<const floatx4*>(&lse_s[8 * a + 4 * h]);
        const floatx4 d4 = *reinterpret_cast<const floatx4*>(&del_s[8 * a + 4 * h]);
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          const int i2 = 4 * a + bb;
          const float p = fast_exp2(__builtin_fmaf(Sa[i2], sc, -l4[bb]));
          Sa[i2] = p;
          dSa[i2] = p * (Pa[i2] - d4[bb]);
        }
      }
    } else {
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const floatx4 l4 = *reinterpret_cast<const floatx4*>(&lse_s[8 * a + 4 * h]);
        const floatx4 d4 = *reinterpret_cast<const floatx4*>(&del_s[8 * a + 4 * h]);
        const int* m4 = &lim_s[8 * a + 4 * h];
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
          const int i2 = 4 * a + bb;
          const float p = fast_exp2((kl <= m4[bb]) ? __builtin_fmaf(Sa[i2], sc, -l4[bb]) : -INFINITY);      // mask in the exponent: no branch around the exponential
          Sa[i2] = p;
          dSa[i2] = p * (Pa[i2] - d4[bb]);
        }
      }
    }
    const bf16x8 Pf0 = pack8(Sa, 0), Pf1 = pack8(Sa, 8);
    const bf16x8 Sf0 = pack8(dSa, 0), Sf1 = pack8(dSa, 8);
    if (FUSE_DQ) {
      // dS^T[key kl][row 8a + 4h + bb]: four consecutive rows per 8-byte store
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        bf16x4 t4;
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) t4[bb] = (__bf16)dSa[4 * a + bb];
        *reinterpret_cast<bf16x4*>(ds_s + kl * RST + 8 * a + 4 * h) = t4;
      }
    }
    // dV^T += dO^T P, dK^T += Q^T dS
    operands_ahead<4 * DT, AHD>(
        [&](int i) { return NSA_SEL_SWZ ? lds_transposed_operand_swz<D>((i & 2) ? xq_s : xg_s, 16 * (i & 1), 32 * (i >> 2), lane) : lds_transposed_operand((i & 2) ? xq_s : xg_s, RS, 16 * (i & 1), 32 * (i >> 2), lane); },
        [&](int i, const bf16x8& a) {
          const int dt = i >> 2, w = i & 3;
          if (w == 0) dVa[dt] = mfma32(a, Pf0, dVa[dt]);
          else if (w == 1) dVa[dt] = mfma32(a, Pf1, dVa[dt]);
          else if (w == 2) dKa[dt] = mfma32(a, Sf0, dKa[dt]);
          else dKa[dt] = mfma32(a, Sf1, dKa[dt]);
        });
    __syncthreads();
    if (FUSE_DQ) {
      // dQ^T[feature][row] = sum_key K^T[feature][key] dS^T[key][row]; this wave: features 32*DTW*kt ...
      floatx16 Qa[DTW];
#pragma unroll
      for (int w = 0; w < DTW; ++w) Qa[w] = zero_acc();
      // per 16 keys: the dS^T operand (lane <-> row, k <-> keys k0 ..), then the DTW K^T operands it multiplies
      bf16x8 Sf = zero_frag();
      operands_ahead<2 * KT * (DTW + 1), AHD>(
          [&](int i) {
            const int k0 = 16 * (i / (DTW + 1)), w = i % (DTW + 1);
            return w == 0 ? lds_transposed_operand(ds_s, RST, k0, 0, lane)
                          : lds_transposed_operand(kb_s, RSK, k0, 32 * (DTW * kt + w - 1), lane);
          },
          [&](int i, const bf16x8& a) {
            const int w = i % (DTW + 1);
            if (w == 0) Sf = a;
            else Qa[w - 1] = mfma32(a, Sf, Qa[w - 1]);
          });
      // Qa[w][4a + bb] = dQ[row n_][feature 32(DTW kt + w) + 8a + 4h + bb]
#pragma unroll
      for (int w = 0; w < DTW; ++w)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          bf16x4 t4;
#pragma unroll
          for (int bb = 0; bb < 4; ++bb) t4[bb] = (__bf16)(Qa[w][4 * a + bb] * P.scale);
          *reinterpret_cast<bf16x4*>(dq_s + n_ * RS + 32 * (DTW * kt + w) + 8 * a + 4 * h) = t4;
        }
      __syncthreads();
      constexpr int CPR = D / 8, RPI = (64 * KT) / CPR;
      bf16x8 vv[32 / RPI];
      size_t rw[32 / RPI];
#pragma unroll
      for (int t = 0; t < 32 / RPI; ++t) {          // all LDS reads first, then all stores
        const int rr = t * RPI + (int)threadIdx.x / CPR, c = threadIdx.x % CPR;
        vv[t] = *reinterpret_cast<const bf16x8*>(dq_s + rr * RS + 8 * c);
        rw[t] = row_s[rr];
      }
#pragma unroll
      for (int t = 0; t < 32 / RPI; ++t)
        __builtin_nontemporal_store(vv[t], reinterpret_cast<bf16x8*>(dqpart + rw[t] * D + 8 * (threadIdx.x % CPR)));
      __syncthreads();
    }
  };
  // whole rounds of NS tiles first: their steps are unconditional, so each wait counts exactly the
  // memory operations issued after the loads it needs
  int vt = ui.v0;
  if (vt + (NS - 1) * ppt < ui.v1) {
    wait_all_loads();      // again: the compiler sinks the later stages' first loads to here, past the wait above
    do {
#pragma unroll
      for (int s2 = 0; s2 < NS; ++s2) step(vt + s2 * ppt, stg[s2]);
      vt += NS * ppt;
    } while (vt + (NS - 1) * ppt < ui.v1);
  }
#pragma unroll
  for (int s2 = 0; s2 < NS - 1; ++s2)
    if (vt + s2 * ppt < ui.v1) step(vt + s2 * ppt, stg[s2]);

  // A block all of whose pairs fit this one unit (most blocks: the later a block lies the fewer queries can select it) has
  // nothing to be summed with: its dK / dV leave as bf16 straight away - what the reduce kernel would make of a single
  // partial, bit for bit - instead of 2 x 32 KT x D floats written here and read back there.
  if (single_unit) {
    const int keys = min(P.B, P.n - ui.j * P.B);
    if (kl < keys) {
      __bf16* ok_ = dk + (((size_t)bh * P.n) + (size_t)ui.j * P.B + kl) * D + 4 * h;
      __bf16* ov_ = dv + (((size_t)bh * P.n) + (size_t)ui.j * P.B + kl) * D + 4 * h;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          store4_bf16(ok_ + 32 * dt + 8 * a, dKa[dt][4 * a] * P.scale, dKa[dt][4 * a + 1] * P.scale, dKa[dt][4 * a + 2] * P.scale, dKa[dt][4 * a + 3] * P.scale);
          store4_bf16(ov_ + 32 * dt + 8 * a, dVa[dt][4 * a], dVa[dt][4 * a + 1], dVa[dt][4 * a + 2], dVa[dt][4 * a + 3]);
        }
    }
    return;
  }
  // partial [unit][2][32*KT keys][D] fp32; dKa/dVa hold [feature 32dt + 8a + 4h + bb][key kl]
  float* part = reinterpret_cast<float*>(bws + P.off_dkvpart) + ((size_t)bh * P.ub_kv + u) * (2 * 32 * KT * D);
  float* pk = part + (size_t)kl * D + 4 * h;
  float* pv = pk + 32 * KT * D;
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

// dk/dv of block j = sum of its units' partials (fixed order -> bit-reproducible)
template <int D, int KT>
__global__ __launch_bounds__(256) void sel_bwd_dkv_reduce_kernel(const SelPlan P, const char* __restrict__ iws, const char* __restrict__ bws,
                                                                __bf16* __restrict__ dk, __bf16* __restrict__ dv) {
  const int j = blockIdx.x, bh = blockIdx.y;
  const int* unit_off = reinterpret_cast<const int*>(iws + P.off_unit[2]) + (size_t)bh * (P.W + 1);
  const int u0 = unit_off[j], u1 = unit_off[j + 1];
  if (u1 - u0 == 1) return;                       // written by the walk itself
  const float* part = reinterpret_cast<const float*>(bws + P.off_dkvpart) + (size_t)bh * P.ub_kv * (2 * 32 * KT * D);
  const int keys = min(P.B, P.n - j * P.B);
  // a unit's partial is 2 x ROWS x D floats in the order (dk | dv, key, feature): the work group reads
  // it as consecutive float4 and every thread keeps its N slices of the sum in registers
  constexpr int CPR = D / 4, ROWS = 32 * KT, UNIT = 2 * ROWS * D, N = 2 * ROWS * CPR / 256;
  floatx4 acc[N];
#pragma unroll
  for (int i = 0; i < N; ++i) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int u = u0; u < u1; ++u) {
    const floatx4* src = reinterpret_cast<const floatx4*>(part + (size_t)u * UNIT) + threadIdx.x;
#pragma unroll
    for (int i = 0; i < N; ++i) acc[i] += __builtin_nontemporal_load(src + 256 * i);
  }
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const int e = threadIdx.x + 256 * i;
    const int which = e / (ROWS * CPR), rem = e % (ROWS * CPR);
    const int key = rem / CPR, dd = (rem % CPR) * 4;
    if (key >= keys) continue;
    const float s = which == 0 ? P.scale : 1.0f;
    __bf16* dst = (which == 0 ? dk : dv) + (((size_t)bh * P.n) + (size_t)j * P.B + key) * D + dd;
    store4_bf16(dst, acc[i][0] * s, acc[i][1] * s, acc[i][2] * s, acc[i][3] * s);
  }
}

}  // namespace nsa

// ----------------------------------------------------------------------------------- host

using namespace nsa;

#define NSA_LAUNCH_CHECK()                         \
  do {                                             \
    hipError_t e_ = hipGetLastError();             \
    if (e_ != hipSuccess) return (int)e_;          \
  } while (0)

// optional phase timing: record caller-created events between the kernels of one call
static inline void mark(void* const* ev, int n, int i, hipStream_t st) {
  if (ev && i < n && ev[i]) (void)hipEventRecord((hipEvent_t)ev[i], st);
}

extern "C" int nsa_select_workspace_bytes(const nsa_select_desc* d, size_t* index_bytes, size_t* fwd_bytes, size_t* bwd_bytes) {
  SelPlan P;
  const int rc = make_plan(d, P);
  if (rc) return rc;
  if (index_bytes) *index_bytes = P.index_total;
  if (fwd_bytes) *fwd_bytes = P.fwd_total;
  if (bwd_bytes) *bwd_bytes = P.bwd_total;
  return 0;
}

extern "C" int nsa_select_build_index(const nsa_select_desc* d, const void* idx, const uint8_t* fmask, void* index_ws, size_t index_bytes, void* stream) {
  SelPlan P;
  const int rc = make_plan(d, P);
  if (rc) return rc;
  if (index_bytes < P.index_total) return NSA_E_WORKSPACE;
  if (!index_ws || (P.S > 0 && (!idx || !fmask))) return NSA_E_ARG;
  hipStream_t st = (hipStream_t)stream;
  char* iws = (char*)index_ws;
  const size_t lds = (size_t)P.W * sizeof(int);
  hipLaunchKernelGGL(sel_count_kernel, dim3(P.nch, P.bh), dim3(256), lds, st, P, idx, fmask, iws);
  NSA_LAUNCH_CHECK();
  hipLaunchKernelGGL(sel_scan_kernel, dim3(P.bh), dim3(256), lds, st, P, iws);
  NSA_LAUNCH_CHECK();
  hipLaunchKernelGGL(sel_units_kernel, dim3(P.bh, 3), dim3(1024), 0, st, P, iws);
  NSA_LAUNCH_CHECK();
  if (4 * lds <= 65536)
    hipLaunchKernelGGL(sel_fill_kernel<4>, dim3(P.nch, P.bh), dim3(256), 4 * lds, st, P, idx, fmask, iws);
  else
    hipLaunchKernelGGL(sel_fill_kernel<1>, dim3(P.nch, P.bh), dim3(64), lds, st, P, idx, fmask, iws);
  NSA_LAUNCH_CHECK();
  return 0;
}

template <int D, int KT>
static int launch_fwd(const SelPlan& P, const void* q, const void* k, const void* v, const void* idx, const uint8_t* fmask,
                      const void* iws, void* fws, void* out, float* lse, hipStream_t st, void* const* ev, int nev) {
  mark(ev, nev, 0, st);
  hipLaunchKernelGGL((sel_fwd_kernel<D, KT>), dim3(xcd_grid(P, 0)), dim3(64), 0, st, P, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v,
                     (const char*)iws, (char*)fws);
  NSA_LAUNCH_CHECK();
  mark(ev, nev, 1, st);
  const long nq = (long)P.bh * P.n, qpb = merge_two_per_wave(P, D / 8) ? 8 : 4;      // queries per work-group of the merge
  hipLaunchKernelGGL((sel_fwd_combine_kernel<D>), dim3((unsigned)((nq + qpb - 1) / qpb)), dim3(256), 0, st, P, idx, fmask, (const char*)fws, (__bf16*)out, lse);
  NSA_LAUNCH_CHECK();
  mark(ev, nev, 2, st);
  return 0;
}

extern "C" int nsa_select_fwd_timed(const nsa_select_desc* d, const void* q, const void* k, const void* v, const void* idx, const uint8_t* fmask,
                                    const void* index_ws, void* fwd_ws, size_t fwd_bytes, void* out, float* lse, void* stream,
                                    void* const* ev, int nev) {
  SelPlan P;
  const int rc = make_plan(d, P);
  if (rc) return rc;
  if (fwd_bytes < P.fwd_total) return NSA_E_WORKSPACE;
  if (!q || !k || !v || !index_ws || !fwd_ws || !out || !lse) return NSA_E_ARG;
  hipStream_t st = (hipStream_t)stream;
  const int KT = (P.B + 31) / 32;
  if (P.D == 64 && KT == 1) return launch_fwd<64, 1>(P, q, k, v, idx, fmask, index_ws, fwd_ws, out, lse, st, ev, nev);
  if (P.D == 64 && KT == 2) return launch_fwd<64, 2>(P, q, k, v, idx, fmask, index_ws, fwd_ws, out, lse, st, ev, nev);
  if (P.D == 128 && KT == 1) return launch_fwd<128, 1>(P, q, k, v, idx, fmask, index_ws, fwd_ws, out, lse, st, ev, nev);
  if (P.D == 128 && KT == 2) return launch_fwd<128, 2>(P, q, k, v, idx, fmask, index_ws, fwd_ws, out, lse, st, ev, nev);
  return NSA_E_UNSUPPORTED;
}

extern "C" int nsa_select_fwd(const nsa_select_desc* d, const void* q, const void* k, const void* v, const void* idx, const uint8_t* fmask,
                              const void* index_ws, void* fwd_ws, size_t fwd_bytes, void* out, float* lse, void* stream) {
  return nsa_select_fwd_timed(d, q, k, v, idx, fmask, index_ws, fwd_ws, fwd_bytes, out, lse, stream, nullptr, 0);
}

template <int D, int KT>
static int launch_bwd(const SelPlan& P, const void* q, const void* k, const void* v, const void* out, const void* dout, const float* dlse, const float* lse,
                      const void* idx, const uint8_t* fmask, const void* iws, void* bws, void* dq, void* dk, void* dv, float* sel_grads, hipStream_t st, void* const* ev, int nev) {
  mark(ev, nev, 0, st);
  float* delta = reinterpret_cast<float*>((char*)bws + P.off_delta);
  const long rows = (long)P.bh * P.g * P.n;
  constexpr int RPB = 256 / (D / 8);
  hipLaunchKernelGGL((sel_delta_kernel<D>), dim3((unsigned)((rows + RPB - 1) / RPB)), dim3(256), 0, st, P, (const __bf16*)out, (const __bf16*)dout, dlse, delta);
  NSA_LAUNCH_CHECK();
  mark(ev, nev, 1, st);
  // without gate gradients the dQ partials come out of the dK/dV walk (one gather of Q and dO
  // instead of two); with them the separate dQ walk, which also emits sel_grads, is used
  const bool fused = sel_grads == nullptr;
  if (!fused) {
    hipLaunchKernelGGL((sel_bwd_dq_kernel<D, KT, true>), dim3(xcd_grid(P, 1)), dim3(64), 0, st, P, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v,
                       (const __bf16*)dout, lse, delta, (const char*)iws, (char*)bws, sel_grads);
    NSA_LAUNCH_CHECK();
  }
  mark(ev, nev, 2, st);
  if (fused) {
    hipLaunchKernelGGL((sel_bwd_dkv_kernel<D, KT, true>), dim3(P.ub_kv, P.bh), dim3(64 * KT), 0, st, P, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v,
                       (const __bf16*)dout, lse, delta, (const char*)iws, (char*)bws, (__bf16*)dk, (__bf16*)dv);
  } else {
    hipLaunchKernelGGL((sel_bwd_dkv_kernel<D, KT, false>), dim3(P.ub_kv, P.bh), dim3(64 * KT), 0, st, P, (const __bf16*)q, (const __bf16*)k, (const __bf16*)v,
                       (const __bf16*)dout, lse, delta, (const char*)iws, (char*)bws, (__bf16*)dk, (__bf16*)dv);
  }
  NSA_LAUNCH_CHECK();
  mark(ev, nev, 3, st);
  const long nq = (long)P.bh * P.n, qpb = merge_two_per_wave(P, D / 8) ? 8 : 4;
  hipLaunchKernelGGL((sel_bwd_dq_combine_kernel<D>), dim3((unsigned)((nq + qpb - 1) / qpb)), dim3(256), 0, st, P, idx, fmask, (const char*)bws, (__bf16*)dq, sel_grads);
  NSA_LAUNCH_CHECK();
  mark(ev, nev, 4, st);
  hipLaunchKernelGGL((sel_bwd_dkv_reduce_kernel<D, KT>), dim3(P.W, P.bh), dim3(256), 0, st, P, (const char*)iws, (const char*)bws, (__bf16*)dk, (__bf16*)dv);
  NSA_LAUNCH_CHECK();
  mark(ev, nev, 5, st);
  return 0;
}

extern "C" int nsa_select_bwd_timed(const nsa_select_desc* d, const void* q, const void* k, const void* v, const void* out, const void* d_out,
                                    const float* d_lse, const float* lse, const void* idx, const uint8_t* fmask, const void* index_ws, void* bwd_ws, size_t bwd_bytes,
                                    void* dq, void* dk, void* dv, float* sel_grads, void* stream, void* const* ev, int nev) {
  SelPlan P;
  const int rc = make_plan(d, P);
  if (rc) return rc;
  if (bwd_bytes < P.bwd_total) return NSA_E_WORKSPACE;
  if (!q || !k || !v || !out || !d_out || !lse || !index_ws || !bwd_ws || !dq || !dk || !dv) return NSA_E_ARG;
  hipStream_t st = (hipStream_t)stream;
  const int KT = (P.B + 31) / 32;
  if (P.D == 64 && KT == 1) return launch_bwd<64, 1>(P, q, k, v, out, d_out, d_lse, lse, idx, fmask, index_ws, bwd_ws, dq, dk, dv, sel_grads, st, ev, nev);
  if (P.D == 64 && KT == 2) return launch_bwd<64, 2>(P, q, k, v, out, d_out, d_lse, lse, idx, fmask, index_ws, bwd_ws, dq, dk, dv, sel_grads, st, ev, nev);
  if (P.D == 128 && KT == 1) return launch_bwd<128, 1>(P, q, k, v, out, d_out, d_lse, lse, idx, fmask, index_ws, bwd_ws, dq, dk, dv, sel_grads, st, ev, nev);
  if (P.D == 128 && KT == 2) return launch_bwd<128, 2>(P, q, k, v, out, d_out, d_lse, lse, idx, fmask, index_ws, bwd_ws, dq, dk, dv, sel_grads, st, ev, nev);
  return NSA_E_UNSUPPORTED;
}

extern "C" int nsa_select_bwd(const nsa_select_desc* d, const void* q, const void* k, const void* v, const void* out, const void* d_out,
                              const float* d_lse, const float* lse, const void* idx, const uint8_t* fmask, const void* index_ws, void* bwd_ws, size_t bwd_bytes,
                              void* dq, void* dk, void* dv, float* sel_grads, void* stream) {
  return nsa_select_bwd_timed(d, q, k, v, out, d_out, d_lse, lse, idx, fmask, index_ws, bwd_ws, bwd_bytes, dq, dk, dv, sel_grads, stream, nullptr, 0);
}

extern "C" int nsa_abi_version(void) { return 6; }
