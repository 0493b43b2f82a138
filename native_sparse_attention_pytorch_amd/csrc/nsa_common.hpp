// Shared device helpers for the gfx950 (CDNA4, wave64) NSA kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nsa {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(8 * sizeof(float)))) float floatx8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t uintx4;
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int intx4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t uintx2;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// D(32x32) += A(32x16) * B(16x32), bf16 inputs, fp32 accumulate.
// Register layout (lane l, half h = l / 32):
//   A: row m = l % 32, k = 8h .. 8h+7          (8 bf16 per lane)
//   B: col n = l % 32, k = 8h .. 8h+7          (8 bf16 per lane)
//   D: col n = l % 32, reg i (0..15) holds row m = 8*(i/4) + 4h + (i%4)
__device__ __forceinline__ floatx16 mfma32(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 zero_frag() {
  uintx4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}

__device__ __forceinline__ floatx16 zero_acc() {
  floatx16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.f;
  return z;
}

// 16-byte global load of 8 consecutive bf16 (address must be 16-byte aligned).
__device__ __forceinline__ bf16x8 load8(const __bf16* p) {
  return *reinterpret_cast<const bf16x8*>(p);
}

// Pack 8 consecutive accumulator registers (first .. first+7) into one bf16 operand.
__device__ __forceinline__ bf16x8 pack8(const floatx16& acc, int first) {
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (__bf16)acc[first + e];
  return r;
}

// Constant B operands that turn an MFMA into a register transpose:
//   ident_lo: B[k][n] = (n == k),      ident_hi: B[k][n] = (n == k + 16)
// mfma32(X_lo, ident_lo, 0) + mfma32(X_hi, ident_hi, .) gives D[m][n] = X[m][n] for a
// 32x32 bf16 tile X held as two A operands (columns 0..15 and 16..31); D then has
// lane <-> column, registers <-> rows, which is the operand layout for a contraction
// over the rows of X.  Products with 0/1 are exact, so the transpose is lossless.
__device__ __forceinline__ void make_ident(int lane, bf16x8& lo, bf16x8& hi) {
  const int n = lane & 31, h = lane >> 5;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    lo[e] = (__bf16)((n == 8 * h + e) ? 1.0f : 0.0f);
    hi[e] = (__bf16)((n == 16 + 8 * h + e) ? 1.0f : 0.0f);
  }
}

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short shortx4;

// Transposed MFMA operand from a row-major bf16 tile X in LDS (row stride RS elements): returns, for lane (m = lane % 32,
// h = lane / 32), the 8 values X[row0 + 8*(e/4) + 4h + e%4][col0 + m], e = 0..7 - i.e. an
// A/B operand whose lane index runs over 32 columns of X and whose k index runs over 16 rows
// of X in the same order in which a 32x32 MFMA result holds its rows (registers 8u .. 8u+7).
// Uses the gfx950 LDS transpose load: in every group of 16 lanes, lane ll receives element
// ll % 4 of the four 8-byte rows addressed by lanes 4e + ll / 4 (e = 0..3) of its group.
// Bank conflicts (measured with the conflict counters, D = 128): this load takes 4 clocks at a row stride of D + 16 and 8 at
// D + 8 (2 would be conflict-free), the 16-byte row reads of lds_row_operand 4 clocks at D + 8 (their minimum) and 8 at D + 16:
// a tile read only one way uses the matching stride, a tile read both ways the swizzled layout below or the stride of the
// read it does more often.
__device__ __forceinline__ bf16x8 lds_transposed_operand(const __bf16* X, int RS, int row0, int col0, int lane) {
  const int ll = lane & 15, e = ll >> 2, qq = ll & 3, mh = (lane >> 4) & 1, h = lane >> 5;
  const __bf16* p0 = X + (row0 + 4 * h + e) * RS + col0 + 16 * mh + 4 * qq;
  typedef shortx4 __attribute__((address_space(3))) * lds_ptr;
  const shortx4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
  const shortx4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0 + 8 * RS));
  typedef __attribute__((__vector_size__(8 * sizeof(short)))) short shortx8;
  shortx8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) { r[i] = a[i]; r[4 + i] = b[i]; }
  return __builtin_bit_cast(bf16x8, r);
}

// MFMA operand (lane <-> row n_, k <-> 8 consecutive features) of k-step ks from a row-major tile
__device__ __forceinline__ bf16x8 lds_row_operand(const __bf16* tile_s, int RS, int ks, int lane) {
  return *reinterpret_cast<const bf16x8*>(tile_s + (lane & 31) * RS + 16 * ks + 8 * (lane >> 5));
}

// Swizzled row-major LDS tile (D = 64 or 128 bf16 per row, no padding) for tiles that are read both ways: the 16-byte
// chunk c of row r is stored at chunk position (c & ~7) | ((c ^ swz(r)) & 7), swz(r) = 2 * (r % 4) + (r / 4) % 2.
// Measured with the bank-conflict counters (gfx950: 64 banks of 4 bytes per clock): a 64-lane 16-byte row read takes 8 clocks
// in this layout (4 is the minimum, reached by a row stride of D + 8), the transpose load 4 clocks at D = 128 and 2 at D = 64
// (2 is the minimum; stride D + 8 takes 8, D + 16 takes 4) - as good as a padded stride can be for a tile read both ways, and
// the only choice for tiles filled by global_load_lds, which cannot pad.  A swizzle over all 16 positions of a row reaches
// both minima but costs an XOR per read (rows r and r + 8 differ, k-steps no longer fold into immediate offsets); it was
// measured no faster in the dense kernels and slower in the selection backward walk.  swz depends on the lane only (not on
// the k-step or the feature tile), so a kernel pays a few address registers.
__device__ __forceinline__ int lds_swz(int row) { return ((row & 3) << 1) | ((row >> 2) & 1); }

template <int D>
__device__ __forceinline__ int lds_swz_off(int row, int chunk) {
  return row * D + 8 * ((chunk & ~7) | ((chunk ^ lds_swz(row)) & 7));
}

template <int D>
__device__ __forceinline__ bf16x8 lds_row_operand_swz(const __bf16* tile_s, int ks, int lane) {
  return *reinterpret_cast<const bf16x8*>(tile_s + lds_swz_off<D>(lane & 31, 2 * ks + (lane >> 5)));
}

// as lds_transposed_operand, from a swizzled tile; row0 must be a multiple of 8 and col0 of 16
template <int D>
__device__ __forceinline__ bf16x8 lds_transposed_operand_swz(const __bf16* X, int row0, int col0, int lane) {
  const int ll = lane & 15, e = ll >> 2, qq = ll & 3, mh = (lane >> 4) & 1, h = lane >> 5;
  const __bf16* p0 = X + lds_swz_off<D>(row0 + 4 * h + e, (col0 >> 3) + 2 * mh + (qq >> 1)) + 4 * (qq & 1);
  typedef shortx4 __attribute__((address_space(3))) * lds_ptr;
  const shortx4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0));
  const shortx4 b = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p0 + 8 * D));      // rows + 8: same swizzle
  typedef __attribute__((__vector_size__(8 * sizeof(short)))) short shortx8;
  shortx8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) { r[i] = a[i]; r[4 + i] = b[i]; }
  return __builtin_bit_cast(bf16x8, r);
}

// A 64-row tile (D bf16 per row) copied from global memory straight into a swizzled LDS tile (the layout read by
// lds_row_operand_swz / lds_transposed_operand_swz) with global_load_lds_dwordx4: no staging registers and no LDS store
// instructions.  One instruction of a wave fills 1 KB of consecutive LDS (lane l writes bytes 16 l .. 16 l + 15 after the
// wave-uniform address in M0), i.e. 1024 / (2 D) whole rows, so the swizzle is applied on the global side: the lane that
// writes chunk position p of row r fetches chunk (p & ~7) | ((p ^ swz(r)) & 7).  NT threads cover the tile in
// 64 * D / (8 * NT) rounds; a lane's rows in different rounds differ by a multiple of 8, which leaves its swizzle (and
// source chunk) alone.  A tile whose 64 rows all exist is addressed as scalar base + one per-lane 32-bit offset that never
// changes: per tile a few scalar additions and no vector arithmetic (per-lane 64-bit row addresses cost more vector
// instructions per tile than a quarter of the softmax).  In a tile that crosses `limit`, rows at or beyond it re-read row
// limit - 1 (finite values; callers mask their scores) through per-lane addresses.
// The copy is asynchronous: it counts in vmcnt, and the tile may be read after s_waitcnt vmcnt(0) by every wave that
// issued a part of it plus a work-group barrier.  A wave must not end while a copy it issued is in flight.
// Inline assembly rather than __builtin_amdgcn_global_load_lds: the compiler makes every later LDS read wait for all the
// copies it knows of (s_waitcnt vmcnt(0) in front of the first operand read of the tile in use), which serialises the
// copy of the next tile with the work on this one.
template <int D, int NT>
struct TileDma {
  static constexpr int CPR = D / 8, RPS = 64 / CPR, WAVES = NT / 64, ROUNDS = (64 / RPS) / WAVES;
  static_assert((WAVES * RPS) % 8 == 0 && ROUNDS >= 1, "a lane's rows must keep their swizzle from round to round");
  int row_in, src_off;
  unsigned voff;        // byte offset of this lane's 16 bytes from the first row of a round
  unsigned lds0;        // LDS byte address of this wave's segment of the first 1 KB copy of a tile (wave-uniform)
  long s_row;
  // lds_base: the LDS array the tiles live in; a tile is addressed by its byte offset from it
  __device__ __forceinline__ void init(int tid, long row_stride, const __bf16* lds_base) {
    typedef __attribute__((address_space(3))) void* lds_p;
    const int lane = tid & 63, pos = lane % CPR, wave = tid >> 6;
    s_row = row_stride;
    row_in = wave * RPS + lane / CPR;
    src_off = 8 * ((pos & ~7) | ((pos ^ lds_swz(row_in)) & 7));
    voff = (unsigned)(row_in * row_stride + src_off) * 2u;
    lds0 = __builtin_amdgcn_readfirstlane((unsigned)(unsigned long)(lds_p)lds_base + wave * 1024);
  }
  // One round (1 KB per wave) of a tile whose 64 rows all exist; tb = address of the tile's first row.  Issuing a copy
  // keeps the wave's instruction stream busy for some 60 cycles; callers with MFMAs to issue put the rounds between them.
  __device__ __forceinline__ void round_full(const __bf16* __restrict__ tb, unsigned tile_off, int r) const {
    // (s_nop 3: five wait states between the last scalar write and the load - enough for M0, and for an address register
    // the compiler may have produced with v_readfirstlane right before: hazards inside inline assembly are not its business)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds0 + tile_off + r * WAVES * 1024), "v"(voff), "s"(tb + r * WAVES * RPS * s_row) : "memory", "m0");
  }
  // The same under an execution mask (all ones: copy; zero: no lane takes part, nothing is read or written and tb may point
  // anywhere): lets a caller keep one straight-line instruction stream whether or not there is a tile to copy.
  // `lanes` is all ones or zero (32 bits, used for both halves of the mask) and wave-uniform.
  __device__ __forceinline__ void round_full_if(unsigned lanes, const __bf16* __restrict__ tb, unsigned tile_off, int r) const {
    asm volatile("s_mov_b32 m0, %0\n\ts_mov_b64 vcc, exec\n\ts_mov_b32 exec_lo, %3\n\ts_mov_b32 exec_hi, %3\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, vcc"
                 :: "s"(lds0 + tile_off + r * WAVES * 1024), "v"(voff), "s"(tb + r * WAVES * RPS * s_row),
                    "s"(__builtin_amdgcn_readfirstlane(lanes)) : "memory", "m0", "vcc");
  }
  // base, first_row, limit and tile_off (bytes from lds_base) must be wave-uniform
  __device__ __forceinline__ void issue(const __bf16* __restrict__ base, long first_row, long limit, unsigned tile_off) const {
    if (first_row + 64 <= limit) {
      const __bf16* tb = base + first_row * s_row;
#pragma unroll
      for (int r = 0; r < ROUNDS; ++r) round_full(tb, tile_off, r);
    } else {
      // (the lane's row passes through an empty volatile statement: this path runs once or twice per work-group, and without
      // the fence the compiler keeps every round's loop-invariant address terms in registers for the whole walk)
      int ri = row_in;
      asm volatile("" : "+v"(ri));
#pragma unroll
      for (int r = 0; r < ROUNDS; ++r) {
        long row = first_row + ri + r * WAVES * RPS;
        row = row < limit ? row : limit - 1;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, off"
                     :: "s"(lds0 + tile_off + r * WAVES * 1024), "v"(base + row * s_row + src_off) : "memory", "m0");
      }
    }
  }
};

// s_waitcnt vmcnt(0) (expcnt / lgkmcnt left at their maxima): all outstanding global loads
// and stores of this wave have completed.
// N operand reads feeding N uses, each read issued AH uses ahead of its own.  The compiler keeps an LDS operand
// read where the source puts it - right before its MFMA it means a full LDS round trip per MFMA - so the distance
// is spelled out here.  `rd(i)` returns operand i, `use(i, a)` consumes it; both are inlined into a fully unrolled loop.
template <int N, int AH, class Read, class Use>
__device__ __forceinline__ void operands_ahead(Read rd, Use use) {
  bf16x8 ring[AH + 1];
#pragma unroll
  for (int i = 0; i < AH && i < N; ++i) ring[i] = rd(i);
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if (i + AH < N) ring[(i + AH) % (AH + 1)] = rd(i + AH);
    use(i, ring[i % (AH + 1)]);
  }
}

// Wait for every outstanding vector memory operation.  The plain s_waitcnt builtin does not order
// loads around itself (the compiler moved gathers issued before it to after it), hence the fence.
__device__ __forceinline__ void wait_all_loads() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0x0F70);      // the builtin, not inline assembly: the compiler's own wait counting sees it
  __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Maximum / sum of a value over the two 32-lane halves of the wave (lane l with lane l ^ 32), left in both halves.
// v_permlane32_swap exchanges the upper half of one register with the lower half of another inside the VALU; the shuffle
// it replaces (ds_bpermute) is an LDS round trip on the critical path of every tile's softmax.  Inline assembly: the
// builtin with the same value for both operands is folded away by the compiler as if the swap did nothing.  The s_nop
// on either side covers the wait states between a VALU write and the swap's read, and the swap's write and a VALU read.
__device__ __forceinline__ void swap_halves(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float halves_max(float v) {
  float a = v, b = v;
  swap_halves(a, b);      // a = lower half's values in both halves, b = upper half's
  return fmaxf(a, b);
}
__device__ __forceinline__ float halves_sum(float v) {
  float a = v, b = v;
  swap_halves(a, b);
  return a + b;
}

// value of lane ^ 1 / lane ^ 2 (DPP quad permutes: VALU speed, no LDS round trip)
__device__ __forceinline__ float dpp_quad_xor1(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
}
__device__ __forceinline__ float dpp_quad_xor2(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
}

// store 4 floats as 4 bf16 (8 bytes)
__device__ __forceinline__ void store4_bf16(__bf16* p, float a, float b, float c, float d) {
  bf16x4 r;
  r[0] = (__bf16)a; r[1] = (__bf16)b; r[2] = (__bf16)c; r[3] = (__bf16)d;
  *reinterpret_cast<bf16x4*>(p) = r;
}

}  // namespace nsa
