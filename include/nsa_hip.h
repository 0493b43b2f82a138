/* C ABI of libnsa_hip.so - the gfx950 (MI355X) kernels for the Native Sparse Attention hot path.
 *
 * Every function is enqueue-only on the given hipStream_t (passed as void*), never allocates or
 * frees device memory, never synchronises and keeps no global state.  The caller owns every
 * buffer, including workspaces, whose sizes come from the *_workspace_bytes functions.
 * Return value: 0 = ok, negative = argument error (NSA_E_*), positive = hipError_t of a launch.
 *
 * Citations are into the reference tree (lucidrains/native-sparse-attention-pytorch v0.2.3):
 *   NSA.py = native_sparse_attention_pytorch/native_sparse_attention.py
 *   TRI.py = native_sparse_attention_pytorch/triton_native_sparse_attention.py
 *
 * Tensors are bf16 (uint16 storage) unless stated; the head dimension always has stride 1 and
 * every row start must be 16-byte aligned.  Strides are in elements: {batch, head, token}.
 */
#ifndef NSA_HIP_H
#define NSA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NSA_E_ARG (-1)         /* inconsistent / out-of-range argument            */
#define NSA_E_UNSUPPORTED (-2) /* shape outside what the kernels are compiled for */
#define NSA_E_WORKSPACE (-3)   /* workspace too small                             */

int nsa_abi_version(void);

/* One-wave hardware self-test of the MFMA register layouts the kernels assume: C[32x32] fp32 =
 * A[32x16] * B[16x32] (row-major bf16) and T[32x32] = X[32x32] (bf16) passed through the
 * identity-operand register transpose.  No reference counterpart (Triton hides layouts). */
int nsa_selftest_mfma(const void* A, const void* B, float* C, const void* X, float* T, void* stream);

/* ------------------------------------------------------------------------------------------
 * Block-selection attention.  Replaces native_sparse_attend / NSA.forward / NSA.backward
 * (TRI.py:1938-1987, 1827-1872, 1875-1925) and the kernels they launch (TRI.py:599-694,
 * 1646-1818); same contract as the pure-torch gather path NSA.py:741-819.
 *
 * Query (b, kv head h, token i) attends - in one softmax - the `block` keys of every slot s
 * with fmask[b,h,i,s] != 0 (block number idx[b,h,i,s], no causal mask inside it, a block named
 * twice counts twice, keys at or beyond `seq` count with logit 0 and value 0) plus, if `causal`,
 * the keys j <= i of its own block (TRI.py include_block_causal).  The `group` query heads
 * h*group .. h*group+group-1 share kv head h and its selection.
 * ------------------------------------------------------------------------------------------ */
typedef struct nsa_select_desc {
  int32_t batch, kv_heads, group, seq, num_sel, block, dim_head, causal;
  int32_t idx_is_int64; /* 1: idx is int64 (what torch.topk returns), 0: int32 */
  float scale;          /* logits multiplier, dim_head^-0.5 in the reference (NSA.py:225) */
  int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3];    /* o: out and d_out */
} nsa_select_desc;

/* Sizes of the three caller-owned workspaces: `index` (inverse index: built by
 * nsa_select_build_index, read by fwd and bwd, must outlive both), `fwd` (per-slot partial
 * outputs, dead after nsa_select_fwd returns) and `bwd` (dead after nsa_select_bwd). */
int nsa_select_workspace_bytes(const nsa_select_desc* d, size_t* index_bytes, size_t* fwd_bytes, size_t* bwd_bytes);

/* Counting sort of (query, slot) pairs by selected block - the inverse map block -> queries that
 * lets forward and backward walk the KV blocks instead of gathering them per query.  Deterministic
 * (no order-dependent atomics).  idx/fmask: contiguous [batch, kv_heads, seq, num_sel];
 * fmask is one byte per slot.  Slots with idx outside [0, ceil(seq/block)) are ignored.
 * Replaces the per-query gather addressing of TRI.py:349-392. */
int nsa_select_build_index(const nsa_select_desc* d, const void* idx, const uint8_t* fmask,
                           void* index_ws, size_t index_bytes, void* stream);

/* out: bf16 [batch, kv_heads*group, seq, dim_head] with strides o_stride; lse: fp32 contiguous
 * [batch, kv_heads*group, seq] (natural log of the softmax normaliser, TRI.py:456-457). */
int nsa_select_fwd(const nsa_select_desc* d, const void* q, const void* k, const void* v,
                   const void* idx, const uint8_t* fmask, const void* index_ws, void* fwd_ws, size_t fwd_bytes,
                   void* out, float* lse, void* stream);

/* dq: bf16 contiguous [batch, kv_heads*group, seq, dim_head]; dk, dv: bf16 contiguous
 * [batch, kv_heads, seq, dim_head].  Atomic-free and bit-reproducible: dK/dV of a KV block are
 * accumulated on chip by the work-groups that own the block, dQ is reduced over a query's slots.
 * (The reference accumulates all three through global fp32 atomics, TRI.py:758-788, 1395-1425.) */
int nsa_select_bwd(const nsa_select_desc* d, const void* q, const void* k, const void* v,
                   const void* out, const void* d_out, const float* lse,
                   const void* idx, const uint8_t* fmask, const void* index_ws, void* bwd_ws, size_t bwd_bytes,
                   void* dq, void* dk, void* dv, void* stream);

/* Same as nsa_select_fwd / nsa_select_bwd, additionally recording the caller's hipEvent_t
 * handles (created with timing enabled) between the kernels of the call, so that a benchmark
 * can time each kernel on the launch stream.  Events: fwd {start, after block walk, after
 * merge}; bwd {start, after delta, after dQ walk, after dQ merge, after dK/dV walk, after dK/dV
 * reduce}.  NULL entries are skipped.  No reference counterpart (measurement hook). */
int nsa_select_fwd_timed(const nsa_select_desc* d, const void* q, const void* k, const void* v,
                         const void* idx, const uint8_t* fmask, const void* index_ws, void* fwd_ws, size_t fwd_bytes,
                         void* out, float* lse, void* stream, void* const* events, int num_events);
int nsa_select_bwd_timed(const nsa_select_desc* d, const void* q, const void* k, const void* v,
                         const void* out, const void* d_out, const float* lse,
                         const void* idx, const uint8_t* fmask, const void* index_ws, void* bwd_ws, size_t bwd_bytes,
                         void* dq, void* dk, void* dv, void* stream, void* const* events, int num_events);

#ifdef __cplusplus
}
#endif
#endif /* NSA_HIP_H */
