/* C ABI of libnsa_hip.so - the gfx950 (MI355X) kernels for the Native Sparse Attention hot path.
 *
 * Every function is enqueue-only on the given hipStream_t (passed as void*), never allocates or
 * frees device memory and never synchronises.  The caller owns every buffer, including
 * workspaces, whose sizes come from the *_workspace_bytes functions.  The library keeps no state
 * between calls, with one exception: nsa_decode_attend_noalloc caches, per device, the address of
 * its fixed scratch array (looked up on the first call on that device, under a mutex).
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

/* Memory-system probe with the access pattern of the block-selection walks (no reference counterpart; used by
 * bench.py to state the ceiling next to the walks' achieved GB/s).  `waves` wavefronts each repeat `iters` times:
 * gather `reads` groups of four 1 KB rows from pseudo-random rows of src (src_rows rows of 1 KB), then scatter
 * `writes` groups of four 1 KB rows to pseudo-random rows of dst (dst_rows rows of 1 KB; ordinary or non-temporal
 * stores).  reads, writes <= 8.  Moves waves * iters * 4 * (reads + writes) KB. */
int nsa_probe_row_traffic(const void* src, size_t src_rows, void* dst, size_t dst_rows, int32_t reads, int32_t writes,
                          int32_t iters, int32_t waves, int32_t nontemporal, uint32_t seed, void* stream);

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
 * Limits (NSA_E_UNSUPPORTED otherwise): dim_head 64 or 128, 1 <= block <= 64, group a power of two <= 32,
 * num_sel <= 62, at most 16384 blocks, head and token strides of q / out below 2^32 elements.
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
 * (The reference accumulates all three through global fp32 atomics, TRI.py:758-788, 1395-1425.)
 * sel_grads: NULL, or fp32 contiguous [batch, kv_heads, seq, num_sel] receiving the gradient of a
 * multiplier of value 1 on each slot's keys (the straight-through top-k gates `sel_scale`,
 * TRI.py:1061-1080, NSA.py:793-797); dead slots get 0.
 * d_lse: NULL, or fp32 contiguous like lse: the upstream gradient of the returned log-sum-exp (the reference's lse
 * output carries none; here it lets a caller merge the results of several calls over disjoint slot sets by their lse
 * and still differentiate the merge). */
int nsa_select_bwd(const nsa_select_desc* d, const void* q, const void* k, const void* v,
                   const void* out, const void* d_out, const float* d_lse, const float* lse,
                   const void* idx, const uint8_t* fmask, const void* index_ws, void* bwd_ws, size_t bwd_bytes,
                   void* dq, void* dk, void* dv, float* sel_grads, void* stream);

/* ------------------------------------------------------------------------------------------
 * Interval-masked GQA flash attention: one kernel family for
 *   mode 0 "band"   - the sliding-window branch.  Replaces LocalAttention(window_size, causal,
 *                     exact_windowsize, autopad) as called at NSA.py:250-257, 841-850: query i
 *                     sees keys j with 0 <= i-j <= window (causal) or |i-j| <= window, which is
 *                     the mask of NSA.py:48-56; k/v have `seq` rows, num_mem = 0;
 *   mode 1 "stride" - the compressed branch.  Replaces attend(q, ck, cv, cmask, return_sim=True)
 *                     (NSA.py:153-184, 632-639): k/v hold num_mem memory rows (always visible)
 *                     followed by num_keys compressed keys; compressed key c is visible to query i
 *                     iff (c+1)*stride - 1 < i when causal, always otherwise.  With `pool` set the
 *                     forward also writes the block-importance logits of NSA.py:652-691 to
 *                     `pooled` (fp32 [batch, kv_heads or heads, seq, nb], nb = num_keys /
 *                     (sel_block/stride)): mean of the scaled logits over the compressed keys of
 *                     fine block j and, if `share`, over the group's heads; -inf where the
 *                     reference's fill values (-finfo.max/10 for an invisible key, -finfo.max for
 *                     the query's own block when stride != sel_block) make the softmax term zero.
 *                     sel_block / stride must be a power of two <= 32 (with sel_block == stride the
 *                     output holds one logit per compressed key, which serves every other ratio).
 *                     pool = 2 (causal only, otherwise as 1): row i of `pooled` is defined only below
 *                     column floor(i / sel_block), the part a causal query can select from; the rest of
 *                     the row (all -inf with pool = 1) is left unwritten - for nsa_topk_prefix.
 * out/lse as for nsa_select_fwd; dq contiguous [batch, heads, seq, d]; dk, dv contiguous
 * [batch, kv_heads, num_mem + num_keys, d] (bf16, or fp32 with dkv_fp32: the compressed keys are few and their
 * gradient feeds sums over every window, where a bf16 rounding per key is the largest error left).
 * bf16 in, fp32 accumulate, bf16 out.  Head and token strides of
 * q / d_out below 2^32 elements, token strides of k / v below 2^26 (NSA_E_UNSUPPORTED otherwise).
 * ------------------------------------------------------------------------------------------ */
typedef struct nsa_dense_desc {
  int32_t batch, kv_heads, group, seq, num_keys, num_mem, dim_head;
  int32_t mode, causal, window, stride;
  int32_t pool, sel_block, share;
  float scale;
  int32_t dkv_fp32; /* backward: 1 = dk and dv are written as fp32 (the fixed-order sums, unrounded), 0 = bf16 */
  int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3], do_stride[3];
} nsa_dense_desc;

int nsa_dense_workspace_bytes(const nsa_dense_desc* d, size_t* bwd_bytes);
int nsa_dense_fwd(const nsa_dense_desc* d, const void* q, const void* k, const void* v,
                  void* out, float* lse, float* pooled, void* stream);
int nsa_dense_bwd(const nsa_dense_desc* d, const void* q, const void* k, const void* v,
                  const void* out, const void* d_out, const float* lse, void* bwd_ws, size_t bwd_bytes,
                  void* dq, void* dk, void* dv, void* stream);

/* Compressed attention with the block selection made inside the forward kernel.  Replaces, in one launch,
 * attend(q, ck, cv, cmask, return_sim=True) (NSA.py:153-184, 632-639), the importance scores (NSA.py:652-691), the
 * padded softmax (NSA.py:693-695), topk (NSA.py:703-713) and the slot mask (NSA.py:721): the block-importance
 * logits are never written to memory.  `d` as for nsa_dense_fwd in mode 1 with pool != 0 (sel_block, share); out /
 * lse as there.  While the key tiles stream by, every query keeps its num_selected best blocks so far; at the end
 * the kernel writes idx int32 and fmask uint8, both [batch, kv_heads, seq, num_selected]: block indices in
 * descending order of their logit (equal logits: lower block first - nsa_topk orders by the softmaxed values, which
 * agrees except where two distinct logits round to the same probability) and fmask = (probability > 1e-10), the
 * probability taken against the selected entries and the -1e3 pad column (every logit left out is at most the
 * smallest selected one, so this moves a probability at the threshold by less than its rounding).  Slots with
 * fmask = 0 hold unspecified valid block indices (as torch.topk's order among the exact zeros is unspecified).
 * Supported (nsa_compress_topk_supported != 0, else NSA_E_UNSUPPORTED): selections shared by the heads of a group
 * (share != 0) of at least 2 heads, num_selected <= min(16, number of selection blocks); other cases go through
 * nsa_dense_fwd + nsa_topk. */
int nsa_compress_topk_supported(const nsa_dense_desc* d, int32_t num_selected);
int nsa_compress_topk_fwd(const nsa_dense_desc* d, const void* q, const void* k, const void* v, void* out, float* lse,
                          int32_t num_selected, int32_t* idx, uint8_t* fmask, void* stream);

/* Block-importance softmax + per-query top-k.  Replaces NSA.py:693-695 (pad -1e3, softmax, drop
 * pad), :713 (topk) and :721 (fmask = value > 1e-10).  scores: fp32 [rows, nb]; with
 * apply_softmax != 0 they are importance logits (-inf = not selectable), otherwise ready
 * probabilities.  Outputs [rows, k]: idx int32 (descending value, ties to the lower block index -
 * torch.topk leaves tie order unspecified), vals fp32, fmask uint8.  A NaN or +inf score is ordered first and
 * comes out as value NaN with fmask 0.  Limits: nb <= 2048, k <= min(nb, 64) (NSA_E_UNSUPPORTED otherwise). */
int nsa_topk(const float* scores, int64_t rows, int32_t nb, int32_t k, int32_t apply_softmax,
             int32_t* idx, float* vals, uint8_t* fmask, void* stream);
/* The same for the logits of a causal compressed forward (nsa_dense_fwd with pool = 2): row r belongs to query
 * r % seq, and only its columns below floor(query / block) - the selection blocks that lie completely before the
 * query, NSA.py:676-689 - are defined; the rest counts as -inf and is never read (about half the matrix).  Same
 * results as nsa_topk on a matrix whose undefined part holds -inf.  rows must be a multiple of seq. */
int nsa_topk_prefix(const float* scores, int64_t rows, int32_t nb, int32_t k, int32_t apply_softmax,
                    int32_t seq, int32_t block, int32_t* idx, float* vals, uint8_t* fmask, void* stream);

/* Fused strategy-gate combine.  Replaces Sigmoid + Rearrange('b n (h s) -> b h n s') + the
 * stack/einsum + merge_heads of NSA.py:323-327, 854-860.  logits: bf16 contiguous [batch, seq,
 * 3*heads] (pre-sigmoid output of the gate projection, column 3*h+s, s = compressed, selected,
 * sliding); c, f, s: bf16 [batch, heads, seq, d] with element strides {batch, head, token};
 * out / d_out: bf16 contiguous [batch, seq, heads*d]; d_logits like logits; dc, df, ds contiguous
 * [batch, heads, seq, d]. */
int nsa_gate_fwd(int32_t batch, int32_t heads, int32_t seq, int32_t dim_head, const void* logits,
                 const void* c, const int64_t* c_stride, const void* f, const int64_t* f_stride,
                 const void* s, const int64_t* s_stride, void* out, void* stream);
int nsa_gate_bwd(int32_t batch, int32_t heads, int32_t seq, int32_t dim_head, const void* logits,
                 const void* c, const int64_t* c_stride, const void* f, const int64_t* f_stride,
                 const void* s, const int64_t* s_stride, const void* d_out,
                 void* d_logits, void* dc, void* df, void* ds, void* stream);

/* Rotary position embedding of queries or keys.  Replaces rotary_emb.rotate_queries_with_cached_keys
 * (NSA.py:643; third-party rotary_embedding_torch defaults: feature pairs (2k, 2k+1) rotated by
 * (i + offset) * freqs[k], fp32 arithmetic).  x: bf16 [batch, heads, seq, d] with element strides
 * {batch, head, token}; freqs: fp32 [d/2]; out: bf16 with element strides out_stride (NULL: contiguous;
 * a slot of a key cache otherwise, NSA.py:384-390).  inverse != 0 rotates by the negative angle (the
 * backward). */
int nsa_rope(const void* x, const int64_t* x_stride, int32_t batch, int32_t heads, int32_t seq, int32_t dim_head,
             const float* freqs, int32_t offset, int32_t inverse, void* out, const int64_t* out_stride, void* stream);

/* Compression windows.  Replaces split_compress_window (pad + unfold, NSA.py:270-275) and the
 * intra-window position add (NSA.py:600-603).  x: bf16 [batch, heads, seq, d] with element strides
 * {batch, head, token}; pos: bf16 [heads, block, d] or NULL; out: bf16 [batch, heads, seq / stride,
 * block, d] contiguous, window w = tokens (w+1)*stride - block .. (w+1)*stride - 1 (zeros left of token
 * 0) + pos.  nsa_windows_bwd: d_windows (same layout as out) -> dx bf16 [batch, heads, seq, d]
 * contiguous (overlap-add in gather form; the gradient of pos is the sum of d_windows over batch and
 * windows, left to the caller). */
int nsa_windows_fwd(const void* x, const int64_t* x_stride, const void* pos, int32_t batch, int32_t heads, int32_t seq,
                    int32_t dim_head, int32_t block, int32_t stride, void* out, void* stream);
int nsa_windows_bwd(const void* d_windows, int32_t batch, int32_t heads, int32_t seq, int32_t dim_head, int32_t block,
                    int32_t stride, void* dx, void* stream);

/* Epilogue of the fused qkv projection.  Replaces, in one pass over the projection's output, the head
 * split (NSA.py:583-587), split_compress_window + the intra-window position add on k and v
 * (NSA.py:589-603, 270-275) and the rotation of queries and keys (NSA.py:643); the backward replaces the
 * backward kernels of all of these plus the gradient sums and the concatenation in front of to_qkv.
 *   qkv     : [batch, seq, (heads + 2 kv_heads) * d] (q heads, then k heads, then v heads of a token;
 *             element strides qkv_stride = {batch, token}), fp32 if `fp32` else bf16
 *   freqs   : fp32 [d/2]; token i is rotated by (i + offset) * freqs[p] on feature pair (2p, 2p+1)
 *   k_pos, v_pos : intra-window positions [kv_heads, block, d] in the dtype of qkv
 *   rq, rk  : bf16 [batch, heads | kv_heads, seq, d] contiguous, rotated queries / keys
 *   q16, v16: bf16 contiguous head-split copies of the un-rotated queries / the values, or NULL (a bf16
 *             qkv is read in place by the attention kernels through strided views)
 *   k_windows, v_windows : [batch, kv_heads, seq / stride, block, d] contiguous in the dtype of qkv, window w
 *             = tokens (w+1)*stride - block .. (w+1)*stride - 1 (zeros left of token 0) + positions;
 *             not touched when block == 0 or seq < stride
 * nsa_qkv_prep_bwd: any of the six gradients (same layouts and dtypes as the outputs above) may be
 * NULL (= zero); d_qkv [batch, seq, (heads + 2 kv_heads) * d] with strides qkv_stride, dtype of qkv.  The
 * gradients of the positions (sums of the window gradients over batch and windows) are left to the caller.
 * dim_head 64 or 128 (NSA_E_UNSUPPORTED otherwise). */
typedef struct nsa_qkv_desc {
  int32_t batch, seq, heads, kv_heads, dim_head;
  int32_t block, stride;  /* compression window length and step (compress_block_size, compress_block_sliding_stride); block 0: no windows */
  int32_t fp32;           /* 1: qkv, positions, windows and d_qkv are fp32; 0: bf16; 2 (forward only): as 1, and rq / rk are
                             written as fp32 too, q16 / v16 are not written (inputs of the fp32 forward kernels below) */
  int32_t offset;         /* rotary position of token 0 */
  int64_t qkv_stride[2];
} nsa_qkv_desc;
int nsa_qkv_prep_fwd(const nsa_qkv_desc* d, const void* qkv, const float* freqs, const void* k_pos, const void* v_pos,
                     void* q16, void* rq, void* rk, void* v16, void* k_windows, void* v_windows, void* stream);
int nsa_qkv_prep_bwd(const nsa_qkv_desc* d, const void* d_q16, const void* d_rq, const void* d_rk, const void* d_v16,
                     const void* d_k_windows, const void* d_v_windows, const float* freqs, void* d_qkv, void* stream);

/* RMS norm over the model dimension in front of the projections.  Replaces self.norm = nn.RMSNorm(dim)
 * (NSA.py:230, applied at NSA.py:369 and 579) and its backward.  x: bf16 [rows, dim], row stride x_row_stride
 * elements; weight: bf16 [dim]; y, dy, dx: bf16 [rows, dim] contiguous; rstd: fp32 [rows], written by the
 * forward and read by the backward.  y = x * rsqrt(mean(x^2) + eps) * weight in fp32, rounded once.
 * nsa_rmsnorm_bwd: dweight (or NULL) is [dim], fp32 if dweight_fp32 else bf16, and then needs partials:
 * fp32 [nsa_rmsnorm_partials(rows) * dim] of scratch.  dim a multiple of 8, at most 4096 (NSA_E_UNSUPPORTED
 * otherwise). */
int nsa_rmsnorm_partials(int64_t rows);
int nsa_rmsnorm_fwd(int64_t rows, int32_t dim, const void* x, int64_t x_row_stride, const void* weight, float eps,
                    void* y, float* rstd, void* stream);
int nsa_rmsnorm_bwd(int64_t rows, int32_t dim, const void* x, int64_t x_row_stride, const void* weight, const float* rstd,
                    const void* dy, void* dx, void* dweight, int32_t dweight_fp32, float* partials, void* stream);

/* Column sums of a bf16 matrix in fp32: the bias gradient of a projection (the sum of d_out over tokens that
 * autograd takes for the nn.Linear layers of NSA.py:244-262, 853) and the gradient of the intra-window positions
 * (the sum of the window gradients over batch and windows, NSA.py:599-600).  Row (o, i) of group g starts at
 * x + g * group_stride + o * outer_stride + i * inner_stride (elements) and has `cols` contiguous entries;
 * out: [groups, cols], fp32 if out_fp32 else bf16, out[g] = sum over o < outer, i < inner.  workspace: fp32,
 * nsa_colsum_workspace(outer * inner, cols, groups) bytes.  cols and the strides multiples of 8
 * (NSA_E_UNSUPPORTED otherwise).  The order of the additions depends on the shape only. */
int64_t nsa_colsum_workspace(int64_t rows, int32_t cols, int32_t groups);
/* out[i] = sum over p < parts of slices[p * n + i] (fp32 in; out fp32 if out_fp32 else bf16): the sum of the partial
 * products of a weight gradient computed as a batched GEMM over slices of the token axis (the gradient autograd takes
 * for the projections of NSA.py:583, 853, 858 in one GEMM).  n a multiple of 4 (NSA_E_UNSUPPORTED otherwise). */
int nsa_sum_slices(const float* slices, int32_t parts, int64_t n, void* out, int32_t out_fp32, void* stream);
int nsa_colsum(const void* x, int32_t groups, int64_t group_stride, int64_t outer, int64_t outer_stride, int64_t inner,
               int64_t inner_stride, int32_t cols, void* out, int32_t out_fp32, float* workspace, void* stream);

/* fp32 forward of the attention branches, for fp32 modules run for inference: products, softmax and
 * accumulation in fp32 on the vector ALUs, so that the result agrees with the reference's fp32 torch path
 * to its own test tolerance (1e-5, tests/test_sparse_attn.py:86), which the bf16 MFMA kernels cannot.
 * Same contracts and descriptors as nsa_dense_fwd (without the importance logits, which are linear in q and
 * the compressed keys and cost one small fp32 GEMM) and nsa_select_fwd (no workspaces, no inverse index);
 * q, k, v: fp32 with element strides {batch, head, token}, key / value rows 16-byte aligned; out: fp32
 * contiguous [batch, heads, seq, d]; lse: fp32 [batch, heads, seq] or NULL.  `seq` of the descriptor is the number
 * of query rows; query row i sits at sequence position i + q_offset (0 for the parallel forward; the cached length
 * for a decode step with seq = 1, NSA.py:338-547), and k / v hold num_mem + num_keys rows (dense) or num_keys rows
 * (selection; idx / fmask are [batch, kv_heads, seq, num_sel]).  Any dim_head <= 128 that is a multiple of 4,
 * any group size, any block size; no backward. */
int nsa_dense_fwd_f32(const nsa_dense_desc* d, const float* q, const float* k, const float* v, float* out, float* lse,
                      int32_t q_offset, void* stream);
int nsa_select_fwd_f32(const nsa_select_desc* d, const float* q, const float* k, const float* v, const void* idx,
                       const uint8_t* fmask, float* out, float* lse, int32_t num_keys, int32_t q_offset, void* stream);

/* Single-token decode attention over cached keys / values.  Replaces the three attention
 * computations of SparseAttention.forward_inference (NSA.py:396-420 compressed, :446-515 selected
 * blocks + own block, :519-530 sliding window).
 *   mode 0: the group's query heads attend keys [start, start + count) of the caches, preceded by
 *           num_mem memory rows (mem_k / mem_v: bf16 [kv_heads, num_mem, d], contiguous; NSA.py:401-405).
 *           logits (optional): fp32 [batch, heads, count] = scale * q.k of the cache keys, the
 *           importance scores of NSA.py:444.
 *   mode 1: keys of blocks idx[slot] (where fmask[slot] != 0 and the block starts before kv_len) plus
 *           the block holding position kv_len - 1 up to that position.  idx / fmask:
 *           [batch, kv_heads, num_sel] or, with per_head_sel, [batch, heads, num_sel].
 * q: bf16 [batch, heads, d] with element strides {batch, head}; k, v: bf16 caches [batch, kv_heads,
 * capacity, d] with element strides {batch, head, token}; out: bf16 [batch, heads, d] contiguous.
 * ws: nsa_decode_workspace_bytes() bytes of device memory (split-K partials).  The caller
 * guarantees start + count <= capacity and kv_len <= capacity. */
typedef struct nsa_decode_desc {
  int32_t batch, kv_heads, group, dim_head;
  int32_t mode;
  int32_t start, count, num_mem;          /* mode 0 */
  int32_t block, num_sel, kv_len;         /* mode 1 */
  int32_t per_head_sel, idx_is_int64;     /* mode 1 */
  float scale;
  int64_t q_stride[2], k_stride[3], v_stride[3];
} nsa_decode_desc;
int nsa_decode_workspace_bytes(const nsa_decode_desc* desc, size_t* bytes);
int nsa_decode_attend(const nsa_decode_desc* desc, const void* q, const void* k, const void* v, const void* mem_k,
                      const void* mem_v, const void* idx, const uint8_t* fmask, void* ws, size_t ws_bytes, void* out,
                      float* logits, void* stream);

/* nsa_decode_attend without a caller workspace and without any allocation: the split-K partials live in a fixed
 * device array of the library (NSA_DECODE_NOALLOC_SCRATCH_BYTES per GPU, held until the process ends).  No
 * counterpart in the reference; it is for callers that cannot allocate device memory - a stream under HIP graph
 * capture, a serving loop or harness that forbids hipMalloc.  Same arguments and results as nsa_decode_attend
 * with out != NULL (out is required: the partials are private).  NSA_E_WORKSPACE when
 * nsa_decode_workspace_bytes(desc) exceeds NSA_DECODE_NOALLOC_SCRATCH_BYTES.  All calls on one GPU share the
 * array: calls that overlap on one GPU (different streams or threads) race; calls ordered on one stream do not.
 * The first call on a device looks the array's address up (hipGetSymbolAddress) and should be made outside a
 * stream capture.  The array used is the current device's (hipGetDevice at the time of the call): `stream` must
 * belong to the current device, as every pointer argument does. */
#define NSA_DECODE_NOALLOC_SCRATCH_BYTES ((size_t)16 << 20)
int nsa_decode_attend_noalloc(const nsa_decode_desc* desc, const void* q, const void* k, const void* v, const void* mem_k,
                              const void* mem_v, const void* idx, const uint8_t* fmask, void* out, float* logits, void* stream);

/* Decode step: block selection from the compressed branch's logits.  Replaces the reduce over the
 * compressed keys of a block and over the heads of a group, the padded softmax, topk and the mask of
 * NSA.py:448-476, 502.  logits: fp32 [batch, heads, num_compressed] as written by nsa_decode_attend;
 * the first (num_compressed / per_block) * per_block columns are used.  share != 0: one selection per
 * kv head (mean over its group heads), rows = batch * kv_heads; otherwise per head, rows = batch * heads.
 * Outputs [rows, k] as for nsa_topk. */
int nsa_decode_topk(const float* logits, int32_t batch, int32_t kv_heads, int32_t group, int32_t num_compressed,
                    int32_t per_block, int32_t share, int32_t k, int32_t* idx, float* vals, uint8_t* fmask, void* stream);

/* Decode step, after three nsa_decode_attend calls with out == NULL (their partials left in the
 * three workspaces): merges each branch, applies the sigmoid strategy gate and writes the merged
 * heads.  Replaces to_strategy_combine's sigmoid + rearrange, the stack / einsum and merge_heads of
 * NSA.py:534-545.  gate_logits: bf16 [batch, 3 * heads], column 3 * head + {0 compressed, 1 selected,
 * 2 sliding}; out: bf16 [batch, heads * d].  A branch whose workspace is NULL contributes zero (the
 * compressed branch before the first compressed key exists, NSA.py:401). */
int nsa_decode_combine(const nsa_decode_desc* compressed, const void* ws_compressed, const nsa_decode_desc* selected,
                       const void* ws_selected, const nsa_decode_desc* sliding, const void* ws_sliding,
                       const void* gate_logits, void* out, void* stream);

/* The attention part of one decode step (NSA.py:377-545 without the projections and the compression of
 * a completed window) as one host call: nsa_decode_prep, the compressed branch, nsa_decode_topk, the
 * selected-block branch, the sliding branch and nsa_decode_combine, with all intermediates in `ws`.
 * pos = rows already in the key / value caches (the new token's position); the caches must have row
 * pos free.  num_sel is the configured number of blocks; min(num_sel, num_compressed / per_block) are
 * selected, their indices (int32) and mask (uint8), [batch, kv_heads or heads, k], are left in the
 * workspace at the offsets nsa_decode_step_workspace_bytes reports.  q, k, v: the new token's
 * projections, bf16 [batch, heads | kv_heads, d], element strides {batch, head}; gate_logits: bf16
 * [batch, 3 * heads]; out: bf16 [batch, heads * d]. */
typedef struct nsa_decode_step_desc {
  int32_t batch, heads, kv_heads, dim_head;
  int32_t pos, num_compressed, num_mem, per_block, block, num_sel, share, window;
  float scale;
  int64_t q_stride[2], k_stride[2], v_stride[2];
  int64_t kc_stride[3], vc_stride[3];     /* key / value caches [batch, kv_heads, capacity, d] */
  int64_t ck_stride[3], cv_stride[3];     /* compressed key / value caches */
  int64_t krun_stride[2], vrun_stride[2]; /* rows of the open compression window (if passed) */
} nsa_decode_step_desc;
int nsa_decode_step_workspace_bytes(const nsa_decode_step_desc* desc, size_t* bytes, size_t* idx_offset, size_t* fmask_offset,
                                    int32_t* num_selected);
int nsa_decode_step(const nsa_decode_step_desc* desc, const void* q, const void* k, const void* v, const float* freqs,
                    void* k_cache, void* v_cache, const void* ck_cache, const void* cv_cache, const void* mem_k,
                    const void* mem_v, void* k_run_row, void* v_run_row, const void* gate_logits, void* ws, size_t ws_bytes,
                    void* out, void* stream);

/* nsa_decode_step with the lengths read from device memory when the kernels run, so that the whole step can be
 * recorded once into a HIP graph and replayed for every token (the host-side cost of a step is otherwise several
 * times the kernels' run time at small batch).  No counterpart in the reference, whose decode step re-derives all
 * shapes on the host (NSA.py:338-547).
 * state: device int32[2] = {rows already in the key / value caches (the new token's position), compressed keys
 * cached}.  `capacity` is a step descriptor whose pos and num_compressed give the LAST position the caches have a
 * row for and the rows of the compressed caches: grids, the workspace and the selection's row stride are sized for
 * them; min(num_sel, state[1] / per_block) blocks are selected.  k_run / v_run (optional, both or neither): rings of
 * run_ring rows per (batch, kv head), element strides capacity->krun_stride / vrun_stride {batch, head} and
 * krun_row_stride / vrun_row_stride; the un-rotated key / value of the new token go to row state[0] % run_ring.
 * gate_logits: bf16, row b at gate_logits + b * gate_row_stride (0: rows are contiguous), gate_bias (optional, bf16
 * [3 * heads]) is added to them - so the gate projection can be columns of the same GEMM as q, k, v.
 * advance != 0: the call's last kernel adds 1 to state[0].  Counters beyond the capacities are clamped (a step replayed
 * past the last cache row writes nothing).  The call neither allocates nor synchronises. */
int nsa_decode_step_dyn(const nsa_decode_step_desc* capacity, int32_t* state, const void* q, const void* k, const void* v,
                        const float* freqs, void* k_cache, void* v_cache, const void* ck_cache, const void* cv_cache,
                        const void* mem_k, const void* mem_v, void* k_run, void* v_run, int64_t krun_row_stride,
                        int64_t vrun_row_stride, int32_t run_ring, const void* gate_logits, int64_t gate_row_stride,
                        const void* gate_bias, void* ws, size_t ws_bytes, void* out, int32_t advance, void* stream);

/* Decode step: rotates the new token's queries (-> rq, bf16 [batch, heads, d] contiguous) and keys to
 * position pos, writes the rotated keys into row pos of the key cache and the values into row pos
 * of the value cache.  Replaces rotate_queries_or_keys x2 and the two cache concatenations of
 * NSA.py:384-393.  q, k, v: bf16 [batch, heads|kv_heads, d] with element strides {batch, head};
 * k_row / v_row: address of row pos of head 0 of batch 0 in the caches, strides {batch, head}.
 * k_run_row / v_run_row (optional, both or neither): where the un-rotated key / value rows of the open
 * compression window go (NSA.py:377-380), same addressing. */
int nsa_decode_prep(const void* q, const int64_t* q_stride, const void* k, const int64_t* k_stride, const void* v,
                    const int64_t* v_stride, int32_t batch, int32_t heads, int32_t kv_heads, int32_t dim_head,
                    const float* freqs, int32_t pos, void* rq, void* k_row, const int64_t* k_row_stride, void* v_row,
                    const int64_t* v_row_stride, void* k_run_row, const int64_t* k_run_stride, void* v_run_row,
                    const int64_t* v_run_stride, void* stream);

/* Same as nsa_select_fwd / nsa_select_bwd, additionally recording the caller's hipEvent_t
 * handles (created with timing enabled) between the kernels of the call, so that a benchmark
 * can time each kernel on the launch stream.  Events: fwd {start, after block walk, after
 * merge}; bwd {start, after delta, after the separate dQ walk (only run when sel_grads is
 * requested), after the dK/dV(+dQ) walk, after dQ merge, after dK/dV reduce}.  NULL entries are skipped.  No reference counterpart (measurement hook). */
int nsa_select_fwd_timed(const nsa_select_desc* d, const void* q, const void* k, const void* v,
                         const void* idx, const uint8_t* fmask, const void* index_ws, void* fwd_ws, size_t fwd_bytes,
                         void* out, float* lse, void* stream, void* const* events, int num_events);
int nsa_select_bwd_timed(const nsa_select_desc* d, const void* q, const void* k, const void* v,
                         const void* out, const void* d_out, const float* d_lse, const float* lse,
                         const void* idx, const uint8_t* fmask, const void* index_ws, void* bwd_ws, size_t bwd_bytes,
                         void* dq, void* dk, void* dv, float* sel_grads, void* stream, void* const* events, int num_events);

#ifdef __cplusplus
}
#endif
#endif /* NSA_HIP_H */
