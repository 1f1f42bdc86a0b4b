/* liblandmark_hip.so — C ABI of the MI355X (gfx950) landmark-attention kernels.
 *
 * Plain pointers and sizes only; the caller (the Python shim in
 * landmark_hip/, or any other host) owns every buffer, passes device pointers
 * and the HIP stream to run on.  Nothing is allocated, nothing synchronises.
 *
 * Return value of every entry point:  0 = launched;  < 0 = argument error
 * detected on the host before any GPU work (LMK_ERR_*, testable without a GPU);
 * > 0 = a hipError_t from the launch.
 *
 * Tensors are 16-bit (bf16 or fp16), logical shape (B, H, L, D) with element
 * strides (stride_b, stride_h, stride_row) and unit stride along D.  Every base
 * pointer and every stride*2 bytes must be a multiple of 16 bytes.
 */
#ifndef LMK_H
#define LMK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LMK_DTYPE_BF16 0
#define LMK_DTYPE_F16 1

#define LMK_OK 0
#define LMK_ERR_NULL (-1)        /* a required pointer is NULL */
#define LMK_ERR_SHAPE (-2)       /* non-positive or inconsistent sizes */
#define LMK_ERR_UNSUPPORTED (-3) /* head dim / block size / dtype outside the built set, or rows * row stride of a slice >= 4 GiB */
#define LMK_ERR_ALIGN (-4)       /* pointer or stride not 16-byte aligned */
#define LMK_ERR_HISTORY (-5)     /* Lk - Lq is not n_prefix * block */
#define LMK_ERR_PARTIAL (-6)     /* backward needs Lq and Lk to be whole blocks */
#define LMK_ERR_SCALE (-7)       /* softmax scale must be finite and > 0 */
#define LMK_ERR_WORKSPACE (-8)   /* workspace too small */
#define LMK_ERR_CACHE (-9)       /* cache holds no complete block (or, for lmk_local_window, no tail) */
#define LMK_ERR_TOPK (-10)       /* top_k outside 1..64 */
#define LMK_ERR_TABLE (-11)      /* rotary tables hold fewer positions than the cache */

typedef struct lmk_tensor4 {
  void* ptr;          /* device pointer */
  int64_t stride_b;   /* element strides */
  int64_t stride_h;
  int64_t stride_row;
} lmk_tensor4;

/* Human-readable text for a return code (static storage). */
const char* lmk_strerror(int code);

/* Library / build identification: "landmark_hip <version> gfx950". */
const char* lmk_version(void);

/* Forward pass.  Replaces the launch of `_fwd_kernel` in
 * FusedLandmarkAttention.forward (llama/ltriton/flash_landmark_attention.py:311-353,
 * kernel :6-122).
 *   q, o: (B,H,Lq,D); k, v: (B,H,Lk,D); L, M: (B*H, Lq) fp32, contiguous.
 *   block: landmark block size (landmark = last key of each block); 32, 64 or 128.
 *   n_prefix: number of history blocks, (Lk - Lq) / block  (:396-398).
 *   L = sum exp(s - M), M = max of the scaled scores over the query's global bucket
 *   (natural-log units, as the reference stores them, :116-119).
 * Lq need not be a multiple of block (the reference masks partial tiles, :44,:118-122). */
int lmk_attn_fwd(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                 float* L, float* M, int B, int H, int Lq, int Lk, int D, float sm_scale, int block,
                 int n_prefix, int dtype, void* stream);

/* Forward pass for callers that do not differentiate (inference prefill): q arrives WITHOUT rotary and is
 * rotated in registers as the kernel loads it, at positions position_ids[b*pos_stride_b + row] (device
 * int64; pos_stride_b = 0 shares one row of positions over the batch), with the same three roundings
 * as lmk_apply_rotary -- the output equals lmk_attn_fwd on the rotated q bit for bit, and q's own pass
 * of apply_rotary_pos_emb (llama/llama_mem.py:298) disappears.  k must already carry its rotary (its
 * rows reach LDS by direct loads that cannot rotate them).  Tables as for lmk_apply_rotary. */
int lmk_attn_fwd_rotary_q(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                          float* L, float* M, const void* cos_table, const void* sin_table, int64_t table_stride_row,
                          int64_t n_pos, const int64_t* position_ids, int64_t pos_stride_b, int B, int H, int Lq, int Lk,
                          int D, float sm_scale, int block, int n_prefix, int dtype, void* stream);

/* Bytes of device workspace lmk_attn_bwd needs (0 for invalid sizes):
 * 2*(B*H*Lq) floats of per-row terms + 3*(B*H*(Lk/block)*Lq) floats of per-(row, block)
 * terms handed from the dQ kernel to the dK/dV kernel. */
size_t lmk_attn_bwd_workspace_bytes(int B, int H, int Lq, int Lk, int block);

/* Bytes of workspace that select the HAND-OVER backward (block 32 only; 0 where it does not apply).
 * Handed a workspace of at least this size, lmk_attn_bwd lets the dQ kernel leave dS of every
 * (query tile, key block) pair behind as 16-bit tiles (2 KB per pair of 32 x 32, about Lq*(Lk+Lq)/2 * 2 bytes
 * per (batch, head): 274 MB at B2 H32 L2048, 8.6 GB at B1 H32 L16384) and the dK/dV kernel reads them
 * instead of forming dP and dS a second time -- each score and each dP is then formed twice per step, not
 * three times.  With a smaller workspace (>= lmk_attn_bwd_workspace_bytes) the recomputing kernels run.
 * The reference forms S and dP once in one kernel (flash_landmark_attention.py:246-299) and pays for it with
 * one program per (batch, head). */
size_t lmk_attn_bwd_handover_workspace_bytes(int B, int H, int Lq, int Lk, int block);

/* Backward pass.  Replaces the launches of `_bwd_preprocess` and `_bwd_kernel` in
 * FusedLandmarkAttention.backward (llama/ltriton/flash_landmark_attention.py:356-389,
 * kernels :125-149 and :152-305).
 *   inputs: q, k, v, o (forward output), dout (gradient of o), L, M (forward statistics);
 *   outputs: dq (B,H,Lq,D), dk, dv (B,H,Lk,D) in the tensors' 16-bit dtype (accumulated in
 *   fp32, rounded once); every element is written, nothing needs zeroing.
 *   workspace: 16-byte aligned device memory of at least lmk_attn_bwd_workspace_bytes(); one of at least
 *   lmk_attn_bwd_handover_workspace_bytes() (when that is not 0) selects the faster hand-over kernels.
 * Lq and Lk must be multiples of block (as in the reference, :359-360). */
int lmk_attn_bwd(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                 const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                 const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B, int H,
                 int Lq, int Lk, int D, float sm_scale, int block, int n_prefix, int dtype, void* stream);

/* Same as lmk_attn_bwd but runs only the kernels selected by `phases` (LMK_BWD_PRE: row terms,
 * LMK_BWD_DQ: dQ and the per-block terms, LMK_BWD_DKDV: dK and dV), in that order.  Each phase
 * consumes what the earlier ones left in `workspace`, so a subset is only meaningful after a
 * full run on the same arguments; it exists to time and profile the kernels one by one.
 * The dQ kernel computes the row terms itself: LMK_BWD_PRE launches the separate row-term kernel
 * only when LMK_BWD_DQ is not selected.
 * No counterpart in the reference (its backward is a single launch, :373-388). */
#define LMK_BWD_PRE 1
#define LMK_BWD_DQ 2
#define LMK_BWD_DKDV 4
#define LMK_BWD_ALL 7
int lmk_attn_bwd_phases(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                        const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B,
                        int H, int Lq, int Lk, int D, float sm_scale, int block, int n_prefix, int dtype, int phases,
                        void* stream);

/* ---- landmark blocks of any size -------------------------------------------------------
 * FusedLandmarkAttention.forward takes any block_size (llama/ltriton/flash_landmark_attention.py:318;
 * the training models use mem_freq + 1 = 51, lm_benchmark/config/rotary.py:57).  The kernels work on
 * blocks of 32, 64 or 128 slots, so a narrower block is stored PADDED: its block_real - 1 normal
 * tokens in front, zero rows, and its landmark in the last of `block` slots.  The padded entry
 * points mask the padding slots in every softmax, so the results at the real rows equal those of the
 * unpadded problem; rows of o / dq / dk / dv at padding slots hold values of no meaning.
 * block is 64 or 128 and 2 <= block_real <= block (block_real == block is the plain call, then 32
 * is accepted too).  Lq, Lk and n_prefix count PADDED rows and stored blocks.
 * dout must be zero at padding rows (lmk_pad_blocks writes zeros there) and o at padding rows must be what
 * lmk_attn_fwd_padded left there (finite): the dK/dV kernel carries no mask of its own and multiplies those rows
 * by zero weights, so a NaN or Inf there would reach real rows of dk and dv.  lmk_attn_*_blocks below have no such
 * requirement. */

/* Rows of a padded tensor that holds `rows` real rows: whole blocks widen to `block`, a partial
 * last block keeps its length.  -1 for invalid sizes. */
int64_t lmk_padded_rows(int64_t rows, int block_real, int block);

/* dst (B,H,lmk_padded_rows(rows),D) <- src (B,H,rows,D): every row of dst is written. */
int lmk_pad_blocks(const lmk_tensor4* src, const lmk_tensor4* dst, int B, int H, int64_t rows, int D,
                   int block_real, int block, void* stream);
/* dst (B,H,rows,D) <- src (B,H,lmk_padded_rows(rows),D): drops the padding rows. */
int lmk_unpad_blocks(const lmk_tensor4* src, const lmk_tensor4* dst, int B, int H, int64_t rows, int D,
                     int block_real, int block, void* stream);

/* lmk_attn_fwd / lmk_attn_bwd on padded tensors (same kernels, same workspace formula with the
 * padded sizes). */
int lmk_attn_fwd_padded(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        float* L, float* M, int B, int H, int Lq, int Lk, int D, float sm_scale, int block,
                        int block_real, int n_prefix, int dtype, void* stream);
int lmk_attn_bwd_padded(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                        const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B,
                        int H, int Lq, int Lk, int D, float sm_scale, int block, int block_real, int n_prefix,
                        int dtype, void* stream);

/* The same without any repacking: q, k, v, o (and dout, dq, dk, dv) keep their rows as they are -- Lq, Lk, L and M
 * count TOKENS of blocks of block_tokens (2..128) -- and the kernels translate the slots they work on into token
 * rows as they load and store (a slot without a token re-reads its block's first token and is masked).  This is what
 * FusedLandmarkAttention.forward / backward do for a block_size that is not 32, 64 or 128
 * (flash_landmark_attention.py:318; lm_benchmark's mem_freq + 1 = 51): no padded copies, no extra launches.
 * block_tokens of 32, 64 or 128 is the plain call.  n_prefix = (Lk - Lq) / block_tokens; the backward needs whole
 * blocks; its workspace (lmk_attn_bwd_blocks_workspace_bytes) is indexed by slots. */
int lmk_attn_fwd_blocks(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        float* L, float* M, int B, int H, int Lq, int Lk, int D, float sm_scale, int block_tokens,
                        int n_prefix, int dtype, void* stream);
size_t lmk_attn_bwd_blocks_workspace_bytes(int B, int H, int Lq, int Lk, int block_tokens);
int lmk_attn_bwd_blocks(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                        const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                        const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes, int B,
                        int H, int Lq, int Lk, int D, float sm_scale, int block_tokens, int n_prefix, int dtype,
                        void* stream);

/* Landmarks at irregular positions: blocks of unequal length.  The reference's fused kernel rejects such masks
 * (flash_landmark_attention.py:393-394); its high-level path takes any is_mem
 * (llama_mem.py:222-243, lm_benchmark/models/landmark.py:88-119) and this is that semantics on the fused kernels.
 * The keys' blocks are described by a table of n_blocks + 1 token offsets: seg[b] = first token of block b,
 * seg[0] = 0, seg[n_blocks] = Lk; every block ends in its landmark except, with last_is_partial, the last one
 * (tokens behind the last landmark, at most max_block_tokens - 1 of them).  A complete block holds
 * 2 .. max_block_tokens (<= 128) tokens.  The table is
 * passed twice: seg_host is read and checked by the call itself (monotone, lengths in range, history made of whole
 * blocks: Lk - Lq == seg[n_prefix]), seg_dev is the copy in device memory the kernels read -- the caller keeps the
 * two identical.  Tensors, L and M are in token rows as in lmk_attn_fwd_blocks; the blocks are worked on in 64 or
 * 128 slots.  The backward needs complete blocks only; workspace: lmk_attn_bwd_segments_workspace_bytes. */
int lmk_attn_fwd_segments(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                          float* L, float* M, const int32_t* seg_host, const int32_t* seg_dev, int n_blocks,
                          int max_block_tokens, int last_is_partial, int B, int H, int Lq, int Lk, int D,
                          float sm_scale, int n_prefix, int dtype, void* stream);
size_t lmk_attn_bwd_segments_workspace_bytes(int B, int H, int n_blocks, int n_prefix, int max_block_tokens);
int lmk_attn_bwd_segments(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                          const lmk_tensor4* dout, const float* L, const float* M, const lmk_tensor4* dq,
                          const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace, size_t workspace_bytes,
                          const int32_t* seg_host, const int32_t* seg_dev, int n_blocks, int max_block_tokens, int B,
                          int H, int Lq, int Lk, int D, float sm_scale, int n_prefix, int dtype, void* stream);

/* Group dropout (lm_benchmark/models/landmark.py:110-113: `dropout(group_prob, p)` on the landmark probabilities
 * that scale the earlier blocks, while the softmax over the landmarks itself stays as it is).  The random draw is
 * the caller's: group_scale is (B*H, Lk/block_tokens, Lq) fp32, contiguous, and entry [bh][b][i] multiplies what
 * earlier block b contributes to query row i -- 0 for a dropped block, 1/(1-p) for a kept one; entries of a row's
 * own and later blocks are not read.  Same tensors, sizes and statistics as lmk_attn_*_blocks; block_tokens 2..128
 * (32 included: it runs in 64 slots here, the block-32 kernels carry no such factor).  The backward must be given
 * the forward's group_scale.  Workspace: lmk_attn_bwd_group_scale_workspace_bytes. */
int lmk_attn_fwd_group_scale(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                             float* L, float* M, const float* group_scale, int B, int H, int Lq, int Lk, int D,
                             float sm_scale, int block_tokens, int n_prefix, int dtype, void* stream);
size_t lmk_attn_bwd_group_scale_workspace_bytes(int B, int H, int Lq, int Lk, int block_tokens);
int lmk_attn_bwd_group_scale(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* v, const lmk_tensor4* o,
                             const lmk_tensor4* dout, const float* L, const float* M, const float* group_scale,
                             const lmk_tensor4* dq, const lmk_tensor4* dk, const lmk_tensor4* dv, void* workspace,
                             size_t workspace_bytes, int B, int H, int Lq, int Lk, int D, float sm_scale,
                             int block_tokens, int n_prefix, int dtype, void* stream);

/* ---- mem-cache retrieval (inference) --------------------------------------------------
 * The reference has no function boundary here: scoring, selection and gather are inline in
 * LlamaAttention.forward (llama/llama_mem.py:318-430) and the attend step follows at :447-477.
 * Conventions kept from there: the cache tuple is (K without rotary, V), each (B,H,S,D)
 * (:424-430); a block is mem_freq+1 tokens whose last token is the landmark; queries arrive
 * rotated; cos/sin are (n_pos, D) tables in the model dtype with the half-split layout of
 * LlamaRotaryEmbedding (:95-124) and `table_stride_row` elements between rows.
 * The cache must hold at least one complete block.  When it ends in an incomplete block
 * (S % block != 0, the state between two landmarks while decoding, :321-324) retrieval works on
 * the S - S % block tokens of the complete blocks, and the tail joins the local window of the
 * attend step (:329-342; see lmk_local_window). */

/* Bytes of device workspace lmk_retrieve_topk needs: rotated landmark keys (kept in tiles of 32 keys,
 * whole tiles per (batch, head)) and their norms, plus two fp32 planes of B*H*T*(S/block) for the
 * per-head selections and the decode path. */
size_t lmk_retrieve_workspace_bytes(int B, int H, int T, int S, int D, int block);

/* Landmark scoring + top-k selection (llama_mem.py:344-384, aggregate=None branch).
 *   idx_out: (B,H,T,k) int64, k = min(top_k, S/block), block indices in ascending order.
 * Score of (query, block) = fp32 dot product accumulated sequentially over the head dim,
 * rounded to the model dtype, divided by sqrt(D) in fp32 and rounded again; the k best
 * under (score descending, index ascending) are selected. */
int lmk_retrieve_topk(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table, const void* sin_table,
                      int64_t table_stride_row, int64_t n_pos, int64_t* idx_out, void* workspace,
                      size_t workspace_bytes, int B, int H, int T, int S, int D, int block, int top_k, int dtype,
                      void* stream);

/* Same as lmk_retrieve_topk when `workspace` still holds the rotated landmark keys a previous
 * lmk_retrieve_topk or lmk_retrieve_topk_reuse call left there for the same B, H, D, block, top_k, tables and
 * S/block, and the complete blocks of the cache have not changed since: the rotation of the landmark keys
 * (llama_mem.py:357-366) is skipped.  That is every decode step between two landmarks -- the positions
 * of :359-365 move only when a block completes -- when the cache is appended to in place.  T may differ from
 * call to call (the keys sit at the front of the workspace); workspace_bytes is checked for this call's T.
 * No counterpart in the reference, which rotates every cached landmark key on every call. */
int lmk_retrieve_topk_reuse(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table,
                            const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                            void* workspace, size_t workspace_bytes, int B, int H, int T, int S, int D, int block,
                            int top_k, int dtype, void* stream);

/* lmk_retrieve_topk for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): same arguments without the workspace, same kernels, same
 * indices.  It has no counterpart in the reference.  The workspace is a fixed array of
 * lmk_retrieve_static_max_bytes() = 16 MiB of device memory inside the library (one copy per GPU the library
 * runs on, held until the process ends); the call allocates and frees nothing.  Sizes whose workspace
 * (lmk_retrieve_workspace_bytes) exceeds that limit are rejected with LMK_ERR_WORKSPACE -- a decode step of
 * 32 heads against 32768 cached tokens needs 8.7 MB, a chunk of 256 queries does not fit.  Every call on a
 * GPU shares that GPU's array: calls that overlap on one GPU (two streams, two threads) race; calls on one
 * stream are ordered.  Nothing in the array needs to start at zero (every kernel writes what it later reads). */
size_t lmk_retrieve_static_max_bytes(void);
/* Looks up the array's address on the CURRENT device (hipGetSymbolAddress, once per device; later calls return at
 * once).  lmk_retrieve_topk_static does the same on its first call on a device, which is a runtime query and not a
 * stream operation: a caller that records the entry point into a HIP graph calls this (or makes one eager call)
 * on that device BEFORE the capture begins.  0, or a hipError_t. */
int lmk_retrieve_static_init(void);
int lmk_retrieve_topk_static(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table,
                             const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out, int B,
                             int H, int T, int S, int D, int block, int top_k, int dtype, void* stream);

/* Gather of the selected K/V blocks with rotary at their slot positions and attention over
 * them (llama_mem.py:386-412), merged with the attention over the local chunk (:447-477).
 *   o_loc, L_loc, M_loc: output and statistics of lmk_attn_fwd run on the local chunk;
 *   stat_stride: floats between consecutive (batch, head) rows of L_loc and M_loc (T when they
 *   are dense; larger when they are the last T columns of a wider window's statistics)
 *   (q against the T new keys/values); out: (B,H,T,D) final attention output.
 * Blocks are read in place from the cache; nothing of size (T, k*block, D) is materialised.
 * Built for D = 64 and 128 and block 32, 64 or 128. */
int lmk_gather_attend(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache, const int64_t* idx,
                      const void* cos_table, const void* sin_table, int64_t table_stride_row, int64_t n_pos,
                      const lmk_tensor4* o_loc, const float* L_loc, const float* M_loc, int64_t stat_stride,
                      const lmk_tensor4* out, int B, int H, int T, int S, int D, float sm_scale, int block, int top_k,
                      int dtype, void* stream);

/* The attend step in one call: lmk_local_window (when S % block > 0), lmk_attn_fwd on the local
 * window and lmk_gather_attend, enqueued back to back with the window, its output and its statistics
 * in `workspace` (at least lmk_attend_workspace_bytes(...) bytes, 16-byte aligned).  Same result as
 * the three calls -- llama_mem.py:321-342 (window), :386-412 and :447-477 (gather, scores, grouped
 * softmax, output) -- for callers whose per-call host cost matters: a decode step spends more time
 * in the binding than on the GPU.  k_loc, v_loc: the new chunk (B,H,T,D), keys rotated.
 * With at most four new tokens and a window inside one block (S % block + T <= block: decoding)
 * the call is ONE launch: the gather kernel attends to the window itself -- cached tail keys rotated at their
 * positions in the model dtype, the new keys as they are, causal, the landmark token not seeing itself -- as one
 * more item of each row's online softmax; nothing is written to `workspace` (its size is still checked). */
size_t lmk_attend_workspace_bytes(int B, int H, int T, int S, int D, int block);
int lmk_attend(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache, const int64_t* idx,
               const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table, const void* sin_table,
               int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* out, void* workspace,
               size_t workspace_bytes, int B, int H, int T, int S, int D, float sm_scale, int block, int top_k,
               int dtype, void* stream);

/* One inference step of the mem-cache path in one call: lmk_retrieve_topk (or lmk_retrieve_topk_reuse
 * when reuse_landmark_keys != 0) followed by lmk_attend on the indices it wrote -- llama_mem.py:321-412
 * and :447-477.  Same results as the two calls; idx_out (B,H,T,k) int64 is an output.  The call takes fewer
 * launches than the two: in decoding (the case lmk_attend serves in one launch) it is two launches -- the slice
 * step of the selection, then a gather that picks a row's k best from the slices' candidates and attends to the
 * row's local window itself; with blocks of 32 and more query rows the forward over the local window shares a
 * launch with a step of the selection (the slice step up to 1024 rows, else the rotation of the landmark keys). */
int lmk_retrieve_and_attend(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache,
                            const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table,
                            const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                            const lmk_tensor4* out, void* retrieve_workspace, size_t retrieve_workspace_bytes,
                            int reuse_landmark_keys, void* attend_workspace, size_t attend_workspace_bytes, int B,
                            int H, int T, int S, int D, float sm_scale, int block, int top_k, int dtype, void* stream);

/* ---- ring cache of blocks (lm_benchmark) -----------------------------------------------
 * Block selection of MemLMCacheStorage.retrieve_for_query
 * (lm_benchmark/models/caches/mem_cache.py:50-85): the cache is a ring buffer of `n_blocks`
 * filled block slots, slot `ring_start` (the reference's cache_iter once the ring is full, 0
 * before) holding the OLDEST block.  Landmark keys are rotated at the positions of :56-61 (the
 * top_k newest blocks at slots 1..top_k, every older block at slot 0, landmark token =
 * slot*block + block-1), scored against the queries, soft-maxed over the blocks in fp32 and
 * reduced as `method` says (:64-70); the top_k best slots are returned in order of age, oldest
 * first -- what the order-restoring sort of :73-84 produces.
 *   kring: (B,H,n_blocks*block,D) view of the filled slots, keys without rotary; the
 *          reference's (B, slot, token, head, dim) buffer is such a view with
 *          stride_row = H*D, stride_h = D.
 *   idx_out: int64 slot numbers; (B,H,T,top_k) for PER_TOKEN_AND_HEAD, (B,T,top_k) for
 *          MAX_OVER_HEADS (shared by the heads), (B,H,top_k) for MAX_OVER_TOKENS.
 *   workspace: lmk_retrieve_workspace_bytes(B,H,T,n_blocks*block,D,block) bytes.
 * top_k > n_blocks is an error (torch.topk raises there, :72).  Ties: (probability descending,
 * slot ascending) for the two aggregated methods; PER_TOKEN_AND_HEAD ranks by (16-bit score descending, slot
 * ascending), which is the probability order wherever two probabilities differ and also orders scores whose
 * exponentials collapse to one fp32 value, where torch.topk leaves the choice open.  Tables in the half-split layout of the other entry points; the benchmark's
 * interleaved pairs map onto it by moving the even head dims in front of the odd ones in q and k. */
#define LMK_SELECT_PER_TOKEN_AND_HEAD 0
#define LMK_SELECT_MAX_OVER_HEADS 1
#define LMK_SELECT_MAX_OVER_TOKENS 2
int lmk_ring_retrieve_topk(const lmk_tensor4* q, const lmk_tensor4* kring, const void* cos_table,
                           const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                           void* workspace, size_t workspace_bytes, int B, int H, int T, int n_blocks, int D, int block,
                           int top_k, int ring_start, int method, int dtype, void* stream);

/* Attention over the picked blocks of the ring, merged with the attention over the current chunk: the part of
 * MemLMCacheStorage.retrieve_for_query behind the selection (lm_benchmark/models/caches/mem_cache.py:86-109:
 * take_along_dim of the picked blocks' keys and values, keys rotated at k_indices = j*block + token, one block
 * further for a block among the top_k newest (:95-97), scores q.k/sqrt(D), is_mem prefix) and what
 * CausalSelfAttention.forward does with it (lm_benchmark/models/landmark.py:196-242: the picked blocks are earlier
 * landmark groups in front of the chunk, grouped softmax, att_prefix @ cache_v added to att @ v).
 *   q: (B,H,T,D) rotated queries; kring, vring: (B,H,n_blocks*block,D) views of the filled slots (keys without
 *   rotary), as for lmk_ring_retrieve_topk; idx: the slots that call returned, in its shape for `method`;
 *   o_loc, L_loc, M_loc, stat_stride: output and statistics of lmk_attn_fwd[_padded] over
 *   [tokens behind the last complete block (last_incomplete_k, rotated; :43-46) ; the chunk], rows of the chunk --
 *   as for lmk_gather_attend; out: (B,H,T,D).
 * block: 2..128 tokens (the benchmark's 51 are worked on in 64 slots; nothing is repacked); D 64 or 128. */
int lmk_ring_gather_attend(const lmk_tensor4* q, const lmk_tensor4* kring, const lmk_tensor4* vring, const int64_t* idx,
                           const void* cos_table, const void* sin_table, int64_t table_stride_row, int64_t n_pos,
                           const lmk_tensor4* o_loc, const float* L_loc, const float* M_loc, int64_t stat_stride,
                           const lmk_tensor4* out, int B, int H, int T, int n_blocks, int D, float sm_scale, int block,
                           int top_k, int ring_start, int method, int dtype, void* stream);

/* Local window of the attend step when the cache ends in an incomplete block of
 * inc = S % block tokens (llama_mem.py:329-342; needs inc > 0 and T + inc <= block, the
 * reference's assert at :330).  Writes, each (B,H,inc+T,D):
 *   k_win = [tail keys rotated at positions S-inc .. S-1 (:337-338) ; k_loc]   (:339)
 *   v_win = [tail values ; v_loc]                                               (:340)
 *   q_win = [inc zero rows ; q]
 * lmk_attn_fwd on (q_win, k_win, v_win) with Lq = Lk = inc + T and n_prefix = 0 then holds, in
 * its last T rows (o, L, M), the attention of the new tokens over the window: the o_loc, L_loc,
 * M_loc that lmk_gather_attend takes.  Replaces the torch.cat / apply_rotary_pos_emb calls of
 * :337-340; the mask rows :331-335 give the tail no landmark and put it in every query's last
 * section, which is what the forward kernel's own block does with rows in front of the queries. */
int lmk_local_window(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache,
                     const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table, const void* sin_table,
                     int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* q_win, const lmk_tensor4* k_win,
                     const lmk_tensor4* v_win, int B, int H, int T, int S, int D, int block, int dtype, void* stream);

/* The same window for the ring cache of lm_benchmark, whose incomplete last block lives outside the ring
 * (last_incomplete_k / last_incomplete_v, lm_benchmark/models/caches/mem_cache.py:43-46, 99-103): the first
 * `tail` rows of k_tail (without positions) are rotated at positions tail_position .. tail_position + tail - 1
 * and put in front of the chunk's keys; v_win = [tail values ; v_loc]; q_win = [tail zero rows ; q].
 * Each window is (B,H,tail+T,D); tail > 0. */
int lmk_ring_local_window(const lmk_tensor4* q, const lmk_tensor4* k_tail, const lmk_tensor4* v_tail,
                          const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table,
                          const void* sin_table, int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* q_win,
                          const lmk_tensor4* k_win, const lmk_tensor4* v_win, int B, int H, int T, int tail,
                          int64_t tail_position, int D, int dtype, void* stream);

/* Landmark scoring + ONE selection per (batch, head), shared by all T queries: the branch
 * `aggregate == "max_over_tokens"` of llama_mem.py:369-384, which the reference takes when the cache
 * is offloaded to the CPU (:369-370).  Per query: scores as in lmk_retrieve_topk, fp32 softmax over
 * the cached blocks, rounded to the model dtype (:376); per block: the maximum over the queries
 * (:377); then the k best blocks under (value descending, index ascending).
 *   idx_out: (B,H,k) int64 ascending (the reference's (B,H,1,k) view, :384);
 *   block_prob_out: NULL, or (B,H,S/block) 16-bit values in the model dtype that receive the
 *   per-head vector the selection ran on (`mem_attn_weights` after :377).
 * torch leaves the exponential's last bit and the order of the sum to its library, so both are
 * fixed here: 2^t by a degree-6 polynomial with separately rounded products and sums, a sum of
 * 64 strided partial sums folded by halves, one correctly rounded division.
 * Workspace: as for lmk_retrieve_topk (lmk_retrieve_workspace_bytes). */
int lmk_retrieve_topk_shared(const lmk_tensor4* q, const lmk_tensor4* kcache, const void* cos_table,
                             const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                             void* block_prob_out, void* workspace, size_t workspace_bytes, int B, int H, int T, int S,
                             int D, int block, int top_k, int dtype, void* stream);

/* lmk_retrieve_topk_shared for a cache whose blocks live elsewhere (host memory, the reference's
 * offload_cache_to_cpu branch, llama/llama_mem.py:326-328,344-356): landmark_keys is the tensor that branch
 * keeps on the GPU as past_key_value[2] -- (B,H,n_blocks,D), one un-rotated landmark key per complete block.
 * Same positions, contract, workspace (lmk_retrieve_workspace_bytes with S = n_blocks * block) and output. */
int lmk_retrieve_topk_shared_landmarks(const lmk_tensor4* q, const lmk_tensor4* landmark_keys, const void* cos_table,
                                       const void* sin_table, int64_t table_stride_row, int64_t n_pos, int64_t* idx_out,
                                       void* block_prob_out, void* workspace, size_t workspace_bytes, int B, int H, int T,
                                       int n_blocks, int D, int block, int top_k, int dtype, void* stream);

/* Keys and values every query of a head attends to after a per-head selection
 * (llama_mem.py:386-388, 393-406): with k = min(top_k, S/block) and inc = S % block,
 *   k_win = [selected blocks' keys rotated at their slot positions ; tail keys rotated at
 *            S-inc .. S-1 ; k_loc]                     (B,H,k*block+inc+T,D)
 *   v_win = [selected blocks' values ; tail values ; v_loc]
 *   q_win = [inc zero rows ; q]                        (B,H,inc+T,D); may be NULL when inc == 0
 * lmk_attn_fwd on (q_win or q, k_win, v_win) with Lq = inc+T, Lk = k*block+inc+T and
 * n_prefix = k is then the reference's fused_landmark_attention call on the concatenated
 * sequence (:441-446); its last T rows are the new tokens' output.  T + inc <= block when inc > 0
 * (:330).  Replaces take_along_dim, apply_rotary_pos_emb and the torch.cat calls of :393-406. */
int lmk_gather_window(const lmk_tensor4* q, const lmk_tensor4* kcache, const lmk_tensor4* vcache, const int64_t* idx,
                      const lmk_tensor4* k_loc, const lmk_tensor4* v_loc, const void* cos_table, const void* sin_table,
                      int64_t table_stride_row, int64_t n_pos, const lmk_tensor4* q_win, const lmk_tensor4* k_win,
                      const lmk_tensor4* v_win, int B, int H, int T, int S, int D, int block, int top_k, int dtype,
                      void* stream);

/* Rotary position embedding of one (B,H,L,D) tensor: out = x*cos[pos] + rotate_half(x)*sin[pos] with
 * pos = position_ids[b*pos_stride_b + l], rounded to the model dtype after each of the three elementwise
 * operations, i.e. bit for bit what apply_rotary_pos_emb (llama/llama_mem.py:127-149) yields for q or
 * for k in a 16-bit model (its call sites: :298 on the projections, :340, :366, :403 on cached keys).
 * position_ids: device int64, (B,L) with pos_stride_b = L, or one row shared by the batch with
 * pos_stride_b = 0; positions outside [0, n_pos) are clamped to the tables' ends.  out may alias x. */
int lmk_apply_rotary(const lmk_tensor4* x, const lmk_tensor4* out, const void* cos_table, const void* sin_table,
                     int64_t table_stride_row, int64_t n_pos, const int64_t* position_ids, int64_t pos_stride_b, int B,
                     int H, int L, int D, int dtype, void* stream);

/* The layer's own call, apply_rotary_pos_emb(query_states, key_states, cos, sin, position_ids)
 * (llama/llama_mem.py:298): q and k, both (B,H,L,D), rotated in ONE launch, each thread using the
 * table rows it fetched for both tensors.  Same bits as two lmk_apply_rotary calls.  Outputs may
 * alias their inputs. */
int lmk_apply_rotary_qk(const lmk_tensor4* q, const lmk_tensor4* k, const lmk_tensor4* q_out, const lmk_tensor4* k_out,
                        const void* cos_table, const void* sin_table, int64_t table_stride_row, int64_t n_pos,
                        const int64_t* position_ids, int64_t pos_stride_b, int B, int H, int L, int D, int dtype,
                        void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LMK_H */
