/* C ABI of the gfx950 block-sparse attention library (libspattn_hip.so).
 *
 * Plain pointers and sizes only.  Every pointer is DEVICE memory (HIP), contiguous,
 * 16-byte aligned.  q, k, v, o are bf16 [B,H,S,D] with D in {64,128}; index tensors are
 * int32; statistics are fp32.  Nothing is allocated or kept between calls; the caller owns
 * every buffer.  Kernels are enqueued asynchronously.
 *
 * Two groups of entry points:
 *   1. the seven functions the reference's binding layer calls, with the reference's own
 *      names and argument order (python/extension.cpp:4-49 declares them, python/cuda_attn.cu
 *      defines them).  They run on the legacy default stream like the reference, return
 *      nothing, and leave their status in spattn_last_status().
 *   2. spattn_* variants that add what the reference lacks: a status return, a stream,
 *      a runtime kv length, a softmax scale, a q-block size, an optional log-sum-exp
 *      output, and KV-block index lists.
 */
#ifndef SPATTN_HIP_H_
#define SPATTN_HIP_H_

#ifdef __cplusplus
extern "C" {
#endif

/* status codes (0 = ok, >0 = hipError_t of the launch) */
#define SPATTN_OK 0
#define SPATTN_ERR_NULL -1       /* a required pointer is null */
#define SPATTN_ERR_HEAD_DIM -2   /* D is not 64 or 128 */
#define SPATTN_ERR_STRIDE -3     /* mask_stride is not a positive multiple of 128 */
#define SPATTN_ERR_QBLK -4       /* q-block is not 64 or 128 */
#define SPATTN_ERR_ALIGN -5      /* a pointer is not 16-byte aligned */
#define SPATTN_ERR_SHAPE -6      /* a size is not positive / inconsistent, or seq >= 2^24 */
#define SPATTN_ERR_SCRATCH -7    /* more q-blocks than SPATTN_BALANCED_MAX_QBLOCKS, or first use on a device inside a stream capture */

/* q-blocks (batch * heads * ceil(seq / qblk)) that spattn_sp_attn_blocks_balanced can order */
#define SPATTN_BALANCED_MAX_QBLOCKS (1 << 20)

/* ---- group 1: the reference's binding surface ------------------------------------ */

/* Dense attention o = softmax(q k^T / sqrt(D)) v.
 * Replaces attn_fwd_wg_impl (python/extension.cpp:4-7, python/cuda_attn.cu:9-38). */
void attn_fwd_wg_impl(void* o, void* q, void* k, void* v, int batch, int heads, int seq, int D);

/* Gathered sparse attention: q-block I (128 rows) attends to the key tokens
 * kv_indices[b][h][I][0 .. num_kv_indices[b][h][I]) ; kv_indices is [B,H,ceil(S/128),mask_stride].
 * Replaces attn_sparse_fwd_wg_impl (python/extension.cpp:10-14, python/cuda_attn.cu:41-75). */
void attn_sparse_fwd_wg_impl(void* o, void* q, void* k, void* v, int* kv_indices, int* num_kv_indices,
                             int mask_stride, int batch, int heads, int seq, int D);

/* Identity lists: kv_indices[b][h][I][s] = s for s < 128*ceil(seq/128), counts = seq.
 * Replaces allindex_mask_impl (python/extension.cpp:17-20, python/cuda_attn.cu:78-94). */
void allindex_mask_impl(int* kv_indices, int* num_kv_indices, int batch, int heads, int seqblocks, int seq);

/* Dense attention that also writes the raw row max and the softmax denominator,
 * both fp32 [B,H,1,128*ceil(S/128)]; pad rows get max 0 and denominator -inf.
 * Replaces attn_maxq_denom_impl (python/extension.cpp:22-27, python/cuda_attn.cu:97-139). */
void attn_maxq_denom_impl(void* d_o, float* d_o_max_q, float* d_o_norm, void* d_q, void* d_k, void* d_v, int batch,
                          int heads, int seq, int D);

/* Row max and denominator only.
 * Replaces maxq_denom_impl (python/extension.cpp:29-33, python/cuda_attn.cu:142-180). */
void maxq_denom_impl(float* d_o_max_q, float* d_o_norm, void* d_q, void* d_k, int batch, int heads, int seq, int D);

/* Vote mask int32 [B,H,ceil(S/128),mask_stride]: entry (I,c) = number of 16-row groups of
 * q-block I in which some row has softmax(r,c) > threshold.  The entry is stored (the
 * reference adds into a caller-zeroed buffer; on a zeroed buffer the results agree).
 * Replaces booleanmask_128_impl (python/extension.cpp:36-41, python/cuda_attn.cu:183-266). */
void booleanmask_128_impl(int* d_booleanmask, float threshold, int mask_stride, float* d_o_max_q, float* d_o_norm,
                          void* d_q, void* d_k, int batch, int heads, int seq, int D);

/* Mask -> index lists: per row the keys c < seq with mask > 0 in ASCENDING order, then the
 * caller's fill; counts are exact.  (The reference's order is whatever its atomics give.)
 * Replaces booleanmask_to_indexmask_impl (python/extension.cpp:44-49, python/cuda_attn.cu:269-301). */
void booleanmask_to_indexmask_impl(int* d_indexmask, int* d_num_indices, int* d_booleanmask, int batch, int heads,
                                   int seq, int seqblocks, int mask_stride);

/* ---- group 2: extended entry points ------------------------------------------------
 * Common conventions: stream is a hipStream_t (NULL = legacy default stream);
 * kv_len <= 0 means seq; scale <= 0 means 1/sqrt(D); lse may be NULL, else fp32 [B,H,S]
 * natural-log log-sum-exp of the scaled scores over the attended keys.
 * Each returns a status code and also records it for spattn_last_status(). */

int spattn_full_attn(void* o, float* lse, const void* q, const void* k, const void* v, int batch, int heads, int seq,
                     int D, int kv_len, float scale, void* stream);

/* qblk in {64,128}: rows per q-block = rows sharing one list; kv_indices is
 * [B,H,ceil(S/qblk),mask_stride]. */
int spattn_sp_attn(void* o, float* lse, const void* q, const void* k, const void* v, const int* kv_indices,
                   const int* num_kv_indices, int mask_stride, int qblk, int batch, int heads, int seq, int D,
                   int kv_len, float scale, void* stream);

/* KV-block lists: blk_indices int32 [B,H,ceil(S/qblk),max_blocks] holds 64-key block ids,
 * blk_counts int32 [B,H,ceil(S/qblk)].  Block j stands for the tokens 64j .. 64j+63 (clipped
 * to kv_len), so this is the token-list op restricted to aligned runs. */
int spattn_sp_attn_blocks(void* o, float* lse, const void* q, const void* k, const void* v, const int* blk_indices,
                          const int* blk_counts, int max_blocks, int qblk, int batch, int heads, int seq, int D,
                          int kv_len, float scale, void* stream);

int spattn_all_index_mask(int* kv_indices, int* num_kv_indices, int batch, int heads, int seqblocks, int seq,
                          int mask_stride, void* stream);

int spattn_fullattn_maxq_denom(void* o, float* max_q, float* denom, const void* q, const void* k, const void* v,
                               int batch, int heads, int seq, int D, int kv_len, float scale, void* stream);

int spattn_maxq_denom(float* max_q, float* denom, const void* q, const void* k, int batch, int heads, int seq, int D,
                      int kv_len, float scale, void* stream);

int spattn_booleanmask_128(int* booleanmask, float threshold, int mask_stride, const float* max_q, const float* denom,
                           const void* q, const void* k, int batch, int heads, int seq, int D, int kv_len, float scale,
                           void* stream);

/* seq is the kv length (python/extension.cpp:326,338). */
int spattn_booleanmask_to_indexmask(int* kv_indices, int* num_kv_indices, const int* booleanmask, int batch, int heads,
                                    int seq, int seqblocks, int mask_stride, void* stream);

/* Bit-packed masks for the mask cache: one bit per key, least significant bit first, rows of
 * mask_stride / 8 bytes -- the layout of `pack` (python/spattn/mask_utils.py:421-430).
 * spattn_pack_mask sets a bit where the int32 vote mask is > 0 (what
 * CompressedBitMaskCache.update_cache stores, python/spattn/mask_utils.py:92-98);
 * spattn_packedmask_to_indexmask is the fused form of `unpack` followed by
 * booleanmask_to_indexmask (CompressedBitMaskCache.get_mask_from_cache,
 * python/spattn/mask_utils.py:86-90): ascending keys c < seq whose bit is set, then the
 * caller's fill; exact counts.  `packed` holds batch*heads*seqblocks*mask_stride/8 bytes. */
int spattn_pack_mask(void* packed, const int* booleanmask, int batch, int heads, int seqblocks, int mask_stride,
                     void* stream);
int spattn_packedmask_to_indexmask(int* kv_indices, int* num_kv_indices, const void* packed, int batch, int heads,
                                   int seq, int seqblocks, int mask_stride, void* stream);

/* The threshold sweep of booleanmask_128 (include/mask_utils.cuh:131-243) with a bit-packed
 * result: one bit per (q-block, key), set where some row r of the q-block has
 * softmax(r, key) > threshold and key < kv_len - the `> 0` view of the vote mask that every
 * consumer of the reference takes (python/spattn/mask_utils.py:269, include/mask_utils.cuh:297),
 * in the layout of `pack` (python/spattn/mask_utils.py:421-430; least significant bit first).
 * qblk = 128: rows are the reference's 128-row q-blocks, packed is
 * [batch,heads,ceil(seq/128),mask_stride/8] bytes and equals spattn_pack_mask of the vote mask.
 * qblk = 64: one row per 64-row q-block, [batch,heads,ceil(seq/64),mask_stride/8]: the votes
 * of the two halves of a 128-row block are kept apart (the lists a 64-row-q-block attention
 * kernel needs).  Every word of every row is written; 1/32 of the bytes of the int32 mask. */
int spattn_booleanmask_packed(void* packed, float threshold, int mask_stride, int qblk, const float* max_q,
                              const float* denom, const void* q, const void* k, int batch, int heads, int seq, int D,
                              int kv_len, float scale, void* stream);

/* Key mask -> KV-block lists.  Key block J (keys 64J .. 64J+63) of a mask row is kept when one
 * of its keys c < seq is set: MB[row,J] = OR_c M[row,c]  (the block form of
 * booleanmask_to_indexmask, include/mask_utils.cuh:273-302; seq is the kv length).
 * blk_indices int32 [batch,heads,seqblocks,max_blocks] receives the kept block ids of each row
 * in ASCENDING order, entries behind them keep the caller's fill; blk_counts int32
 * [batch,heads,seqblocks] the number of kept blocks (if it exceeds max_blocks only the first
 * max_blocks ids are written; the attention entry points clamp a count to max_blocks).
 * blockmask may be NULL, else uint8 [batch,heads,seqblocks,mask_stride/64] receives MB (0/1).
 * The outputs feed spattn_sp_attn_blocks directly.  Sources: the bit-packed mask
 * (seqblocks rows of mask_stride/8 bytes) or the int32 vote mask. */
int spattn_packedmask_to_blocklists(int* blk_indices, int* blk_counts, void* blockmask, const void* packed, int batch,
                                    int heads, int seq, int seqblocks, int mask_stride, int max_blocks, void* stream);
int spattn_booleanmask_to_blocklists(int* blk_indices, int* blk_counts, void* blockmask, const int* booleanmask,
                                     int batch, int heads, int seq, int seqblocks, int mask_stride, int max_blocks,
                                     void* stream);

/* Block-level pre-pass without a second score sweep.  The statistics sweeps can also write, next
 * to max_q and denom, the raw score maximum of every row over every 64-key block:
 * blockmax bf16 [batch,heads,Sp/64,Sp] with Sp = 128*ceil(seq/128), entry [J][r] = max over the
 * keys c of block J with c < kv_len of q[r].k[c], rounded toward +infinity to bf16 (never below the
 * fp32 maximum, at most a factor 1 + 2^-7 above it in magnitude; blocks without such a key are not
 * written): 2*Sp*Sp/64 bytes per head, e.g. 0.81 GB at (1,24,32768), 4.3 GB at (1,24,75856),
 * 7.2 GB at (1,40,75600).
 * The reference's threshold test  exp2((s[r,c] - max_q[r]) sf) / denom[r] > threshold
 * (include/mask_utils.cuh:231-238) holds for some key of block J exactly when it holds for the
 * block's maximum, so spattn_blockmax_to_blocklists derives the block mask
 *   MB[I,J] = OR_{r in q-block I, r < seq} ( blockmax[J][r] passes the test of row r )
 * and the ascending block lists from those bytes instead of the 2*Sp*Sp*D flops of
 * the sweep (include/mask_utils.cuh:131-243 + 273-302 for block-level masks); thresholds can be
 * changed without another sweep.  Because the stored maxima are rounded up, the lists hold every
 * block of the sweep's block mask and may hold a block whose best key misses the threshold by
 * less than one bf16 step of its raw score.  qblk = 64 or 128 rows per list; outputs as
 * spattn_packedmask_to_blocklists: blk_indices [batch,heads,ceil(seq/qblk),max_blocks] (entries
 * behind the count keep the caller's fill), blk_counts [batch,heads,ceil(seq/qblk)], optional
 * blockmask uint8 [batch,heads,ceil(seq/qblk),Sp/64].  max_q / denom are those of the same sweep
 * ([batch,heads,1,Sp]); scale and kv_len must be the ones the sweep was given.
 * The _blockmax sweeps replace maxq_denom_impl / attn_maxq_denom_impl
 * (python/extension.cpp:22-33) with the extra output. */
int spattn_maxq_denom_blockmax(float* max_q, float* denom, void* blockmax, const void* q, const void* k, int batch,
                               int heads, int seq, int D, int kv_len, float scale, void* stream);
int spattn_fullattn_maxq_denom_blockmax(void* o, float* max_q, float* denom, void* blockmax, const void* q, const void* k,
                                        const void* v, int batch, int heads, int seq, int D, int kv_len, float scale,
                                        void* stream);
int spattn_blockmax_to_blocklists(int* blk_indices, int* blk_counts, void* blockmask, const void* blockmax,
                                  const float* max_q, const float* denom, float threshold, int qblk, int batch, int heads,
                                  int seq, int D, int kv_len, float scale, int max_blocks, void* stream);

/* The threshold sweep restricted to listed key blocks.  blk_indices int32
 * [batch,heads,ceil(seq/128),max_blocks] holds, per 128-row q-block, ascending ids of 64-key
 * blocks, blk_counts [batch,heads,ceil(seq/128)] how many.  Only the keys of the listed blocks are
 * multiplied and tested; every other entry of the mask row is written as zero.  With lists that
 * hold every block in which some key passes the test - what spattn_blockmax_to_blocklists gives at
 * qblk = 128 for the same statistics, threshold, scale and kv_len - the result is the mask of
 * spattn_booleanmask_128 / spattn_booleanmask_packed (include/mask_utils.cuh:131-243), vote for
 * vote, at the cost of the kept blocks only (about 8 % of the sweep at the density the reference
 * runs at).  A block missing from a list loses its votes; an id outside the row is read as the row's
 * last pair of key blocks, whose votes are then written as the full sweep would write them (the
 * result stays within the full sweep's votes).
 * booleanmask / packed, mask_stride, qblk as in the full sweeps (qblk is the row granularity of
 * the bit output; the lists are per 128-row q-block in both cases). */
int spattn_booleanmask_128_blocks(int* booleanmask, float threshold, int mask_stride, const float* max_q,
                                  const float* denom, const void* q, const void* k, const int* blk_indices,
                                  const int* blk_counts, int max_blocks, int batch, int heads, int seq, int D, int kv_len,
                                  float scale, void* stream);
int spattn_booleanmask_packed_blocks(void* packed, float threshold, int mask_stride, int qblk, const float* max_q,
                                     const float* denom, const void* q, const void* k, const int* blk_indices,
                                     const int* blk_counts, int max_blocks, int batch, int heads, int seq, int D,
                                     int kv_len, float scale, void* stream);

/* Top-k mask generator (python/spattn/mask_utils.py:389-417, qk_topkmask_indices): per
 * q-block of `blocksz` rows the select_k keys c < kv_len (0 = seq) with the largest
 * (block mean of q / sqrt(D)) . k[c], every step rounded to bf16 as the reference's bf16 torch
 * ops do.  Outputs: qmean bf16 [batch,heads,SB,D]; score bf16 [batch,heads,SB,score_stride]
 * (columns >= kv_len hold unspecified values; score_stride a multiple of 8); kv_indices
 * [batch,heads,SB,idx_stride] receives min(select_k, kv_len) keys per row in ASCENDING key
 * order (the reference orders them by descending score; sp_attn does not depend on the
 * order), entries behind them keep the caller's fill; num_kv_indices the count.  Among equal
 * scores the lower key wins.  SB = ceil(seq / blocksz), blocksz 64 or 128. */
int spattn_qk_topkmask_indices(int* kv_indices, int* num_kv_indices, void* score, void* qmean, const void* q,
                               const void* k, int batch, int heads, int seq, int D, int blocksz, int kv_len,
                               int select_k, int score_stride, int idx_stride, void* stream);

/* Work order for lists of very uneven length.  No counterpart in the reference, whose grid is
 * fixed to (q-block, head, batch) (include/sparseattn_asyncgatherload_padded.cuh:273).
 * spattn_qblock_order writes into order[0..n) a permutation of 0..n-1 (n = batch*heads*SB, the
 * flat q-block index of the count tensor): longest lists first, in quarter-octave classes of the
 * count, stable inside a class; if the longest list is less than twice the shortest, the default order.  The
 * _ordered forms of the two list-driven attention entry points let workgroup i take q-block
 * order[i]; results are bit-identical to the plain forms, only the schedule changes.
 * order must be a permutation of 0..n-1: an entry outside that range is skipped by the kernel
 * (nothing is read or written for it), a q-block that no entry names keeps whatever o held, and
 * a q-block named twice is computed twice. */
int spattn_qblock_order(int* order, const int* counts, int n, void* stream);
int spattn_sp_attn_ordered(void* o, float* lse, const void* q, const void* k, const void* v, const int* kv_indices,
                           const int* num_kv_indices, const int* order, int mask_stride, int qblk, int batch, int heads,
                           int seq, int D, int kv_len, float scale, void* stream);
int spattn_sp_attn_blocks_ordered(void* o, float* lse, const void* q, const void* k, const void* v,
                                  const int* blk_indices, const int* blk_counts, const int* order, int max_blocks,
                                  int qblk, int batch, int heads, int seq, int D, int kv_len, float scale, void* stream);

/* Block-list attention in balanced (longest list first) order for callers that cannot
 * allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference.  It is spattn_qblock_order followed by
 * spattn_sp_attn_blocks_ordered, bit for bit, with the work order kept in a device array that
 * belongs to the library (4 MiB per device, held until the process ends) instead of a buffer
 * the caller provides; it calls no allocating routine.  At most SPATTN_BALANCED_MAX_QBLOCKS
 * q-blocks, else SPATTN_ERR_SCRATCH and nothing is launched.  All calls on one device share
 * that array: calls that overlap on one device (two streams, two threads) race on it - run
 * them one after the other, or use the _ordered form with a buffer per stream.
 * spattn_init looks the array's address up for the current device and raises the dynamic-LDS limit
 * of every attention kernel there - the two things a first call on a device otherwise does; it is
 * optional, except that after it every entry point only launches kernels, which is what a caller
 * needs who records his first calls on a device into a HIP graph.  A first call on a device made
 * while its stream is being captured, without spattn_init before it, returns SPATTN_ERR_SCRATCH
 * and records nothing (the address lookup is not a call to make inside a capture); a graph that
 * holds this entry point replays on one stream at a time like the eager calls. */
int spattn_init(void);
int spattn_sp_attn_blocks_balanced(void* o, float* lse, const void* q, const void* k, const void* v,
                                   const int* blk_indices, const int* blk_counts, int max_blocks, int qblk, int batch,
                                   int heads, int seq, int D, int kv_len, float scale, void* stream);

/* Status of the most recent call on this host thread, and its text. */
int spattn_last_status(void);
const char* spattn_status_string(int status);
int spattn_version(void);

#ifdef __cplusplus
}
#endif
#endif /* SPATTN_HIP_H_ */
