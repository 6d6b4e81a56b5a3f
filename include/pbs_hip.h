/* C ABI of libpbs_hip.so -- the gfx950 (MI355X) kernels behind PBS-Attn's
 * permuted block-sparse prefill attention.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless named otherwise; tensors are bf16
 *     (uint16 storage) with head_dim 128 and block_size 128;
 *   - strides are in ELEMENTS (batch, head, sequence); the innermost dimension has
 *     stride 1 and every row must start 16-byte aligned;
 *   - K/V may be given at Hkv heads (query head h reads KV head h / (Hq / Hkv)) or
 *     already repeated to Hq heads (pass Hkv = Hq);
 *   - `stream` is a hipStream_t; all work is enqueued on it, nothing synchronises,
 *     nothing allocates; scratch memory comes in through `workspace`;
 *   - return 0 on success, a negative value for an argument error, a positive
 *     hipError_t for a launch error; pbs_last_error() gives the message (thread local).
 *
 * File:line citations name the reference code (xinghaow99/pbs-attn) each entry
 * point replaces.
 */
#ifndef PBS_HIP_H
#define PBS_HIP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

int pbs_abi_version(void);
const char* pbs_last_error(void);

/* Key scoring: scores[b,h,k] = mean over the last 128 queries of
 * softmax_k(bf16(bf16(q.k) / sqrt(D))) over the keys of the complete segments.
 * scores: (B, Hq, Sc) float32, Sc = (S / segment_size) * segment_size.  Strides in elements, rows 16-byte
 * aligned, key row stride in [128, 2^28).
 * Replaces pbs_attn/src/permute_states.py:44-50. */
size_t pbs_score_keys_workspace_bytes(int B, int Hq, int Hkv, int S, int segment_size);
int pbs_score_keys(const void* q, const void* k, float* scores, int B, int Hq, int Hkv, int S, int head_dim,
                   int block_size, int segment_size, int64_t q_sb, int64_t q_sh, int64_t q_ss, int64_t k_sb,
                   int64_t k_sh, int64_t k_ss, void* workspace, size_t workspace_bytes, void* stream);

/* pbs_score_keys without a workspace argument and without any allocation.  It has no counterpart in
 * the reference: it is for callers that cannot allocate device memory around the call (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  The chunk partials and row
 * statistics live in a library-owned device array of PBS_SCORE_KEYS_STATIC_SCRATCH_BYTES per GPU (held
 * until the process ends); shapes whose pbs_score_keys_workspace_bytes exceeds it are rejected with an
 * argument error (-1).  The device address of the array is looked up on the first call on each device
 * (-2 if that fails): make that first call outside any stream capture.  All calls on one GPU share the array: calls that overlap on one GPU (two streams,
 * two threads) race; calls on one stream are ordered and safe.  Same arguments, results and error
 * behaviour as pbs_score_keys otherwise. */
#define PBS_SCORE_KEYS_STATIC_SCRATCH_BYTES ((size_t)8 << 20)
int pbs_score_keys_static(const void* q, const void* k, float* scores, int B, int Hq, int Hkv, int S, int head_dim,
                          int block_size, int segment_size, int64_t q_sb, int64_t q_sh, int64_t q_ss, int64_t k_sb,
                          int64_t k_sh, int64_t k_ss, void* stream);

/* Per-segment stable descending argsort (ties keep ascending index).
 * scores: (rows, Sc); key_indices: (rows, S_pad) int32 global key positions;
 * positions >= Sc (trailing partial segment, block padding) keep identity order.
 * Replaces pbs_attn/src/permute_states.py:52-56,71-81 and the index padding of
 * pbs_attn/src/pbs.py:80-84. */
int pbs_segment_argsort(const float* scores, int32_t* key_indices, int rows, int S, int S_pad, int segment_size,
                        void* stream);

/* Gather K and V into permuted order and pool the permuted key blocks.
 * perm_k: (B, Hq, nb*128, 128) rows past S zero; perm_vt: (B, Hq, nb, 128, 128)
 * holding each V block transposed [d][key]; pooled_k: (B, Hq, nb, 128) bf16, may be null (no pooling).  block_needed (may be null): (B*Hq, nb) bytes as written by
 * pbs_select_blocks; permuted blocks whose byte is zero are skipped and their perm_k / perm_vt
 * tiles left unwritten (the attention kernel reads only the blocks on some visit list).
 * Replaces pbs_attn/src/permute_states.py:59-69, pbs_attn/src/pbs.py:213-215,
 * the key padding of pbs.py:78-79 and the key pooling of pbs_attn/src/utils.py:24-29. */
int pbs_gather_kv(const void* k, const void* v, const int32_t* key_indices, void* perm_k, void* perm_vt,
                  void* pooled_k, int B, int Hq, int Hkv, int S, int head_dim, int block_size, int64_t k_sb,
                  int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss, int key_pool_max,
                  const uint8_t* block_needed, void* stream);

/* pooled_k of pbs_gather_kv (the same bits) without gathering anything: the permuted key blocks are
 * pooled straight from k through key_indices.  block_needed (may be null): (B*Hq, nb) bytes, cleared
 * here, for pbs_select_blocks to set.  With this the permutation of pbs_attn/src/pbs.py:185-190 can be
 * deferred until the selection (pbs.py:195-209) has said which permuted blocks are read at all. */
int pbs_pool_k_permuted(const void* k, const int32_t* key_indices, void* pooled_k, uint8_t* block_needed, int B,
                        int Hq, int Hkv, int S, int head_dim, int block_size, int64_t k_sb, int64_t k_sh,
                        int64_t k_ss, int key_pool_max, void* stream);

/* pbs_pool_q and pbs_pool_k_permuted in one launch (the same bits as the two calls): the two kinds of
 * workgroup alternate in launch order, so the key pooling's scattered row reads and the query pooling's
 * streaming reads run side by side. */
int pbs_pool_blocks(const void* q, const void* k, const int32_t* key_indices, void* pooled_q, void* pooled_k,
                    uint8_t* block_needed, int B, int Hq, int Hkv, int S, int head_dim, int block_size,
                    int64_t q_sb, int64_t q_sh, int64_t q_ss, int64_t k_sb, int64_t k_sh, int64_t k_ss,
                    int query_pool_max, int key_pool_max, void* stream);

/* Query-block pooling (mean with divisor 128, or max; rows past S count as zero).
 * pooled_q: (B, Hq, nb, 128) bf16.  Replaces pbs_attn/src/pbs.py:67-71 and
 * pbs_attn/src/utils.py:18-23. */
int pbs_pool_q(const void* q, void* pooled_q, int B, int Hq, int S, int head_dim, int block_size, int64_t q_sb,
               int64_t q_sh, int64_t q_ss, int query_pool_max, void* stream);

/* Block logits + masked fp32 softmax.  block_attn_scores: (rows, nb, nb) float32;
 * candidates of query block qb are the key blocks of strictly earlier segments;
 * rows without candidates are NaN.  Replaces pbs_attn/src/pbs.py:97-107 and
 * pbs_attn/src/utils.py:30-33. */
int pbs_block_logits_softmax(const void* pooled_q, const void* pooled_k, float* block_attn_scores, int rows, int nb,
                             int head_dim, int blocks_per_segment, void* stream);

/* pbs_block_logits_softmax for a consumer that reads a row's candidate entries only (pbs_select_blocks with
 * candidate_rule 1 on at most 1024 blocks): the zeros outside the candidates and the NaN rows are not written, which
 * halves the kernel's stores.  The candidate entries are the bits pbs_block_logits_softmax writes.  Replaces the
 * same lines, pbs_attn/src/pbs.py:97-107 and pbs_attn/src/utils.py:30-33. */
int pbs_block_logits_softmax_candidates_only(const void* pooled_q, const void* pooled_k, float* block_attn_scores, int rows,
                                             int nb, int head_dim, int blocks_per_segment, void* stream);

/* The same with the candidate rule of the reference's un-permuted MeanPooling baseline: query block qb
 * scores every key block kb <= qb (the causal lower triangle INCLUDING the diagonal), so no row is NaN.
 * Replaces pbs_attn/baselines/MeanPooling.py:43-48 (mask) + pbs_attn/src/utils.py:30-33. */
int pbs_block_logits_softmax_causal(const void* pooled_q, const void* pooled_k, float* block_attn_scores, int rows,
                                    int nb, int head_dim, void* stream);

/* Cumulative-threshold selection.  threshold_per_row (rows floats) overrides
 * `threshold` when non-null; threshold_is_int_one selects every candidate.
 * sel_mask = selected | first-token block; final_mask = sel_mask | own segment
 * (both (rows, nb, nb) bytes, either may be null); csr_cols (rows, nb, nb) /
 * csr_cnt (rows, nb): the ascending key blocks of sel_mask that lie in segments
 * strictly before the query block's -- the permuted tiles the attention kernel
 * visits (it adds the causal part of the query block's own segment itself).
 * candidate_rule says which entries of a row of block_attn_scores can be non-zero, so that only those are
 * sorted: 0 = any (the whole row is sorted, as the reference does), 1 = key blocks of segments strictly
 * before the query block's (rows written by pbs_block_logits_softmax), 2 = key blocks up to and including
 * the query block (pbs_block_logits_softmax_causal).  Entries outside the rule must be exactly zero; the
 * result is then the same as with rule 0.
 * block_needed (may be null): (rows, nb) bytes, cleared by the caller (pbs_pool_k_permuted does);
 * the byte of every key block that appears on some query block's visit list is set to 1.
 * Replaces pbs_attn/src/utils.py:38-86 and pbs_attn/src/pbs.py:10-25,119-127,209. */
size_t pbs_select_blocks_workspace_bytes(int rows);
int pbs_select_blocks(const float* block_attn_scores, const float* threshold_per_row, float threshold,
                      int threshold_is_int_one, int force_select_first_block, int candidate_rule,
                      const int32_t* key_indices, int rows, int S, int block_size, int segment_size, uint8_t* sel_mask, uint8_t* final_mask,
                      int32_t* csr_cols, int32_t* csr_cnt, uint8_t* block_needed, void* workspace,
                      size_t workspace_bytes, void* stream);

/* Visit lists from a block mask somebody else made: csr_cols / csr_cnt as pbs_select_blocks writes them (the set
 * key blocks of strictly earlier segments of every query block, ascending) from block_mask ((rows, nb, nb) bytes,
 * non-zero = attend; entries of later segments are ignored: none of their keys is visible).  *own_missing (one int32
 * the caller zeroes) receives the number of blocks of a query block's own segment the mask leaves out:
 * pbs_sparse_attn_fwd always attends to the visible keys of the whole own segment, so a mask with own_missing != 0
 * is not one it can serve.  For callers of the reference's attention stage that bring
 * their own mask (pbs_attn/src/kernels/permuted_block_sparse_attention.py:134-157,314-323: block_mask argument). */
int pbs_block_mask_to_csr(const uint8_t* block_mask, int32_t* csr_cols, int32_t* csr_cnt, int32_t* own_missing, int rows,
                          int nb, int blocks_per_segment, void* stream);

/* Block-sparse flash-attention forward.  Query block qb attends to the permuted K /
 * transposed V tiles listed in csr_cols (earlier segments, no element mask) and to
 * its own segment: blocks first-of-segment .. qb of the ORIGINAL k and v (B, Hkv, S, 128,
 * caller's strides, read in place), with the causal triangle on block qb.  The keys a
 * query sees are exactly those of the reference's final mask and element mask
 * (a segment's permuted blocks hold the same keys as its original blocks).
 * out: (B, Hq, S, 128) bf16 with its own strides, original query order.
 * workspace: pbs_sparse_attn_workspace_bytes(B, Hq, S, segment_size) bytes of device memory, 256-byte
 * aligned (work counters and the merged visit list of every pair of query blocks, rewritten by each call).
 * Two launches: the list merge, then one persistent workgroup per CU.
 * Replaces pbs_attn/src/kernels/permuted_block_sparse_attention.py:134-311
 * (launch at pbs_attn/src/pbs.py:220-246). */
size_t pbs_sparse_attn_workspace_bytes(int B, int Hq, int S, int segment_size);
int pbs_sparse_attn_fwd(const void* q, const void* perm_k, const void* perm_vt, const void* k, const void* v,
                        const int32_t* csr_cols, const int32_t* csr_cnt, void* out, int B, int Hq, int Hkv, int S,
                        int head_dim, int block_size, int segment_size, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                        int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss,
                        int64_t o_sb, int64_t o_sh, int64_t o_ss, float softmax_scale, void* workspace, void* stream);

/* pbs_sparse_attn_fwd for one-block segments (segment_size = block_size: the un-permuted MeanPooling mode) with an
 * OPTIONAL diagonal block: query block qb of head row r attends to its own block (with the causal triangle) only
 * where own_block_needed[r * nb + qb] != 0 ((B*Hq, nb) bytes), and to the blocks of csr_cols as before.  A query
 * block left without any block gets zeros, like a row without selected blocks in
 * pbs_attn/src/kernels/permuted_block_sparse_attention.py:340-343.  Workspace: pbs_sparse_attn_workspace_bytes(B, Hq, S,
 * block_size).  Replaces the attention call of pbs_attn/baselines/MeanPooling.py:80-96 when
 * force_select_current_block (:54-58) is off. */
int pbs_sparse_attn_fwd_optional_diagonal(const void* q, const void* perm_k, const void* perm_vt, const void* k,
                                          const void* v, const int32_t* csr_cols, const int32_t* csr_cnt,
                                          const uint8_t* own_block_needed, void* out, int B, int Hq, int Hkv, int S,
                                          int head_dim, int block_size, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                                          int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh,
                                          int64_t v_ss, int64_t o_sb, int64_t o_sh, int64_t o_ss, float softmax_scale,
                                          void* workspace, void* stream);

/* out[b,h,q_idx[b,h,i],:] = o_perm[b,h,i,:] (o_perm contiguous).  q_idx null with
 * o_perm == out is the identity fast path (no launch): the reference does not
 * permute queries (pbs_attn/src/pbs.py:191-193), so this is what it takes. */
int pbs_unpermute(const void* o_perm, const int32_t* q_idx, void* out, int B, int H, int S, int head_dim,
                  int64_t o_sb, int64_t o_sh, int64_t o_ss, void* stream);

/* key_indices[r, i] = i for every row: the order of a sequence that is not permuted
 * (pbs_attn/src/permute_states.py:36-38). */
int pbs_identity_indices(int32_t* key_indices, int rows, int S_pad, void* stream);

/* The whole path in one call: key scoring, segment sort, gather, estimation, selection and sparse
 * attention enqueued back to back on `stream`, intermediates in `workspace` (256-byte aligned,
 * pbs_prefill_attn_workspace_bytes).  S <= segment_size gives plain causal attention, as the
 * reference does.  Replaces pbs_attn/src/pbs.py:132-257 as a whole. */
size_t pbs_prefill_attn_workspace_bytes(int B, int Hq, int Hkv, int S, int head_dim, int block_size,
                                        int segment_size);
int pbs_prefill_attn_fwd(const void* q, const void* k, const void* v, void* out, int B, int Hq, int Hkv, int S,
                         int head_dim, int block_size, int segment_size, int64_t q_sb, int64_t q_sh, int64_t q_ss,
                         int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss,
                         int64_t o_sb, int64_t o_sh, int64_t o_ss, float threshold, const float* threshold_per_row,
                         int threshold_is_int_one, int force_select_first_block, int query_pool_max,
                         int key_pool_max, float softmax_scale, void* workspace, size_t workspace_bytes,
                         void* stream);

/* Rotary position embedding of Q and K in one pass: out = bf16(bf16(x * cos) + bf16(rotate_half(x) * sin)),
 * bit-identical to the bf16 tensor expression of pbs_attn/patch/huggingface.py:14-25 (called at :203).
 * q (B, Hq, S, 128) and k (B, Hkv, S, 128) with their strides (e.g. the (B, S, H, D) memory of the
 * projections); cos / sin (B or 1, S, 128) with batch stride c_sb (0 to broadcast) and row stride c_ss;
 * q_out (B, Hq, S, 128) and k_out (B, Hkv, S, 128) contiguous, head-major. */
int pbs_rope_qk(const void* q, const void* k, const void* cos, const void* sin, void* q_out, void* k_out, int B, int Hq,
                int Hkv, int S, int head_dim, int64_t q_sb, int64_t q_sh, int64_t q_ss, int64_t k_sb, int64_t k_sh,
                int64_t k_ss, int64_t c_sb, int64_t c_ss, void* stream);

#ifdef __cplusplus
}
#endif
#endif
