// Whole PBS prefill attention in one call: every stage enqueued on one stream out of one caller-provided
// workspace (no allocation, no synchronisation, one host round trip instead of ten).
#include "pbs_common.h"

#include "../../include/pbs_hip.h"   // the stage entry points, type-checked against the public ABI

namespace {

__global__ void identity_indices_kernel(int32_t* idx, int S_pad, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < total) idx[i] = (int32_t)(i % S_pad);
}

struct Layout {
  size_t scores, score_ws, idx, perm_k, perm_vt, pooled_k, pooled_q, probs, cols, cnt, needed, select_ws, attn_ws, total;
};

size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

Layout make_layout(int B, int Hq, int Hkv, int S, int D, int block_size, int segment_size) {
  Layout L;
  const size_t rows = (size_t)B * Hq;
  const size_t nb = (size_t)(S + block_size - 1) / block_size, s_pad = nb * block_size;
  const size_t sc = (size_t)(S / segment_size) * segment_size;
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t o = off; off = align256(off + bytes); return o; };
  L.scores = take(rows * sc * 4);
  L.score_ws = take(pbs_score_keys_workspace_bytes(B, Hq, Hkv, S, segment_size));
  L.idx = take(rows * s_pad * 4);
  L.perm_k = take(rows * s_pad * D * 2);
  L.perm_vt = take(rows * s_pad * D * 2);
  L.pooled_k = take(rows * nb * D * 2);
  L.pooled_q = take(rows * nb * D * 2);
  L.probs = take(rows * nb * nb * 4);
  L.cols = take(rows * nb * nb * 4);
  L.cnt = take(rows * nb * 4);
  L.needed = take(rows * nb);
  L.select_ws = take(pbs_select_blocks_workspace_bytes((int)rows));
  L.attn_ws = take(pbs_sparse_attn_workspace_bytes(B, Hq, S, segment_size));
  L.total = off;
  return L;
}

// A sequence that fits inside one segment is plain causal attention (pbs_attn/src/pbs.py:175-182): identity key
// order, every causal block visited.  With that order and every candidate selected the result does not depend on the
// segment size, so the kernels run with one segment spanning the sequence or, beyond the attention kernel's 511
// blocks per segment, with segments of 256 blocks.  Returns the segment size to run with.
int one_segment_size(int S, int block_size) {
  const int nb = (S + block_size - 1) / block_size;
  return (nb <= 511 ? nb : 256) * block_size;
}

}  // namespace

extern "C" int pbs_identity_indices(int32_t* key_indices, int rows, int S_pad, void* stream) {
  PBS_REQUIRE(key_indices && rows > 0 && S_pad > 0, "pbs_identity_indices: bad arguments");
  const int64_t total = (int64_t)rows * S_pad;
  hipLaunchKernelGGL(identity_indices_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     key_indices, S_pad, total);
  return pbs_check_launch("pbs_identity_indices");
}

extern "C" size_t pbs_prefill_attn_workspace_bytes(int B, int Hq, int Hkv, int S, int head_dim, int block_size, int segment_size) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || S <= 0 || head_dim <= 0 || block_size <= 0 || segment_size <= 0) return 0;
  if (S <= segment_size) segment_size = one_segment_size(S, block_size);   // as pbs_prefill_attn_fwd
  return make_layout(B, Hq, Hkv, S, head_dim, block_size, segment_size).total;
}

extern "C" int pbs_prefill_attn_fwd(const void* q, const void* k, const void* v, void* out, int B, int Hq, int Hkv, int S,
                                    int head_dim, int block_size, int segment_size, int64_t q_sb, int64_t q_sh,
                                    int64_t q_ss, int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh,
                                    int64_t v_ss, int64_t o_sb, int64_t o_sh, int64_t o_ss, float threshold,
                                    const float* threshold_per_row, int threshold_is_int_one,
                                    int force_select_first_block, int query_pool_max, int key_pool_max,
                                    float softmax_scale, void* workspace, size_t workspace_bytes, void* stream) {
  PBS_REQUIRE(q && k && v && out, "pbs_prefill_attn_fwd: null tensor pointer");
  PBS_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && S > 0, "pbs_prefill_attn_fwd: bad shape");
  PBS_REQUIRE(block_size > 0 && segment_size > 0 && segment_size % block_size == 0,
              "pbs_prefill_attn_fwd: segment_size must be a multiple of block_size");
  // sequences that fit one segment: plain causal attention = one segment spanning the sequence,
  // identity order, every causal block visited
  const bool one_segment = S <= segment_size;
  if (one_segment) {
    segment_size = one_segment_size(S, block_size);
    threshold_is_int_one = 1;
  }
  // checked here, before anything is enqueued (the attention kernel holds one segment's blocks in its list)
  PBS_REQUIRE(segment_size / block_size <= 511,
              "pbs_prefill_attn_fwd: a segment of %d blocks exceeds the limit of 511 (use a smaller segment_size)",
              segment_size / block_size);
  const Layout L = make_layout(B, Hq, Hkv, S, head_dim, block_size, segment_size);
  PBS_REQUIRE(workspace && workspace_bytes >= L.total, "pbs_prefill_attn_fwd: workspace too small (%zu < %zu bytes)",
              workspace_bytes, L.total);
  PBS_REQUIRE(((uintptr_t)workspace % 256) == 0, "pbs_prefill_attn_fwd: workspace must be 256-byte aligned");
  uint8_t* w = (uint8_t*)workspace;
  const int rows = B * Hq, nb = (S + block_size - 1) / block_size, s_pad = nb * block_size;
  const int nseg = S / segment_size, rem = S % segment_size;
  int rc;
  if (one_segment || nseg == 0 || (nseg == 1 && rem == 0)) {
    if ((rc = pbs_identity_indices((int32_t*)(w + L.idx), rows, s_pad, stream))) return rc;
  } else {
    if ((rc = pbs_score_keys(q, k, (float*)(w + L.scores), B, Hq, Hkv, S, head_dim, block_size, segment_size, q_sb, q_sh,
                             q_ss, k_sb, k_sh, k_ss, w + L.score_ws, L.idx - L.score_ws, stream))) return rc;
    if ((rc = pbs_segment_argsort((const float*)(w + L.scores), (int32_t*)(w + L.idx), rows, S, s_pad, segment_size, stream))) return rc;
  }
  // With a real threshold the permuted K / V are gathered AFTER the selection, and only the blocks some query
  // block visits: the estimate needs no more than the pooled permuted key blocks, which come straight from K.
  // (Every candidate selected: everything is visited, one full gather.)
  uint8_t* needed = threshold_is_int_one ? nullptr : w + L.needed;
  if (threshold_is_int_one) {
    if ((rc = pbs_gather_kv(k, v, (const int32_t*)(w + L.idx), w + L.perm_k, w + L.perm_vt, nullptr, B, Hq, Hkv,
                            S, head_dim, block_size, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, key_pool_max, nullptr, stream))) return rc;
  } else {
    if ((rc = pbs_pool_blocks(q, k, (const int32_t*)(w + L.idx), w + L.pooled_q, w + L.pooled_k, needed, B, Hq, Hkv, S,
                              head_dim, block_size, q_sb, q_sh, q_ss, k_sb, k_sh, k_ss, query_pool_max, key_pool_max,
                              stream))) return rc;
    // (up to 1024 blocks the selection reads a row's candidate entries only: the others are not written)
    if (nb <= 1024) {
      if ((rc = pbs_block_logits_softmax_candidates_only(w + L.pooled_q, w + L.pooled_k, (float*)(w + L.probs), rows, nb,
                                                         head_dim, segment_size / block_size, stream))) return rc;
    } else {
      if ((rc = pbs_block_logits_softmax(w + L.pooled_q, w + L.pooled_k, (float*)(w + L.probs), rows, nb, head_dim,
                                         segment_size / block_size, stream))) return rc;
    }
  }
  if ((rc = pbs_select_blocks((const float*)(w + L.probs), threshold_per_row, threshold, threshold_is_int_one,
                              force_select_first_block, /*candidate_rule=*/1, (const int32_t*)(w + L.idx), rows, S, block_size,
                              segment_size,
                              nullptr, nullptr, (int32_t*)(w + L.cols), (int32_t*)(w + L.cnt), needed, w + L.select_ws,
                              L.attn_ws - L.select_ws, stream))) return rc;
  if (!threshold_is_int_one) {
    if ((rc = pbs_gather_kv(k, v, (const int32_t*)(w + L.idx), w + L.perm_k, w + L.perm_vt, nullptr, B, Hq, Hkv,
                            S, head_dim, block_size, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, key_pool_max, needed, stream))) return rc;
  }
  return pbs_sparse_attn_fwd(q, w + L.perm_k, w + L.perm_vt, k, v, (const int32_t*)(w + L.cols),
                             (const int32_t*)(w + L.cnt), out, B, Hq, Hkv, S, head_dim, block_size, segment_size, q_sb,
                             q_sh, q_ss, k_sb, k_sh, k_ss, v_sb, v_sh, v_ss, o_sb, o_sh, o_ss, softmax_scale, w + L.attn_ws,
                             stream);
}
