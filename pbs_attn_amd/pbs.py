"""PBS-Attn prefill attention on MI355X: host orchestration of the HIP stages.

``permuted_block_sparse_attn_fwd`` mirrors the reference's operator (pbs_attn/src/pbs.py:132-257): same
name, arguments, defaults and assertions.  ``apply_permutation`` and ``permuted_block_selection`` here are
this build's own staged API (device-side ``PermutedKV`` bundle, CSR visit list); the functions with the
reference's signatures and return values are in ``pbs_attn_amd.compat`` and are what
``pbs_attn.src.pbs`` / ``pbs_attn.src.permute_states`` / ``pbs_attn.src.utils`` export.  Every stage runs
in hand-written gfx950 kernels reached through the C ABI of libpbs_hip.so; nothing here computes on
the CPU and nothing falls back to another implementation.

Differences a caller can see:
  * K/V may arrive at the KV-head count (the reference wants them repeated to the
    query-head count; that still works);
  * both sorts are stable (ties keep ascending index order), the order torch's
    GPU sort produces and the reference leaves unspecified;
  * ``use_triton`` is accepted for signature compatibility; there is a single
    implementation (HIP) whatever its value.
"""
from __future__ import annotations

import math
import warnings
from dataclasses import dataclass
from typing import Optional, Union

import torch

from . import ops

_warned_use_triton = False

# Optional profiling hook: an object with ``mark(stage_name)``, called after each
# stage has been enqueued (the benchmark records a HIP event there).
stage_timer = None


def _mark(name):
    if stage_timer is not None:
        stage_timer.mark(name)


@dataclass
class PermutedKV:
    """Device-side product of the permutation phase."""
    key_indices: torch.Tensor   # (B, Hq, S_pad) int32, positions >= S are their own index
    perm_k: torch.Tensor        # (B, Hq, S_pad, D) rows >= S zero
    perm_vt: torch.Tensor       # (B, Hq, nb, D, 128): V blocks transposed [d][key]
    pooled_k: torch.Tensor      # (B, Hq, nb, D)
    seq_len: int
    key_states: torch.Tensor = None     # the caller's K and V (B, Hkv or Hq, S, D), read in place for own-segment tiles
    value_states: torch.Tensor = None

    def attention(self, query_states, csr_cols, csr_cnt, segment_size, softmax_scale=None, out=None):
        """Sparse attention over this permutation (see ops.sparse_attn_fwd)."""
        return ops.sparse_attn_fwd(query_states, self.perm_k, self.perm_vt, self.key_states, self.value_states,
                                   csr_cols, csr_cnt, segment_size, softmax_scale, out)

    def permuted_keys(self):
        return self.perm_k[:, :, :self.seq_len]

    def permuted_values(self):
        """(B, Hq, S, D) view-free copy in the reference's layout (for inspection)."""
        b, h, nb, d, bs = self.perm_vt.shape
        return self.perm_vt.transpose(-1, -2).reshape(b, h, nb * bs, d)[:, :, :self.seq_len]


def _identity_indices(B, H, s_pad, device):
    return torch.arange(s_pad, dtype=torch.int32, device=device).view(1, 1, -1).expand(B, H, -1).contiguous()


def apply_permutation(query_states, key_states, value_states, block_size, segment_size, key_pool_mode="mean",
                      scores: Optional[torch.Tensor] = None, identity: bool = False) -> PermutedKV:
    """Permutation phase (pbs.py:185-190 + :213-215): score keys with the last query
    block, sort inside each segment, gather K and V.  ``scores`` can be injected
    to run the sort on a given score tensor; ``identity`` keeps the keys in their order."""
    B, Hq, S, D = query_states.shape
    nseg, rem = S // segment_size, S % segment_size
    s_pad = (S + block_size - 1) // block_size * block_size
    if identity or nseg == 0 or (nseg == 1 and rem == 0):               # permute_states.py:36-38
        idx = _identity_indices(B, Hq, s_pad, query_states.device)
    else:
        if scores is None:
            scores = ops.score_keys(query_states, key_states, block_size, segment_size)
            _mark("score")
        idx = ops.segment_argsort(scores, S, segment_size, block_size)
        _mark("sort")
    perm_k, perm_vt, pooled_k = ops.gather_kv(key_states, value_states, idx, Hq, key_pool_mode)
    _mark("gather")
    return PermutedKV(idx, perm_k, perm_vt, pooled_k, S, key_states, value_states)


def permuted_block_selection(query_states, perm: PermutedKV, block_size, segment_size, threshold=0.9, causal=True,
                             force_select_first_block=True, query_pool_mode="mean", key_pool_mode="mean",
                             want_masks=True, block_attn_scores: Optional[torch.Tensor] = None):
    """Selection phase (pbs.py:29-130 + :209).  Returns a dict with
    block_attn_scores, block_mask (selected | first token), final_mask
    (| own segment), csr_cols / csr_cnt (the selected blocks of strictly earlier
    segments, ascending: the permuted tiles the attention kernel visits)."""
    assert causal
    assert segment_size % block_size == 0, "segment_size must be a multiple of block_size"
    if query_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid query_pool_mode: {query_pool_mode}")
    if key_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid key_pool_mode: {key_pool_mode}")
    S = query_states.shape[2]
    is_int_one = isinstance(threshold, int) and threshold == 1   # pbs.py:120 (True counts, as there)
    P = block_attn_scores
    rule = 0   # scores handed in: any values, the whole row is sorted
    if P is None and (not is_int_one or want_masks):
        pooled_q = ops.pool_q(query_states, query_pool_mode)
        P = ops.block_logits_softmax(pooled_q, perm.pooled_k, segment_size // block_size)
        rule = 1   # zero outside the blocks of earlier segments
        _mark("estimate")
    sel, fin, cols, cnt = ops.select_blocks(P, threshold, perm.key_indices, S, block_size, segment_size,
                                            force_select_first_block, want_masks=want_masks, candidate_rule=rule)
    _mark("select")
    return dict(block_attn_scores=P, block_mask=sel, final_mask=fin, csr_cols=cols, csr_cnt=cnt)


def _select_then_gather(query_states, key_states, value_states, block_size, segment_size, threshold,
                        force_select_first_block, query_pool_mode, key_pool_mode, candidates_only=False):
    B, Hq, S, _ = query_states.shape
    s_pad = (S + block_size - 1) // block_size * block_size
    nseg, rem = S // segment_size, S % segment_size
    if nseg == 0 or (nseg == 1 and rem == 0):
        idx = _identity_indices(B, Hq, s_pad, query_states.device)
    else:
        scores = ops.score_keys(query_states, key_states, block_size, segment_size)
        _mark("score")
        idx = ops.segment_argsort(scores, S, segment_size, block_size)
        _mark("sort")
    pooled_q, pooled_k, needed = ops.pool_blocks(query_states, key_states, idx, query_pool_mode, key_pool_mode)
    _mark("pool")
    # candidates_only (the single-call path's form, up to 1024 blocks): the selection reads a row's candidate entries only
    P = ops.block_logits_softmax(pooled_q, pooled_k, segment_size // block_size,
                                 candidates_only=candidates_only and s_pad // block_size <= 1024)
    _mark("estimate")
    _, _, cols, cnt = ops.select_blocks(P, threshold, idx, S, block_size, segment_size, force_select_first_block,
                                        want_masks=False, block_needed=needed, candidate_rule=1)
    _mark("select")
    perm_k, perm_vt, _ = ops.gather_kv(key_states, value_states, idx, Hq, key_pool_mode,
                                                block_needed=needed, want_pooled=False)
    _mark("gather")
    perm = PermutedKV(idx, perm_k, perm_vt, pooled_k, S, key_states, value_states)
    return perm, dict(block_attn_scores=P, csr_cols=cols, csr_cnt=cnt, block_needed=needed)


def permuted_block_sparse_attn_fwd(
    query_states: torch.Tensor,
    key_states: torch.Tensor,
    value_states: torch.Tensor,
    block_size: int,
    segment_size: int,
    threshold: Union[float, int, torch.Tensor],
    causal: bool,
    force_select_first_block: bool = True,
    use_triton: bool = True,
    query_pool_mode: str = "mean",
    key_pool_mode: str = "mean",
):
    """Permuted block-sparse attention forward (pbs.py:132-257).

    query_states (B, Hq, S, D); key/value_states (B, Hkv or Hq, S, D); bf16 on the
    GPU.  Returns (B, Hq, S, D) in original query order."""
    global _warned_use_triton
    batch_size, num_q_heads, q_len, head_dim = query_states.shape
    _, num_kv_heads, kv_len, _ = key_states.shape
    assert num_q_heads % num_kv_heads == 0
    assert causal
    assert q_len == kv_len
    assert segment_size % block_size == 0, "segment_size must be a multiple of block_size"
    if not use_triton and not _warned_use_triton:
        warnings.warn("use_triton=False: this build has a single implementation (HIP kernels); the flag is ignored")
        _warned_use_triton = True

    if stage_timer is None:
        # the whole path in one library call; the staged path below does the same work stage by
        # stage so that a profiler hook can stamp each one
        return ops.prefill_attn_fwd(query_states, key_states, value_states, block_size, segment_size, threshold,
                                    force_select_first_block, query_pool_mode, key_pool_mode)

    one_segment = q_len <= segment_size
    if one_segment:
        # pbs.py:175-182: plain causal attention.  Same kernel, identity order, every causal block visited: one
        # segment spanning the sequence or, beyond the kernel's 511 blocks per segment, segments of 256 blocks
        # (with that order and everything selected the result does not depend on the segment size).
        nb = (q_len + block_size - 1) // block_size
        segment_size = (nb if nb <= 511 else 256) * block_size
        threshold = 1

    if isinstance(threshold, int) and threshold == 1:
        # every candidate is selected: no estimate, one full gather
        perm = apply_permutation(query_states, key_states, value_states, block_size, segment_size, key_pool_mode,
                                 identity=one_segment)
        sel = permuted_block_selection(query_states, perm, block_size, segment_size, threshold, causal,
                                       force_select_first_block, query_pool_mode, key_pool_mode, want_masks=False)
    else:
        # the order of the single-call path: the estimate runs on key blocks pooled straight from K, and K / V
        # are gathered after the selection, only the blocks some query block visits
        perm, sel = _select_then_gather(query_states, key_states, value_states, block_size, segment_size, threshold,
                                        force_select_first_block, query_pool_mode, key_pool_mode, candidates_only=True)
    out = perm.attention(query_states, sel["csr_cols"], sel["csr_cnt"], segment_size, 1.0 / math.sqrt(head_dim))
    _mark("sparse_attn")
    # queries are not permuted (pbs.py:191-193): un-permutation is the identity
    out = ops.unpermute(out)
    _mark("unpermute")
    return out


# the patched Hugging Face forward may hand K/V over at the KV-head count
permuted_block_sparse_attn_fwd.native_gqa = True
