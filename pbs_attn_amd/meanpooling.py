"""The reference's un-permuted MeanPooling baseline through the PBS HIP kernels.

Mirrors pbs_attn/baselines/MeanPooling.py:7-99 (``MeanPooling_prefill``: same name, arguments and
defaults): block probabilities from mean-pooled Q and K blocks over the causal lower triangle of
blocks INCLUDING the diagonal, cumulative-threshold selection, block 0 and the diagonal block forced,
block-sparse causal attention.  It is PBS without the permutation, which makes it the ablation that
shows what the permutation buys.  The reference runs its attention on an external CUDA extension;
here the identity key order goes through the same gather / estimate / select / attention kernels
(one block per "segment": the diagonal block is the own segment, read with the causal triangle,
every selected earlier block is read unmasked).

Differences a caller can see: any batch size and K/V at the KV-head count are accepted (the
reference asserts batch 1 and expanded heads).  With ``force_select_current_block=False`` a query block
attends to its diagonal block only where the threshold selected it (MeanPooling.py:54-58)."""
from __future__ import annotations

import torch

from . import ops


def MeanPooling_prefill(
    query_states: torch.Tensor,
    key_states: torch.Tensor,
    value_states: torch.Tensor,
    block_size: int = 128,
    segment_size: int = 1024,
    threshold: float = 0.9,
    causal: bool = True,
    force_select_first_block: bool = True,
    force_select_current_block: bool = True,
    return_masks: bool = False,
):
    batch_size, num_q_heads, q_len, head_dim = query_states.shape
    _, num_kv_heads, kv_len, _ = key_states.shape
    assert num_q_heads % num_kv_heads == 0
    assert q_len == kv_len, "Only support prefilling for now, q_len: {}, kv_len: {}".format(q_len, kv_len)
    assert causal
    s_pad = (q_len + block_size - 1) // block_size * block_size
    idx = torch.arange(s_pad, dtype=torch.int32, device=query_states.device).view(1, 1, -1)
    idx = idx.expand(batch_size, num_q_heads, -1).contiguous()
    perm_k, perm_vt, pooled_k = ops.gather_kv(key_states, value_states, idx, num_q_heads, "mean")
    pooled_q = ops.pool_q(query_states, "mean")
    scores = ops.block_logits_softmax(pooled_q, pooled_k, 1, causal_candidates=True)
    # MeanPooling.py:50 hands the threshold to select_blocks as it is: there is no "int 1 = everything" rule here
    thr = threshold if isinstance(threshold, torch.Tensor) else float(threshold)
    # one block per segment: the visit list holds the selected blocks before the diagonal, the diagonal
    # block (MeanPooling.py:54-58) is the attention kernel's own-segment tile
    sel, fin, cols, cnt = ops.select_blocks(scores, thr, idx, q_len, block_size, block_size, force_select_first_block,
                                            want_masks=return_masks or not force_select_current_block, candidate_rule=2)
    own = None
    if not force_select_current_block:
        # the diagonal block only where the threshold chose it (or it is block 0 and that one is forced): the plain
        # selection mask says where
        fin = sel   # the selection with the forced first column, without the forced diagonal
        own = fin.diagonal(dim1=-2, dim2=-1).to(torch.uint8).contiguous()
    out = ops.sparse_attn_fwd(query_states, perm_k, perm_vt, key_states, value_states, cols, cnt, block_size, own_block_needed=own)
    if return_masks:
        return out, dict(block_attn_scores=scores, block_mask=fin, csr_cnt=cnt)
    return out


MeanPooling_prefill.native_gqa = True
