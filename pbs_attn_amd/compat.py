"""The reference's stage-level functions with the reference's own signatures and return values, on the HIP
kernels.  They exist for callers that import the stages (``pbs_attn.src.permute_states``,
``pbs_attn.src.utils``, ``pbs_attn.src.pbs``); the prefill path itself runs fused through
``pbs_attn_amd.pbs`` and never materialises these intermediates in the reference's layouts.

Tensors are bf16 on the GPU, head_dim 128, block_size 128; K/V heads may equal the query heads (the
reference's requirement) or divide them.  Sorts are stable (ties keep ascending index order)."""
from __future__ import annotations

from typing import Tuple, Union

import torch

from . import ops


def last_block_attn_sorting(queries: torch.Tensor, keys: torch.Tensor, block_size: int,
                            segment_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """pbs_attn/src/permute_states.py:6-83 -> (permuted_keys (B, H, S, D), indices (B, H, S) int64)."""
    assert segment_size > 0 and block_size > 0
    B, H, S, _ = queries.shape
    nseg, rem = S // segment_size, S % segment_size
    if nseg == 0 or (nseg == 1 and rem == 0):               # permute_states.py:36-38
        idx = torch.arange(S, device=keys.device).view(1, 1, -1).expand(B, H, -1)
        return (keys if keys.shape[1] == H else keys.repeat_interleave(H // keys.shape[1], dim=1)), idx
    scores = ops.score_keys(queries, keys, block_size, segment_size)
    idx = ops.segment_argsort(scores, S, segment_size, block_size)
    perm_k, _, _ = ops.gather_kv(keys, keys, idx, H)
    return perm_k[:, :, :S], idx[:, :, :S].long()


def apply_permutation(query_states: torch.Tensor, key_states: torch.Tensor, block_size: int,
                      segment_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """pbs_attn/src/permute_states.py:87-106 -> (permuted_keys, indices)."""
    return last_block_attn_sorting(queries=query_states, keys=key_states, block_size=block_size,
                                   segment_size=segment_size)


def first_token_mask(key_indices: torch.Tensor, block_size: int) -> torch.Tensor:
    """pbs_attn/src/pbs.py:10-25 -> (B, H, 1, num_kv_blocks) bool."""
    m = (key_indices.view(key_indices.shape[0], key_indices.shape[1], -1, block_size) == 0).any(dim=-1)
    return m[:, :, None, :]


def _candidate_rule(mask: torch.Tensor):
    """Which of the two candidate rules the kernels implement a (nb, nb) block mask states:
    ("causal", 1) = lower triangle with the diagonal; ("segments", bps) = blocks of strictly earlier
    segments of bps blocks (pbs.py:97-107)."""
    nb = mask.shape[-1]
    assert mask.shape[-2] == nb, "only square (prefill) block masks are supported"
    m = mask.to(torch.bool).cpu()
    qb, kb = torch.arange(nb).unsqueeze(1), torch.arange(nb).unsqueeze(0)
    if torch.equal(m, kb <= qb):
        return "causal", 1
    for bps in range(1, nb + 1):
        if torch.equal(m, ((qb // bps) != (kb // bps)) & (kb <= qb)):
            return "segments", bps
    raise ValueError("block_pooled_attn: this mask is neither the causal lower triangle nor the "
                     "earlier-segments rule; the HIP estimate kernel implements those two")


def block_pooled_attn(query_states: torch.Tensor, key_states: torch.Tensor, block_size: int, mask: torch.Tensor,
                      query_pool_mode: str = "mean", key_pool_mode: str = "mean") -> torch.Tensor:
    """pbs_attn/src/utils.py:6-34 for sequences that are whole blocks (the caller pads, as there)."""
    if query_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid query_pool_mode: {query_pool_mode}")
    if key_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid key_pool_mode: {key_pool_mode}")
    rule, bps = _candidate_rule(mask)
    H = query_states.shape[1]
    if key_states.shape[1] != H:
        key_states = key_states.repeat_interleave(H // key_states.shape[1], dim=1)
    pooled_q = ops.pool_q(query_states, query_pool_mode)
    pooled_k = ops.pool_q(key_states, key_pool_mode)
    return ops.block_logits_softmax(pooled_q, pooled_k, bps, causal_candidates=(rule == "causal"))


def select_blocks(block_attn_scores: torch.Tensor, threshold: Union[float, torch.Tensor],
                  causal: bool = True) -> torch.Tensor:
    """pbs_attn/src/utils.py:38-86 -> (B, H, nb, nb) bool."""
    assert causal == True, "This implementation variant strictly supports causal=True."  # noqa: E712
    B, H, nb, nk = block_attn_scores.shape
    assert nb == nk, "only square (prefill) score matrices are supported"
    dev = block_attn_scores.device
    idx = torch.arange(nb * ops.BLOCK, dtype=torch.int32, device=dev).view(1, 1, -1).expand(B, H, -1).contiguous()
    thr = threshold if isinstance(threshold, torch.Tensor) else float(threshold)
    sel, _, _, _ = ops.select_blocks(block_attn_scores.float(), thr, idx, nb * ops.BLOCK, ops.BLOCK, ops.BLOCK,
                                     force_select_first_block=False, want_masks=True, want_csr=False)
    return sel


def permuted_block_selection(permuted_query_states: torch.Tensor, permuted_key_states: torch.Tensor,
                             query_indices: torch.Tensor, key_indices: torch.Tensor, block_size: int,
                             segment_size: int, threshold: float = 0.9, causal: bool = True,
                             force_select_first_block: bool = True, query_pool_mode: str = "mean",
                             key_pool_mode: str = "mean") -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """pbs_attn/src/pbs.py:29-130 -> (block_attn_scores, block_mask, segment_mask)."""
    assert causal
    assert segment_size % block_size == 0, "segment_size must be a multiple of block_size"
    if query_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid query_pool_mode: {query_pool_mode}")
    if key_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid key_pool_mode: {key_pool_mode}")
    B, H, S, _ = permuted_query_states.shape
    assert S == permuted_key_states.shape[2], "Only support prefilling for now"
    dev = permuted_query_states.device
    nb = (S + block_size - 1) // block_size
    bps = segment_size // block_size
    k = permuted_key_states
    if k.shape[1] != H:
        k = k.repeat_interleave(H // k.shape[1], dim=1)
    pooled_q = ops.pool_q(permuted_query_states, query_pool_mode)      # rows past S count as zeros (pbs.py:67-79)
    pooled_k = ops.pool_q(k, key_pool_mode)
    scores = ops.block_logits_softmax(pooled_q, pooled_k, bps)
    pad_idx = torch.cat([key_indices.to(device=dev, dtype=torch.int32).expand(B, H, -1),
                         torch.arange(S, nb * block_size, dtype=torch.int32, device=dev).expand(B, H, -1)], dim=-1)
    sel, _, _, _ = ops.select_blocks(scores, threshold, pad_idx.contiguous(), S, block_size, segment_size,
                                     force_select_first_block, want_masks=True, want_csr=False)
    qb = torch.arange(nb, device=dev).unsqueeze(1)
    kb = torch.arange(nb, device=dev).unsqueeze(0)
    segment_mask = (qb // bps) == (kb // bps)
    return scores, sel, segment_mask
