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


def sparse_attention_on_block_mask(perm_Q, perm_K, perm_V, perm_O, perm_Q_indices, perm_K_indices, perm_V_indices,
                                   block_mask, block_size=128, segment_size=1024, causal=True):
    """The reference's attention stage with its own argument list
    (pbs_attn/src/kernels/permuted_block_sparse_attention.py:314-323, and the Triton launch of pbs.py:220-246):
    queries in original order, K / V already permuted, their original positions, and a block mask in permuted
    block coordinates.  Query i attends to permuted key j iff block_mask[block(i), block(j)] and
    perm_K_indices[j] <= perm_Q_indices[i].  Fills and returns perm_O.

    Runs on the HIP attention kernel, which reads a query block's own segment in original key order and always
    attends to all of its visible keys: a mask that leaves out a block of a query block's own segment (the
    reference's orchestrator never makes one, pbs.py:209) raises ValueError, as do permuted queries."""
    assert causal
    assert segment_size % block_size == 0, "segment_size must be a multiple of block_size"
    B, H, S, D = perm_Q.shape
    assert perm_K.shape[2] == S, "Only support prefilling for now"
    dev = perm_Q.device
    nb = (S + block_size - 1) // block_size
    pos = torch.arange(S, device=dev)
    if not bool((perm_Q_indices.to(dev) == pos.view(1, 1, -1)).all()):
        raise ValueError("the HIP attention kernel takes queries in their original order (the reference never permutes them)")
    if block_mask.shape[-2:] != (nb, nb):
        raise ValueError(f"block_mask must be (..., {nb}, {nb}) for {S} tokens in blocks of {block_size}")
    k, v = perm_K, perm_V
    if k.shape[1] != H:
        k = k.repeat_interleave(H // k.shape[1], dim=1)
        v = v.repeat_interleave(H // v.shape[1], dim=1)
    k_idx = perm_K_indices.to(device=dev, dtype=torch.int32).expand(B, H, -1).contiguous()
    v_idx = perm_V_indices.to(device=dev, dtype=torch.int32).expand(B, H, -1).contiguous()
    # back to original key order (the scatter kernel of the output un-permutation), then the kernels' own layouts
    k_orig = ops.unpermute(k.contiguous(), k_idx, torch.empty_like(k, memory_format=torch.contiguous_format))
    v_orig = ops.unpermute(v.contiguous(), v_idx, torch.empty_like(v, memory_format=torch.contiguous_format))
    pad_idx = torch.cat([k_idx, torch.arange(S, nb * block_size, dtype=torch.int32, device=dev).expand(B, H, -1)], dim=-1)
    perm_k, perm_vt, _ = ops.gather_kv(k_orig, v_orig, pad_idx.contiguous(), H, want_pooled=False)
    cols, cnt, missing = ops.block_mask_to_csr(block_mask.to(dev).expand(B, H, nb, nb), segment_size // block_size)
    if int(missing.item()) != 0:
        raise ValueError("block_mask leaves out blocks of a query block's own segment: the HIP attention kernel "
                         "always attends to the visible keys of the whole own segment (as pbs.py:209 arranges)")
    out = ops.sparse_attn_fwd(perm_Q, perm_k, perm_vt, k_orig, v_orig, cols, cnt, segment_size, 1.0 / (D ** 0.5))
    perm_O.copy_(out)
    return perm_O


class _TritonStyleLauncher:
    """``kernel[grid](...)`` with the positional list of the reference's Triton kernel
    (pbs_attn/src/pbs.py:220-246): the tensors and the two size constants are used, strides come from the tensors."""

    def __getitem__(self, grid):
        def launch(Q, K, V, O, block_mask, q_idx, k_idx, v_idx, *strides_and_sizes, LOGICAL_BLOCK_SIZE=128,
                   SEGMENT_SIZE=1024, **meta):
            sparse_attention_on_block_mask(Q, K, V, O, q_idx, k_idx, v_idx, block_mask, LOGICAL_BLOCK_SIZE, SEGMENT_SIZE, True)
        return launch


permuted_block_sparse_attn_kernel = _TritonStyleLauncher()
