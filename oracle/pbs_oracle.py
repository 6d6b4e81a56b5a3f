"""CPU restatement of PBS-Attn's permuted block-sparse prefill attention.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
module; it is the checker that tests, the smoke entry and the benchmark's
``cpu_baseline`` leg compare the HIP path against.  It restates, in plain
torch ops on the CPU, the algorithm of the reference files

    pbs_attn/src/pbs.py                               (orchestrator, selection)
    pbs_attn/src/permute_states.py                    (key scoring, segment sort)
    pbs_attn/src/utils.py                             (block pooling, selection)
    pbs_attn/src/kernels/permuted_block_sparse_attention.py:314-383 (naive path)

Two deliberate, documented differences from the reference text:

* both sorts are STABLE (descending by value, ties by ascending index).  The
  reference calls ``argsort``/``sort`` without ``stable=True``; on GPU torch's
  sort behaves stably, on CPU it does not for rows >= 32 wide, and ties are
  common (bf16 block logits).  Stable order is the one defined here.
* indices are carried as int64 like the reference, K/V may be passed at the
  KV-head count (they are expanded exactly like ``repeat_kv`` does).

How each function is pinned (no reference test exists for this path, the
reference ships no golden vectors):

* ``key_scores``: closed form in float64 (tests/test_oracle.py::test_key_scores_*),
  rows sum to one.
* ``segment_argsort``: brute force ``sorted(range, key=(-score, index))``.
* ``gather_rows``: ``K[idx]`` by explicit python loops.
* ``block_pooled_attn``: textbook mean pool + softmax in float64.
* ``select_blocks``: brute-force minimal descending prefix with a sequential
  float64 running sum; invariants (mass >= thr, minimality, empty on zero rows).
* ``first_token_mask`` / masks: closed-form integer construction.
* ``sparse_attn_naive`` and the whole pipeline: dense fp32 masked attention on
  the token mask, ``threshold=1`` (int) == ``scaled_dot_product_attention``
  (library routine), ``S <= segment`` == SDPA, one-hot V recovers the weights,
  an independent pure-python pipeline on tiny inputs (tests/golden).
"""
from __future__ import annotations

import math
from typing import Optional, Union

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------

def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(B, Hkv, S, D) -> (B, Hkv*n_rep, S, D); pbs_attn/patch/huggingface.py:28-37."""
    if n_rep == 1:
        return x
    b, h, s, d = x.shape
    return x[:, :, None].expand(b, h, n_rep, s, d).reshape(b, h * n_rep, s, d)


def _expand_to(q: torch.Tensor, kv: torch.Tensor) -> torch.Tensor:
    hq, hkv = q.shape[1], kv.shape[1]
    assert hq % hkv == 0
    return repeat_kv(kv, hq // hkv)


# --------------------------------------------------------------------------
# (a2) key scoring -- permute_states.py:26-54
# --------------------------------------------------------------------------

def key_scores(q: torch.Tensor, k: torch.Tensor, block_size: int, segment_size: int) -> torch.Tensor:
    """Mean attention each key of the complete segments receives from the last
    ``block_size`` queries.  Returns (B, H, Sc) float32, Sc = (S // seg) * seg.

    permute_states.py:44    last_block_queries = queries[:, :, -block_size:, :]
    permute_states.py:47-48 logits = matmul(lastQ, Kc^T) / sqrt(D)   (input dtype)
    permute_states.py:49    softmax(dim=-1, dtype=float32)           (no causal mask)
    permute_states.py:50    mean over the query rows
    """
    k = _expand_to(q, k)
    s, d = k.shape[2], k.shape[3]
    sc = (s // segment_size) * segment_size
    last_q = q[:, :, -block_size:, :]
    logits = torch.matmul(last_q, k[:, :, :sc, :].transpose(-1, -2)) / math.sqrt(d)
    probs = F.softmax(logits, dim=-1, dtype=torch.float32)
    return probs.mean(dim=-2)


# --------------------------------------------------------------------------
# (a3) per-segment stable descending argsort -- permute_states.py:52-56,71-81
# --------------------------------------------------------------------------

def segment_argsort(scores: torch.Tensor, seq_len: int, segment_size: int) -> torch.Tensor:
    """scores (B, H, Sc) -> global key indices (B, H, S) int64.  Keys never leave
    their segment; the trailing partial segment keeps identity order."""
    b, h, sc = scores.shape
    nseg = sc // segment_size
    local = torch.argsort(scores.reshape(b, h, nseg, segment_size), dim=-1, descending=True, stable=True)
    starts = torch.arange(0, sc, segment_size).view(1, 1, nseg, 1)
    idx = (local + starts).reshape(b, h, sc)
    if sc < seq_len:
        rem = torch.arange(sc, seq_len).view(1, 1, -1).expand(b, h, -1)
        idx = torch.cat([idx, rem], dim=2)
    return idx


def gather_rows(x: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """x (B, H, S, D), idx (B, H, S) -> x[b, h, idx[b, h, i], :];
    permute_states.py:59-62, pbs.py:213-214."""
    return torch.gather(x, 2, idx.unsqueeze(-1).expand(-1, -1, -1, x.shape[-1]))


def last_block_attn_sorting(q, k, block_size, segment_size, scores: Optional[torch.Tensor] = None):
    """permute_states.py:6-83.  Returns (perm_k, idx int64).  ``scores`` may be
    injected so the sort can be checked on a given score tensor."""
    k = _expand_to(q, k)
    b, h, s, _ = k.shape
    nseg, rem = s // segment_size, s % segment_size
    if nseg == 0 or (nseg == 1 and rem == 0):          # permute_states.py:36-38
        idx = torch.arange(s).view(1, 1, -1).expand(b, h, -1)
        return k, idx
    if scores is None:
        scores = key_scores(q, k, block_size, segment_size)
    idx = segment_argsort(scores, s, segment_size)
    return gather_rows(k, idx), idx


# --------------------------------------------------------------------------
# (a5-a8) block selection -- pbs.py:29-130, utils.py
# --------------------------------------------------------------------------

def pad_to_block(x: torch.Tensor, idx: torch.Tensor, block_size: int):
    """Zero-pad the sequence to a multiple of the block and extend the index with
    its own positions; pbs.py:67-92."""
    s = x.shape[2]
    pad = (-s) % block_size
    if pad == 0:
        return x, idx
    x = F.pad(x, (0, 0, 0, pad), value=0)
    ext = torch.arange(s, s + pad).view(1, 1, -1).expand(idx.shape[0], idx.shape[1], -1)
    return x, torch.cat([idx, ext], dim=-1)


def candidate_masks(nb: int, blocks_per_segment: int):
    """pbs.py:97-107 (square, causal).  Returns (candidate, segment_mask), both (nb, nb) bool."""
    qb = torch.arange(nb).unsqueeze(1)
    kb = torch.arange(nb).unsqueeze(0)
    segment_mask = (qb // blocks_per_segment) == (kb // blocks_per_segment)
    cand = (~segment_mask) & (kb <= qb)
    return cand, segment_mask


def pool_blocks(x: torch.Tensor, block_size: int, mode: str) -> torch.Tensor:
    """utils.py:18-29; x already padded.  Result keeps x's dtype."""
    b, h, s, d = x.shape
    x5 = x.reshape(b, h, s // block_size, block_size, d)
    if mode == "mean":
        return x5.mean(dim=-2)
    if mode == "max":
        return x5.max(dim=-2).values
    raise ValueError(f"Invalid pool mode: {mode}")


def block_logits_softmax(pooled_q: torch.Tensor, pooled_k: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """utils.py:30-33 from already pooled states."""
    d = pooled_q.shape[-1]
    logits = torch.einsum("bhqd,bhkd->bhqk", pooled_q, pooled_k)
    logits = logits / math.sqrt(d)
    logits = logits.masked_fill(~mask, float("-inf"))
    return F.softmax(logits, dim=-1, dtype=torch.float32)


def block_pooled_attn(q, k, block_size, mask, query_pool_mode="mean", key_pool_mode="mean"):
    """utils.py:6-34."""
    if query_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid query_pool_mode: {query_pool_mode}")
    if key_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid key_pool_mode: {key_pool_mode}")
    return block_logits_softmax(pool_blocks(q, block_size, query_pool_mode),
                                pool_blocks(k, block_size, key_pool_mode), mask)


def select_blocks(block_attn_scores: torch.Tensor, threshold: Union[float, torch.Tensor]) -> torch.Tensor:
    """utils.py:38-86: smallest descending prefix whose running sum reaches the
    threshold; nothing if the row never reaches it.

    The running sum is the CPU one: sequential float64 accumulation, every
    prefix rounded to float32, compared with float32(threshold)."""
    p = torch.nan_to_num(block_attn_scores.float(), nan=0.0)
    nk = p.shape[-1]
    if p.shape[-2] == 0 or nk == 0:
        return torch.zeros_like(p, dtype=torch.bool)
    sorted_scores, sorted_idx = torch.sort(p, dim=-1, descending=True, stable=True)
    cum = torch.cumsum(sorted_scores.double(), dim=-1).float()
    if isinstance(threshold, torch.Tensor):
        # utils.py:70-72: compared after torch's type promotion (a float64 tensor makes it a float64 compare)
        thr = threshold.reshape(threshold.shape + (1, 1))
    else:
        thr = torch.tensor(float(threshold), dtype=torch.float32)
    exceed = cum >= thr
    first = torch.argmax(exceed.int(), dim=-1, keepdim=True)
    any_exceeds = exceed.any(dim=-1, keepdim=True)
    ramp = torch.arange(nk).view(1, 1, 1, nk)
    sel_sorted = (ramp <= first) & any_exceeds
    out = torch.empty_like(p, dtype=torch.bool)
    out.scatter_(dim=-1, index=sorted_idx, src=sel_sorted)
    return out


def first_token_mask(key_indices: torch.Tensor, block_size: int) -> torch.Tensor:
    """pbs.py:10-25: the kv block(s) holding original key 0 -> (B, H, 1, nb)."""
    b, h, _ = key_indices.shape
    return (key_indices.reshape(b, h, -1, block_size) == 0).any(dim=-1)[:, :, None, :]


def permuted_block_selection(q, perm_k, key_indices, block_size, segment_size, threshold=0.9,
                             force_select_first_block=True, query_pool_mode="mean", key_pool_mode="mean"):
    """pbs.py:29-130 (queries are not permuted).  Returns
    (block_attn_scores, block_mask, segment_mask)."""
    assert q.shape[1] == perm_k.shape[1]
    assert q.shape[2] == perm_k.shape[2], "Only support prefilling for now"
    assert segment_size % block_size == 0, "segment_size must be a multiple of block_size"
    b, h, s, _ = q.shape
    q_idx = torch.arange(s).view(1, 1, -1).expand(b, h, -1)
    pq, _ = pad_to_block(q, q_idx, block_size)
    pk, pidx = pad_to_block(perm_k, key_indices, block_size)
    nb = pq.shape[2] // block_size
    cand, segment_mask = candidate_masks(nb, segment_size // block_size)
    scores = block_pooled_attn(pq, pk, block_size, cand, query_pool_mode, key_pool_mode)
    if isinstance(threshold, int) and threshold == 1:           # pbs.py:120-121
        block_mask = cand.view(1, 1, nb, nb).expand_as(scores).clone()
    else:
        block_mask = select_blocks(scores, threshold)
    if force_select_first_block:                                 # pbs.py:125-127
        block_mask = block_mask | first_token_mask(pidx, block_size)
    return scores, block_mask, segment_mask


# --------------------------------------------------------------------------
# (a10) naive sparse attention -- kernels/permuted_block_sparse_attention.py:314-383
# --------------------------------------------------------------------------

def sparse_attn_naive(q, perm_k, perm_v, key_indices, block_mask, block_size):
    """Per (batch, head, query block): concatenate the selected K/V blocks, mask
    ``q_idx >= k_idx``, softmax in float32, cast to the input dtype, multiply V."""
    b, h, s, d = q.shape
    nb = (s + block_size - 1) // block_size
    out = torch.empty_like(q)
    q_pos = torch.arange(s)
    for bi in range(b):
        for hi in range(h):
            for qb in range(nb):
                q0, q1 = qb * block_size, min((qb + 1) * block_size, s)
                sel = torch.where(block_mask[bi, hi, qb])[0]
                if len(sel) == 0:
                    out[bi, hi, q0:q1] = 0
                    continue
                cols = torch.cat([torch.arange(int(kb) * block_size, min((int(kb) + 1) * block_size, s)) for kb in sel])
                kk = perm_k[bi, hi, cols]
                vv = perm_v[bi, hi, cols]
                ki = key_indices[bi, hi, cols]
                logits = torch.matmul(q[bi, hi, q0:q1], kk.transpose(-2, -1)) / math.sqrt(d)
                allowed = q_pos[q0:q1].unsqueeze(-1) >= ki.unsqueeze(0)
                logits = logits.masked_fill(~allowed, float("-inf"))
                w = torch.softmax(logits, dim=-1, dtype=torch.float32).to(q.dtype)
                out[bi, hi, q0:q1] = torch.matmul(w, vv)
    return out


def token_mask(key_indices: torch.Tensor, block_mask: torch.Tensor, seq_len: int, block_size: int) -> torch.Tensor:
    """(B, H, S, S) bool over (query position, PERMUTED key position): the block is
    selected and the key's original position is not after the query."""
    pos = torch.arange(seq_len)
    blk = pos // block_size
    bm = block_mask[:, :, blk][:, :, :, blk]
    causal = key_indices[:, :, None, :seq_len] <= pos.view(1, 1, -1, 1)
    return bm & causal


def dense_masked_attention_fp32(q, perm_k, perm_v, key_indices, block_mask, block_size) -> torch.Tensor:
    """Dense float32 attention restricted to ``token_mask``; the independent check
    for both the naive path and the HIP kernel.  Returns float32."""
    s, d = q.shape[2], q.shape[3]
    tm = token_mask(key_indices, block_mask, s, block_size)
    logits = torch.matmul(q.float(), perm_k.float().transpose(-1, -2)) / math.sqrt(d)
    logits = logits.masked_fill(~tm, float("-inf"))
    return torch.matmul(torch.softmax(logits, dim=-1), perm_v.float())


# --------------------------------------------------------------------------
# (a1) orchestrator -- pbs.py:132-257
# --------------------------------------------------------------------------

def permuted_block_sparse_attn_fwd(q, k, v, block_size, segment_size, threshold, causal=True,
                                   force_select_first_block=True, query_pool_mode="mean",
                                   key_pool_mode="mean", return_intermediates=False):
    """The reference's ``use_triton=False`` pipeline.  Output (B, H, S, D) in the
    input dtype, original query order."""
    assert causal
    k = _expand_to(q, k)
    v = _expand_to(q, v)
    assert q.shape[2] == k.shape[2]
    s = q.shape[2]
    if s <= segment_size:                                        # pbs.py:175-182
        out = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        return (out, {}) if return_intermediates else out
    perm_k, idx = last_block_attn_sorting(q, k, block_size, segment_size)
    scores, block_mask, segment_mask = permuted_block_selection(
        q, perm_k, idx, block_size, segment_size, threshold, force_select_first_block,
        query_pool_mode, key_pool_mode)
    final_mask = block_mask | segment_mask[None, None]           # pbs.py:209
    perm_v = gather_rows(v, idx)
    out = sparse_attn_naive(q, perm_k, perm_v, idx, final_mask, block_size)
    if return_intermediates:
        return out, dict(key_indices=idx, perm_k=perm_k, perm_v=perm_v, block_attn_scores=scores,
                         block_mask=block_mask, final_mask=final_mask)
    return out


def visited_block_pairs(final_mask: torch.Tensor, blocks_per_segment: int) -> int:
    """Number of (q block, k block) tiles the sparse kernel visits: mask true and
    the key block's segment not after the query block's."""
    nb = final_mask.shape[-1]
    qb = torch.arange(nb).unsqueeze(1) // blocks_per_segment
    kb = torch.arange(nb).unsqueeze(0) // blocks_per_segment
    return int((final_mask & (kb <= qb)).sum())


# --------------------------------------------------------------------------
# MeanPooling baseline (no permutation) -- baselines/MeanPooling.py:7-99
# --------------------------------------------------------------------------

def meanpooling_selection(q, k, block_size, threshold, force_select_first_block=True,
                          force_select_current_block=True):
    """baselines/MeanPooling.py:24-58: pad to whole blocks, candidates = the causal lower triangle of blocks
    INCLUDING the diagonal (:43-46), block_pooled_attn + select_blocks on the un-permuted keys (:48-50),
    column 0 forced (:52-53), diagonal forced (:54-58).  Returns (block_attn_scores, block_mask)."""
    k = _expand_to(q, k)
    b, h, s, _ = q.shape
    ident = torch.arange(s).view(1, 1, -1).expand(b, h, -1)
    pq, _ = pad_to_block(q, ident, block_size)
    pk, _ = pad_to_block(k, ident, block_size)
    nb = pq.shape[2] // block_size
    cand = torch.tril(torch.ones(nb, nb, dtype=torch.bool))
    scores = block_pooled_attn(pq, pk, block_size, cand)
    block_mask = select_blocks(scores, threshold)
    if force_select_first_block:
        block_mask[:, :, :, 0] = True
    if force_select_current_block:
        block_mask = block_mask | torch.eye(nb, dtype=torch.bool).view(1, 1, nb, nb)
    return scores, block_mask


def meanpooling_prefill(q, k, v, block_size=128, segment_size=1024, threshold=0.9, causal=True,
                        force_select_first_block=True, force_select_current_block=True,
                        return_intermediates=False):
    """baselines/MeanPooling.py:7-99 with the external block-sparse kernel (:80-96, ``is_causal=True``)
    restated as what it computes: attention over the selected blocks with the token-level causal mask, here
    through the same naive per-block path as PBS (identity key order).  ``segment_size`` is accepted and
    unused, as there."""
    assert causal
    k, v = _expand_to(q, k), _expand_to(q, v)
    assert q.shape[2] == k.shape[2]
    b, h, s, _ = q.shape
    scores, block_mask = meanpooling_selection(q, k, block_size, threshold, force_select_first_block,
                                               force_select_current_block)
    ident = torch.arange(s).view(1, 1, -1).expand(b, h, -1)
    out = sparse_attn_naive(q, k, v, ident, block_mask, block_size)
    if return_intermediates:
        return out, dict(block_attn_scores=scores, block_mask=block_mask, key_indices=ident)
    return out
