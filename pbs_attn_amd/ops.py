"""Stage-level torch wrappers over the C ABI (device pointers, strides, current
stream).  Tensors are bf16, head_dim 128, block_size 128; all outputs are
allocated through torch's caching allocator."""
from __future__ import annotations

import math

import torch

from . import _lib

BLOCK = 128
HEAD_DIM = 128


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return t.data_ptr() if t is not None else None


def _rows16(t: torch.Tensor) -> torch.Tensor:
    """Kernels need unit stride on head_dim and 16-byte aligned rows."""
    if t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:-1]) or t.data_ptr() % 16:
        t = t.contiguous()
    return t


def _check_bf16_cuda(*ts):
    for t in ts:
        if not t.is_cuda:
            raise _lib.PbsHipError("PBS HIP kernels need tensors on the GPU (there is no CPU path)")
        if t.dtype != torch.bfloat16:
            raise _lib.PbsHipError(f"PBS HIP kernels are bf16 only, got {t.dtype}")


def _threshold_args(threshold, B, H, device):
    """(is_int_one, per-row fp32 tensor or None, python float) with the reference's comparison semantics
    (pbs_attn/src/pbs.py:120, pbs_attn/src/utils.py:67-72): ``isinstance(threshold, int) and threshold == 1``
    (True included) selects every candidate; a python float is compared in float32; a tensor is compared
    after type promotion with the float32 running sum -- for a float64 tensor that is a float64 compare,
    which equals a float32 compare with the smallest float32 not below the threshold."""
    if isinstance(threshold, torch.Tensor):
        t = threshold.to(device=device)
        if t.dtype == torch.float64:
            t32 = t.float()
            t32 = torch.where(t32.double() < t, torch.nextafter(t32, torch.full_like(t32, float("inf"))), t32)
        elif t.is_floating_point():
            t32 = t.float()
        else:
            t32 = t.double().float()   # integer tensors: exact for every value a threshold can sensibly take
        return False, t32.expand(B, H).contiguous(), 0.0
    if isinstance(threshold, int) and threshold == 1:
        return True, None, 0.0
    return False, None, float(threshold)


def score_keys(q, k, block_size, segment_size):
    """(B, Hq, Sc) float32 key scores; permute_states.py:44-50."""
    _check_bf16_cuda(q, k)
    lib = _lib.load()
    q, k = _rows16(q), _rows16(k)
    B, Hq, S, D = q.shape
    Hkv = k.shape[1]
    Sc = (S // segment_size) * segment_size
    scores = torch.empty((B, Hq, Sc), dtype=torch.float32, device=q.device)
    ws_bytes = lib.pbs_score_keys_workspace_bytes(B, Hq, Hkv, S, segment_size)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=q.device)
    _lib.check(lib.pbs_score_keys(_ptr(q), _ptr(k), _ptr(scores), B, Hq, Hkv, S, D, block_size, segment_size,
                                  q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
                                  _ptr(ws), ws.numel(), _stream()), "pbs_score_keys")
    return scores


def segment_argsort(scores, seq_len, segment_size, block_size=BLOCK):
    """scores (B, H, Sc) float32 -> int32 key indices (B, H, S_pad), S_pad = S rounded
    up to the block; permute_states.py:56,71-81."""
    lib = _lib.load()
    B, H = scores.shape[:2]
    scores = scores.contiguous().float()
    s_pad = (seq_len + block_size - 1) // block_size * block_size
    idx = torch.empty((B, H, s_pad), dtype=torch.int32, device=scores.device)
    _lib.check(lib.pbs_segment_argsort(_ptr(scores), _ptr(idx), B * H, seq_len, s_pad, segment_size, _stream()),
               "pbs_segment_argsort")
    return idx


def gather_kv(k, v, idx, num_q_heads, key_pool_mode="mean", block_needed=None, want_pooled=True):
    """Returns perm_k (B, Hq, S_pad, D), perm_vt (B, Hq, nb, D, 128) and pooled_k (B, Hq, nb, D).
    ``block_needed`` ((B, Hq, nb) uint8, from ``select_blocks(..., block_needed=...)``) restricts the gather to
    the blocks whose byte is set: the other tiles of perm_k / perm_vt stay uninitialised.  ``want_pooled=False``
    returns None for pooled_k."""
    _check_bf16_cuda(k, v)
    if key_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid key_pool_mode: {key_pool_mode}")
    lib = _lib.load()
    k, v = _rows16(k), _rows16(v)
    B, Hkv, S, D = k.shape
    Hq = num_q_heads
    nb = (S + BLOCK - 1) // BLOCK
    assert idx.shape == (B, Hq, nb * BLOCK) and idx.dtype == torch.int32 and idx.is_contiguous()
    perm_k = torch.empty((B, Hq, nb * BLOCK, D), dtype=k.dtype, device=k.device)
    perm_vt = torch.empty((B, Hq, nb, D, BLOCK), dtype=k.dtype, device=k.device)
    pooled_k = torch.empty((B, Hq, nb, D), dtype=k.dtype, device=k.device) if want_pooled else None
    if block_needed is not None:
        assert block_needed.shape == (B, Hq, nb) and block_needed.dtype == torch.uint8 and block_needed.is_contiguous()
    _lib.check(lib.pbs_gather_kv(_ptr(k), _ptr(v), _ptr(idx), _ptr(perm_k), _ptr(perm_vt), _ptr(pooled_k),
                                 B, Hq, Hkv, S, D, BLOCK, k.stride(0), k.stride(1), k.stride(2),
                                 v.stride(0), v.stride(1), v.stride(2), int(key_pool_mode == "max"),
                                 _ptr(block_needed), _stream()),
               "pbs_gather_kv")
    return perm_k, perm_vt, pooled_k


def pool_k_permuted(k, idx, num_q_heads, key_pool_mode="mean"):
    """pooled_k of ``gather_kv`` (the same bits) without gathering: the permuted key blocks are pooled straight
    from ``k`` through ``idx``.  Also returns a cleared (B, Hq, nb) uint8 tensor for ``select_blocks`` to mark
    the key blocks that are visited at all."""
    _check_bf16_cuda(k)
    if key_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid key_pool_mode: {key_pool_mode}")
    lib = _lib.load()
    k = _rows16(k)
    B, Hkv, S, D = k.shape
    Hq = num_q_heads
    nb = (S + BLOCK - 1) // BLOCK
    assert idx.shape == (B, Hq, nb * BLOCK) and idx.dtype == torch.int32 and idx.is_contiguous()
    pooled_k = torch.empty((B, Hq, nb, D), dtype=k.dtype, device=k.device)
    needed = torch.empty((B, Hq, nb), dtype=torch.uint8, device=k.device)
    _lib.check(lib.pbs_pool_k_permuted(_ptr(k), _ptr(idx), _ptr(pooled_k), _ptr(needed), B, Hq, Hkv, S, D, BLOCK,
                                       k.stride(0), k.stride(1), k.stride(2), int(key_pool_mode == "max"), _stream()),
               "pbs_pool_k_permuted")
    return pooled_k, needed


def pool_blocks(q, k, idx, query_pool_mode="mean", key_pool_mode="mean"):
    """``pool_q`` and ``pool_k_permuted`` in one launch: returns (pooled_q, pooled_k, block_needed)."""
    _check_bf16_cuda(q, k)
    for mode in (query_pool_mode, key_pool_mode):
        if mode not in ("mean", "max"):
            raise ValueError(f"Invalid pool mode: {mode}")
    lib = _lib.load()
    q, k = _rows16(q), _rows16(k)
    B, Hq, S, D = q.shape
    Hkv = k.shape[1]
    nb = (S + BLOCK - 1) // BLOCK
    assert idx.shape == (B, Hq, nb * BLOCK) and idx.dtype == torch.int32 and idx.is_contiguous()
    pooled_q = torch.empty((B, Hq, nb, D), dtype=q.dtype, device=q.device)
    pooled_k = torch.empty((B, Hq, nb, D), dtype=q.dtype, device=q.device)
    needed = torch.empty((B, Hq, nb), dtype=torch.uint8, device=q.device)
    _lib.check(lib.pbs_pool_blocks(_ptr(q), _ptr(k), _ptr(idx), _ptr(pooled_q), _ptr(pooled_k), _ptr(needed), B, Hq, Hkv,
                                   S, D, BLOCK, q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1),
                                   k.stride(2), int(query_pool_mode == "max"), int(key_pool_mode == "max"), _stream()),
               "pbs_pool_blocks")
    return pooled_q, pooled_k, needed


def pool_q(q, query_pool_mode="mean"):
    _check_bf16_cuda(q)
    if query_pool_mode not in ("mean", "max"):
        raise ValueError(f"Invalid query_pool_mode: {query_pool_mode}")
    lib = _lib.load()
    q = _rows16(q)
    B, Hq, S, D = q.shape
    nb = (S + BLOCK - 1) // BLOCK
    pooled = torch.empty((B, Hq, nb, D), dtype=q.dtype, device=q.device)
    _lib.check(lib.pbs_pool_q(_ptr(q), _ptr(pooled), B, Hq, S, D, BLOCK, q.stride(0), q.stride(1), q.stride(2),
                              int(query_pool_mode == "max"), _stream()), "pbs_pool_q")
    return pooled


def block_logits_softmax(pooled_q, pooled_k, blocks_per_segment, causal_candidates=False, candidates_only=False):
    """(B, H, nb, nb) float32 block probabilities; utils.py:30-33.  Candidates of a query block are the key
    blocks of strictly earlier segments (pbs.py:97-107) or, with ``causal_candidates``, every block up to and
    including the diagonal one (baselines/MeanPooling.py:43-48).  ``candidates_only`` (earlier-segment rule): the
    entries outside a row's candidates stay unwritten -- for ``select_blocks(..., candidate_rule=1)`` on at most 1024
    blocks, which reads no others."""
    _check_bf16_cuda(pooled_q, pooled_k)
    lib = _lib.load()
    pooled_q, pooled_k = pooled_q.contiguous(), pooled_k.contiguous()
    B, H, nb, D = pooled_q.shape
    P = torch.empty((B, H, nb, nb), dtype=torch.float32, device=pooled_q.device)
    if candidates_only:
        assert not causal_candidates
        _lib.check(lib.pbs_block_logits_softmax_candidates_only(_ptr(pooled_q), _ptr(pooled_k), _ptr(P), B * H, nb, D,
                                                                blocks_per_segment, _stream()),
                   "pbs_block_logits_softmax_candidates_only")
    elif causal_candidates:
        _lib.check(lib.pbs_block_logits_softmax_causal(_ptr(pooled_q), _ptr(pooled_k), _ptr(P), B * H, nb, D, _stream()),
                   "pbs_block_logits_softmax_causal")
    else:
        _lib.check(lib.pbs_block_logits_softmax(_ptr(pooled_q), _ptr(pooled_k), _ptr(P), B * H, nb, D,
                                                blocks_per_segment, _stream()), "pbs_block_logits_softmax")
    return P


def select_blocks(block_attn_scores, threshold, idx, seq_len, block_size, segment_size,
                  force_select_first_block=True, want_masks=True, want_csr=True, rows_shape=None, block_needed=None,
                  candidate_rule=0):
    """Returns (sel_mask, final_mask, csr_cols, csr_cnt).  ``threshold`` may be a
    python float, the python int 1 (all candidates) or a (B, H) tensor.  ``block_needed``: a cleared
    (B, H, nb) uint8 tensor; the byte of every key block on some visit list is set.  ``candidate_rule``: 0 = the
    whole row is sorted (any score tensor); 1 / 2 = the scores come from ``block_logits_softmax`` without / with
    ``causal_candidates`` and are zero outside its candidates, so only those are sorted (same result)."""
    lib = _lib.load()
    B, H = idx.shape[:2]
    dev = idx.device
    nb = (seq_len + block_size - 1) // block_size
    is_int_one, thr_rows, thr = _threshold_args(threshold, B, H, dev)
    P = None
    if not is_int_one:
        P = block_attn_scores.contiguous()
        assert P.dtype == torch.float32 and P.shape == (B, H, nb, nb)
    sel = torch.empty((B, H, nb, nb), dtype=torch.bool, device=dev) if want_masks else None
    fin = torch.empty((B, H, nb, nb), dtype=torch.bool, device=dev) if want_masks else None
    cols = torch.empty((B, H, nb, nb), dtype=torch.int32, device=dev) if want_csr else None
    cnt = torch.empty((B, H, nb), dtype=torch.int32, device=dev)
    ws = torch.empty(max(lib.pbs_select_blocks_workspace_bytes(B * H), 16), dtype=torch.uint8, device=dev)
    if block_needed is not None:
        assert block_needed.shape == (B, H, nb) and block_needed.dtype == torch.uint8 and block_needed.is_contiguous()
    _lib.check(lib.pbs_select_blocks(_ptr(P), _ptr(thr_rows), thr, int(is_int_one), int(bool(force_select_first_block)),
                                     int(candidate_rule), _ptr(idx), B * H, seq_len, block_size, segment_size, _ptr(sel), _ptr(fin),
                                     _ptr(cols), _ptr(cnt), _ptr(block_needed), _ptr(ws), ws.numel(), _stream()),
               "pbs_select_blocks")
    return sel, fin, cols, cnt


def block_mask_to_csr(block_mask, blocks_per_segment):
    """Visit lists (csr_cols, csr_cnt) of a (B, H, nb, nb) bool block mask made elsewhere, and the number of
    own-segment blocks it leaves out (a device tensor of one int32; the attention kernel always attends to the
    visible keys of the whole own segment)."""
    lib = _lib.load()
    if not block_mask.is_cuda:
        raise _lib.PbsHipError("PBS HIP kernels need tensors on the GPU (there is no CPU path)")
    B, H, nb, nb2 = block_mask.shape
    assert nb == nb2, "only square (prefill) block masks are supported"
    m = block_mask.to(torch.uint8).contiguous()
    cols = torch.empty((B, H, nb, nb), dtype=torch.int32, device=m.device)
    cnt = torch.empty((B, H, nb), dtype=torch.int32, device=m.device)
    missing = torch.zeros(1, dtype=torch.int32, device=m.device)
    _lib.check(lib.pbs_block_mask_to_csr(_ptr(m), _ptr(cols), _ptr(cnt), _ptr(missing), B * H, nb, blocks_per_segment,
                                         _stream()), "pbs_block_mask_to_csr")
    return cols, cnt, missing


def sparse_attn_fwd(q, perm_k, perm_vt, k, v, csr_cols, csr_cnt, segment_size, softmax_scale=None, out=None,
                    own_block_needed=None):
    """Attention of every query block over the permuted tiles listed in the CSR (earlier segments) and
    over the causal part of its own segment, read in place from the original ``k`` and ``v`` (B, Hkv or Hq, S, D).
    ``own_block_needed`` ((B, Hq, nb) uint8, one-block segments only) makes the diagonal block
    optional per query block."""
    _check_bf16_cuda(q, perm_k, perm_vt, k, v)
    lib = _lib.load()
    q, k, v = _rows16(q), _rows16(k), _rows16(v)
    B, Hq, S, D = q.shape
    Hkv = k.shape[1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    if out is None:
        out = torch.empty((B, Hq, S, D), dtype=q.dtype, device=q.device)
    nb = (S + BLOCK - 1) // BLOCK
    assert perm_k.is_contiguous() and perm_vt.is_contiguous()
    assert perm_k.shape == (B, Hq, nb * BLOCK, D) and perm_vt.shape == (B, Hq, nb, D, BLOCK)
    assert k.shape == (B, Hkv, S, D) and v.shape == (B, Hkv, S, D)
    assert csr_cols.is_contiguous() and csr_cnt.is_contiguous()
    assert csr_cols.shape == (B, Hq, nb, nb) and csr_cnt.shape == (B, Hq, nb)
    ws = torch.empty(max(lib.pbs_sparse_attn_workspace_bytes(B, Hq, S, segment_size), 256), dtype=torch.uint8, device=q.device)
    strides = (q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1), v.stride(2),
               out.stride(0), out.stride(1), out.stride(2))
    if own_block_needed is not None:
        if segment_size != BLOCK:
            raise ValueError("own_block_needed: only for one-block segments (segment_size == block_size)")
        assert own_block_needed.shape == (B, Hq, nb) and own_block_needed.dtype == torch.uint8 and own_block_needed.is_contiguous()
        _lib.check(lib.pbs_sparse_attn_fwd_optional_diagonal(
            _ptr(q), _ptr(perm_k), _ptr(perm_vt), _ptr(k), _ptr(v), _ptr(csr_cols), _ptr(csr_cnt), _ptr(own_block_needed),
            _ptr(out), B, Hq, Hkv, S, D, BLOCK, *strides, softmax_scale, _ptr(ws), _stream()), "pbs_sparse_attn_fwd_optional_diagonal")
        return out
    _lib.check(lib.pbs_sparse_attn_fwd(_ptr(q), _ptr(perm_k), _ptr(perm_vt), _ptr(k), _ptr(v), _ptr(csr_cols),
                                       _ptr(csr_cnt), _ptr(out), B, Hq, Hkv, S, D, BLOCK, segment_size, *strides,
                                       softmax_scale, _ptr(ws), _stream()),
               "pbs_sparse_attn_fwd")
    return out


def prefill_attn_fwd(q, k, v, block_size, segment_size, threshold, force_select_first_block=True,
                     query_pool_mode="mean", key_pool_mode="mean", softmax_scale=None):
    """Every stage in one library call (pbs.py:132-257): one workspace allocation, one
    host round trip.  Returns (B, Hq, S, D)."""
    _check_bf16_cuda(q, k, v)
    for mode, what in ((query_pool_mode, "query_pool_mode"), (key_pool_mode, "key_pool_mode")):
        if mode not in ("mean", "max"):
            raise ValueError(f"Invalid {what}: {mode}")
    lib = _lib.load()
    q, k, v = _rows16(q), _rows16(k), _rows16(v)
    B, Hq, S, D = q.shape
    Hkv = k.shape[1]
    if softmax_scale is None:
        softmax_scale = 1.0 / math.sqrt(D)
    is_int_one, thr_rows, thr = _threshold_args(threshold, B, Hq, q.device)
    if S > segment_size and segment_size // block_size > 511:
        raise _lib.PbsHipError(
            f"a segment of {segment_size // block_size} blocks exceeds the attention kernel's limit of 511: "
            f"use a smaller segment_size")
    out = torch.empty((B, Hq, S, D), dtype=q.dtype, device=q.device)
    ws_bytes = lib.pbs_prefill_attn_workspace_bytes(B, Hq, Hkv, S, D, block_size, segment_size)
    ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=q.device)
    _lib.check(lib.pbs_prefill_attn_fwd(
        _ptr(q), _ptr(k), _ptr(v), _ptr(out), B, Hq, Hkv, S, D, block_size, segment_size,
        q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
        v.stride(0), v.stride(1), v.stride(2), out.stride(0), out.stride(1), out.stride(2),
        thr, _ptr(thr_rows), int(is_int_one), int(bool(force_select_first_block)),
        int(query_pool_mode == "max"), int(key_pool_mode == "max"), softmax_scale,
        _ptr(ws), ws.numel(), _stream()), "pbs_prefill_attn_fwd")
    return out


def rope_qk(q, k, cos, sin):
    """Rotary embedding of q (B, Hq, S, D) and k (B, Hkv, S, D) with cos / sin (B or 1, S, D): the bits of
    ``x * cos + rotate_half(x) * sin`` in bf16 (pbs_attn/patch/huggingface.py:14-25), in one pass, returned
    contiguous and head-major."""
    _check_bf16_cuda(q, k, cos, sin)
    lib = _lib.load()
    q, k, cos, sin = _rows16(q), _rows16(k), _rows16(cos), _rows16(sin)
    B, Hq, S, D = q.shape
    Hkv = k.shape[1]
    assert k.shape == (B, Hkv, S, D) and cos.shape == sin.shape and cos.shape[-2:] == (S, D)
    assert cos.dim() == 3 and cos.shape[0] in (1, B) and cos.stride() == sin.stride()
    q_out = torch.empty((B, Hq, S, D), dtype=q.dtype, device=q.device)
    k_out = torch.empty((B, Hkv, S, D), dtype=q.dtype, device=q.device)
    c_sb = cos.stride(0) if cos.shape[0] == B and B > 1 else 0
    _lib.check(lib.pbs_rope_qk(_ptr(q), _ptr(k), _ptr(cos), _ptr(sin), _ptr(q_out), _ptr(k_out), B, Hq, Hkv, S, D,
                               q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
                               c_sb, cos.stride(1), _stream()), "pbs_rope_qk")
    return q_out, k_out


def unpermute(o_perm, q_idx=None, out=None):
    """out[b, h, q_idx[b, h, i]] = o_perm[b, h, i]; identity (no launch) when the
    queries were not permuted."""
    lib = _lib.load()
    if q_idx is None and out is None:
        out = o_perm
    o_perm = o_perm if (q_idx is None and out is o_perm) else o_perm.contiguous()
    if out is None:
        out = torch.empty_like(o_perm)
    B, H, S, D = o_perm.shape
    _lib.check(lib.pbs_unpermute(_ptr(o_perm), _ptr(q_idx), _ptr(out), B, H, S, D,
                                 out.stride(0), out.stride(1), out.stride(2), _stream()), "pbs_unpermute")
    return out
