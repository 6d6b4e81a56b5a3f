"""The operator as a PyTorch custom op: ``torch.ops.pbs_hip.prefill_attn_fwd``.

Registers the whole-path library call (``ops.prefill_attn_fwd`` -> ``pbs_prefill_attn_fwd`` of libpbs_hip.so,
the replacement of pbs_attn/src/pbs.py:132-257) with the dispatcher: a schema, the GPU implementation and a
shape-only implementation for tracing (fake / meta tensors), so that graph capture tools (``torch.compile``,
``torch.export``) see one opaque node instead of ctypes calls.  There is no CPU implementation: CPU tensors
fail in the dispatcher.  The threshold is split into the three forms the reference's argument can take: a
float, the python int 1 (``threshold_is_int_one``), or a per-head tensor (``threshold_per_head``, (B, Hq)).

    import pbs_attn_amd.torch_ops            # registers the op
    out = torch.ops.pbs_hip.prefill_attn_fwd(q, k, v, 128, 256, 0.9, False, None, True, "mean", "mean")
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops

_LIB = torch.library.Library("pbs_hip", "DEF")
_LIB.define(
    "prefill_attn_fwd(Tensor q, Tensor k, Tensor v, int block_size, int segment_size, float threshold, "
    "bool threshold_is_int_one, Tensor? threshold_per_head, bool force_select_first_block, "
    "str query_pool_mode, str key_pool_mode) -> Tensor")


def _threshold(threshold: float, is_int_one: bool, per_head: Optional[torch.Tensor]):
    if is_int_one:
        return 1
    return per_head if per_head is not None else float(threshold)


def _prefill_attn_fwd_gpu(q, k, v, block_size, segment_size, threshold, threshold_is_int_one, threshold_per_head,
                          force_select_first_block, query_pool_mode, key_pool_mode):
    return ops.prefill_attn_fwd(q, k, v, block_size, segment_size,
                                _threshold(threshold, threshold_is_int_one, threshold_per_head),
                                force_select_first_block, query_pool_mode, key_pool_mode)


_LIB.impl("prefill_attn_fwd", _prefill_attn_fwd_gpu, "CUDA")


@torch.library.register_fake("pbs_hip::prefill_attn_fwd")
def _prefill_attn_fwd_fake(q, k, v, block_size, segment_size, threshold, threshold_is_int_one, threshold_per_head,
                           force_select_first_block, query_pool_mode, key_pool_mode):
    torch._check(q.dim() == 4 and k.dim() == 4 and v.dim() == 4, lambda: "q, k, v must be (B, H, S, D)")
    torch._check(q.shape[1] % k.shape[1] == 0, lambda: "query heads must be a multiple of the KV heads")
    torch._check(k.shape == v.shape and q.shape[2] == k.shape[2], lambda: "prefill only: q_len == kv_len")
    return torch.empty(q.shape, dtype=q.dtype, device=q.device)


def prefill_attn_fwd(q, k, v, block_size=128, segment_size=256, threshold=0.9, force_select_first_block=True,
                     query_pool_mode="mean", key_pool_mode="mean"):
    """Same arguments as ``ops.prefill_attn_fwd``, routed through the dispatcher."""
    is_one = isinstance(threshold, int) and threshold == 1
    per_head = threshold if isinstance(threshold, torch.Tensor) else None
    scalar = 0.0 if (is_one or per_head is not None) else float(threshold)
    return torch.ops.pbs_hip.prefill_attn_fwd(q, k, v, block_size, segment_size, scalar, is_one, per_head,
                                              force_select_first_block, query_pool_mode, key_pool_mode)
