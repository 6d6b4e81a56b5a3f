"""Plug-in boundary: swaps the prefill attention of Hugging Face Llama / Qwen2
decoder layers for a caller-supplied ``prefill_fn(q, k, v)``.

Same surface as the reference's pbs_attn/patch/huggingface.py:
``get_permuted_block_sparse_attn_fwd`` (:141-167), ``patched_attention_forward``
(:169-241), ``apply_patch_with_prefill`` (:243-307), ``is_model_supported`` /
``get_supported_model_types`` (:305-316).  Prompts (q_len > 1) go through
projections -> RoPE -> KV-cache update -> prefill_fn -> o_proj; single-token
decode steps go to the module's original forward.

Two extensions: a prefill function whose underlying python function carries
``native_gqa = True`` receives K/V at the KV-head count, which saves the
``repeat_kv`` copies (the PBS HIP path reads KV head h // group itself); and bf16
head-dim-128 prompts on the GPU get their rotary embedding from one HIP kernel
that produces the same bits as the tensor expression.
"""
from __future__ import annotations

import types
from functools import partial
from typing import Callable, Optional

import torch

SUPPORTED_MODEL_TYPES = ("LlamaForCausalLM", "Qwen2ForCausalLM")


# ---- rotary / GQA helpers (pbs_attn/patch/huggingface.py:14-37) ---------------

def rotate_half(x):
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rotary_pos_emb(q, k, cos, sin, position_ids=None, unsqueeze_dim=1):
    cos, sin = cos.unsqueeze(unsqueeze_dim), sin.unsqueeze(unsqueeze_dim)
    return q * cos + rotate_half(q) * sin, k * cos + rotate_half(k) * sin


def repeat_kv(hidden_states: torch.Tensor, n_rep: int) -> torch.Tensor:
    if n_rep == 1:
        return hidden_states
    b, h, s, d = hidden_states.shape
    return hidden_states.unsqueeze(2).expand(b, h, n_rep, s, d).reshape(b, h * n_rep, s, d)


# ---- prefill kernel factories --------------------------------------------------

def get_meanpooling_prefill(block_size=128, segment_size=1024, threshold=0.9,
                            force_select_first_block=True, force_select_current_block=True):
    """The un-permuted MeanPooling baseline (pbs_attn/patch/huggingface.py:43-58), through the PBS HIP kernels."""
    try:
        from pbs_attn_amd.meanpooling import MeanPooling_prefill as _MeanPooling_prefill
    except Exception as e:
        raise RuntimeError("MeanPooling unavailable.") from e
    return partial(
        _MeanPooling_prefill,
        block_size=block_size,
        segment_size=segment_size,
        threshold=threshold,
        causal=True,
        force_select_first_block=force_select_first_block,
        force_select_current_block=force_select_current_block,
    )


def _unavailable(name):
    # the reference builds these baselines on external CUDA packages (minference, block_sparse_attn, flash_attn)
    # and raises this error when the package is missing (pbs_attn/patch/huggingface.py:60-138); this build
    # never has them
    raise RuntimeError(f"{name} unavailable.")


def get_minference_prefill(vertical_size=1000, slash_size=6096, adaptive_budget=None):
    """pbs_attn/patch/huggingface.py:60-88: needs the `minference` CUDA package."""
    _unavailable("Minference")


def get_xattention_prefill(stride, norm=1, threshold=0.8, block_size=128, use_triton=True,
                           kdb=1, chunk_size=None, keep_sink=False, keep_recent=False):
    """pbs_attn/patch/huggingface.py:91-110: needs the `block_sparse_attn` CUDA package."""
    _unavailable("XAttention")


def get_flexprefill_prefill(gamma=0.9, tau=0, min_budget=None, max_budget=None,
                            gqa_interleave=False, softmax_scale=None, block_size=128):
    """pbs_attn/patch/huggingface.py:112-127: needs the `flash_attn` CUDA package."""
    _unavailable("FlexPrefill")


def get_flashattn_prefill(causal=True):
    """pbs_attn/patch/huggingface.py:129-138: needs the `flash_attn` CUDA package."""
    _unavailable("FlashAttn")



def get_permuted_block_sparse_attn_fwd(
    block_size=128,
    segment_size=256,
    threshold=0.9,
    causal=True,
    force_select_first_block=True,
    use_triton=True,
    query_pool_mode: str = "mean",
    key_pool_mode: str = "mean",
):
    """Returns ``functools.partial`` of the PBS attention forward with these settings."""
    try:
        from pbs_attn_amd.pbs import permuted_block_sparse_attn_fwd as impl
    except Exception as exc:  # pragma: no cover - import failure is environment specific
        raise RuntimeError("PBS unavailable.") from exc
    settings = dict(block_size=block_size, segment_size=segment_size, threshold=threshold, causal=causal,
                    force_select_first_block=force_select_first_block, use_triton=use_triton,
                    query_pool_mode=query_pool_mode, key_pool_mode=key_pool_mode)
    return partial(impl, **settings)


def _underlying(fn):
    return fn.func if isinstance(fn, partial) else fn


# ---- patched forward ------------------------------------------------------------

def _split_heads(x, bsz, q_len, head_dim):
    n_local = x.shape[-1] // head_dim            # local head count under tensor parallel
    return x.view(bsz, q_len, n_local, head_dim).transpose(1, 2), n_local


def _fused_rope_applies(q, k, cos, sin):
    return (q.is_cuda and q.dtype == torch.bfloat16 and k.dtype == q.dtype and cos.dtype == q.dtype
            and sin.dtype == q.dtype and q.shape[-1] == 128 and cos.dim() == 3 and cos.shape == sin.shape
            and cos.shape[0] in (1, q.shape[0]) and tuple(cos.shape[-2:]) == (q.shape[2], 128)
            and cos.stride() == sin.stride())


def patched_attention_forward(
    self,
    hidden_states: torch.Tensor,
    position_embeddings,
    attention_mask: Optional[torch.Tensor],
    past_key_values=None,
    cache_position: Optional[torch.LongTensor] = None,
    prefill_fn: Optional[Callable] = None,
    **kwargs,
):
    """Replacement for ``LlamaAttention.forward`` / ``Qwen2Attention.forward``."""
    bsz, q_len, _ = hidden_states.size()
    if q_len <= 1:
        return self.original_forward(hidden_states=hidden_states, position_embeddings=position_embeddings,
                                     attention_mask=attention_mask, past_key_values=past_key_values,
                                     cache_position=cache_position, **kwargs)

    q, n_q = _split_heads(self.q_proj(hidden_states), bsz, q_len, self.head_dim)
    k, n_kv = _split_heads(self.k_proj(hidden_states), bsz, q_len, self.head_dim)
    v, _ = _split_heads(self.v_proj(hidden_states), bsz, q_len, self.head_dim)

    cos, sin = position_embeddings
    if _fused_rope_applies(q, k, cos, sin):
        # same bits as apply_rotary_pos_emb, one kernel instead of ten, head-major contiguous outputs
        from pbs_attn_amd import ops
        q, k = ops.rope_qk(q, k, cos, sin)
    else:
        q, k = apply_rotary_pos_emb(q, k, cos, sin)
    if past_key_values is not None:
        past_key_values.update(k, v, self.layer_idx, {"sin": sin, "cos": cos, "cache_position": cache_position})

    if prefill_fn is None:
        raise RuntimeError("prefill_fn required.")
    kernel_fn = _underlying(prefill_fn)
    if not getattr(kernel_fn, "native_gqa", False):
        n_rep = max(1, n_q // max(1, n_kv))
        k, v = repeat_kv(k, n_rep), repeat_kv(v, n_rep)

    if "layer_idx" in kernel_fn.__code__.co_varnames:
        attn = prefill_fn(q, k, v, layer_idx=self.layer_idx)
    else:
        attn = prefill_fn(q, k, v)

    attn = attn.transpose(1, 2).reshape(bsz, q_len, n_q * self.head_dim)
    return self.o_proj(attn), None


# ---- patcher ----------------------------------------------------------------------

def get_supported_model_types():
    return list(SUPPORTED_MODEL_TYPES)


def is_model_supported(model):
    return type(model).__name__ in SUPPORTED_MODEL_TYPES


def _make_forward(prefill_fn):
    def new_forward(self, hidden_states, position_embeddings, attention_mask=None, past_key_values=None,
                    cache_position=None, **kwargs):
        return patched_attention_forward(self, hidden_states=hidden_states, position_embeddings=position_embeddings,
                                         attention_mask=attention_mask, past_key_values=past_key_values,
                                         cache_position=cache_position, prefill_fn=prefill_fn, **kwargs)
    return new_forward


def apply_patch_with_prefill(model, prefill_fn: Optional[Callable] = None, skip_layers: Optional[list] = None):
    """Monkey-patches every decoder layer's self-attention (except ``skip_layers``)
    so that prompts run through ``prefill_fn``.  Returns the model."""
    skip = set(skip_layers or [])
    if not is_model_supported(model):
        raise ValueError(f"Model type {type(model).__name__} is not supported. "
                         f"Supported types: {get_supported_model_types()}")
    layers = model.model.layers
    attn_type = type(layers[0].self_attn).__name__ if len(layers) > 0 else "Unknown"
    fn_name = _underlying(prefill_fn).__name__ if prefill_fn else "None"
    print(f"\nApplying monkey patch to {type(model).__name__} with {attn_type}")
    print(f"Prefill function: {fn_name}")
    if skip:
        print(f"Skipping layers: {sorted(skip)}")

    patched = 0
    for layer_idx, layer in enumerate(layers):
        if layer_idx in skip:
            print(f"  Skipping layer {layer_idx}")
            continue
        attn = layer.self_attn
        attn.original_forward = attn.forward
        attn.forward = types.MethodType(_make_forward(prefill_fn), attn)
        patched += 1
    print(f"Monkey patch applied. Patched {patched}/{len(layers)} layers.")
    return model
