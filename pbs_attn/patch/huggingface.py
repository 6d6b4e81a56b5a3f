"""Alias of pbs_attn_amd.patch.huggingface under the reference's module path."""
from pbs_attn_amd.patch.huggingface import *  # noqa: F401,F403
from pbs_attn_amd.patch.huggingface import (  # noqa: F401
    apply_patch_with_prefill,
    get_permuted_block_sparse_attn_fwd,
    get_supported_model_types,
    is_model_supported,
    patched_attention_forward,
)
