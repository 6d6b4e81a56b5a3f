"""Alias of pbs_attn_amd.patch.huggingface under the reference's module path."""
from pbs_attn_amd.patch.huggingface import *  # noqa: F401,F403
from pbs_attn_amd.patch.huggingface import (  # noqa: F401
    apply_patch_with_prefill,
    get_flashattn_prefill,
    get_flexprefill_prefill,
    get_meanpooling_prefill,
    get_minference_prefill,
    get_permuted_block_sparse_attn_fwd,
    get_supported_model_types,
    get_xattention_prefill,
    is_model_supported,
    patched_attention_forward,
)
