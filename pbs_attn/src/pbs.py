"""Alias of pbs_attn_amd.pbs under the reference's module path."""
from pbs_attn_amd.pbs import (  # noqa: F401
    apply_permutation,
    permuted_block_selection,
    permuted_block_sparse_attn_fwd,
)
