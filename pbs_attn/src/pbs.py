"""The reference's module path pbs_attn.src.pbs: the attention forward, and the stage functions with the
reference's signatures."""
from pbs_attn_amd.compat import apply_permutation, first_token_mask, permuted_block_selection  # noqa: F401
from pbs_attn_amd.pbs import permuted_block_sparse_attn_fwd  # noqa: F401
