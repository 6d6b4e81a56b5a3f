"""The reference's module path pbs_attn.src.permute_states."""
from pbs_attn_amd.compat import apply_permutation, last_block_attn_sorting  # noqa: F401
