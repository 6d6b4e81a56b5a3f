"""The reference's module path pbs_attn.src.utils."""
from pbs_attn_amd.compat import block_pooled_attn, select_blocks  # noqa: F401
