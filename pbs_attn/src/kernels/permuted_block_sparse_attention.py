"""The reference's module path pbs_attn.src.kernels.permuted_block_sparse_attention (imported by its
pbs_attn/src/pbs.py:6): the attention stage under its two names, both on the HIP attention kernel."""
from pbs_attn_amd.compat import permuted_block_sparse_attn_kernel as _permuted_block_sparse_attn_fwd  # noqa: F401
from pbs_attn_amd.compat import sparse_attention_on_block_mask as _permuted_block_sparse_attn_fwd_torch_naive  # noqa: F401
