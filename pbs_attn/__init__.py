"""Import-path alias: ``pbs_attn`` is the name the reference package is used under
(README.md:47, pbs_attn/__init__.py:4).  The implementation lives in pbs_attn_amd."""
from pbs_attn_amd.pbs import permuted_block_sparse_attn_fwd  # noqa: F401
