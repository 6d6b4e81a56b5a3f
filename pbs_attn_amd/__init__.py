"""MI355X-native PBS-Attn prefill attention (hand-written gfx950 HIP kernels)."""
from .pbs import permuted_block_sparse_attn_fwd  # noqa: F401

__all__ = ["permuted_block_sparse_attn_fwd"]
