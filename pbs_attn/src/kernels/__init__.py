"""pbs_attn.src.kernels alias package."""
