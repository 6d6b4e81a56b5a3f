"""pbs_attn.src alias package."""
