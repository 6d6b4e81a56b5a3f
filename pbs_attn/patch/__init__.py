"""pbs_attn.patch alias package."""
