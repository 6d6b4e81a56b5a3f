"""Alias of pbs_attn_amd.meanpooling under the reference's module path."""
from pbs_attn_amd.meanpooling import MeanPooling_prefill  # noqa: F401
