"""Shared helpers for the parity tests."""
import math

import torch

from pbs_attn_amd.synth import make_qkv


def small_case(B=1, Hq=4, Hkv=2, S=1024, D=128, kind="uniform_heavy", seed=0):
    return make_qkv(B, Hq, Hkv, S, D, kind=kind, seed=seed, device="cpu")


def expand_kv(q, x):
    from oracle.pbs_oracle import repeat_kv
    return repeat_kv(x, q.shape[1] // x.shape[1])


def assert_attn_close(out, ref, max_abs=2e-2, mean_abs=2e-3, what=""):
    """North-star tolerance for bf16 attention outputs."""
    diff = (out.float().cpu() - ref.float().cpu()).abs()
    assert torch.isfinite(out.float()).all(), f"{what}: non-finite output"
    assert diff.max().item() <= max_abs, f"{what}: max-abs {diff.max().item():.4g} > {max_abs}"
    assert diff.mean().item() <= mean_abs, f"{what}: mean-abs {diff.mean().item():.4g} > {mean_abs}"


def quantised_scores(shape, levels, seed):
    """Random scores on a coarse grid: plenty of exact ties."""
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, levels, shape, generator=g).float() / levels
