"""Seeded synthetic Q/K/V for the benchmark workloads.

All tensors are drawn in float32 from a ``torch.Generator`` on the requested
device, then cast to bf16.  K and V are produced at the KV-head count; the
query heads of a group share their KV head's heavy-hitter direction ``u``.

workloads
---------
``uniform_heavy``   2 % of key positions (uniform) get ``K += 3u``; every query
                    gets ``Q += 1.5u``.
``span_heavy``      1 % of key positions, clustered into 64 equal-length random
                    spans, get ``K += 3u``; every query gets ``Q += 1.5u``.
``local_window``    ``uniform_heavy`` plus a per-head local-window bias: one random
                    unit direction ``w_r`` per 512-token window r; ``Q_i += w_r(i)``
                    and ``K_j += w_r(j)`` so same-window pairs gain about +1 in
                    the logit before the 1/sqrt(D) scale.
``strong_heavy``    ``uniform_heavy`` with a 10x stronger signal (K += 30u,
                    Q += 15u) clustered in spans: the supplementary input on
                    which permutation visibly raises block sparsity.
``strong_uniform``  the 10x signal on 2 % of the key positions drawn uniformly (no spans):
                    every 128-key block holds a few heavy keys, so without the
                    permutation no block stands out; sorting inside a segment moves
                    them into the segment's first block.
"""
from __future__ import annotations

import torch

WORKLOADS = {
    # name: (B, Hq, Hkv, S, D, generator kind, block, segment, threshold)
    "cfg0": dict(B=1, Hq=32, Hkv=8, S=4096, D=128, kind="uniform_heavy", block=128, segment=256, threshold=0.9),
    "cfg1": dict(B=1, Hq=32, Hkv=8, S=32768, D=128, kind="uniform_heavy", block=128, segment=256, threshold=0.9),
    "cfg2": dict(B=1, Hq=32, Hkv=8, S=131072, D=128, kind="span_heavy", block=128, segment=1024, threshold=0.9),
    "cfg3": dict(B=4, Hq=28, Hkv=4, S=16384, D=128, kind="local_window", block=128, segment=256, threshold=0.9),
}


def _unit(shape, gen, device):
    x = torch.randn(shape, generator=gen, device=device, dtype=torch.float32)
    return x / x.norm(dim=-1, keepdim=True)


def make_qkv(B, Hq, Hkv, S, D, kind="uniform_heavy", seed=0, device="cpu", dtype=torch.bfloat16):
    """Returns q (B, Hq, S, D), k, v (B, Hkv, S, D)."""
    assert Hq % Hkv == 0
    G = Hq // Hkv
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    pos_gen = torch.Generator(device="cpu")
    pos_gen.manual_seed(seed + 1)

    q = torch.randn((B, Hkv, G, S, D), generator=gen, device=device, dtype=torch.float32)
    k = torch.randn((B, Hkv, S, D), generator=gen, device=device, dtype=torch.float32)
    v = torch.randn((B, Hkv, S, D), generator=gen, device=device, dtype=torch.float32)
    u = _unit((B, Hkv, D), gen, device)

    heavy = torch.zeros(S, dtype=torch.bool)
    if kind in ("uniform_heavy", "local_window", "strong_uniform"):
        n = max(1, int(round(0.02 * S)))
        heavy[torch.randperm(S, generator=pos_gen)[:n]] = True
        kq_gain = (30.0, 15.0) if kind == "strong_uniform" else (3.0, 1.5)
    elif kind in ("span_heavy", "strong_heavy"):
        n_spans = min(64, max(1, S // 128))
        span = max(1, int(round(0.01 * S / n_spans)))
        starts = torch.randint(0, max(1, S - span), (n_spans,), generator=pos_gen)
        for st in starts.tolist():
            heavy[st:st + span] = True
        kq_gain = (3.0, 1.5) if kind == "span_heavy" else (30.0, 15.0)
    else:
        raise ValueError(f"unknown workload kind: {kind}")
    heavy = heavy.to(device)

    k += kq_gain[0] * heavy.view(1, 1, S, 1).float() * u.view(B, Hkv, 1, D)
    q += kq_gain[1] * u.view(B, Hkv, 1, 1, D)

    if kind == "local_window":
        win = 512
        n_win = (S + win - 1) // win
        w = _unit((B, Hkv, n_win, D), gen, device)
        wpos = (torch.arange(S, device=device) // win)
        wk = w[:, :, wpos, :]                       # (B, Hkv, S, D)
        k += wk
        q += wk.unsqueeze(2)

    q = q.reshape(B, Hq, S, D).to(dtype)
    return q, k.to(dtype), v.to(dtype)


def make_workload(name, seed=0, device="cpu", **override):
    cfg = dict(WORKLOADS[name])
    cfg.update(override)
    q, k, v = make_qkv(cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["S"], cfg["D"], cfg["kind"], seed, device)
    return cfg, q, k, v
