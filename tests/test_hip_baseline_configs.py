"""GPU: BASELINE.json's configurations 1, 2 and 3 at their OWN parameters (shape, head grouping, generator,
segment size, threshold), the whole path as the benchmark runs it: the single-call entry point against the staged
path, the selection invariants on every head, the visit lists and the key blocks marked for the filtered gather
against the masks, sampled query blocks against dense float32 attention on the path's own mask, and the key
scores / key order of some heads against the CPU oracle."""
import math

import pytest
import torch

from oracle import pbs_oracle as O
from pbs_attn_amd import ops
from pbs_attn_amd import pbs as P
from pbs_attn_amd.synth import make_workload
from tests.util import assert_attn_close

pytestmark = pytest.mark.gpu


class _NullTimer:
    def mark(self, name):
        pass


def _check_selection(Pm, chosen, final, cnt, cols, needed, first_col, thr, nb, bps, dev):
    """The invariants of utils.py:38-86 + pbs.py:119-127,209 on every (batch, head, query block) row."""
    B, H = Pm.shape[:2]
    qb = torch.arange(nb, device=dev)
    cand = (qb.view(1, -1) // bps) < (qb.view(-1, 1) // bps)
    own = (qb.view(1, -1) // bps) == (qb.view(-1, 1) // bps)
    assert torch.isnan(Pm[:, :, :bps]).all() and not torch.isnan(Pm[:, :, bps:]).any()
    assert (torch.nan_to_num(Pm, nan=0.0)[..., ~cand] == 0).all()
    forced = torch.zeros_like(chosen)
    forced.scatter_(-1, first_col.view(B, H, 1, 1).expand(B, H, nb, 1), True)   # the block of token 0, every row
    by_threshold = chosen & ~forced
    assert not (by_threshold & ~cand).any()                 # the threshold only ever selects candidates
    assert (chosen & forced).eq(forced).all()               # the first-token block is in every row
    assert torch.equal(final, chosen | own)
    # `chosen` is the threshold's minimal descending prefix T united with the forced block; where that block is a
    # candidate T is either `chosen` without it or with it: one of the two must satisfy the prefix invariants
    def prefix_ok(Pz, pick):
        mass = (Pz * pick).sum(-1)
        smallest = torch.where(pick, Pz, torch.full_like(Pz, 2.0)).min(-1).values
        largest_out = torch.where(cand & ~pick, Pz, torch.full_like(Pz, -1.0)).max(-1).values
        return ((mass >= thr - 1e-5)                       # the threshold is reached ...
                & (mass - smallest < thr + 1e-5)           # ... and not without the smallest selected block
                & (largest_out <= smallest + 1e-12))       # a descending prefix
    for b in range(B):
        for h0 in range(0, H, 8):                           # float64 copies of a few heads at a time
            hs = slice(h0, min(h0 + 8, H))
            Pz = torch.nan_to_num(Pm[b, hs], nan=0.0).double()
            without = by_threshold[b, hs]
            ok = prefix_ok(Pz, without) | prefix_ok(Pz, without | (forced[b, hs] & cand))
            assert ok[:, bps:].all(), (b, h0, (~ok[:, bps:]).nonzero()[:5])
    visited = chosen & cand
    assert torch.equal(cnt, visited.sum(-1).int())
    # the visit list of every row: ascending, exactly the selected blocks of earlier segments
    valid = torch.arange(nb, device=dev).view(1, 1, 1, nb) < cnt.unsqueeze(-1)
    listed = torch.zeros(chosen.shape, dtype=torch.int32, device=dev)
    listed.scatter_add_(-1, torch.where(valid, cols, torch.zeros_like(cols)).long(), valid.int())
    assert torch.equal(listed, visited.int())              # every listed block once, nothing else
    c = torch.where(valid, cols, torch.full_like(cols, nb))
    assert (c[..., 1:] >= c[..., :-1]).all()
    assert torch.equal(needed.bool(), visited.any(-2))      # marked for the gather <=> on some query block's list


def _assert_close_with_large_values(out, ref, what):
    """max-abs 2e-2 / mean-abs 2e-3, except that an element whose reference value is large may be off by 1.5 units in
    the last place of bf16 (the rule of the random-configuration sweep: the strong_heavy inputs produce outputs beyond
    +-4, where one bf16 step is 0.031 and the rounding of the output alone can take 0.016)."""
    diff = (out.float() - ref.float()).abs()
    assert torch.isfinite(out.float()).all(), what
    ulp = torch.exp2(torch.floor(torch.log2(ref.abs().clamp_min(1e-30))) - 7)
    assert (diff <= torch.maximum(torch.full_like(diff, 2e-2), 1.5 * ulp)).all(), (what, diff.max().item())
    assert diff.mean().item() <= 2e-3, (what, diff.mean().item())


def _check_config(dev, name, sample_blocks, oracle_heads, large_outputs=False, **override):
    cfg, q, k, v = make_workload(name, device=dev, **override)
    B, Hq, Hkv, S, seg, thr = cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["S"], cfg["segment"], cfg["threshold"]
    nb, bps, G = S // 128, seg // 128, Hq // Hkv
    # the product path (one library call) against the same work stage by stage: the same bits
    assert P.stage_timer is None
    one = P.permuted_block_sparse_attn_fwd(q, k, v, 128, seg, thr, True)
    P.stage_timer = _NullTimer()
    try:
        staged = P.permuted_block_sparse_attn_fwd(q, k, v, 128, seg, thr, True)
    finally:
        P.stage_timer = None
    assert torch.equal(one, staged)
    assert torch.isfinite(one.float()).all()
    del staged
    # the stages once more, keeping what they produce
    perm, sel = P._select_then_gather(q, k, v, 128, seg, thr, True, "mean", "mean")
    assert torch.equal(perm.attention(q, sel["csr_cols"], sel["csr_cnt"], seg), one)
    idx = perm.key_indices
    chosen, final, cols, cnt = ops.select_blocks(sel["block_attn_scores"], thr, idx, S, 128, seg, True, candidate_rule=1)
    assert torch.equal(cnt, sel["csr_cnt"])
    first_col = (idx[:, :, :S] == 0).int().argmax(-1) // 128
    _check_selection(sel["block_attn_scores"], chosen, final, cnt, cols, sel["block_needed"], first_col, thr, nb, bps, dev)
    density = (int(cnt.sum()) + sum(min(qb % bps, nb) + 1 for qb in range(nb)) * B * Hq) / (B * Hq * nb * (nb + 1) / 2)
    print(f"\n{name} {override}: density of executed tiles {density:.4f}")
    # a permutation of every segment's own range
    srt = idx[:, :, :S].long().view(B, Hq, -1, seg).sort(-1).values
    assert torch.equal(srt, torch.arange(S, device=dev).view(1, 1, -1, seg).expand_as(srt))

    # sampled query blocks, every head: dense float32 attention over the ORIGINAL K / V with the path's own mask
    # carried to original key positions (key j sits in permuted block pos_of_key[j] // 128)
    pos_of_key = torch.empty_like(idx, dtype=torch.int64)
    pos_of_key.scatter_(-1, idx.long(), torch.arange(idx.shape[-1], device=dev).expand_as(idx))
    key_block = pos_of_key[:, :, :S] // 128
    pos = torch.arange(S, device=dev)
    worst = 0.0
    for qb in sample_blocks:
        rows = slice(qb * 128, qb * 128 + 128)
        for h0 in range(0, Hq, G):                          # one KV group at a time
            hs = slice(h0, h0 + G)
            kf = k[:, h0 // G].float().unsqueeze(1)
            vf = v[:, h0 // G].float().unsqueeze(1)
            logits = q[:, hs, rows].float() @ kf.transpose(-1, -2) / math.sqrt(128)
            allowed = torch.gather(final[:, hs, qb], -1, key_block[:, hs]).unsqueeze(2) & (pos.view(1, 1, 1, S) <= pos[rows].view(1, 1, -1, 1))
            ref = torch.softmax(logits.masked_fill(~allowed, float("-inf")), -1) @ vf
            what = f"{name}: query block {qb}, heads {h0}..{h0 + G - 1}"
            if large_outputs:
                _assert_close_with_large_values(one[:, hs, rows], ref, what)
            else:
                assert_attn_close(one[:, hs, rows], ref, what=what)
            worst = max(worst, (one[:, hs, rows].float() - ref).abs().max().item())
    print(f"{name}: {len(sample_blocks)} query blocks x {B * Hq} heads against dense fp32 on the path's mask: max-abs {worst:.2e}")

    # key scores and key order of some heads against the CPU oracle (permute_states.py:44-56)
    scores = ops.score_keys(q, k, 128, seg)
    agree = []
    for (b, h) in oracle_heads:
        ref = O.key_scores(q[b:b + 1, h:h + 1].cpu(), k[b:b + 1, h // G:h // G + 1].cpu(), 128, seg)[0, 0]
        got = scores[b, h].cpu()
        rel = ((got - ref).abs() / ref.clamp_min(1e-30))
        print(f"{name}: key scores of head {(b, h)} against the oracle: max rel {rel.max():.2e}, mean rel {rel.mean():.2e}")
        assert rel.max() < 3e-2 and rel.mean() < 2e-3, (rel.max(), rel.mean())
        ref_idx = O.segment_argsort(ref.view(1, 1, -1), S, seg)[0, 0]
        agree.append((idx[b, h, :S].cpu().long() == ref_idx).float().mean().item())
        # the sort itself is exact: the oracle's order of the HIP scores is the HIP order
        assert torch.equal(O.segment_argsort(got.view(1, 1, -1), S, seg)[0, 0], idx[b, h, :S].cpu().long())
    print(f"{name}: key-index agreement with the oracle at S={S} on heads {oracle_heads}: {['%.4f' % a for a in agree]}")
    assert min(agree) > 0.9


def test_cfg2_at_its_own_parameters(dev):
    # S = 131072, 32 / 8 heads, segment 1024, threshold 0.9, span_heavy: the headline configuration
    _check_config(dev, "cfg2", sample_blocks=(8, 517, 1023), oracle_heads=[(0, 0), (0, 21)])


def test_cfg3_at_its_own_parameters(dev):
    # batch 4, 28 / 4 heads (7:1), S = 16384, local_window, segment 256
    _check_config(dev, "cfg3", sample_blocks=(2, 77, 127), oracle_heads=[(0, 0), (3, 27)])


def test_cfg1_full_layer_threshold_09_segment_1024(dev):
    # the 32-head layer at 32k, and the (0.9, 1024) cell of config 1's sweep
    _check_config(dev, "cfg1", sample_blocks=(9, 130, 255), oracle_heads=[(0, 5)], segment=1024)


def test_cfg1_full_layer_segment_256(dev):
    _check_config(dev, "cfg1", sample_blocks=(1, 200), oracle_heads=[(0, 30)])


def test_cfg2_shape_in_the_sparse_regime(dev):
    # the supplementary strong_heavy input at cfg2's shape and parameters: 1.5 % of the causal blocks, 2 % of the
    # permuted key blocks gathered, rows decided without a sort, items of 8 tiles
    _check_config(dev, "cfg2", sample_blocks=(8, 517, 1023), oracle_heads=[(0, 3)], large_outputs=True, kind="strong_heavy")
