"""Pins the CPU oracle: closed forms in float64, brute force on small inputs,
library routines for the special cases, invariants, and the independent
pure-python vectors under tests/golden.  No GPU."""
import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import pbs_oracle as O
from tests.util import assert_attn_close, expand_kv, quantised_scores, small_case

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "tiny_pipeline.json")


# ------------------------------------------------------------------ key scores
def test_key_scores_closed_form_fp64():
    q, k, _ = small_case(1, 2, 1, 768, seed=1)
    seg = 256
    got = O.key_scores(q, k, 128, seg)
    ke = expand_kv(q, k).double()
    logits = q.double()[:, :, -128:] @ ke.transpose(-1, -2) / math.sqrt(128)
    ref = torch.softmax(logits, -1).mean(-2)
    assert got.dtype == torch.float32 and got.shape == (1, 2, 768)
    assert torch.allclose(got.sum(-1), torch.ones(1, 2), atol=1e-4)
    rel = (got.double() - ref).abs() / ref
    assert rel.max() < 3e-2 and rel.mean() < 3e-3      # logits are rounded to bf16 twice


def test_key_scores_ignore_partial_segment_and_use_last_block():
    q, k, _ = small_case(1, 1, 1, 700, seed=2)
    s = O.key_scores(q, k, 128, 256)
    assert s.shape[-1] == 512
    # only the last 128 queries matter
    q2 = q.clone()
    q2[:, :, :-128] = 0
    assert torch.equal(O.key_scores(q2, k, 128, 256), s)
    # keys of the partial segment do not take part in the softmax
    k2 = k.clone()
    k2[:, :, 512:] += 5
    assert torch.equal(O.key_scores(q, k2, 128, 256), s)


# ------------------------------------------------------------------ segment sort
@pytest.mark.parametrize("S,seg", [(64, 16), (70, 16), (48, 48), (100, 32)])
def test_segment_argsort_bruteforce_with_ties(S, seg):
    sc = (S // seg) * seg
    scores = quantised_scores((2, 2, sc), levels=5, seed=S)
    idx = O.segment_argsort(scores, S, seg)
    for b in range(2):
        for h in range(2):
            want = []
            for s0 in range(0, sc, seg):
                want += sorted(range(s0, s0 + seg), key=lambda j: (-scores[b, h, j].item(), j))
            want += list(range(sc, S))
            assert idx[b, h].tolist() == want


def test_gather_rows_explicit():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((2, 2, 10, 3), generator=g)
    idx = torch.stack([torch.stack([torch.randperm(10, generator=g) for _ in range(2)]) for _ in range(2)])
    got = O.gather_rows(x, idx)
    for b in range(2):
        for h in range(2):
            for i in range(10):
                assert torch.equal(got[b, h, i], x[b, h, idx[b, h, i]])


def test_no_permutation_cases():
    q, k, _ = small_case(1, 2, 2, 256, seed=3)
    pk, idx = O.last_block_attn_sorting(q, k, 128, 256)       # exactly one segment
    assert torch.equal(pk, k) and torch.equal(idx[0, 0], torch.arange(256))
    pk, idx = O.last_block_attn_sorting(q[:, :, :200], k[:, :, :200], 128, 256)   # none complete
    assert torch.equal(idx[0, 0], torch.arange(200))
    _, idx = O.last_block_attn_sorting(*small_case(1, 1, 1, 300, seed=4)[:2], 128, 256)   # one + remainder: sorts
    assert not torch.equal(idx[0, 0, :256], torch.arange(256))
    assert torch.equal(idx[0, 0, 256:], torch.arange(256, 300))


# ------------------------------------------------------------------ masks
def test_candidate_and_segment_masks_closed_form():
    cand, segm = O.candidate_masks(7, 3)
    for qb in range(7):
        for kb in range(7):
            assert segm[qb, kb].item() == (qb // 3 == kb // 3)
            assert cand[qb, kb].item() == (kb // 3 < qb // 3)


def test_first_token_mask_bruteforce():
    g = torch.Generator().manual_seed(5)
    idx = torch.stack([torch.randperm(32, generator=g) for _ in range(6)]).view(2, 3, 32)
    m = O.first_token_mask(idx, 4)
    assert m.shape == (2, 3, 1, 8)
    for b in range(2):
        for h in range(3):
            blk = idx[b, h].tolist().index(0) // 4
            assert m[b, h, 0].tolist() == [i == blk for i in range(8)]


# ------------------------------------------------------------------ block probabilities
@pytest.mark.parametrize("mode", ["mean", "max"])
def test_block_pooled_attn_textbook(mode):
    q, k, _ = small_case(1, 2, 2, 1024, seed=6)
    cand, _ = O.candidate_masks(8, 2)
    got = O.block_pooled_attn(q, k, 128, cand, mode, mode)
    red = (lambda x: x.mean(-2)) if mode == "mean" else (lambda x: x.max(-2).values)
    pq = red(q.double().view(1, 2, 8, 128, 128))
    pk = red(k.double().view(1, 2, 8, 128, 128))
    dots = pq @ pk.transpose(-1, -2)
    assert torch.isnan(got[:, :, :2]).all()                   # segment 0 has no candidate
    if mode == "mean":
        ref = torch.softmax((dots / math.sqrt(128)).masked_fill(~cand, float("-inf")), -1)
        assert torch.allclose(got[:, :, 2:].double(), ref[:, :, 2:], rtol=5e-2, atol=1e-4)
    else:
        # max-pooled logits are ~70: one bf16 ulp is 0.5, so apply the two bf16 roundings the
        # path makes (matmul output, then the divide) to the float64 dot products
        lg = (dots.float().bfloat16().float() / torch.tensor(math.sqrt(128), dtype=torch.float32)).bfloat16().double()
        ref = torch.softmax(lg.masked_fill(~cand, float("-inf")), -1)
        close = torch.isclose(got[:, :, 2:].double(), ref[:, :, 2:], rtol=1e-3, atol=1e-6)
        assert close.float().mean() > 0.9     # a rare rounding flip of one logit moves its whole row
    assert (got[:, :, 2:][..., ~cand[2:]] == 0).all()
    with pytest.raises(ValueError):
        O.block_pooled_attn(q, k, 128, cand, "median", "mean")


# ------------------------------------------------------------------ selection
def _select_bruteforce(row, thr32):
    order = sorted(range(len(row)), key=lambda i: (-row[i], i))
    c = np.float64(0.0)
    for rank, i in enumerate(order):
        c = c + np.float64(row[i])
        if np.float32(c) >= thr32:
            return set(order[:rank + 1])
    return set()


@pytest.mark.parametrize("thr", [0.0, 0.3, 0.9, 0.95, 1.0])
def test_select_blocks_bruteforce_and_invariants(thr):
    g = torch.Generator().manual_seed(7)
    logits = (torch.randn((2, 2, 12, 40), generator=g) * 2).bfloat16().float()     # ties
    p = torch.softmax(logits, -1)
    p[0, 0, 0] = float("nan")
    p[0, 0, 1] = 0.0
    sel = O.select_blocks(p, thr)
    thr32 = np.float32(thr)
    pn = torch.nan_to_num(p, nan=0.0)
    for b in range(2):
        for h in range(2):
            for r in range(12):
                want = _select_bruteforce([np.float32(x) for x in pn[b, h, r].tolist()], thr32)
                got = set(torch.where(sel[b, h, r])[0].tolist())
                assert got == want
                if want and thr > 0:
                    vals = sorted((pn[b, h, r, i].item() for i in want), reverse=True)
                    assert sum(vals) >= thr - 1e-5
                    assert sum(vals[:-1]) < thr + 1e-5       # minimal prefix
    assert sel[0, 0, 0].sum() == (1 if thr <= 0 else 0) and sel[0, 0, 1].sum() == (1 if thr <= 0 else 0)


def test_select_blocks_tensor_threshold_and_fp32_compare():
    p = torch.tensor([0.5, 0.25, 0.125, 0.125]).view(1, 1, 1, 4).repeat(1, 2, 1, 1)
    thr = torch.tensor([[0.75, 0.76]])
    sel = O.select_blocks(p, thr)
    assert sel[0, 0, 0].tolist() == [True, True, False, False]
    assert sel[0, 1, 0].tolist() == [True, True, True, False]
    # the comparison is made in float32: float32(0.9) <= 0.9 as a float32 prefix
    a, b = np.float32(0.9), np.float32(0.9) - np.float32(0.5)
    p2 = torch.tensor([0.5, float(b), 0.05]).view(1, 1, 1, 3)
    assert np.float32(np.float64(0.5) + np.float64(b)) == a
    assert O.select_blocks(p2, 0.9)[0, 0, 0].tolist() == [True, True, False]


def test_cumsum_is_sequential_fp64_rounded_per_prefix():
    g = torch.Generator().manual_seed(8)
    x = torch.softmax(torch.randn((64, 1000), generator=g) * 3, -1).sort(-1, descending=True).values
    seq = np.cumsum(x.numpy().astype(np.float64), -1).astype(np.float32)
    assert np.array_equal(torch.cumsum(x.double(), -1).float().numpy(), seq)
    assert np.array_equal(torch.cumsum(x, -1).numpy(), seq)      # what torch's CPU cumsum does on float32


# ------------------------------------------------------------------ attention
def test_naive_path_matches_dense_fp32_oracle():
    q, k, v = small_case(1, 2, 1, 1024, seed=9)
    ke, ve = expand_kv(q, k), expand_kv(q, v)
    out, mid = O.permuted_block_sparse_attn_fwd(q, ke, ve, 128, 256, 0.9, return_intermediates=True)
    dense = O.dense_masked_attention_fp32(q, mid["perm_k"], mid["perm_v"], mid["key_indices"], mid["final_mask"], 128)
    d = (out.float() - dense).abs()
    assert d.max() < 3e-2 and d.mean() < 2e-3


@pytest.mark.parametrize("S,seg", [(1024, 256), (1000, 256), (640, 512), (200, 256), (256, 256)])
def test_threshold_int_one_is_dense_causal(S, seg):
    q, k, v = small_case(1, 2, 2, S, seed=S)
    out = O.permuted_block_sparse_attn_fwd(q.float(), k.float(), v.float(), 128, seg, 1)
    ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    assert torch.allclose(out, ref, atol=2e-5)


def test_float_one_selects_fewer_blocks_than_int_one():
    q, k, v = small_case(1, 2, 2, 1024, seed=10)
    _, a = O.permuted_block_sparse_attn_fwd(q, k, v, 128, 256, 1, return_intermediates=True)
    _, b = O.permuted_block_sparse_attn_fwd(q, k, v, 128, 256, 1.0, return_intermediates=True)
    assert (b["final_mask"] & ~a["final_mask"]).sum() == 0
    assert a["final_mask"].sum() >= b["final_mask"].sum()


def test_one_hot_values_recover_attention_weights():
    # V = identity rows: the output IS the attention weight matrix over permuted key positions
    S, bs, seg = 16, 2, 4
    g = torch.Generator().manual_seed(11)
    q = torch.randn((1, 1, S, S), generator=g)
    k = torch.randn((1, 1, S, S), generator=g)
    v = torch.eye(S).view(1, 1, S, S)
    out, mid = O.permuted_block_sparse_attn_fwd(q, k, v, bs, seg, 0.7, return_intermediates=True)
    idx, fm = mid["key_indices"][0, 0], mid["final_mask"][0, 0]
    assert torch.allclose(out.sum(-1), torch.ones(1, 1, S), atol=1e-5)
    for qi in range(S):
        for pos in range(S):
            allowed = fm[qi // bs, pos // bs] and idx[pos] <= qi
            w = out[0, 0, qi, idx[pos]]        # weight on the key whose ORIGINAL position is idx[pos]
            assert (w > 0) == bool(allowed)


def test_visited_block_pairs():
    fm = torch.ones((1, 1, 4, 4), dtype=torch.bool)
    assert O.visited_block_pairs(fm, 2) == 2 * 2 + 2 * 4


# ------------------------------------------------------------------ independent pure-python vectors
def test_against_pure_python_vectors():
    cases = json.load(open(GOLDEN))
    assert len(cases) >= 6
    for c in cases:
        t = lambda x: torch.tensor(x, dtype=torch.float32).view(1, 1, c["S"], c["D"])  # noqa: E731
        q, k, v = t(c["q"]), t(c["k"]), t(c["v"])
        thr = c["threshold"]
        exp = c["expected"]
        out, mid = O.permuted_block_sparse_attn_fwd(q, k, v, c["block_size"], c["segment_size"], thr,
                                                    force_select_first_block=c["force_first"], return_intermediates=True)
        assert torch.allclose(out[0, 0], torch.tensor(exp["out"], dtype=torch.float32), atol=1e-5), c["S"]
        if c["S"] <= c["segment_size"]:
            continue
        assert mid["key_indices"][0, 0].tolist() == exp["key_indices"]
        assert mid["block_mask"][0, 0].tolist() == exp["block_mask"]
        assert mid["final_mask"][0, 0].tolist() == exp["final_mask"]
        probs = torch.nan_to_num(mid["block_attn_scores"][0, 0], nan=0.0)
        assert torch.allclose(probs, torch.tensor(exp["block_probs"], dtype=torch.float32), atol=1e-6)


# ---------------------------------------------------------------- MeanPooling baseline (no permutation)
def _brute_meanpooling_mask(q, k, bs, thr, force_first, force_current):
    """Independent restatement with explicit loops: float64 pooled logits rounded the way the bf16 tensor
    path rounds them, softmax over kb <= qb, minimal descending prefix (sequential float64 sum rounded to
    float32 per step), column 0, diagonal."""
    import numpy as np
    B, H, S, D = q.shape
    nb = (S + bs - 1) // bs
    out = torch.zeros((B, H, nb, nb), dtype=torch.bool)
    qf = torch.zeros((B, H, nb * bs, D)); qf[:, :, :S] = q.float()
    kf = torch.zeros((B, H, nb * bs, D)); kf[:, :, :S] = k.float()
    pq = qf.view(B, H, nb, bs, D).mean(-2).bfloat16()
    pk = kf.view(B, H, nb, bs, D).mean(-2).bfloat16()
    for b in range(B):
        for h in range(H):
            logit = (pq[b, h] @ pk[b, h].T)                      # bf16 matmul, as the tensor path
            logit = (logit / math.sqrt(D))                        # bf16 divide
            for qb in range(nb):
                row = logit[qb, :qb + 1].float()
                p = torch.softmax(row, -1).numpy().astype(np.float32)
                order = sorted(range(qb + 1), key=lambda i: (-p[i], i))
                c, chosen, reached = np.float64(0.0), [], False
                for i in order:
                    c = c + np.float64(p[i])
                    chosen.append(i)
                    if np.float32(c) >= np.float32(thr):
                        reached = True
                        break
                if reached:
                    out[b, h, qb, chosen] = True
                if force_first:
                    out[b, h, qb, 0] = True
                if force_current:
                    out[b, h, qb, qb] = True
    return out


@pytest.mark.parametrize("S,thr,ff", [(1024, 0.9, True), (900, 0.8, True), (640, 0.95, False)])
def test_meanpooling_selection_matches_brute_force(S, thr, ff):
    q, k, _ = small_case(1, 2, 2, S, seed=S)
    scores, mask = O.meanpooling_selection(q, k, 128, thr, ff, True)
    assert not torch.isnan(scores).any()                        # the diagonal is a candidate: no empty rows
    nb = mask.shape[-1]
    assert torch.allclose(scores.sum(-1), torch.ones(1, 2, nb), atol=1e-5)
    assert (scores.triu(1) == 0).all()
    brute = _brute_meanpooling_mask(q, k, 128, thr, ff, True)
    # rows where two blocks tie exactly on the threshold step are the only place the two may differ
    assert (mask != brute).float().mean().item() < 2e-2
    assert (mask.diagonal(dim1=-2, dim2=-1)).all() and not mask.triu(1).any()
    if ff:
        assert mask[..., 0].all()


def test_meanpooling_prefill_is_dense_attention_on_its_mask():
    q, k, v = small_case(1, 2, 1, 1000, seed=8)
    out, mid = O.meanpooling_prefill(q, k, v, 128, 1024, 0.9, return_intermediates=True)
    ke, ve = expand_kv(q, k), expand_kv(q, v)
    dense = O.dense_masked_attention_fp32(q, ke, ve, mid["key_indices"], mid["block_mask"], 128)
    assert_attn_close(out, dense, max_abs=2.5e-2, what="MeanPooling naive vs dense fp32")
    # threshold 1.0 on a row whose float32 running sum reaches 1: everything selected -> causal attention
    full, mid1 = O.meanpooling_prefill(q, k, v, 128, 1024, 0.0, return_intermediates=True)
    assert mid1["block_mask"].sum() <= mid["block_mask"].sum()  # threshold 0: the top block (+ forced ones) only
