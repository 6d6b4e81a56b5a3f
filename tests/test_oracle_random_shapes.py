"""Property tests of the CPU oracle over random small shapes (hypothesis, derandomised): ragged lengths,
segment == block, one segment plus a remainder, batch > 1, head grouping, tensor thresholds, max pooling.
No GPU."""
import numpy as np
import torch
import torch.nn.functional as F
from hypothesis import given, settings, strategies as st

from oracle import pbs_oracle as O

SETTINGS = dict(max_examples=40, deadline=None, derandomize=True)


@st.composite
def shapes(draw):
    bs = draw(st.sampled_from([4, 8, 16]))
    bps = draw(st.integers(1, 4))
    seg = bs * bps
    S = draw(st.integers(1, 6 * seg + bs))
    hkv = draw(st.integers(1, 2))
    hq = hkv * draw(st.integers(1, 3))
    return dict(B=draw(st.integers(1, 2)), Hq=hq, Hkv=hkv, S=S, D=draw(st.sampled_from([8, 16])), bs=bs, seg=seg,
                seed=draw(st.integers(0, 10 ** 6)))


def _qkv(c, dtype=torch.float32):
    g = torch.Generator().manual_seed(c["seed"])
    q = torch.randn((c["B"], c["Hq"], c["S"], c["D"]), generator=g)
    k = torch.randn((c["B"], c["Hkv"], c["S"], c["D"]), generator=g)
    v = torch.randn((c["B"], c["Hkv"], c["S"], c["D"]), generator=g)
    return q.to(dtype), k.to(dtype), v.to(dtype)


@settings(**SETTINGS)
@given(shapes())
def test_full_selection_is_causal_attention_for_any_shape(c):
    # threshold int 1: every causal block is attended to, whatever permutation the scores produce
    q, k, v = _qkv(c)
    out = O.permuted_block_sparse_attn_fwd(q, k, v, c["bs"], c["seg"], 1)
    ke, ve = O.repeat_kv(k, c["Hq"] // c["Hkv"]), O.repeat_kv(v, c["Hq"] // c["Hkv"])
    ref = F.scaled_dot_product_attention(q, ke, ve, is_causal=True)
    assert out.shape == q.shape and torch.allclose(out, ref, atol=3e-5)


@settings(**SETTINGS)
@given(shapes(), st.sampled_from([0.3, 0.8, 0.9, 1.0, "rows"]), st.sampled_from(["mean", "max"]), st.booleans())
def test_pipeline_equals_dense_attention_on_its_own_mask(c, thr, pool, force):
    q, k, v = _qkv(c)
    if thr == "rows":
        thr = torch.linspace(0.2, 0.95, c["B"] * c["Hq"]).view(c["B"], c["Hq"])
    ke, ve = O.repeat_kv(k, c["Hq"] // c["Hkv"]), O.repeat_kv(v, c["Hq"] // c["Hkv"])
    out, mid = O.permuted_block_sparse_attn_fwd(q, ke, ve, c["bs"], c["seg"], thr, True, force, pool, pool,
                                                return_intermediates=True)
    S, bs, seg = c["S"], c["bs"], c["seg"]
    sc = (S // seg) * seg
    if S > seg:
        idx = mid["key_indices"]
        # the permutation stays inside segments, the remainder keeps its order
        srt = idx[:, :, :sc].view(c["B"], c["Hq"], -1, seg).sort(-1).values
        assert torch.equal(srt, torch.arange(sc).view(1, 1, -1, seg).expand_as(srt))
        assert torch.equal(idx[:, :, sc:], torch.arange(sc, S).expand(c["B"], c["Hq"], -1))
        # masks: own segment always there, nothing from later segments is ever needed
        nb, bps = (S + bs - 1) // bs, seg // bs
        cand, segm = O.candidate_masks(nb, bps)
        assert (mid["final_mask"] | ~segm[None, None]).all()
        assert not (mid["block_mask"] & ~cand[None, None] & ~O.first_token_mask(
            torch.cat([idx, torch.arange(S, nb * bs).expand(c["B"], c["Hq"], -1)], -1), bs)).any()
        dense = O.dense_masked_attention_fp32(q, mid["perm_k"], mid["perm_v"], idx, mid["final_mask"], bs)
        assert torch.allclose(out, dense, atol=3e-5)
    else:
        assert torch.allclose(out, F.scaled_dot_product_attention(q, ke, ve, is_causal=True), atol=3e-5)


@settings(**SETTINGS)
@given(st.integers(1, 3), st.integers(1, 40), st.sampled_from([0.0, 0.25, 0.5, 0.9, 0.999, 1.0]), st.integers(0, 10 ** 6))
def test_select_blocks_is_the_minimal_descending_prefix(rows, n, thr, seed):
    g = torch.Generator().manual_seed(seed)
    p = torch.softmax((torch.randn((1, 1, rows, n), generator=g) * 2).bfloat16().float(), -1)   # ties on purpose
    sel = O.select_blocks(p, thr)
    thr32 = np.float32(thr)
    for r in range(rows):
        vals = [np.float32(x) for x in p[0, 0, r].tolist()]
        order = sorted(range(n), key=lambda i: (-vals[i], i))
        acc, want = np.float64(0.0), set()
        for rank, i in enumerate(order):
            acc += np.float64(vals[i])
            if np.float32(acc) >= thr32:
                want = set(order[:rank + 1])
                break
        assert set(torch.where(sel[0, 0, r])[0].tolist()) == want
