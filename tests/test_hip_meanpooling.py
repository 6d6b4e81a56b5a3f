"""GPU parity of the un-permuted MeanPooling mode (baselines/MeanPooling.py) and of the stage adapters with
the reference's signatures, against the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import pbs_oracle as O
from pbs_attn_amd import compat, ops
from pbs_attn_amd.meanpooling import MeanPooling_prefill
from tests.util import assert_attn_close, expand_kv, small_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("nb", [8, 33, 100])
def test_causal_candidate_block_probabilities(dev, nb):
    g = torch.Generator().manual_seed(nb)
    pq = (torch.randn((2, 3, nb, 128), generator=g) * 0.5).bfloat16()
    pk = (torch.randn((2, 3, nb, 128), generator=g) * 0.5).bfloat16()
    ref = O.block_logits_softmax(pq, pk, torch.tril(torch.ones(nb, nb, dtype=torch.bool)))
    got = ops.block_logits_softmax(pq.to(dev), pk.to(dev), 1, causal_candidates=True).cpu()
    assert not torch.isnan(got).any() and (got.triu(1) == 0).all()
    assert torch.allclose(got.sum(-1), torch.ones(2, 3, nb), atol=1e-4)
    assert torch.allclose(got, ref, rtol=3e-2, atol=1e-6)


@pytest.mark.parametrize("B,Hq,Hkv,S,thr,ff", [(1, 4, 2, 2048, 0.9, True), (2, 2, 2, 1000, 0.8, True),
                                               (1, 7, 1, 1536, 0.95, False)])
def test_meanpooling_masks_bit_exact_and_output_vs_dense(dev, B, Hq, Hkv, S, thr, ff):
    q, k, v = small_case(B, Hq, Hkv, S, seed=S + Hq)
    ke, ve = expand_kv(q, k), expand_kv(q, v)
    ref_out, mid = O.meanpooling_prefill(q, ke, ve, 128, 1024, thr, True, ff, True, return_intermediates=True)
    nb = (S + 127) // 128
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    idx = torch.arange(nb * 128, dtype=torch.int32, device=dev).view(1, 1, -1).expand(B, Hq, -1).contiguous()
    # the selection on the ORACLE's block probabilities: masks must be bit-exact
    sel, fin, cols, cnt = ops.select_blocks(mid["block_attn_scores"].to(dev), float(thr), idx, S, 128, 128, ff)
    assert torch.equal(fin.cpu(), mid["block_mask"])
    perm_k, perm_vt, _ = ops.gather_kv(kd, vd, idx, Hq)
    out = ops.sparse_attn_fwd(qd, perm_k, perm_vt, kd, vd, cols, cnt, 128).cpu()
    dense = O.dense_masked_attention_fp32(q, ke, ve, mid["key_indices"], mid["block_mask"], 128)
    assert_attn_close(out, dense, what="MeanPooling HIP vs dense fp32 on the oracle's mask")
    assert_attn_close(ref_out, dense, max_abs=2.5e-2, what="oracle naive vs dense fp32")
    # the whole mode from raw Q, K, V: its own mask differs from the oracle's only where a block probability
    # sits on the threshold step; its output is dense attention on ITS mask
    out2, got = MeanPooling_prefill(qd, kd, vd, 128, 1024, thr, True, ff, True, return_masks=True)
    own_mask = got["block_mask"].cpu()
    agree = (own_mask == mid["block_mask"]).float().mean().item()
    assert agree >= 0.995, agree
    dense2 = O.dense_masked_attention_fp32(q, ke, ve, mid["key_indices"], own_mask, 128)
    assert_attn_close(out2.cpu(), dense2, what="MeanPooling_prefill vs dense fp32 on its own mask")


def test_meanpooling_through_the_factory_and_patch(dev):
    from pbs_attn.patch.huggingface import get_meanpooling_prefill
    q, k, v = small_case(1, 4, 4, 1024, seed=3)
    fn = get_meanpooling_prefill(threshold=0.9)
    out = fn(q.to(dev), k.to(dev), v.to(dev))
    assert out.shape == q.shape and torch.isfinite(out.float()).all()
    out = get_meanpooling_prefill(force_select_current_block=False)(q.to(dev), k.to(dev), v.to(dev))
    assert out.shape == q.shape and torch.isfinite(out.float()).all()


@pytest.mark.parametrize("B,Hq,Hkv,S,thr,ff", [(1, 4, 2, 2048, 0.3, True), (2, 2, 2, 1000, 0.5, True), (1, 7, 1, 1536, 0.2, False),
                                               (1, 2, 2, 1280, 0.9, True)])
def test_meanpooling_with_an_optional_diagonal_block(dev, B, Hq, Hkv, S, thr, ff):
    """force_select_current_block=False (MeanPooling.py:54-58 skipped): a query block attends to its diagonal block
    only where the threshold selected it.  Masks bit-exact on the oracle's block probabilities, output against dense
    attention on that mask; low thresholds so that many diagonals are in fact dropped."""
    q, k, v = small_case(B, Hq, Hkv, S, seed=S + Hq + 1)
    ke, ve = expand_kv(q, k), expand_kv(q, v)
    ref_out, mid = O.meanpooling_prefill(q, ke, ve, 128, 1024, thr, True, ff, False, return_intermediates=True)
    nb = (S + 127) // 128
    eye = torch.eye(nb, dtype=torch.bool)
    dropped = (~mid["block_mask"] & eye).sum().item()
    if thr < 0.9:
        assert dropped > 0, "the case is meant to drop diagonal blocks"
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    idx = torch.arange(nb * 128, dtype=torch.int32, device=dev).view(1, 1, -1).expand(B, Hq, -1).contiguous()
    sel, fin, cols, cnt = ops.select_blocks(mid["block_attn_scores"].to(dev), float(thr), idx, S, 128, 128, ff, candidate_rule=2)
    assert torch.equal(sel.cpu(), mid["block_mask"])
    own = sel.diagonal(dim1=-2, dim2=-1).to(torch.uint8).contiguous()
    perm_k, perm_vt, _ = ops.gather_kv(kd, vd, idx, Hq)
    out = ops.sparse_attn_fwd(qd, perm_k, perm_vt, kd, vd, cols, cnt, 128, own_block_needed=own).cpu()
    dense = O.dense_masked_attention_fp32(q, ke, ve, mid["key_indices"], mid["block_mask"], 128)
    assert_attn_close(out, dense, what="optional diagonal: HIP vs dense fp32 on the oracle's mask")
    assert_attn_close(ref_out, dense, max_abs=2.5e-2, what="oracle naive vs dense fp32")
    # with every flag set the entry point is the plain one
    ones = torch.ones_like(own)
    a = ops.sparse_attn_fwd(qd, perm_k, perm_vt, kd, vd, cols, cnt, 128, own_block_needed=ones)
    b = ops.sparse_attn_fwd(qd, perm_k, perm_vt, kd, vd, cols, cnt, 128)
    assert torch.equal(a, b)
    # the whole mode from raw Q, K, V
    out2, got = MeanPooling_prefill(qd, kd, vd, 128, 1024, thr, True, ff, False, return_masks=True)
    own_mask = got["block_mask"].cpu()
    assert (own_mask == mid["block_mask"]).float().mean().item() >= 0.99
    dense2 = O.dense_masked_attention_fp32(q, ke, ve, mid["key_indices"], own_mask, 128)
    assert_attn_close(out2.cpu(), dense2, what="MeanPooling_prefill (optional diagonal) vs dense fp32 on its own mask")


def test_stage_adapters_with_the_reference_signatures(dev):
    B, H, S, seg, thr = 1, 4, 1536, 512, 0.9
    q, k, v = small_case(B, H, H, S, seed=17)
    qd, kd = q.to(dev), k.to(dev)
    perm_k, idx = compat.apply_permutation(qd, kd, 128, seg)
    assert perm_k.shape == k.shape and idx.shape == (B, H, S) and idx.dtype == torch.int64
    # a permutation inside every segment, and the gathered rows are the rows of K
    assert torch.equal(idx.view(B, H, S // seg, seg).sort(-1).values.cpu(),
                       torch.arange(S).view(1, 1, S // seg, seg).expand(B, H, -1, -1))
    assert torch.equal(perm_k.cpu(), O.gather_rows(k, idx.cpu()))
    # selection on these permuted keys: probabilities close to the oracle's, mask bit-exact on the oracle's scores
    scores, block_mask, segment_mask = compat.permuted_block_selection(qd, perm_k, None, idx, 128, seg, thr)
    ref_scores, ref_mask, ref_segm = O.permuted_block_selection(q, perm_k.cpu(), idx.cpu(), 128, seg, thr)
    assert torch.equal(segment_mask.cpu(), ref_segm)
    nan = torch.isnan(ref_scores)
    assert torch.equal(torch.isnan(scores.cpu()), nan)
    assert torch.allclose(scores.cpu()[~nan], ref_scores[~nan], rtol=3e-2, atol=1e-6)
    assert (block_mask.cpu() == ref_mask).float().mean().item() >= 0.99
    sel = compat.select_blocks(ref_scores.to(dev), thr)
    assert torch.equal(sel.cpu(), O.select_blocks(ref_scores, thr))
    cand, _ = O.candidate_masks(S // 128, seg // 128)
    P = compat.block_pooled_attn(qd, perm_k, 128, cand.to(dev))
    assert torch.allclose(P.cpu()[~nan], ref_scores[~nan], rtol=3e-2, atol=1e-6)
    assert torch.equal(compat.first_token_mask(idx, 128).cpu(), O.first_token_mask(idx.cpu(), 128))


@pytest.mark.parametrize("B,Hq,Hkv,S,thr", [(1, 4, 2, 2048, 1.5), (2, 2, 2, 1000, 1.0), (1, 3, 1, 1536, 1.0), (1, 2, 2, 128, 2.0),
                                            (1, 1, 1, 4096, 1.5)])
def test_query_blocks_that_select_nothing_give_zeros(dev, B, Hq, Hkv, S, thr):
    """force_select_first_block=False and force_select_current_block=False with a threshold the running sum never
    reaches (above 1, or 1.0 against a float32 sum that tops out below it): select_blocks picks nothing for such a
    row (utils.py:74-84) and the attention gives zeros for it (kernels/...:340-343).  Whole launches without a single
    tile, pairs of query blocks where one or both visit nothing, and rows that do reach the threshold, side by side."""
    q, k, v = small_case(B, Hq, Hkv, S, seed=S + Hq + 5)
    ke, ve = expand_kv(q, k), expand_kv(q, v)
    ref_out, mid = O.meanpooling_prefill(q, ke, ve, 128, 1024, thr, True, False, False, return_intermediates=True)
    empty_rows = ~mid["block_mask"].any(-1)
    assert empty_rows.any(), "the case is meant to leave query blocks without a block"
    if thr > 1.0:
        assert empty_rows.all() and (ref_out == 0).all()
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    nb = (S + 127) // 128
    idx = torch.arange(nb * 128, dtype=torch.int32, device=dev).view(1, 1, -1).expand(B, Hq, -1).contiguous()
    sel, fin, cols, cnt = ops.select_blocks(mid["block_attn_scores"].to(dev), float(thr), idx, S, 128, 128, False, candidate_rule=2)
    assert torch.equal(sel.cpu(), mid["block_mask"])
    own = sel.diagonal(dim1=-2, dim2=-1).to(torch.uint8).contiguous()
    perm_k, perm_vt, _ = ops.gather_kv(kd, vd, idx, Hq)
    out = torch.full_like(qd, float("nan"))
    ops.sparse_attn_fwd(qd, perm_k, perm_vt, kd, vd, cols, cnt, 128, own_block_needed=own, out=out)
    out = out.cpu()
    dense = torch.nan_to_num(O.dense_masked_attention_fp32(q, ke, ve, mid["key_indices"], mid["block_mask"], 128), nan=0.0)
    assert_attn_close(out, dense, what="rows without blocks: HIP vs dense fp32 (zeros where nothing is selected)")
    row_empty = empty_rows.repeat_interleave(128, -1)[..., :S]
    assert (out[row_empty] == 0).all()
    # the whole mode from raw Q, K, V, twice (the second call finds the first one's lists in the workspace)
    for _ in range(2):
        out2, got = MeanPooling_prefill(qd, kd, vd, 128, 1024, thr, True, False, False, return_masks=True)
        own_mask = got["block_mask"].cpu()
        dense2 = torch.nan_to_num(O.dense_masked_attention_fp32(q, ke, ve, mid["key_indices"], own_mask, 128), nan=0.0)
        assert_attn_close(out2.cpu(), dense2, what="MeanPooling_prefill with unreachable threshold vs dense fp32 on its own mask")


def test_attention_stage_with_the_reference_argument_list(dev):
    """pbs_attn.src.kernels.permuted_block_sparse_attention: the attention stage under the reference's two names
    (the naive function's argument list, kernels/...:314-323, and the Triton kernel's launch form, pbs.py:220-246), fed
    with what the reference's orchestrator hands it: permuted K / V, their original positions, block_mask | segment_mask."""
    from pbs_attn.src.kernels.permuted_block_sparse_attention import (
        _permuted_block_sparse_attn_fwd, _permuted_block_sparse_attn_fwd_torch_naive)
    B, H, S, seg, thr = 2, 3, 1664, 512, 0.7
    q, k, v = small_case(B, H, H, S, seed=29)
    ref_out, mid = O.permuted_block_sparse_attn_fwd(q, k, v, 128, seg, thr, return_intermediates=True)
    idx, mask = mid["key_indices"], mid["final_mask"]
    perm_k, perm_v = O.gather_rows(k, idx), O.gather_rows(v, idx)
    dense = O.dense_masked_attention_fp32(q, perm_k, perm_v, idx, mask, 128)
    q_idx = torch.arange(S).view(1, 1, -1).expand(B, H, -1)
    args = [t.to(dev) for t in (q, perm_k, perm_v)]
    out = torch.empty_like(args[0])
    got = _permuted_block_sparse_attn_fwd_torch_naive(*args, out, q_idx.to(dev), idx.to(dev), idx.to(dev), mask.to(dev), 128, seg, True)
    assert got is out
    assert_attn_close(out.cpu(), dense, what="attention stage on the oracle's mask vs dense fp32")
    assert_attn_close(out.cpu(), ref_out, max_abs=2.5e-2, what="attention stage vs the oracle's naive path")
    out2 = torch.zeros_like(out)
    strides = [0] * 29
    _permuted_block_sparse_attn_fwd[(13, H, B)](*args, out2, mask.to(dev), q_idx.to(dev), idx.to(dev), idx.to(dev), *strides, S, S,
                                               128 ** -0.5, H=H, num_kv_groups=1, HEAD_DIM=128, SEGMENT_SIZE=seg,
                                               LOGICAL_BLOCK_SIZE=128, STAGE=3)
    assert torch.equal(out2, out)
    # the visit lists made from the mask are the selection's own
    cols, cnt, missing = ops.block_mask_to_csr(mask.to(dev), seg // 128)
    nb, bps = mask.shape[-1], seg // 128
    qb = torch.arange(nb)
    earlier = (qb.view(1, -1) // bps) < (qb.view(-1, 1) // bps)
    assert int(missing.item()) == 0 and torch.equal(cnt.cpu(), (mask & earlier).sum(-1).int())
    row = cols[1, 2, nb - 1, :cnt[1, 2, nb - 1]].cpu()
    assert torch.equal(row, torch.where(mask[1, 2, nb - 1] & earlier[nb - 1])[0].int())
    # a mask without a block of the own segment, and permuted queries, are refused
    bad = mask.clone()
    bad[0, 0, 5, 5] = False
    with pytest.raises(ValueError, match="own segment"):
        _permuted_block_sparse_attn_fwd_torch_naive(*args, out, q_idx.to(dev), idx.to(dev), idx.to(dev), bad.to(dev), 128, seg, True)
    with pytest.raises(ValueError, match="original order"):
        _permuted_block_sparse_attn_fwd_torch_naive(*args, out, q_idx.flip(-1).to(dev), idx.to(dev), idx.to(dev), mask.to(dev), 128, seg, True)
