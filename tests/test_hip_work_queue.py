"""GPU: the attention kernel's work distribution (one persistent workgroup per CU, items claimed from per-XCD
counters, other XCDs' items taken at the end, the next item's list / queries / first tiles requested during the
current item).  Shapes chosen for the corners of that machinery: items of one and two tiles (their look-ahead
steps run after the tile loop), an odd number of query blocks (the last item has one query block), fewer items
than workgroups, head counts that leave XCD ranges uneven, many short items per workgroup."""
import math

import pytest
import torch

from pbs_attn_amd import pbs as P
from tests.util import assert_attn_close, small_case

pytestmark = pytest.mark.gpu


def _dense_causal(q, k, v):
    B, Hq, S, D = q.shape
    G = Hq // k.shape[1]
    kf, vf = k.float().repeat_interleave(G, 1), v.float().repeat_interleave(G, 1)
    logits = q.float() @ kf.transpose(-1, -2) / math.sqrt(D)
    mask = torch.ones(S, S, dtype=torch.bool, device=q.device).tril()
    return torch.softmax(logits.masked_fill(~mask, float("-inf")), -1) @ vf


@pytest.mark.parametrize("S", [1, 5, 127, 128, 129, 255, 256, 257, 384, 385, 640])
@pytest.mark.parametrize("seg", [128, 256])
def test_short_sequences_every_block_selected(dev, S, seg):
    q, k, v = small_case(1, 2, 1, S, seed=S)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out = P.permuted_block_sparse_attn_fwd(qd, kd, vd, 128, seg, 1, True)
    assert_attn_close(out, _dense_causal(qd, kd, vd), what=f"S={S} seg={seg}")


@pytest.mark.parametrize("B,Hq,Hkv,S,seg,thr", [
    (3, 5, 1, 640, 256, 0.5),        # 45 items of 1-5 tiles: fewer items than workgroups
    (1, 3, 3, 8192, 1024, 0.9),      # 96 items in eight uneven ranges
    (2, 7, 1, 4096 + 77, 512, 0.8),  # ragged length, odd head count
    (4, 8, 2, 2048, 256, 0.3),       # 256 short items
    (1, 1, 1, 16384 + 128, 256, 0.9),  # one head, odd block count: the last item is a single query block
    (1, 32, 8, 4096, 256, 0.9),      # few items per workgroup, 4 whole heads per range: tickets handed out pair-major
    (2, 8, 8, 2048 + 300, 512, 0.7),   # same with 2 heads per range, ragged length, odd block count (160 items)
    (1, 8, 2, 1024, 256, 0.9),       # one head per range: pair-major is head-major
])
def test_work_distribution_shapes_against_dense_attention_on_the_mask(dev, B, Hq, Hkv, S, seg, thr):
    q, k, v = small_case(B, Hq, Hkv, S, kind="strong_heavy", seed=B * 100 + Hq)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    out = P.permuted_block_sparse_attn_fwd(qd, kd, vd, 128, seg, thr, True)
    again = P.permuted_block_sparse_attn_fwd(qd, kd, vd, 128, seg, thr, True)
    assert torch.equal(out, again)      # which workgroup takes which item does not touch the arithmetic
    # dense fp32 attention restricted to the keys the kernel's own masks allow
    perm = P.apply_permutation(qd, kd, vd, 128, seg)
    sel = P.permuted_block_selection(qd, perm, 128, seg, thr)
    nb = (S + 127) // 128
    fin = sel["final_mask"]                                           # (B, Hq, nb, nb) over PERMUTED key blocks
    idx = perm.key_indices.long()                                     # permuted position -> original key
    G = Hq // Hkv
    kf, vf = kd.float().repeat_interleave(G, 1), vd.float().repeat_interleave(G, 1)
    s_pad = nb * 128
    pos_of_key = torch.empty_like(idx)
    pos_of_key.scatter_(-1, idx, torch.arange(s_pad, device=dev).expand_as(idx))
    key_block = pos_of_key[..., :S] // 128                            # (B, Hq, S): permuted block of every key
    qblock = torch.arange(S, device=dev) // 128
    allowed = torch.gather(fin[:, :, qblock], -1, key_block.unsqueeze(2).expand(B, Hq, S, S))
    causal = torch.ones(S, S, dtype=torch.bool, device=dev).tril()
    logits = qd.float() @ kf.transpose(-1, -2) / math.sqrt(128)
    ref = torch.softmax(logits.masked_fill(~(allowed & causal), float("-inf")), -1) @ vf
    assert_attn_close(out, ref, what=f"B={B} Hq={Hq} S={S}")


def test_tile_pipeline_probe_runs_and_reports_clocks(dev):
    """The measurement entry point: a short run on zero and on random tiles returns finite sums and both clock counters."""
    import bench
    from pbs_attn_amd import _lib
    lib = bench.load_probe_library()
    sink = torch.empty(256 * 512, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    for ring in (torch.zeros(4 * 32768, dtype=torch.bfloat16, device=dev),
                 torch.randn(4 * 32768, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16).to(dev)):
        for copies in (0, 1):
            clocks = torch.zeros(2, dtype=torch.int64, device=dev)
            _lib.check(lib.pbs_attn_tile_probe(ring.data_ptr(), 4, 50, copies, sink.data_ptr(), clocks.data_ptr(), st), "probe")
            torch.cuda.synchronize()
            c = clocks.tolist()
            assert torch.isfinite(sink).all() and c[0] > 50 * 4096 and c[1] > 0   # at least the matrix pipe's cycles per tile
    assert lib.pbs_attn_tile_probe(None, 4, 50, 0, sink.data_ptr(), clocks.data_ptr(), st) < 0
