"""pbs_score_keys_static (the entry point that allocates nothing: its chunk partials live in a
library-owned device array) against pbs_score_keys, through the C ABI.

Same kernels on the same inputs, so the scores must be bit-identical.  Two calls in a row, the second
on a smaller input: the array keeps the first call's contents and the second must not be disturbed by
them.  The file is collected last so that a failure here hides no other test."""
import pytest
import torch

from oracle import pbs_oracle as O
from pbs_attn_amd import _lib
from tests.util import small_case

pytestmark = pytest.mark.gpu


def _score(entry, q, k, seg, ws=None):
    lib = _lib.load()
    B, Hq, S, D = q.shape
    Hkv = k.shape[1]
    sc = (S // seg) * seg
    scores = torch.full((B, Hq, sc), float("nan"), dtype=torch.float32, device=q.device)
    st = torch.cuda.current_stream().cuda_stream
    common = (q.data_ptr(), k.data_ptr(), scores.data_ptr(), B, Hq, Hkv, S, D, 128, seg,
              q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2))
    if entry == "static":
        rc = lib.pbs_score_keys_static(*common, st)
    else:
        rc = lib.pbs_score_keys(*common, ws.data_ptr(), ws.numel(), st)
    return rc, scores


def _workspace(q, k, seg):
    lib = _lib.load()
    n = lib.pbs_score_keys_workspace_bytes(q.shape[0], q.shape[1], k.shape[1], q.shape[2], seg)
    return torch.empty(max(n, 16), dtype=torch.uint8, device=q.device)


def test_static_scratch_entry_point_equals_workspace_entry_point(dev):
    cases = [(2, 8, 2, 8192, 1024, 31), (1, 4, 2, 1024 + 200, 256, 32)]   # the second call is the smaller one
    for B, Hq, Hkv, S, seg, seed in cases:
        q, k, _ = small_case(B, Hq, Hkv, S, seed=seed)
        qd, kd = q.to(dev), k.to(dev)
        rc, want = _score("workspace", qd, kd, seg, _workspace(qd, kd, seg))
        assert rc == 0, _lib.load().pbs_last_error()
        rc, got = _score("static", qd, kd, seg)
        assert rc == 0, _lib.load().pbs_last_error()
        torch.cuda.synchronize()
        assert not torch.isnan(got).any()
        assert torch.equal(got, want), (S, (got - want).abs().max().item())
        # and both agree with the oracle to the scoring tolerance
        ref = O.key_scores(q, O.repeat_kv(k, Hq // Hkv), 128, seg)
        rel = (got.cpu() - ref).abs() / ref.abs().clamp_min(1e-12)
        assert rel.max().item() < 3e-2 and rel.mean().item() < 2e-3


def test_static_scratch_entry_point_rejects_shapes_beyond_its_buffer(dev):
    lib = _lib.load()
    B, Hq, Hkv, S, seg = 4, 64, 8, 131072, 1024
    need = lib.pbs_score_keys_workspace_bytes(B, Hq, Hkv, S, seg)
    assert need > (8 << 20)
    # argument checks only: the pointers are never dereferenced because the size check comes first
    x = torch.zeros(16, dtype=torch.bfloat16, device=dev)
    s = torch.zeros(16, dtype=torch.float32, device=dev)
    rc = lib.pbs_score_keys_static(x.data_ptr(), x.data_ptr(), s.data_ptr(), B, Hq, Hkv, S, 128, 128, seg,
                                   Hq * S * 128, S * 128, 128, Hkv * S * 128, S * 128, 128,
                                   torch.cuda.current_stream().cuda_stream)
    assert rc == -1
    assert b"library-owned buffer" in lib.pbs_last_error()
