"""GPU: the plug-in boundary with the real HIP prefill function on a Llama-3.1-8B-shaped layer stack
(random weights): a patched model with every causal block selected must reproduce the unpatched model."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["llama31_8b", "qwen25_7b"])
def test_patched_model_matches_unpatched_on_gpu(dev, name):
    from pbs_attn.patch.huggingface import apply_patch_with_prefill, get_permuted_block_sparse_attn_fwd
    from pbs_attn_amd.ttft import build_model
    model = build_model(name, layers=2, device=dev)
    ids = torch.randint(0, 1000, (2, 1500), generator=torch.Generator().manual_seed(0)).to(dev)
    with torch.no_grad():
        ref = model(ids).logits.float()
        apply_patch_with_prefill(model, get_permuted_block_sparse_attn_fwd(segment_size=256, threshold=1))
        got = model(ids).logits.float()
        # bf16 model: two attention kernels with different summation orders differ by a few bf16 ulps of the
        # logits (|logit| up to ~7: one ulp is 0.03); a wrong mask or permutation moves them by O(1)
        assert (got - ref).abs().max() < 0.15, (got - ref).abs().max()
        assert (got - ref).abs().mean() < 0.02, (got - ref).abs().mean()
        assert torch.equal(got[:, 0], ref[:, 0])            # the first token attends to itself only
        # prefill with the sparse path, then decode through the module's original forward
        out = model.generate(ids[:1], max_new_tokens=3, do_sample=False)
        assert out.shape == (1, 1503)
    model2 = build_model(name, layers=1, device=dev)
    apply_patch_with_prefill(model2, get_permuted_block_sparse_attn_fwd())
    with torch.no_grad():
        lg = model2(ids).logits
    assert torch.isfinite(lg.float()).all()
