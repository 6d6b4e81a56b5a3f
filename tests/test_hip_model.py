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


def test_llama31_8b_prompt_of_65536_tokens(dev):
    """BASELINE.json's config 4 at its own prompt length (65 536 uniform random token ids, the Llama-3.1-8B
    architecture with random weights; two of the 32 identical layers): patched with every causal block selected
    the model must reproduce the unpatched one on the logits of the last 256 positions; patched with the default
    threshold (which drops a tenth of the estimated attention mass) it must stay finite; the distance is printed."""
    from pbs_attn.patch.huggingface import apply_patch_with_prefill, get_permuted_block_sparse_attn_fwd
    from pbs_attn_amd.ttft import build_model
    model = build_model("llama31_8b", layers=2, device=dev)
    ids = torch.randint(0, 128256, (1, 65536), generator=torch.Generator().manual_seed(4)).to(dev)
    with torch.no_grad():
        ref = model(ids, logits_to_keep=256).logits.float()
        assert ref.shape == (1, 256, 128256)
        apply_patch_with_prefill(model, get_permuted_block_sparse_attn_fwd(segment_size=256, threshold=1))
        got = model(ids, logits_to_keep=256).logits.float()
        d = (got - ref).abs()
        print(f"\n64k prompt, threshold=1 against the unpatched model: max {d.max():.4f} mean {d.mean():.5f}")
        assert d.max() < 0.15 and d.mean() < 0.02, (d.max(), d.mean())
        for layer in model.model.layers:            # patch again with the factory's defaults (threshold 0.9)
            layer.self_attn.forward = layer.self_attn.original_forward
        apply_patch_with_prefill(model, get_permuted_block_sparse_attn_fwd())
        sparse = model(ids, logits_to_keep=256).logits.float()
        assert torch.isfinite(sparse).all()
        d = (sparse - ref).abs()
        print(f"64k prompt, threshold=0.9 against the unpatched model: max {d.max():.4f} mean {d.mean():.5f}")
        out = model.generate(ids, max_new_tokens=1, do_sample=False)
        assert out.shape == (1, 65537)


@pytest.mark.parametrize("method", ["pbs", "meanpooling", "dense"])
def test_ttft_harness_writes_the_reference_result_record(dev, method, tmp_path, capsys):
    """The offline harness follows eval/efficiency/eval_efficiency.py: one JSON line on stdout and a result
    file <output_dir>/<method>_<len>.json with the fields of its results dict (:261-290)."""
    import json
    from pbs_attn_amd import ttft
    argv = ["--method", method, "--layers", "2", "--len", "4096", "--iters", "2", "--warmup", "1",
            "--output-dir", str(tmp_path)]
    assert ttft.main(argv) == 0
    line = capsys.readouterr().out.strip().splitlines()[-1]
    printed = json.loads(line)
    path = tmp_path / f"{method}_4096.json"
    assert printed["result_file"] == str(path) and path.exists()
    saved = json.loads(path.read_text())
    for key in ("script_args", "method_args", "model_name", "tokenizer_name", "num_tokens", "avg_e2e_latency", "e2e_std"):
        assert key in saved, key
    assert saved["num_tokens"] == 4096 and saved["model_name"] == "llama31_8b"
    assert saved["script_args"]["method"] == method and saved["script_args"]["len"] == 4096
    assert saved["script_args"]["n_examples"] == 2 and saved["script_args"]["num_warmup_iter"] == 1
    assert len(saved["e2e_latencies"]) == 2 and all(t > 0 for t in saved["e2e_latencies"])
    assert abs(saved["avg_e2e_latency"] - sum(saved["e2e_latencies"]) / 2) < 1e-9
    assert printed["ttft_s"] == saved["avg_e2e_latency"]
    if method == "dense":
        assert saved["method_args"] == {}
    else:
        assert saved["method_args"]["segment_size"] == (256 if method == "pbs" else 1024)
        assert saved["method_args"]["threshold"] == 0.9 and saved["method_args"]["block_size"] == 128


def test_ttft_harness_defaults_follow_the_protocol():
    """30 warm-up generations and 10 examples unless overridden (eval_efficiency.py:36-37)."""
    import inspect
    from pbs_attn_amd import ttft
    src = inspect.getsource(ttft.main)
    assert 'default=30, dest="num_warmup_iter"' in src and 'default=10, dest="n_examples"' in src


def test_dispatcher_op_equals_the_direct_call_and_traces(dev):
    """torch.ops.pbs_hip.prefill_attn_fwd gives the bits of the ctypes call, for the three threshold forms, and a
    function that uses it can be captured by torch.compile's tracer (the op is one opaque node)."""
    import pbs_attn_amd.torch_ops as T
    from pbs_attn_amd import ops
    from tests.util import small_case
    q, k, v = small_case(2, 4, 2, 1500, seed=61)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    per_head = torch.tensor([[0.5, 0.7, 0.9, 0.95], [0.6, 0.8, 0.85, 0.99]], device=dev)
    for thr in (0.9, 1, per_head):
        direct = ops.prefill_attn_fwd(qd, kd, vd, 128, 256, thr)
        via_op = T.prefill_attn_fwd(qd, kd, vd, 128, 256, thr)
        assert torch.equal(direct, via_op)

    def f(a, b, c):
        return torch.ops.pbs_hip.prefill_attn_fwd(a * 1, b, c, 128, 256, 0.9, False, None, True, "mean", "mean") + 0

    traced = torch.compile(f, backend="eager", fullgraph=True)
    assert torch.equal(traced(qd, kd, vd), ops.prefill_attn_fwd(qd, kd, vd, 128, 256, 0.9))
