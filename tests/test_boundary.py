"""Host-side logic without a GPU: the C ABI exports what the header declares, the
import paths and factory of the plug-in boundary, the Hugging Face patcher on tiny
random-init models (with the CPU oracle standing in as prefill_fn), and that the
product path refuses to run without the GPU."""
import ctypes
import os
import re
from functools import partial

import pytest
import torch

from oracle import pbs_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pbs_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pbs_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from pbs_attn_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from pbs_attn_amd.build import build_library
        build_library()
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/pbs_hip.h but not exported"
    assert set(names) == set(_lib.SIGNATURES), "ctypes signatures and header disagree"
    assert _lib.load().pbs_abi_version() == 1


def test_ctypes_signatures_match_the_header_parameter_by_parameter():
    # a wrong ctypes signature passes garbage to a kernel launch: compare every declaration's return
    # type and parameter types with the table the host code calls through
    from pbs_attn_amd import _lib
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    decls = re.findall(r"\b(int|size_t|double|const char\s*\*)\s+(pbs_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S)
    assert len(decls) == len(_lib.SIGNATURES)

    def ctype_of(param):
        param = " ".join(param.split())
        if param == "void":
            return None
        if "*" in param:
            return ctypes.c_void_p
        base = param.rsplit(" ", 1)[0].replace("const ", "")
        return {"int": ctypes.c_int, "int64_t": ctypes.c_int64, "float": ctypes.c_float, "size_t": ctypes.c_size_t,
                "double": ctypes.c_double}[base]

    ret_map = {"int": ctypes.c_int, "size_t": ctypes.c_size_t, "double": ctypes.c_double}
    for ret, name, params in decls:
        want_args = [t for t in (ctype_of(x) for x in params.split(",")) if t is not None]
        res, args = _lib.SIGNATURES[name]
        assert list(args) == want_args, f"{name}: ctypes argument types differ from the header"
        if "char" in ret:
            assert res is ctypes.c_char_p
        else:
            assert res is ret_map[ret], f"{name}: return type differs from the header"


def test_argument_errors_are_reported_without_a_gpu():
    from pbs_attn_amd import _lib
    lib = _lib.load()
    # argument validation happens before any launch: safe on a CPU-only host
    rc = lib.pbs_segment_argsort(None, None, 1, 128, 128, 128, None)
    assert rc < 0 and b"null" in lib.pbs_last_error()
    rc = lib.pbs_pool_q(1, 1, 1, 1, 128, 64, 128, 0, 0, 0, 0, None)
    assert rc < 0 and b"head_dim" in lib.pbs_last_error()
    with pytest.raises(_lib.PbsHipError):
        _lib.check(rc, "pbs_pool_q")
    # a key row stride the scoring kernel's 32-bit copy offsets cannot hold (pointers are only checked, never read)
    fake = 4096
    rc = lib.pbs_score_keys(fake, fake, fake, 1, 4, 2, 1024, 128, 128, 256, 0, 0, 128, 0, 0, 1 << 28, fake, 1 << 30, None)
    assert rc < 0 and b"key row stride" in lib.pbs_last_error()


def test_reference_import_paths():
    from pbs_attn import permuted_block_sparse_attn_fwd as a
    from pbs_attn.patch.huggingface import apply_patch_with_prefill, get_permuted_block_sparse_attn_fwd
    from pbs_attn.src.pbs import permuted_block_sparse_attn_fwd as b
    assert a is b and callable(apply_patch_with_prefill) and callable(get_permuted_block_sparse_attn_fwd)


def test_reference_callers_import_lines_work():
    # the import statements of the reference's own callers (eval/efficiency/eval_efficiency.py:21-29,
    # eval/benchmarks/opencompass_models.py:14-21) and of its stage modules
    from pbs_attn.patch.huggingface import (  # noqa: F401
        apply_patch_with_prefill,
        get_flexprefill_prefill,
        get_minference_prefill,
        get_xattention_prefill,
        get_meanpooling_prefill,
        get_permuted_block_sparse_attn_fwd,
        get_flashattn_prefill,
    )
    from pbs_attn.src.permute_states import apply_permutation, last_block_attn_sorting
    from pbs_attn.src.utils import block_pooled_attn, select_blocks
    from pbs_attn.src.pbs import first_token_mask, permuted_block_selection
    from pbs_attn.src.pbs import apply_permutation as ap2
    from pbs_attn.baselines.MeanPooling import MeanPooling_prefill
    # pbs_attn/src/pbs.py:6 of the reference
    from pbs_attn.src.kernels.permuted_block_sparse_attention import (  # noqa: F401
        _permuted_block_sparse_attn_fwd, _permuted_block_sparse_attn_fwd_torch_naive)
    assert callable(_permuted_block_sparse_attn_fwd_torch_naive) and callable(_permuted_block_sparse_attn_fwd[(1, 1, 1)])
    assert ap2 is apply_permutation

    def params(fn):
        return fn.__code__.co_varnames[:fn.__code__.co_argcount]
    # the reference's signatures (permute_states.py:6-11,87-93; utils.py:6-13,38-42; pbs.py:10-13,29-41)
    assert params(last_block_attn_sorting) == ("queries", "keys", "block_size", "segment_size")
    assert params(apply_permutation) == ("query_states", "key_states", "block_size", "segment_size")
    assert params(block_pooled_attn) == ("query_states", "key_states", "block_size", "mask", "query_pool_mode",
                                         "key_pool_mode")
    assert params(select_blocks) == ("block_attn_scores", "threshold", "causal")
    assert params(first_token_mask) == ("key_indices", "block_size")
    assert params(permuted_block_selection) == (
        "permuted_query_states", "permuted_key_states", "query_indices", "key_indices", "block_size", "segment_size",
        "threshold", "causal", "force_select_first_block", "query_pool_mode", "key_pool_mode")
    assert params(MeanPooling_prefill)[:9] == (
        "query_states", "key_states", "value_states", "block_size", "segment_size", "threshold", "causal",
        "force_select_first_block", "force_select_current_block")
    # the baselines built on external CUDA packages fail the way the reference does without them
    for factory, name in ((get_flashattn_prefill, "FlashAttn"), (get_minference_prefill, "Minference"),
                          (get_flexprefill_prefill, "FlexPrefill")):
        with pytest.raises(RuntimeError, match=f"{name} unavailable."):
            factory()
    with pytest.raises(RuntimeError, match="XAttention unavailable."):
        get_xattention_prefill(stride=8)
    mp = get_meanpooling_prefill()
    assert isinstance(mp, partial) and mp.func.__name__ == "MeanPooling_prefill"
    assert mp.keywords == dict(block_size=128, segment_size=1024, threshold=0.9, causal=True,
                               force_select_first_block=True, force_select_current_block=True)
    assert "layer_idx" not in mp.func.__code__.co_varnames


def test_candidate_rule_detection_of_the_stage_adapter():
    from pbs_attn_amd.compat import _candidate_rule
    from oracle import pbs_oracle as O
    assert _candidate_rule(torch.tril(torch.ones(9, 9, dtype=torch.bool))) == ("causal", 1)
    for nb, bps in ((8, 2), (12, 4), (7, 1), (9, 9)):
        assert _candidate_rule(O.candidate_masks(nb, bps)[0]) == ("segments", bps)
    with pytest.raises(ValueError):
        _candidate_rule(torch.ones(4, 4, dtype=torch.bool))


def test_threshold_argument_semantics():
    from pbs_attn_amd.ops import _threshold_args
    dev = torch.device("cpu")
    assert _threshold_args(1, 1, 2, dev)[0] is True
    assert _threshold_args(True, 1, 2, dev)[0] is True       # isinstance(True, int): the reference's rule (pbs.py:120)
    assert _threshold_args(1.0, 1, 2, dev) == (False, None, 1.0)
    # a float64 tensor is compared in float64 there: the smallest float32 not below it gives the same decisions
    t64 = torch.tensor([[0.9, 0.5]], dtype=torch.float64)
    _, rows, _ = _threshold_args(t64, 1, 2, dev)
    assert rows.dtype == torch.float32 and (rows.double() >= t64).all()
    assert rows[0, 0].item() == torch.nextafter(torch.tensor(0.9, dtype=torch.float32), torch.tensor(2.0)).item()
    assert rows[0, 1].item() == 0.5
    c = torch.tensor([0.9], dtype=torch.float32)            # float32(0.9) < 0.9 in float64
    assert not bool((c.double() >= t64[0, 0]).item()) and not bool((c >= rows[0, 0]).item())
    _, rows32, _ = _threshold_args(torch.tensor([[0.9, 0.5]]), 1, 2, dev)
    assert rows32[0, 0].item() == torch.tensor(0.9, dtype=torch.float32).item()


def test_factory_defaults_and_introspection():
    from pbs_attn.patch.huggingface import get_permuted_block_sparse_attn_fwd
    fn = get_permuted_block_sparse_attn_fwd()
    assert isinstance(fn, partial)
    assert fn.func.__name__ == "permuted_block_sparse_attn_fwd"
    assert fn.keywords == dict(block_size=128, segment_size=256, threshold=0.9, causal=True,
                               force_select_first_block=True, use_triton=True, query_pool_mode="mean",
                               key_pool_mode="mean")
    names = fn.func.__code__.co_varnames[:fn.func.__code__.co_argcount]
    assert names == ("query_states", "key_states", "value_states", "block_size", "segment_size", "threshold",
                     "causal", "force_select_first_block", "use_triton", "query_pool_mode", "key_pool_mode")
    assert "layer_idx" not in fn.func.__code__.co_varnames


def test_product_path_has_no_cpu_fallback():
    from pbs_attn_amd import permuted_block_sparse_attn_fwd
    from pbs_attn_amd._lib import PbsHipError
    q = torch.zeros((1, 2, 512, 128), dtype=torch.bfloat16)
    with pytest.raises(PbsHipError):
        permuted_block_sparse_attn_fwd(q, q, q, 128, 256, 0.9, True)


# ------------------------------------------------------------------ patcher on tiny models
def _tiny(kind, layers=2):
    from transformers import LlamaConfig, LlamaForCausalLM, Qwen2Config, Qwen2ForCausalLM
    torch.manual_seed(0)
    common = dict(hidden_size=64, intermediate_size=128, num_hidden_layers=layers, num_attention_heads=4,
                  num_key_value_heads=2, vocab_size=97, max_position_embeddings=512)
    if kind == "llama":
        return LlamaForCausalLM(LlamaConfig(head_dim=16, **common)).eval()
    return Qwen2ForCausalLM(Qwen2Config(**common)).eval()


def _oracle_prefill(**kw):
    def oracle_prefill(query_states, key_states, value_states):
        return O.permuted_block_sparse_attn_fwd(query_states, key_states, value_states, **kw)
    return oracle_prefill


@pytest.mark.parametrize("kind", ["llama", "qwen2"])
def test_patched_model_with_full_selection_equals_unpatched(kind):
    from pbs_attn.patch.huggingface import apply_patch_with_prefill
    model = _tiny(kind)
    ids = torch.randint(0, 97, (2, 48), generator=torch.Generator().manual_seed(1))
    with torch.no_grad():
        ref = model(ids).logits
        apply_patch_with_prefill(model, _oracle_prefill(block_size=8, segment_size=16, threshold=1))
        got = model(ids).logits
    assert torch.allclose(got, ref, atol=2e-4)
    for layer in model.model.layers:
        assert hasattr(layer.self_attn, "original_forward")


def test_skip_layers_and_errors():
    from pbs_attn.patch.huggingface import apply_patch_with_prefill
    model = _tiny("llama", layers=3)
    apply_patch_with_prefill(model, _oracle_prefill(block_size=8, segment_size=16, threshold=1), skip_layers=[1])
    assert hasattr(model.model.layers[0].self_attn, "original_forward")
    assert not hasattr(model.model.layers[1].self_attn, "original_forward")
    with pytest.raises(ValueError):
        apply_patch_with_prefill(torch.nn.Linear(2, 2), _oracle_prefill(block_size=8, segment_size=16, threshold=1))
    m2 = _tiny("llama")
    apply_patch_with_prefill(m2, None)
    with pytest.raises(RuntimeError, match="prefill_fn required"):
        m2(torch.randint(0, 97, (1, 8)))


def test_generate_prefill_then_decode_uses_unpermuted_cache():
    from pbs_attn.patch.huggingface import apply_patch_with_prefill
    model = _tiny("llama")
    ids = torch.randint(0, 97, (1, 40), generator=torch.Generator().manual_seed(2))
    with torch.no_grad():
        ref = model.generate(ids, max_new_tokens=4, do_sample=False)
        apply_patch_with_prefill(model, _oracle_prefill(block_size=8, segment_size=16, threshold=1))
        got = model.generate(ids, max_new_tokens=4, do_sample=False)
    assert torch.equal(got, ref)


def test_layer_idx_is_passed_when_the_kernel_asks_for_it():
    from pbs_attn.patch.huggingface import apply_patch_with_prefill
    seen = []

    def prefill_with_layer(query_states, key_states, value_states, layer_idx=None):
        seen.append((layer_idx, key_states.shape[1]))
        return torch.nn.functional.scaled_dot_product_attention(query_states, key_states, value_states, is_causal=True)

    model = _tiny("qwen2")
    apply_patch_with_prefill(model, partial(prefill_with_layer))
    with torch.no_grad():
        model(torch.randint(0, 97, (1, 12)))
    assert seen == [(0, 4), (1, 4)]            # K/V repeated to the 4 query heads


def test_native_gqa_kernels_get_unrepeated_kv():
    from pbs_attn.patch.huggingface import apply_patch_with_prefill
    shapes = []

    def gqa_prefill(query_states, key_states, value_states):
        shapes.append(key_states.shape[1])
        return O.permuted_block_sparse_attn_fwd(query_states, key_states, value_states, 8, 16, 1)
    gqa_prefill.native_gqa = True
    model = _tiny("llama")
    ids = torch.randint(0, 97, (1, 40), generator=torch.Generator().manual_seed(3))
    with torch.no_grad():
        ref = model(ids).logits
        apply_patch_with_prefill(model, gqa_prefill)
        got = model(ids).logits
    assert shapes == [2, 2] and torch.allclose(got, ref, atol=2e-4)


def test_synthetic_generators_are_seeded_and_shaped():
    from pbs_attn_amd.synth import WORKLOADS, make_qkv
    a = make_qkv(1, 4, 2, 256, 128, "uniform_heavy", seed=5)
    b = make_qkv(1, 4, 2, 256, 128, "uniform_heavy", seed=5)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    assert a[0].shape == (1, 4, 256, 128) and a[1].shape == (1, 2, 256, 128) and a[0].dtype == torch.bfloat16
    for kind in ("span_heavy", "local_window", "strong_heavy", "strong_uniform"):
        q, k, v = make_qkv(2, 4, 1, 640, 128, kind, seed=1)
        assert q.shape == (2, 4, 640, 128) and torch.isfinite(q.float()).all()
    assert set(WORKLOADS) >= {"cfg0", "cfg1", "cfg2", "cfg3"}


def test_bench_refuses_more_than_one_gpu_and_cpu_only_hosts():
    import subprocess
    import sys
    bench = os.path.join(ROOT, "bench.py")
    r = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout.strip() == ""
    if not torch.cuda.is_available():
        r = subprocess.run([sys.executable, bench], capture_output=True, text=True, timeout=120)
        assert r.returncode == 1 and "no GPU" in r.stderr and r.stdout.strip() == ""


def test_ttft_model_specs_match_the_named_architectures():
    from pbs_attn_amd.ttft import MODELS
    m = MODELS["llama31_8b"]
    assert (m["hidden_size"], m["num_hidden_layers"], m["num_attention_heads"], m["num_key_value_heads"],
            m["head_dim"], m["intermediate_size"], m["vocab_size"], m["rope_theta"]) == \
        (4096, 32, 32, 8, 128, 14336, 128256, 500000.0)
    q = MODELS["qwen25_7b"]
    assert (q["num_attention_heads"], q["num_key_value_heads"], q["hidden_size"] // q["num_attention_heads"]) == (28, 4, 128)


def test_operator_is_registered_with_the_dispatcher():
    """torch.ops.pbs_hip.prefill_attn_fwd: schema, shape-only implementation for tracing, no CPU kernel."""
    import pbs_attn_amd.torch_ops as T
    schema = str(torch.ops.pbs_hip.prefill_attn_fwd.default._schema)
    assert schema.startswith("pbs_hip::prefill_attn_fwd(Tensor q, Tensor k, Tensor v, int block_size, int segment_size")
    assert "Tensor? threshold_per_head" in schema and schema.endswith("-> Tensor")
    q = torch.empty(2, 4, 300, 128, dtype=torch.bfloat16, device="meta")
    k = torch.empty(2, 2, 300, 128, dtype=torch.bfloat16, device="meta")
    out = T.prefill_attn_fwd(q, k, k, 128, 256, 0.9)
    assert out.shape == q.shape and out.dtype == q.dtype and out.device.type == "meta"
    out = T.prefill_attn_fwd(q, k, k, 128, 256, torch.full((2, 4), 0.8, device="meta"))
    assert out.shape == q.shape
    with pytest.raises(RuntimeError):     # the shape checks of the tracing implementation
        T.prefill_attn_fwd(q, k[:, :, :200], k[:, :, :200])
    qc = torch.zeros(1, 2, 256, 128, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError, match="CPU"):   # no CPU kernel, no fallback
        T.prefill_attn_fwd(qc, qc, qc)
