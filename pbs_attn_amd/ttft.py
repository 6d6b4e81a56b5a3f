"""Offline time-to-first-token harness: the measurement protocol of the reference's
eval/efficiency/eval_efficiency.py without its network dependencies.

Same protocol: ``num_warmup_iter`` (default 30, :37) warm-up ``generate(max_new_tokens=1)`` calls on
one random prompt (:136-144), then ``n_examples`` (default 10, :36) prompts of exactly ``len`` tokens,
each timed with device events around ``generate(max_new_tokens=1, do_sample=False)`` after a
synchronize (:147-157), mean and standard deviation (:243-258), and a result file
``<output_dir>/<method>_<len>.json`` holding script_args, method_args, model_name, num_tokens,
avg_e2e_latency and e2e_std (:261-290).  What differs, because there is no network: the model is
random-initialised from a local config of the named architecture instead of ``from_pretrained``, and
the prompts are uniform random token ids instead of tokenised LongBench-v2 contexts (both recorded
in the result).

    python -m pbs_attn_amd.ttft --method pbs --len 65536
    python -m pbs_attn_amd.ttft --method dense --len 65536          # unpatched model, torch SDPA
    python -m pbs_attn_amd.ttft --method meanpooling --len 32768

Methods: ``pbs`` (:68-73 PBSArgs), ``meanpooling`` (:60-66 MeanPoolingArgs), ``dense`` (the unpatched
model; the reference's ``flash`` baseline needs the flash_attn package).  Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

MODELS = {
    # Llama-3.1-8B architecture (the 64k time-to-first-token configuration)
    "llama31_8b": dict(family="llama", hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
                       num_attention_heads=32, num_key_value_heads=8, head_dim=128, vocab_size=128256,
                       rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=131072),
    # Qwen2.5-7B architecture
    "qwen25_7b": dict(family="qwen2", hidden_size=3584, intermediate_size=18944, num_hidden_layers=28,
                      num_attention_heads=28, num_key_value_heads=4, vocab_size=152064,
                      rms_norm_eps=1e-6, rope_theta=1000000.0, max_position_embeddings=131072),
}

METHODS = ("pbs", "meanpooling", "dense")


def build_model(name, layers=None, device="cuda", seed=0):
    import torch
    from transformers import LlamaConfig, LlamaForCausalLM, Qwen2Config, Qwen2ForCausalLM
    spec = dict(MODELS[name])
    family = spec.pop("family")
    if layers:
        spec["num_hidden_layers"] = layers
    torch.manual_seed(seed)
    cfg_cls, model_cls = (LlamaConfig, LlamaForCausalLM) if family == "llama" else (Qwen2Config, Qwen2ForCausalLM)
    cfg = cfg_cls(attn_implementation="sdpa", **spec)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(device):
            model = model_cls(cfg)
    finally:
        torch.set_default_dtype(prev)
    return model.eval()


def build_prefill_fn(method, method_args):
    """eval_efficiency.py:75-110 for the methods this build has."""
    from pbs_attn_amd.patch.huggingface import get_meanpooling_prefill, get_permuted_block_sparse_attn_fwd
    if method == "pbs":
        return get_permuted_block_sparse_attn_fwd(**method_args)
    if method == "meanpooling":
        return get_meanpooling_prefill(**method_args)
    raise ValueError(f"Unknown method: {method}")


def warmup_generate(model, length, num_iter, seed=0):
    """eval_efficiency.py:136-144: one random prompt, generated `num_iter` times."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    vocab = model.get_input_embeddings().weight.size(0)
    ids = torch.randint(0, vocab, (1, length), generator=g).to(model.device)
    with torch.no_grad():
        for _ in range(num_iter):
            model.generate(input_ids=ids, max_new_tokens=1, do_sample=False)


def measure_prefill_latency(model, input_ids):
    """eval_efficiency.py:147-157."""
    import torch
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    with torch.no_grad():
        model.generate(input_ids=input_ids, max_new_tokens=1, do_sample=False)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / 1000.0


def measure(model, length, warmup, iters, seed=1):
    """Warm-up, then `iters` fresh random prompts of `length` tokens; returns the latencies in seconds."""
    import torch
    warmup_generate(model, length, warmup, seed=seed - 1)
    g = torch.Generator(device="cpu").manual_seed(seed)
    vocab = model.get_input_embeddings().weight.size(0)
    times = []
    for _ in range(iters):
        ids = torch.randint(0, vocab, (1, length), generator=g).to(model.device)
        times.append(measure_prefill_latency(model, ids))
    return times


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--method", default="pbs", choices=METHODS)
    ap.add_argument("--len", type=int, default=65536, dest="length", help="length of the input sequence")
    ap.add_argument("--n-examples", "--iters", type=int, default=10, dest="n_examples")
    ap.add_argument("--num-warmup-iter", "--warmup", type=int, default=30, dest="num_warmup_iter")
    ap.add_argument("--no-save", action="store_true")
    ap.add_argument("--output-dir", default="results")
    ap.add_argument("--model", default="llama31_8b", choices=sorted(MODELS), dest="model_name")
    ap.add_argument("--layers", type=int, default=None, help="override the number of decoder layers")
    ap.add_argument("--block-size", type=int, default=128)
    ap.add_argument("--segment-size", type=int, default=None, help="default 256 for pbs, 1024 for meanpooling")
    ap.add_argument("--threshold", type=float, default=0.9)
    ap.add_argument("--no-force-select-first-block", action="store_true")
    args = ap.parse_args(argv)

    import torch
    if not torch.cuda.is_available():
        print("ttft: needs the GPU", file=sys.stderr)
        return 1
    method_args = {}
    if args.method in ("pbs", "meanpooling"):
        method_args = dict(block_size=args.block_size,
                           segment_size=args.segment_size or (256 if args.method == "pbs" else 1024),
                           threshold=args.threshold, force_select_first_block=not args.no_force_select_first_block)
    t0 = time.time()
    model = build_model(args.model_name, args.layers)
    if args.method != "dense":
        import contextlib
        from pbs_attn_amd.patch.huggingface import apply_patch_with_prefill
        with contextlib.redirect_stdout(sys.stderr):   # keep stdout to the one JSON line
            apply_patch_with_prefill(model, build_prefill_fn(args.method, method_args))
    print(f"[ttft] model built in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    times = measure(model, args.length, args.num_warmup_iter, args.n_examples)
    avg = sum(times) / len(times)
    script_args = dict(method=args.method, len=args.length, n_examples=args.n_examples,
                       num_warmup_iter=args.num_warmup_iter, no_save=args.no_save, output_dir=args.output_dir,
                       model_name=args.model_name)
    results = {
        "script_args": script_args,
        "method_args": method_args,
        "model_name": args.model_name,
        "tokenizer_name": None,
        "num_tokens": args.length,
        "avg_e2e_latency": avg,
    }
    if len(times) > 1:
        results["e2e_std"] = torch.tensor(times).std().item()
    # what the offline harness adds to the reference's record
    results.update(e2e_latencies=times, layers=model.config.num_hidden_layers, weights="random init",
                   prompts="uniform random token ids", dtype="bf16")
    file_path = None
    if not args.no_save:
        results_dir = args.output_dir if os.path.isabs(args.output_dir) else os.path.join(os.getcwd(), args.output_dir)
        os.makedirs(results_dir, exist_ok=True)
        file_path = os.path.join(results_dir, f"{args.method}_{args.length}.json")
        with open(file_path, "w") as f:
            json.dump(results, f, indent=4)
        print(f"Results saved to {file_path}", file=sys.stderr)
    print(json.dumps({"metric": "ttft_s", "ttft_s": avg, "result_file": file_path, **results}), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
