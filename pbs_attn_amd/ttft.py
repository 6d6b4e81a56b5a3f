"""Offline time-to-first-token harness: the measurement protocol of the reference's
eval/efficiency/eval_efficiency.py (:136-157 -- warm-up generates on random ids, then
`generate(max_new_tokens=1)` timed with device events) without its network
dependencies: the model is random-initialised from a local config and the prompt is
uniform random token ids.

    python -m pbs_attn_amd.ttft --len 65536 --method pbs          # patched with the HIP path
    python -m pbs_attn_amd.ttft --len 65536 --method dense        # unpatched, torch SDPA

prints one JSON line per run.
"""
from __future__ import annotations

import argparse
import json
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


def measure(model, length, warmup, iters, seed=1):
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    vocab = model.get_input_embeddings().weight.size(0)
    times = []
    with torch.no_grad():
        for i in range(warmup + iters):
            ids = torch.randint(0, vocab, (1, length), generator=g).to(model.device)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            model.generate(input_ids=ids, max_new_tokens=1, do_sample=False)
            e1.record()
            torch.cuda.synchronize()
            if i >= warmup:
                times.append(e0.elapsed_time(e1) / 1e3)
    return times


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", default="llama31_8b", choices=sorted(MODELS))
    ap.add_argument("--layers", type=int, default=None, help="override the number of decoder layers")
    ap.add_argument("--len", type=int, default=65536, dest="length")
    ap.add_argument("--method", default="pbs", choices=["pbs", "dense"])
    ap.add_argument("--block-size", type=int, default=128)
    ap.add_argument("--segment-size", type=int, default=256)
    ap.add_argument("--threshold", type=float, default=0.9)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--iters", type=int, default=3)
    args = ap.parse_args(argv)

    import torch
    if not torch.cuda.is_available():
        print("ttft: needs the GPU", file=sys.stderr)
        return 1
    t0 = time.time()
    model = build_model(args.model, args.layers)
    if args.method == "pbs":
        import contextlib
        from pbs_attn_amd.patch.huggingface import apply_patch_with_prefill, get_permuted_block_sparse_attn_fwd
        with contextlib.redirect_stdout(sys.stderr):   # keep stdout to the one JSON line
            apply_patch_with_prefill(model, get_permuted_block_sparse_attn_fwd(
                block_size=args.block_size, segment_size=args.segment_size, threshold=args.threshold))
    print(f"[ttft] model built in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    times = measure(model, args.length, args.warmup, args.iters)
    mean = sum(times) / len(times)
    print(json.dumps({"metric": "ttft_s", "model": args.model, "layers": model.config.num_hidden_layers,
                      "prompt_len": args.length, "method": args.method, "ttft_s": mean, "runs": times,
                      "block_size": args.block_size, "segment_size": args.segment_size, "threshold": args.threshold,
                      "weights": "random init", "prompt": "uniform random token ids", "dtype": "bf16"}), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
