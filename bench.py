#!/usr/bin/env python3
"""PBS-Attn prefill-attention benchmark on one MI355X.

A step = one full pass of the hot path (key scoring, segment sort, key-block pooling,
block estimation + selection, K/V gather, block-sparse attention, un-permutation) over one
synthetic Llama-3.1-8B-shaped attention layer already resident in HBM.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2]

prints ONE JSON line.  The K timed steps are K calls of the operator as a caller
makes them (`permuted_block_sparse_attn_fwd`, one library call each); `value` is the
effective TFLOP/s of that pass (4 * 128 * 128 * 128 FLOP per visited block pair /
step time).  A second, untimed-for-`value` pass runs the same work stage by stage with
a HIP event after every stage: `stage_ms`, and `roofline`, which prices the dominant
kernel (the block-sparse attention) against the bf16 dense MFMA peak.  `cpu_baseline`
times the CPU restatement of the reference's torch path on a bounded sample on this
host's cores.  The default run adds the other configurations as extra keys: `cfg0` (4k), `cfg1`
(the 32k layer: segment 256, threshold 0.9), `cfg1_sweep` (threshold x segment size at 32k), `cfg3`
(the batched 7:1 layer), `permutation_ablation` (PBS against the un-permuted MeanPooling mode) and
`ttft_llama31_8b_64k` (time to first token of the 32-layer architecture on a 64k prompt, patched
against unpatched).
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
FLOP_PER_BLOCK_PAIR = 4.0 * 128 * 128 * 128
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary of the default workload; the attention kernel's HBM bytes per
# launch are read from its "traffic_bytes_per_launch" line when the run is that workload
TRAFFIC_PROFILE = "profiles/pipeline_cfg2_hbm_traffic.txt"


def measured_traffic(workload, kind, segment, threshold):
    """(bytes per launch, source file) of sparse_attn_kernel from the committed counter summary, or (None, None)."""
    import re
    if (workload, kind, segment, threshold) != ("cfg2", None, 1024, 0.9):
        return None, None
    try:
        with open(os.path.join(ROOT, TRAFFIC_PROFILE)) as f:
            m = re.search(r"^traffic_bytes_per_launch\s+sparse_attn_kernel\s+([0-9.eE+]+)\s*$", f.read(), re.M)
    except OSError:
        return None, None
    return (float(m.group(1)), TRAFFIC_PROFILE) if m else (None, None)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class StageTimer:
    """Records a HIP event after every stage of every step on the launch stream."""

    def __init__(self, torch):
        self.torch = torch
        self.steps = []

    def begin(self):
        ev = self.torch.cuda.Event(enable_timing=True)
        ev.record()
        self.steps.append([("start", ev)])

    def mark(self, name):
        ev = self.torch.cuda.Event(enable_timing=True)
        ev.record()
        self.steps[-1].append((name, ev))

    def summary(self):
        tot = {}
        for marks in self.steps:
            for (_, e0), (name, e1) in zip(marks[:-1], marks[1:]):
                tot.setdefault(name, []).append(e0.elapsed_time(e1))
        return {k: sum(v) / len(v) for k, v in tot.items()}


_probe_lib = None


def load_probe_library():
    """libpbs_probe.so: the measurement kernels (an MFMA-only loop, the attention kernel's tile pipeline alone).
    Bench-only: built next to the operator's library, not part of its ABI."""
    global _probe_lib
    if _probe_lib is None:
        import ctypes
        from ctypes import c_double, c_int, c_void_p
        from pbs_attn_amd import _lib
        _lib.load()   # the probe library takes its error helpers from the operator's library
        lib = ctypes.CDLL(os.path.join(os.path.dirname(_lib.LIB_PATH), "libpbs_probe.so"))
        lib.pbs_mfma_probe.restype, lib.pbs_mfma_probe.argtypes = c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p]
        lib.pbs_mfma_probe_flop.restype, lib.pbs_mfma_probe_flop.argtypes = c_double, [c_int]
        lib.pbs_attn_tile_probe.restype = c_int
        lib.pbs_attn_tile_probe.argtypes = [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
        _probe_lib = lib
    return _probe_lib


def mfma_ceiling(torch, iters=100000):
    """What the matrix cores sustain on this GPU by themselves, on all-zero operands and on normally distributed
    ones (the rate depends on the values: the chip lowers its clock to stay inside its power limit), with the
    attention kernel's instruction (v_mfma_f32_16x16x32_bf16) and, for comparison, with v_mfma_f32_32x32x16_bf16.
    `normal` is the practical ceiling for a kernel fed with data like attention's."""
    from pbs_attn_amd import _lib
    lib = load_probe_library()
    dev = torch.device("cuda")
    sink = torch.empty(256 * 512, dtype=torch.float32, device=dev)
    gen = torch.Generator(device="cpu").manual_seed(7)
    pools = {"zeros": torch.zeros(65536, dtype=torch.bfloat16, device=dev),
             "normal": torch.randn(65536, generator=gen).to(torch.bfloat16).to(dev)}
    st = torch.cuda.current_stream().cuda_stream
    out = {"unit": "TFLOP/s", "kernel": "matrix instructions only, 256 workgroups x 8 waves: v_mfma_f32_16x16x32_bf16 "
                                        "(the attention kernel's; keys `zeros`, `normal`) and v_mfma_f32_32x32x16_bf16 (`*_32x32x16`)"}
    for shape, suffix in ((0, ""), (1, "_32x32x16")):
        for name, pool in pools.items():
            clocks = torch.zeros(2, dtype=torch.int64, device=dev)
            _lib.check(lib.pbs_mfma_probe(pool.data_ptr(), 2000, shape, sink.data_ptr(), clocks.data_ptr(), st), "pbs_mfma_probe")
            torch.cuda.synchronize()
            clocks.zero_()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _lib.check(lib.pbs_mfma_probe(pool.data_ptr(), iters, shape, sink.data_ptr(), clocks.data_ptr(), st), "pbs_mfma_probe")
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            c = clocks.tolist()
            out[name + suffix] = lib.pbs_mfma_probe_flop(iters) / ms / 1e9
            out[name + suffix + "_shader_clock_mhz"] = 100.0 * c[0] / max(1, c[1])
    return out


def tile_pipeline(torch, iters=6000):
    """The attention kernel's tile pipeline by itself (pbs_attn_tile_probe: fast tiles out of LDS with the
    kernel's barrier and copies per tile, no lists, items or write-out), on all-zero and on normally distributed
    K / V / Q: cycles per tile (the same on both), the time per tile and the shader clock the chip holds.  On data
    the clock falls with the power limit; what the attention kernel reaches of this rate is the cost of
    everything around the pipeline."""
    from pbs_attn_amd import _lib
    lib = load_probe_library()
    dev = torch.device("cuda")
    n_src = 256                                     # 16 MB ring of tile pairs
    sink = torch.empty(256 * 512, dtype=torch.float32, device=dev)
    gen = torch.Generator(device="cpu").manual_seed(11)
    rings = {"zeros": torch.zeros(n_src * 32768, dtype=torch.bfloat16, device=dev),
             "normal": torch.randn(n_src * 32768, generator=gen).to(torch.bfloat16).to(dev)}
    st = torch.cuda.current_stream().cuda_stream
    out = {"kernel": "fast tiles of 128 keys x 256 queries per workgroup, 256 workgroups x 8 waves, barrier per tile",
           "flop_per_tile_step": 2 * FLOP_PER_BLOCK_PAIR}
    for name, ring in rings.items():
        for copies in (1, 0):
            clocks = torch.zeros(2, dtype=torch.int64, device=dev)
            args = (ring.data_ptr(), n_src, None, copies, sink.data_ptr(), clocks.data_ptr(), st)
            _lib.check(lib.pbs_attn_tile_probe(*args[:2], iters // 8, *args[3:]), "pbs_attn_tile_probe")
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _lib.check(lib.pbs_attn_tile_probe(*args[:2], iters, *args[3:]), "pbs_attn_tile_probe")
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            c = clocks.tolist()
            key = name + ("" if copies else "_no_copies")
            out[key] = {"us_per_tile_step": ms * 1e3 / iters, "cycles_per_tile_step": c[0] / iters,
                        "shader_clock_mhz": 100.0 * c[0] / max(1, c[1]),
                        "tflops": 256 * 2 * FLOP_PER_BLOCK_PAIR * iters / (ms * 1e-3) / 1e12}
    return out


def block_pair_counts(csr_cnt, B, Hq, nb, bps):
    """(executed, reference) numbers of 128 x 128 tiles of one launch.  executed = what the HIP kernel
    multiplies: the selected blocks of earlier segments plus the causal part of the own segment (blocks
    first-of-segment .. query block, read in original key order).  reference = the tiles the reference's
    kernel visits for the same masks: the same selected blocks plus EVERY block of the own segment (in
    permuted order a block of the segment can hold visible keys wherever it lies)."""
    earlier = int(csr_cnt.sum().item())
    own_exec = sum(qb - (qb // bps) * bps + 1 for qb in range(nb))
    own_all = sum(min((qb // bps) * bps + bps, nb) - (qb // bps) * bps for qb in range(nb))
    return earlier + B * Hq * own_exec, earlier + B * Hq * own_all


def cpu_baseline(cfg, q, k, v, seconds_budget=20.0):
    """The reference's torch CPU path (restated in oracle/) on the SAME workload,
    bounded to whole query heads: head after head until `seconds_budget` is spent
    (at least one).  The rate is visited-block FLOPs per second of CPU time."""
    import torch
    from oracle import pbs_oracle as O
    G = cfg["Hq"] // cfg["Hkv"]
    flops, spent, heads = 0.0, 0.0, 0
    for h in range(cfg["Hq"]):
        qs = q[:1, h:h + 1].cpu()
        ks, vs = k[:1, h // G:h // G + 1].cpu(), v[:1, h // G:h // G + 1].cpu()
        t0 = time.perf_counter()
        _, mid = O.permuted_block_sparse_attn_fwd(qs, ks, vs, cfg["block"], cfg["segment"], cfg["threshold"],
                                                  return_intermediates=True)
        spent += time.perf_counter() - t0
        flops += O.visited_block_pairs(mid["final_mask"], cfg["segment"] // cfg["block"]) * FLOP_PER_BLOCK_PAIR
        heads += 1
        log(f"[bench] cpu baseline: head {h} done, {spent:.1f} s so far")
        if spent > seconds_budget:
            break
    return {"value": flops / spent / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle torch CPU path on {heads} of {cfg['B'] * cfg['Hq']} (batch, query head) slices of the "
                      f"same workload (S={cfg['S']}, segment {cfg['segment']}, threshold {cfg['threshold']}), "
                      f"{spent:.1f} s, os.cpu_count()={os.cpu_count()}",
            "ms_per_head": spent / heads * 1e3}


def dense_sdpa_ms(torch, q, k, v, reps=3):
    """Dense causal flash attention of the torch ROCm wheel on the same tensors."""
    F = torch.nn.functional
    try:
        from torch.nn.attention import SDPBackend, sdpa_kernel
        ctx = lambda: sdpa_kernel([SDPBackend.FLASH_ATTENTION])  # noqa: E731
        with ctx():
            F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        with ctx():
            for _ in range(reps):
                F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps
    except Exception as exc:  # the baseline is informative only
        log(f"[bench] dense SDPA baseline unavailable: {type(exc).__name__}: {exc}")
        return None


def run_workload(torch, name, steps, warmup, seed=0, overrides=None, with_dense=True, with_zero_operands=False, min_warm_ms=0.0):
    from pbs_attn_amd import pbs as P
    from pbs_attn_amd.synth import make_workload
    dev = torch.device("cuda:0")
    cfg, q, k, v = make_workload(name, seed=seed, device=dev, **(overrides or {}))
    B, Hq, Hkv, S, D = cfg["B"], cfg["Hq"], cfg["Hkv"], cfg["S"], cfg["D"]
    bs, seg, thr = cfg["block"], cfg["segment"], cfg["threshold"]
    nb = (S + bs - 1) // bs

    def step():
        return P.permuted_block_sparse_attn_fwd(q, k, v, bs, seg, thr, True)

    # the timed region: the operator as a caller makes it (no profiling hook: one library call per step)
    assert P.stage_timer is None
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # short steps (the side measurements of small workloads): keep warming until the chip has been under load for
    # min_warm_ms, or the first timed steps run at the clock of an idle GPU
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < min_warm_ms:
        step()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = step()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    # the same work stage by stage, a HIP event on the launch stream after every stage
    timer = StageTimer(torch)
    P.stage_timer = timer
    try:
        timer.begin()
        step()
        torch.cuda.synchronize()
        timer.steps.clear()
        t0 = time.perf_counter()
        for _ in range(steps):
            timer.begin()
            out = step()
        torch.cuda.synchronize()
        staged_ms = (time.perf_counter() - t0) * 1e3 / steps
    finally:
        P.stage_timer = None
    stages = timer.summary()

    # visited block pairs of this input (one extra selection pass, outside the timed region)
    perm = P.apply_permutation(q, k, v, bs, seg)
    sel = P.permuted_block_selection(q, perm, bs, seg, thr, want_masks=False)
    n_vis, n_ref = block_pair_counts(sel["csr_cnt"], B, Hq, nb, seg // bs)
    causal_pairs = B * Hq * nb * (nb + 1) // 2
    flops = n_vis * FLOP_PER_BLOCK_PAIR
    attn_ms = stages["sparse_attn"]
    res = {
        "workload": name, "B": B, "Hq": Hq, "Hkv": Hkv, "S": S, "D": D, "block": bs, "segment": seg,
        "threshold": thr, "generator": cfg["kind"], "seed": seed,
        "ms_per_step": wall_ms, "ms_per_step_staged": staged_ms, "stage_ms": stages, "visited_block_pairs": n_vis,
        "reference_block_pairs": n_ref,
        "density_vs_causal": n_vis / causal_pairs,
        "effective_tflops_pipeline": flops / (wall_ms * 1e-3) / 1e12,
        "effective_tflops_attn_kernel": flops / (attn_ms * 1e-3) / 1e12,
        "dense_causal_flop": 4.0 * S * S * D / 2 * Hq * B,
    }
    # HBM-bound stages: algorithmic bytes / stage time.  With a real threshold the gather runs after the
    # selection and moves only the key blocks some query block visits (fraction f of all permuted blocks)
    e = 2
    f = 1.0
    if "pool" in stages:
        _, sel2 = P._select_then_gather(q, k, v, bs, seg, thr, True, "mean", "mean")
        f = float(sel2["block_needed"].float().mean().item())
        del sel2
    res["gathered_block_fraction"] = f
    kv_once = B * Hkv * S * D * e                       # one of K, V at the KV heads
    score_b = kv_once + B * Hq * bs * D * e + B * Hq * S * 4
    pool_b = kv_once + B * Hq * S * 4 + 2 * B * Hq * nb * D * e + B * Hq * S * D * e    # K, indices, Q in; pooled out
    # reads: the K and V rows of the gathered blocks (each row counted once per KV head at most) and their indices;
    # writes: the gathered tiles.
    gather_b = 2 * min(f * B * Hq, B * Hkv) * S * D * e + f * B * Hq * S * 4 + 2 * f * B * Hq * S * D * e
    est_b = (0 if "pool" in stages else B * Hq * S * D * e) + 2 * B * Hq * nb * D * e + B * Hq * nb * nb * 4
    res["hbm_gbs"] = {
        "score": score_b / (stages["score"] * 1e-3) / 1e9 if "score" in stages else None,
        "pool": pool_b / (stages["pool"] * 1e-3) / 1e9 if "pool" in stages else None,
        "gather": gather_b / (stages["gather"] * 1e-3) / 1e9,
        "estimate": est_b / (stages["estimate"] * 1e-3) / 1e9 if "estimate" in stages else None,
    }
    if with_zero_operands:
        # the same launch (same visit lists, same schedule) on all-zero Q, K, V: what the kernel's schedule
        # delivers when the matrix cores draw the least power
        from pbs_attn_amd import ops
        zq, zk, zv = torch.zeros_like(q), torch.zeros_like(perm.perm_k), torch.zeros_like(perm.perm_vt)
        zargs = (zq, zk, zv, torch.zeros_like(k), torch.zeros_like(v), sel["csr_cols"], sel["csr_cnt"], seg)
        ops.sparse_attn_fwd(*zargs)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(2):
            ops.sparse_attn_fwd(*zargs)
        e1.record()
        torch.cuda.synchronize()
        res["attn_ms_zero_operands"] = e0.elapsed_time(e1) / 2
        del zq, zk, zv
    if with_dense:
        res["dense_sdpa_ms"] = dense_sdpa_ms(torch, q, k, v)
        # the build's own kernel on the full causal mask (every candidate selected, one block per segment)
        for _ in range(2):
            P.permuted_block_sparse_attn_fwd(q, k, v, bs, bs, 1, True)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        P.permuted_block_sparse_attn_fwd(q, k, v, bs, bs, 1, True)
        e1.record()
        torch.cuda.synchronize()
        res["dense_own_kernel_ms"] = e0.elapsed_time(e1)
        if res["dense_sdpa_ms"]:
            res["speedup_vs_dense_sdpa"] = res["dense_sdpa_ms"] / wall_ms
    del out
    return res, (cfg, q, k, v)


def meanpooling_mode(torch, cfg, q, k, v, reps=2):
    """The reference's MeanPooling baseline on the same tensors (`get_meanpooling_prefill`: PBS without the
    permutation; same block size and threshold): block density of its mask and the time of one pass."""
    from pbs_attn_amd.meanpooling import MeanPooling_prefill
    B, Hq, S, bs, thr = cfg["B"], cfg["Hq"], cfg["S"], cfg["block"], cfg["threshold"]
    nb = (S + bs - 1) // bs
    _, mid = MeanPooling_prefill(q, k, v, bs, cfg["segment"], thr, return_masks=True)
    pairs = int(mid["csr_cnt"].sum().item()) + B * Hq * nb          # selected earlier blocks + the diagonal block
    del mid
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        MeanPooling_prefill(q, k, v, bs, cfg["segment"], thr)
    e1.record()
    torch.cuda.synchronize()
    return pairs / (B * Hq * nb * (nb + 1) // 2), e0.elapsed_time(e1) / reps


def side_summary(torch, name, overrides, steps, warmup, with_dense=True):
    """One more configuration measured like the headline one, condensed to the figures of a table row."""
    r, inputs = run_workload(torch, name, steps, warmup, overrides=overrides, with_dense=with_dense, min_warm_ms=150.0)
    del inputs
    torch.cuda.empty_cache()
    log(f"[bench] {name} {overrides} " + json.dumps(r))
    a = r["visited_block_pairs"] * FLOP_PER_BLOCK_PAIR / (r["stage_ms"]["sparse_attn"] * 1e-3) / 1e12
    out = {"workload": f"{name}: B={r['B']} Hq={r['Hq']} Hkv={r['Hkv']} S={r['S']}, block {r['block']}, segment {r['segment']}, "
                       f"threshold {r['threshold']}, generator {r['generator']} seed {r['seed']}",
           "segment": r["segment"], "threshold": r["threshold"],
           "ms_per_step": r["ms_per_step"], "value": r["effective_tflops_pipeline"], "unit": "TFLOP/s",
           "density_vs_causal": r["density_vs_causal"], "stage_ms": r["stage_ms"],
           "attn_kernel_tflops": a, "attn_kernel_frac_of_peak": a / PEAK_BF16_TFLOPS}
    if with_dense:
        out.update(dense_sdpa_ms=r.get("dense_sdpa_ms"), dense_own_kernel_ms=r.get("dense_own_kernel_ms"),
                   speedup_vs_dense_sdpa=r.get("speedup_vs_dense_sdpa"))
    return out


def ablation(torch, name, overrides, res):
    """PBS (permuted) against MeanPooling_prefill (the same estimate and selection without the permutation) on one
    input: block density of the two masks and the time of one pass each."""
    from pbs_attn_amd.synth import make_workload
    if res is None:
        res, (cfg, q, k, v) = run_workload(torch, name, 3, 2, overrides=overrides, with_dense=False)
    else:
        cfg, q, k, v = make_workload(name, seed=0, device=torch.device("cuda:0"), **overrides)
    mp_density, mp_ms = meanpooling_mode(torch, cfg, q, k, v)
    del q, k, v
    torch.cuda.empty_cache()
    return {"workload": f"{name}: S={cfg['S']}, segment {cfg['segment']}, threshold {cfg['threshold']}, generator {cfg['kind']}",
            "pbs_density": res["density_vs_causal"], "pbs_ms": res["ms_per_step"],
            "meanpooling_density": mp_density, "meanpooling_ms": mp_ms}


def ttft_pair(torch, length=65536, runs=3, warmup=1, model_name="llama31_8b", layers=None):
    """Time to first token of the random-init architecture on a `length`-token prompt of uniform random ids:
    the unpatched model (torch SDPA) and the same model patched with the PBS prefill (defaults: block 128,
    segment 256, threshold 0.9).  `runs` timed generations each after `warmup` untimed ones."""
    import contextlib
    from pbs_attn_amd import ttft
    from pbs_attn_amd.patch.huggingface import apply_patch_with_prefill, get_permuted_block_sparse_attn_fwd
    t0 = time.perf_counter()
    model = ttft.build_model(model_name, layers)
    out = {"model": model_name, "layers": model.config.num_hidden_layers, "num_tokens": length, "runs": runs,
           "warmup": warmup, "weights": "random init", "prompts": "uniform random token ids", "unit": "s"}
    dense = ttft.measure(model, length, warmup, runs)
    with contextlib.redirect_stdout(sys.stderr):
        apply_patch_with_prefill(model, get_permuted_block_sparse_attn_fwd())
    pbs = ttft.measure(model, length, warmup, runs)
    out.update(pbs_s=sum(pbs) / runs, dense_s=sum(dense) / runs, pbs_runs=pbs, dense_runs=dense,
               speedup_vs_dense=sum(dense) / sum(pbs), wall_s=time.perf_counter() - t0)
    del model
    torch.cuda.empty_cache()
    return out


def run_report(torch, path, steps, warmup):
    """Every single-layer benchmark configuration + sweeps, written as a markdown table."""
    runs = [("cfg0", {}), ("cfg1", {})]
    runs += [("cfg1", {"segment": sg, "threshold": th}) for sg in (256, 1024) for th in (0.8, 0.9, 0.95)
             if not (sg == 256 and th == 0.9)]
    runs += [("cfg2", {}), ("cfg3", {}), ("cfg3", {"segment": 1024}),
             ("cfg1", {"kind": "strong_heavy", "segment": 1024}), ("cfg2", {"kind": "strong_heavy"}),
             ("cfg2", {"kind": "strong_uniform"})]
    lines = ["| workload | generator | S | B x Hq/Hkv | segment | thr | density | MeanPooling density | MeanPooling ms | pass ms | "
             "attn ms | attn TFLOP/s | % MFMA peak | dense SDPA ms | speed-up vs dense | score/sort/pool/estimate/select/gather ms |",
             "|---|---|---|---|---|---|---|---|---|---|---|---|---|---|---|---|"]
    out = []
    for name, ov in runs:
        res, (cfg, q, k, v) = run_workload(torch, name, steps, warmup, overrides=ov, with_dense=True, min_warm_ms=150.0)
        res["density_unpermuted"], res["meanpooling_ms"] = meanpooling_mode(torch, cfg, q, k, v)
        del q, k, v
        torch.cuda.empty_cache()
        st = res["stage_ms"]
        lines.append(
            f"| {name} | {res['generator']} | {res['S']} | {res['B']} x {res['Hq']}/{res['Hkv']} | {res['segment']} | "
            f"{res['threshold']} | {res['density_vs_causal']:.3f} | {res['density_unpermuted']:.3f} | {res['meanpooling_ms']:.2f} | {res['ms_per_step']:.2f} | "
            f"{st['sparse_attn']:.2f} | {res['effective_tflops_attn_kernel']:.0f} | "
            f"{100 * res['effective_tflops_attn_kernel'] / PEAK_BF16_TFLOPS:.1f} | "
            f"{res['dense_sdpa_ms']:.2f} | {res['dense_sdpa_ms'] / res['ms_per_step']:.2f} | "
            f"{st.get('score', 0):.2f}/{st.get('sort', 0):.2f}/{st.get('pool', 0):.2f}/{st.get('estimate', 0):.2f}/"
            f"{st['select']:.2f}/{st['gather']:.2f} |")
        log(lines[-1])
        out.append(res)
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="cfg2", help="cfg0 | cfg1 | cfg2 | cfg3 (see pbs_attn_amd/synth.py)")
    ap.add_argument("--segment", type=int, default=None)
    ap.add_argument("--threshold", type=float, default=None)
    ap.add_argument("--kind", default=None, help="override the input generator, e.g. strong_heavy")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-dense", action="store_true")
    ap.add_argument("--no-mfma-probe", action="store_true", help="skip the MFMA-only ceiling measurement")
    ap.add_argument("--cpu-seconds", type=float, default=20.0)
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the extra measurements of the default run (the other configurations, the ablation, the 64k time to first token)")
    ap.add_argument("--report", default=None, metavar="FILE.md",
                    help="run every single-layer configuration and the sweeps, write a markdown table, and exit")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="also run one plain device copy of Q (known bytes) so that rocprofv3 --pmc FETCH_SIZE / "
                         "WRITE_SIZE readings can be scaled")
    args = ap.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this path is measured on ONE GPU (it shards over heads with no exchange); "
            "run with --gpus 1.")
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible; the HIP path has no CPU fallback.")
        sys.exit(1)
    from pbs_attn_amd import _lib
    _lib.load()

    if args.report:
        res = run_report(torch, args.report, args.steps, args.warmup)
        print(json.dumps({"report": args.report, "rows": len(res)}), flush=True)
        return
    overrides = {}
    if args.segment:
        overrides["segment"] = args.segment
    if args.threshold is not None:
        overrides["threshold"] = args.threshold
    if args.kind:
        overrides["kind"] = args.kind
    res, inputs = run_workload(torch, args.workload, args.steps, args.warmup, overrides=overrides,
                               with_dense=not args.no_dense, with_zero_operands=not args.no_mfma_probe)
    log("[bench] " + json.dumps(res))
    if args.traffic_calibration:
        cfg, q = inputs[0], inputs[1]
        dst = torch.empty_like(q)
        dst.copy_(q)
        torch.cuda.synchronize()
        log(f"[bench] calibration copy: {q.numel() * q.element_size()} bytes read and written by one copy kernel")

    attn_s = res["stage_ms"]["sparse_attn"] * 1e-3
    achieved = res["visited_block_pairs"] * FLOP_PER_BLOCK_PAIR / attn_s / 1e12
    traffic, traffic_source = measured_traffic(args.workload, args.kind, res["segment"], res["threshold"])
    line = {
        "metric": "pbs_prefill_attn_effective_tflops",
        "value": res["effective_tflops_pipeline"],
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: Llama-3.1-8B attention layer B={res['B']} Hq={res['Hq']} "
                               f"Hkv={res['Hkv']} D={res['D']} S={res['S']}, block {res['block']}, segment "
                               f"{res['segment']}, threshold {res['threshold']}, generator {res['generator']} seed {res['seed']}",
                   "density_vs_causal": res["density_vs_causal"],
                   "visited_block_pairs": res["visited_block_pairs"],
                   "reference_block_pairs": res["reference_block_pairs"]},
        "roofline": {"bound": "mfma", "kernel": "sparse_attn_kernel", "achieved": achieved, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS,
                     "traffic": traffic, "traffic_unit": "bytes/launch", "traffic_source": traffic_source,
                     "kernel_ms": res["stage_ms"]["sparse_attn"]},
        "stage_ms": res["stage_ms"],
        "ms_per_step_staged": res["ms_per_step_staged"],
        "hbm_gbs": res["hbm_gbs"],
        "gathered_block_fraction": res["gathered_block_fraction"],
        "dense_sdpa_ms": res.get("dense_sdpa_ms"),
        "dense_own_kernel_ms": res.get("dense_own_kernel_ms"),
        "speedup_vs_dense_sdpa": res.get("speedup_vs_dense_sdpa"),
    }
    if not args.no_mfma_probe:
        # context for roofline.frac: `peak` stays the published figure, this is what the matrix cores
        # sustain on this GPU on their own
        line["mfma_ceiling"] = mfma_ceiling(torch)
        line["roofline"]["frac_of_measured_ceiling"] = achieved / line["mfma_ceiling"]["normal"]
        line["roofline"]["kernel_ms_zero_operands"] = res["attn_ms_zero_operands"]
        line["tile_pipeline"] = tile_pipeline(torch)
        line["roofline"]["frac_of_tile_pipeline"] = achieved / line["tile_pipeline"]["normal"]["tflops"]
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(*inputs, seconds_budget=args.cpu_seconds)
    del inputs
    torch.cuda.empty_cache()
    if not (args.no_extras or overrides or args.workload != "cfg2"):
        # the other figures the headline metric names and the other configurations, measured the same way in the same run
        line["cfg1"] = side_summary(torch, "cfg1", {}, steps=max(args.steps, 10), warmup=max(args.warmup, 3))
        line["cfg0"] = side_summary(torch, "cfg0", {}, steps=20, warmup=5)
        line["cfg3"] = side_summary(torch, "cfg3", {}, steps=10, warmup=3)
        # config 1's sweep: threshold x segment size on the 32k layer (the dense baseline is the one of `cfg1`)
        line["cfg1_sweep"] = [side_summary(torch, "cfg1", {"threshold": th, "segment": sg}, steps=5, warmup=2, with_dense=False)
                              for sg in (256, 1024) for th in (0.8, 0.9, 0.95)]
        # the sparse regime: the headline shape on an input whose attention has the structure PBS exploits
        line["cfg2_strong_heavy"] = side_summary(torch, "cfg2", {"kind": "strong_heavy"}, steps=10, warmup=3, with_dense=False)
        # what the permutation buys: PBS against the reference's un-permuted MeanPooling baseline (same block size
        # and threshold through the same kernels) on the headline input and on one whose heavy keys are scattered
        line["permutation_ablation"] = [ablation(torch, "cfg2", {}, res), ablation(torch, "cfg2", {"kind": "strong_uniform"}, None)]
        line["ttft_llama31_8b_64k"] = ttft_pair(torch)
        log("[bench] ttft " + json.dumps(line["ttft_llama31_8b_64k"]))
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
