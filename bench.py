#!/usr/bin/env python3
"""Benchmark of the MoBA attention path on one MI355X.

A step is one forward pass of ``moba_attn_varlen`` (chunk-mean, gate + top-k, gather
lists, fused attention, merge) over one synthetic batch already resident in HBM.
The default workload is the headline configuration: one sequence of 131072 tokens,
32 query heads (8 KV heads repeated to 32 before the operator, outside the timed
region), head_dim 128, chunk 4096, top-k 12, bf16.

Prints one JSON line: whole-operator effective TFLOP/s on the FLOPs actually required
(4*D per attended query/key pair), ms per layer, the roofline figures of the dominant
kernel measured with device events inside the timed region, per-stage times, and a CPU
baseline (the dense-mask oracle on a bounded sample, timed on this host's cores).
"""

from __future__ import annotations

import argparse
import json
import os
import random
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of moba_fwd_kernel come from rocprofv3 FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of
# known size: a counter run of its own, whose summary (for the headline workload only) is this file; the figure
# is read from its line "traffic_bytes_per_launch = <number>"
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "moba_fwd_128k_hbm_traffic.txt")

WORKLOADS = {
    # name: (seq lens or None, heads, kv_heads, chunk, topk, normalise, backward)
    "cfg1_L4096_h4_c512_k3": ([4096], 4, 4, 512, 3, False, False),
    "cfg2_L32768_h1_c2048_k3": ([32768], 1, 1, 2048, 3, False, True),
    "cfg3_varlen8_h32_c2048_k3": (None, 32, 32, 2048, 3, False, True),
    "cfg4_L131072_h32_c4096_k12": ([131072], 32, 8, 4096, 12, True, False),
    "cfg5_L1048576_h32_c4096_k12": ([1048576], 32, 8, 4096, 12, False, False),
    # the default shape of the reference's speed script (tests/test_moba_speedup.py:84)
    "speedscript_L32768_h1_c512_k3": ([32768], 1, 1, 512, 3, False, True),
}
DEFAULT = "cfg4_L131072_h32_c4096_k12"


def make_inputs(name, device, gqa=False):
    lens, H, Hkv, B, topk, normalise, _ = WORKLOADS[name]
    if lens is None:
        rng = random.Random(0)
        lens = [rng.randint(4096, 65536) for _ in range(8)]
    S = sum(lens)
    g = torch.Generator(device=device).manual_seed(0)

    def draw(h):
        x = torch.randn((S, h, 128), generator=g, device=device, dtype=torch.float32)
        if normalise:
            x = x / x.pow(2).mean(dim=-1, keepdim=True).sqrt()
        return x.to(torch.bfloat16)

    q = draw(H)
    k = draw(Hkv)
    v = draw(Hkv)
    if Hkv != H and not gqa:  # the wrapper's repeat_kv (moba/wrapper.py:59-61), outside the timed region
        k = torch.repeat_interleave(k, H // Hkv, dim=1).contiguous()
        v = torch.repeat_interleave(v, H // Hkv, dim=1).contiguous()
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    return q, k, v, cu, max(lens), B, topk


def cpu_baseline(q, k, v, B, topk, budget_tokens=32768, heads=8):
    """Dense-mask oracle (restatement of moba_naive) on the first ``budget_tokens`` tokens of
    ``heads`` heads of the same data, one head at a time, on this host's cores."""
    from oracle import moba_oracle as O

    L = min(budget_tokens, q.shape[0])
    heads = min(heads, q.shape[1])
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    dt = 0.0
    for h in range(heads):
        qc, kc, vc = (x[:L, h:h + 1].cpu().contiguous() for x in (q, k, v))
        t0 = time.perf_counter()
        O.moba_attn_varlen_naive(qc, kc, vc, [0, L], L, B, topk)
        dt += time.perf_counter() - t0
    flops = O.attention_flops([0, L], B, topk, heads, 128)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{heads} heads x first {L} tokens of the same q/k/v, chunk {B}, top-k {topk}, dense-mask fp32 "
                      f"algorithm of moba_naive, {dt:.1f} s"}


def bench_decode(dev, skv, heads, kv_heads=8, iters=50):
    """One query token per sequence against a cache of skv keys: the HIP decode kernel and PyTorch's
    scaled_dot_product_attention on the same tensors.  HBM-bound: K and V are read once."""
    import torch.nn.functional as F

    from moba_amd.decode import decode_attention
    kv_heads = min(kv_heads, heads)
    g = torch.Generator(device=dev).manual_seed(2)
    q = torch.randn((1, heads, 1, 128), generator=g, device=dev).to(torch.bfloat16)
    k = torch.randn((1, kv_heads, skv, 128), generator=g, device=dev).to(torch.bfloat16)
    v = torch.randn((1, kv_heads, skv, 128), generator=g, device=dev).to(torch.bfloat16)

    def timed(fn):
        for _ in range(5):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / iters

    ms = timed(lambda: decode_attention(q, k, v))
    ms_sdpa = timed(lambda: F.scaled_dot_product_attention(q, k, v, enable_gqa=heads != kv_heads))
    gbs = 2 * k.numel() * 2 / (ms * 1e-3) / 1e9
    return {"tokens_in_cache": skv, "heads": heads, "kv_heads": kv_heads, "ms": ms, "sdpa_ms": ms_sdpa,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": gbs / HBM_PEAK_GBS}}


def traffic_from_profile(workload):
    """HBM bytes per launch of the dominant kernel, as the committed counter profile states them (None if it does
    not cover this workload)."""
    if workload != DEFAULT or not os.path.exists(TRAFFIC_PROFILE):
        return None
    for line in open(TRAFFIC_PROFILE):
        if line.strip().startswith("traffic_bytes_per_launch"):
            return float(line.split("=")[1].split()[0])
    return None


def mfma_ceiling(dev, iters=40000):
    """What the chip's matrix pipes sustain when they do nothing else, on this box, now: a register-resident loop
    of v_mfma_f32_32x32x16_bf16 on every compute unit (eight waves each, as the forward kernel runs), once on
    constant operands and once on random bf16 N(0,1) operands.  The clock the chip holds at its power limit depends
    on how much the multipliers' inputs toggle, so the second figure, not the published peak, is the ceiling of any
    kernel that multiplies real data."""
    import ctypes
    from moba_amd import _lib
    lib = _lib.load()
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    flops = cus * 8 * iters * 16 * 32768.0
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    out = {"kernel": "mfma_probe_kernel", "workgroups": cus, "waves_per_workgroup": 8, "unit": "TFLOP/s",
           "peak": MFMA_BF16_PEAK_TFLOPS}
    g = torch.Generator(device=dev).manual_seed(3)
    for name, data in (("constant_operands", torch.ones(8192, device=dev, dtype=torch.bfloat16)),
                       ("random_bf16_operands", torch.randn(8192, generator=g, device=dev).to(torch.bfloat16))):
        best = None
        for _ in range(4):   # (about 10 ms each: long enough for the clock to settle at the power limit)
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            _lib.check(lib.moba_mfma_probe(ctypes.c_void_p(data.data_ptr()), ctypes.c_void_p(sink.data_ptr()), iters, 0,
                                           stream), "moba_mfma_probe")
            b.record()
            torch.cuda.synchronize()
            ms = a.elapsed_time(b)
            best = ms if best is None else min(best, ms)
        out[name] = flops / (best * 1e-3) / 1e12
    out["random_frac_of_peak"] = out["random_bf16_operands"] / MFMA_BF16_PEAK_TFLOPS
    return out


def quick_measure(name, dev, steps, warmup, backward, dtype=torch.bfloat16, topk=None):
    """Forward (and forward + backward) time of one of the other workloads, a few steps each: wall clock around
    the steps, bracketed by synchronisations, like the headline figure.  topk overrides the workload's
    (topk = 1: full causal attention through the same operator)."""
    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan

    q, k, v, cu, max_seqlen, B, topk0 = make_inputs(name, dev)
    topk = topk0 if topk is None else topk
    q, k, v = (x.to(dtype) for x in (q, k, v))
    S, H, D = q.shape
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    flops = make_plan(cu_t, B, topk).flops_per_head * D * H

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    with torch.no_grad():
        fwd_ms = timed(lambda: E.moba_attn_varlen(q, k, v, cu_t, max_seqlen, B, topk))
    out = {"tokens": S, "heads": H, "chunk": B, "topk": topk, "sequences": len(cu) - 1, "fwd_flops": flops,
           "fwd_ms": fwd_ms, "fwd_tflops": flops / (fwd_ms * 1e-3) / 1e12}
    if backward:
        g = torch.Generator(device=dev).manual_seed(1)
        do = torch.randn(q.shape, generator=g, device=dev, dtype=torch.float32).to(dtype)
        qg, kg, vg = (x.requires_grad_(True) for x in (q, k, v))

        def both():
            qg.grad = kg.grad = vg.grad = None
            E.moba_attn_varlen(qg, kg, vg, cu_t, max_seqlen, B, topk).backward(do)

        ms = timed(both)
        # the backward's algorithmic work is 2.5 x the forward's (5 products against 2)
        out.update(fwd_bwd_ms=ms, fwd_bwd_tflops=3.5 * flops / (ms * 1e-3) / 1e12)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=DEFAULT, help="one of %s, or its cfgN prefix" % ", ".join(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--backward", action="store_true", help="also time forward + backward")
    ap.add_argument("--decode", action="store_true",
                    help="also time the decode kernel (one token against a cache of the workload's length, "
                         "8 KV heads) next to PyTorch SDPA")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="with the default workload: do not also time the other BASELINE configurations")
    ap.add_argument("--no-ceiling", action="store_true", help="do not run the matrix-pipe ceiling probe")
    ap.add_argument("--gqa", action="store_true",
                    help="keep the key/value heads unexpanded (grouped-query operator) instead of the reference "
                         "wrapper's repeat_kv; not the headline configuration")
    args = ap.parse_args()
    if args.workload not in WORKLOADS:
        match = [w for w in WORKLOADS if w.split("_")[0] == args.workload]
        if len(match) != 1:
            ap.error("unknown workload %r" % args.workload)
        args.workload = match[0]
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    from moba_amd import moba_efficient as E
    from moba_amd.plan import make_plan

    dev = torch.device("cuda:0")
    q, k, v, cu, max_seqlen, B, topk = make_inputs(args.workload, dev, args.gqa)
    S, H, D = q.shape
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    plan = make_plan(cu_t, B, topk)
    flops = plan.flops_per_head * D * H

    for _ in range(args.warmup):
        E.moba_attn_varlen_with_lse(q, k, v, cu_t, max_seqlen, B, topk, gqa=args.gqa)
    torch.cuda.synchronize()
    # The timed region: K steps, with device events around the dominant kernel only (recording a pair of events
    # costs the host tens of microseconds; one pair per step is invisible at this size, five would not be).
    kernel_timer = E.StageTimer(only=("fwd_partials",))
    t0 = time.perf_counter()
    for _ in range(args.steps):
        E.moba_attn_varlen_with_lse(q, k, v, cu_t, max_seqlen, B, topk, timer=kernel_timer, gqa=args.gqa)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    kern_ms = sum(kernel_timer.ms()["fwd_partials"]) / args.steps
    # the other stages, from K more steps of the same work with events around every stage
    timer = E.StageTimer()
    for _ in range(args.steps):
        E.moba_attn_varlen_with_lse(q, k, v, cu_t, max_seqlen, B, topk, timer=timer, gqa=args.gqa)
    torch.cuda.synchronize()
    per_stage = timer.ms()
    stage_ms = {name: sum(x) / len(x) for name, x in per_stage.items()}
    stage_ms["fwd_partials"] = kern_ms
    # device time of each step (sum of its stage spans): median and minimum over those steps
    step_ms = sorted(sum(x[i] for x in per_stage.values()) for i in range(args.steps))

    # forward + backward (reported beside the forward figure for the workloads that name it)
    fwd_bwd_ms = None
    others = args.workload == DEFAULT and not args.gqa and not args.no_other_configs
    if WORKLOADS[args.workload][6] or args.backward or others:
        g = torch.Generator(device=dev).manual_seed(1)
        do = torch.randn(q.shape, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        qg, kg, vg = (x.clone().requires_grad_(True) for x in (q, k, v))
        op = E.moba_attn_varlen_gqa if args.gqa else E.moba_attn_varlen
        bsteps = args.steps if (WORKLOADS[args.workload][6] or args.backward) else min(args.steps, 3)
        for _ in range(max(1, min(args.warmup, bsteps))):
            op(qg, kg, vg, cu_t, max_seqlen, B, topk).backward(do)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(bsteps):
            qg.grad = kg.grad = vg.grad = None
            op(qg, kg, vg, cu_t, max_seqlen, B, topk).backward(do)
        torch.cuda.synchronize()
        fwd_bwd_ms = (time.perf_counter() - t1) / bsteps * 1e3
        del qg, kg, vg, do

    achieved = flops / (kern_ms * 1e-3) / 1e12
    result = {
        "metric": "moba_fwd_effective_tflops_128k" if args.workload == DEFAULT else "moba_fwd_effective_tflops",
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": args.workload, "tokens": S, "heads": H, "kv_heads": k.shape[1], "head_dim": D, "chunk": B, "topk": topk,
                   "sequences": len(cu) - 1, "fwd_flops": flops},
        "pct_mfma_peak_whole_op": 100.0 * flops / dt / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        "stage_ms": stage_ms,
        "device_ms_per_step": {"median": step_ms[len(step_ms) // 2], "min": step_ms[0]},
        "roofline": {"kernel": "moba_fwd_kernel", "bound": "mfma", "achieved": achieved,
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": traffic_from_profile(args.workload),
                     "traffic_source": "profiles/moba_fwd_128k_hbm_traffic.txt (rocprofv3 counter runs of this "
                                       "workload; not measured in this run)"},
    }
    if not args.no_ceiling:
        # the same box, the same minute: what the matrix pipes sustain with nothing else to do
        result["mfma_ceiling"] = mfma_ceiling(dev)
        result["roofline"]["frac_of_random_operand_ceiling"] = achieved / result["mfma_ceiling"]["random_bf16_operands"]
    if fwd_bwd_ms is not None:
        # algorithmic backward work is 2.5x the forward's
        result["fwd_bwd"] = {"ms_per_step": fwd_bwd_ms, "tflops": 3.5 * flops / (fwd_bwd_ms * 1e-3) / 1e12,
                             "pct_mfma_peak": 100.0 * 3.5 * flops / (fwd_bwd_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS}
    if "chunk_mean" in stage_ms:
        gbs = k.numel() * 2 / (stage_ms["chunk_mean"] * 1e-3) / 1e9
        result["chunk_mean_hbm"] = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                    "frac": gbs / HBM_PEAK_GBS}
    if args.decode:
        result["decode"] = bench_decode(dev, S if len(cu) == 2 else max_seqlen, H)
    if others:
        # the other BASELINE configurations, 200 steps of the two small ones, a few of the others
        # (cfg5: BASELINE asks for the forward; the backward runs too)
        del q, k, v
        torch.cuda.empty_cache()
        result["other_configs"] = {}
        for name, steps, warmup in (("cfg1_L4096_h4_c512_k3", 200, 20), ("cfg2_L32768_h1_c2048_k3", 200, 20),
                                    ("speedscript_L32768_h1_c512_k3", 200, 20),
                                    ("cfg3_varlen8_h32_c2048_k3", 3, 1), ("cfg5_L1048576_h32_c4096_k12", 2, 1)):
            result["other_configs"][name] = quick_measure(name, dev, steps, warmup, backward=True)
            torch.cuda.empty_cache()
        # the headline shape in fp16 (the dtype of the reference's example, examples/llama.py:26)
        result["other_configs"]["cfg4_fp16"] = quick_measure(DEFAULT, dev, 5, 2, backward=False, dtype=torch.float16)
        torch.cuda.empty_cache()
        # Full causal attention through the same operator (moba_topk = 1) beside MoBA: the ratio the reference's
        # report plots (full FlashAttention / MoBA forward time: 1.19x at 128K, 6.5x at 1M tokens, on its hardware)
        result["full_attention"] = {}
        for name, steps, warmup, published in (("cfg2_L32768_h1_c2048_k3", 50, 5, None), (DEFAULT, 3, 1, 1.19),
                                               ("cfg5_L1048576_h32_c4096_k12", 1, 1, 6.5)):
            full = quick_measure(name, dev, steps, warmup, backward=False, topk=1)
            moba_ms = dt * 1e3 if name == DEFAULT else result["other_configs"][name]["fwd_ms"]
            result["full_attention"][name] = {"full_fwd_ms": full["fwd_ms"], "full_fwd_tflops": full["fwd_tflops"],
                                              "moba_fwd_ms": moba_ms, "full_over_moba": full["fwd_ms"] / moba_ms,
                                              "report_full_over_moba": published}
            torch.cuda.empty_cache()
        q, k, v, cu, max_seqlen, B, topk = make_inputs(args.workload, dev, args.gqa)   # for the CPU baseline's sample
    if not args.no_cpu_baseline:
        rep = H // k.shape[1]
        nkv = (8 + rep - 1) // rep  # key/value heads behind the first 8 query heads
        result["cpu_baseline"] = cpu_baseline(q, k if rep == 1 else torch.repeat_interleave(k[:, :nkv], rep, dim=1),
                                              v if rep == 1 else torch.repeat_interleave(v[:, :nkv], rep, dim=1), B, topk)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
