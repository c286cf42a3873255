#!/usr/bin/env python3
"""Benchmark of the vTensor KV-cache hot path on one MI355X.

A step is one decode step of one layer over one batch: per-sequence range bookkeeping (map a
2 MiB chunk where a sequence crosses a boundary), upload of the byte offsets and sequence
lengths, `reshape_and_cache` of one new token per sequence, and decode attention over the whole
context.  Inputs are synthetic (N(0,1) cast to the KV dtype) and resident in HBM before timing.

Prints one JSON line: the BASELINE metric, a `roofline` object for the dominant kernel (HIP-event
timed inside this process) and a `cpu_baseline` object (the reference's CPU attention timed on this
host on a bounded sample of the same workload).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes moved per launch of the dominant kernel relative to its algorithmic bytes, measured with
# rocprofv3 (FETCH_SIZE and WRITE_SIZE in separate runs, each scaled by what the counter reads for the
# calibration copy of known size that this script runs before timing).  Counters cannot be read from
# inside this process: the ratios below were measured once per workload with the commands given in the
# named summaries, and `roofline.traffic` is the launch's algorithmic bytes times that stored ratio (the
# JSON says so: "traffic_replayed_from_profile").
# workload: (fetch bytes, write bytes, algorithmic bytes of the profiled launches, MFMA-busy share, summary)
MEASURED_TRAFFIC = {
    "c2": (634797463, 2403448, 635113472, 0.0663, "profiles/decode_attn_stream_kernel_c2_llama3_8b_decode.md"),
    "c3": (926249383, 1144900, 926629888, 0.0681, "profiles/decode_attn_stream_kernel_c3_c4_c5.md"),
    "c4": (1212193147, 10957685, 1213501440, 0.1253, "profiles/decode_attn_stream_kernel_c3_c4_c5.md"),
    "c5": (1236069922, 5777604, 1235329024, 0.0651, "profiles/decode_attn_stream_kernel_c3_c4_c5.md"),
}


def measured_traffic(config: str):
    """(traffic / algorithmic bytes, MFMA-busy fraction, source) for `config`, or (None, None, None)."""
    if config not in MEASURED_TRAFFIC:
        return None, None, None
    fetch, write, algo, mfma, source = MEASURED_TRAFFIC[config]
    return (fetch + write) / algo, mfma, source


CONFIGS = {
    # BASELINE.json configs[1]: Llama-3-8B-shaped single-layer decode, bf16
    "c2": dict(name="llama3-8b-decode-bf16 B=64 Hq=32 Hkv=8 D=128 ctx~U[512,4096]", batch=64, hq=32, hkv=8, d=128,
               lo=512, hi=4096, seed=1001, kv="bf16"),
    # configs[2]: long-context split-K decode
    "c3": dict(name="long-context-decode-bf16 B=4 Hq=32 Hkv=8 D=128 ctx~U[32768,131072]", batch=4, hq=32, hkv=8,
               d=128, lo=32768, hi=131072, seed=1002, kv="bf16"),
    # configs[3]: fp8-e4m3 KV at the Llama-3-70B per-layer shape
    "c4": dict(name="llama3-70b-layer-decode-fp8kv B=128 Hq=64 Hkv=8 D=128 ctx~U[1024,8192]", batch=128, hq=64,
               hkv=8, d=128, lo=1024, hi=8192, seed=1003, kv="fp8"),
    # configs[4]: 256 sequences that grow; as a plain workload (--config c5) without its swap events, with them
    # in growth_and_swap_protocol()
    "c5": dict(name="growth-bf16 B=256 Hq=32 Hkv=8 D=128 ctx~U[256,2048]", batch=256, hq=32, hkv=8, d=128, lo=256,
               hi=2048, seed=1004, kv="bf16"),
    # outside BASELINE.json: very many short sequences (every workgroup meets many segment starts and ends)
    "t1k": dict(name="many-short-bf16 B=1024 Hq=32 Hkv=8 D=128 ctx~U[64,512]", batch=1024, hq=32, hkv=8, d=128, lo=64,
                hi=512, seed=1007, kv="bf16"),
    # BASELINE.json configs[0] (the reference's CPU-runnable case) on the GPU, and configs[1]'s batch in float32:
    # float32 queries over float32 rows through the float32 kernels
    "c1": dict(name="fp32 B=8 Hq=32 Hkv=8 D=128 ctx~U[128,1024]", batch=8, hq=32, hkv=8, d=128, lo=128, hi=1024,
               seed=1000, kv="f32", f32=True),
    "c2f32": dict(name="llama3-8b-decode-fp32 B=64 Hq=32 Hkv=8 D=128 ctx~U[512,4096]", batch=64, hq=32, hkv=8, d=128,
                  lo=512, hi=4096, seed=1001, kv="f32", f32=True),
    # outside BASELINE.json: a prompt run (cache write + causal attention over the ranges), 8 prompts of 2048
    "p2k": dict(name="llama3-8b-prompt-run-bf16 B=8 Hq=32 Hkv=8 D=128 prompt=2048", batch=8, hq=32, hkv=8, d=128,
                lo=2048, hi=2048, seed=1006, kv="bf16", prefill=True),
}

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 rate


def prompt_run(args, cfg) -> int:
    """One step = one prompt run of one layer: reshape_and_cache of every prompt row, then causal
    attention of all prompt tokens over the ranges.  Reported in TFLOP/s (4*Hq*D flop per visible
    (query, key) pair) against the dense bf16 MFMA peak."""
    import torch

    from glake_amd import _custom_ops as ops, vmm_allocator as vmm
    from glake_amd.worker.cache_engine import CacheEngine

    B, Hq, Hkv, D = cfg["batch"], cfg["hq"], cfg["hkv"], cfg["d"]
    K, W = args.steps, args.warmup
    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    gen = torch.Generator().manual_seed(cfg["seed"])
    lens = torch.randint(cfg["lo"], cfg["hi"] + 1, (B,), generator=gen).tolist()
    row = Hkv * D * 2
    chunks = (max(lens) * row + (2 << 20) - 1) // (2 << 20) + 1
    vmm.init_physical_handle(2 * B * chunks + 16, 0)
    engine = CacheEngine(num_layers=1, num_kv_heads=Hkv, head_size=D, dtype=torch.bfloat16, max_num_seqs=B,
                         max_num_batched_tokens=max(lens) + 128, swap_space_bytes=0)
    segs = engine.vmm_kvcache_segment
    n_tok = sum(lens)
    ggen = torch.Generator(device=dev).manual_seed(cfg["seed"])
    q = torch.randn(n_tok, Hq, D, generator=ggen, device=dev).to(torch.bfloat16)
    k = torch.randn(n_tok, Hkv, D, generator=ggen, device=dev).to(torch.bfloat16)
    v = torch.randn(n_tok, Hkv, D, generator=ggen, device=dev).to(torch.bfloat16)
    out = torch.empty_like(q)
    slot_ids = list(range(B))
    slot_t = torch.arange(B, dtype=torch.int64, device=dev)
    lens_t = torch.tensor(lens, dtype=torch.int32, device=dev)
    starts = torch.tensor([sum(lens[:i]) for i in range(B)], dtype=torch.int32, device=dev)
    zeros_t = torch.zeros(B, dtype=torch.int64, device=dev)
    # rows are reserved once (the prompt's chunks are mapped by the step prologue before the first layer)
    vmm.extend_kv_cache_batch(None, None, slot_ids, [n * row for n in lens], segs, [0] * B, row, False)
    scale = float(D) ** -0.5
    torch.cuda.synchronize()
    torch.cuda.set_stream(torch.cuda.Stream(device=dev))

    def step():
        ops.reshape_and_cache(k, v, engine.k_cache_ptr[0], engine.v_cache_ptr[0], zeros_t, slot_t, lens_t, starts,
                              max(lens), Hkv, D)
        ops.prefill_attention(out, q, engine.k_cache_ptr[0], engine.v_cache_ptr[0], Hkv, scale, lens, lens, slot_t)

    for _ in range(W):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / K
    # attention alone, with HIP events on the stream it runs on
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    ev[0].record()
    for _ in range(K):
        ops.prefill_attention(out, q, engine.k_cache_ptr[0], engine.v_cache_ptr[0], Hkv, scale, lens, lens, slot_t)
    ev[1].record()
    torch.cuda.synchronize()
    attn_ms = ev[0].elapsed_time(ev[1]) / K
    pairs = sum(n * (n + 1) // 2 for n in lens)
    flops = 4 * Hq * D * pairs
    achieved = flops / (attn_ms * 1e-3) / 1e12
    result = {
        "metric": "prompt-run attention TFLOP/s (causal, over contiguous ranges)", "value": round(flops / dt / 1e12, 2),
        "unit": "TFLOP/s", "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(dt * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": cfg["name"], "layers": 1, "prompt_tokens": n_tok},
        "tokens_per_s": round(n_tok / dt, 1),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "kernel": "prefill_attn_kernel", "avg_call_ms": round(attn_ms, 4),
                     "algorithmic_flops_per_call": flops},
    }
    if args.workgroup_trace:
        # the tracing build keeps {XCC id, start, first stage in LDS, end of the stages, end, stages} of every workgroup
        # of the last launch (100 MHz clock)
        from glake_amd import _C
        fn = _C.lib().vtkv_debug_prefill_trace
        fn.argtypes = [C.c_void_p, C.c_int]
        per_unit = max(1, 128 // (Hq // Hkv))
        n_wg = min(4096, sum((n + per_unit - 1) // per_unit for n in lens) * Hkv)
        buf = (C.c_ulonglong * (4096 * 6))()
        _C.check(fn(buf, 4096))
        t = np.array(list(buf), dtype=np.int64).reshape(4096, 6)[:n_wg]
        t0 = t[:, 1].min()
        us = lambda a: (a - t0) / 100.0
        life = (t[:, 4] - t[:, 1]) / 100.0
        pro, loop, epi = (t[:, 2] - t[:, 1]) / 100.0, (t[:, 3] - t[:, 2]) / 100.0, (t[:, 4] - t[:, 3]) / 100.0
        span = float(us(t[:, 4]).max())
        q = lambda a: [round(float(np.percentile(a, x)), 2) for x in (10, 50, 90)]
        result["workgroup_trace"] = {
            "workgroups": int(n_wg), "kernel_span_us": round(span, 1),
            "prologue_us_p10_p50_p90": q(pro), "epilogue_us_p10_p50_p90": q(epi),
            "stage_ns_p10_p50_p90": q(loop * 1e3 / np.maximum(t[:, 5], 1)),
            "sum_of_lifetimes_over_span_times_512": round(float(life.sum() / (span * 512)), 3),
            "share_of_lifetime_in_prologue_and_epilogue": round(float((pro.sum() + epi.sum()) / life.sum()), 3),
            "last_start_us": round(float(us(t[:, 1]).max()), 1),
            "end_us_mean_by_xcc": [round(float(us(t[:, 4])[t[:, 0] == x].max()), 1) for x in range(8)]}
    print(json.dumps(result))
    engine.close()
    return 0


def f32_run(args, cfg) -> int:
    """A float32 model: one step = reshape_and_cache of one new float32 row per sequence + decode attention over
    float32 rows (two launches, three where partitions are merged), through DecodeStepPlan.  Reported like the 16-bit
    workloads: algorithmic bytes (rows + q + out, 4 bytes per element) per second of whole steps, and for the
    attention call alone by HIP events on the stream it runs on."""
    import torch

    from glake_amd import _custom_ops as ops, vmm_allocator as vmm
    from glake_amd.worker.cache_engine import CacheEngine
    from glake_amd.worker.step import DecodeStepPlan

    B, Hq, Hkv, D = cfg["batch"], cfg["hq"], cfg["hkv"], cfg["d"]
    K, W = args.steps, args.warmup
    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    ctx0 = torch.randint(cfg["lo"], cfg["hi"] + 1, (B,), generator=torch.Generator().manual_seed(cfg["seed"])).tolist()
    row = Hkv * D * 4
    total_steps = 2 * (W + K) + 4
    chunk = vmm.chunkBytes()
    chunks_per_range = ((max(ctx0) + total_steps + 1) * row + args.value_skew + chunk - 1) // chunk
    vmm.init_physical_handle(2 * B * chunks_per_range + 16, 0)
    engine = CacheEngine(num_layers=1, num_kv_heads=Hkv, head_size=D, dtype=torch.float32, max_num_seqs=B,
                         max_num_batched_tokens=max(ctx0) + total_steps + 1, swap_space_bytes=0,
                         value_skew=args.value_skew)
    segs = engine.vmm_kvcache_segment
    ggen = torch.Generator(device=dev).manual_seed(cfg["seed"])
    for b in range(B):
        nbytes = ctx0[b] * row
        segs[b].ensure_mapped(nbytes)
        for base in (segs[b].getKeyDevicePtr(0), segs[b].getValueDevicePtr(0)):
            t = torch.randn(ctx0[b], Hkv, D, generator=ggen, device=dev, dtype=torch.float32)
            ops.swap_ranges([t.data_ptr()], [base], [nbytes], "d2d")
            torch.cuda.synchronize()
        segs[b].set_used_size(nbytes)
    q = torch.randn(B, Hq, D, generator=ggen, device=dev, dtype=torch.float32)
    new_k = torch.randn(B, Hkv * D, generator=ggen, device=dev, dtype=torch.float32)
    new_v = torch.randn(B, Hkv * D, generator=ggen, device=dev, dtype=torch.float32)
    out = torch.empty(B, Hq, D, dtype=torch.float32, device=dev)
    plan = DecodeStepPlan(segs, list(range(B)), engine.k_cache_ptr[0], engine.v_cache_ptr[0], Hq, Hkv, D, D ** -0.5,
                          model_dtype=torch.float32, device=dev)
    torch.cuda.set_stream(torch.cuda.Stream(device=dev))
    step_bytes = lambda lens: sum(lens) * 2 * row + 2 * B * Hq * D * 4
    lens = list(ctx0)
    for _ in range(W):
        plan.run(q, new_k, new_v, out)
        lens = [n + 1 for n in lens]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    moved = 0
    for _ in range(K):
        plan.run(q, new_k, new_v, out)
        lens = [n + 1 for n in lens]
        moved += step_bytes(lens)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    # the attention call alone (the lengths stay what they are), with HIP events on its stream
    lens_t = torch.tensor(lens, dtype=torch.int32, device=dev)
    slot_t = torch.arange(B, dtype=torch.int64, device=dev)
    attend = lambda: ops.paged_attention_v1(out, q, engine.k_cache_ptr[0], engine.v_cache_ptr[0], Hkv, D ** -0.5, lens_t, 1,
                                            max(lens), None, "auto", 1.0, slot_t)
    for _ in range(W):
        attend()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    ev[0].record()
    for _ in range(K):
        attend()
    ev[1].record()
    torch.cuda.synchronize()
    attn_ms = ev[0].elapsed_time(ev[1]) / K
    achieved = step_bytes(lens) / (attn_ms * 1e-3) / 1e9
    value = moved / dt / 1e9
    result = {
        "metric": "decode-attn HBM GB/s (% peak) + tokens/s, float32 model", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": round(dt / K * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": cfg["name"], "layers": 1, "new_tokens_per_step": B, "kv_chunk": "2MiB VMM",
                   "mean_ctx": round(sum(ctx0) / B, 1)},
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2), "tokens_per_s": round(B * K / dt, 1),
        "algorithmic_bytes_per_step": step_bytes(lens),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "decode_attn_f32_kernel (+ merge_attn_f32_kernel)", "avg_call_us": round(attn_ms * 1e3, 2),
                     "algorithmic_bytes_per_launch": step_bytes(lens)},
    }
    print(json.dumps(result))
    engine.close()
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--partition-tokens", type=int, default=0)
    ap.add_argument("--host-path", default="plan", choices=["plan", "ops", "backend"],
                    help="plan: DecodeStepPlan (arguments prepared once); ops: the separate reference-style op calls; "
                         "backend: the reference's own call sequence, one prepare_step then --layers x "
                         "VTensorImpl.forward per step")
    ap.add_argument("--layers", type=int, default=32, help="layers of a step with --host-path backend")
    ap.add_argument("--repeats", type=int, default=0,
                    help="timed regions of exactly --steps steps each, synchronised on both sides; the median one is "
                         "reported (0 = 21 for regions of up to 50 steps, else 3)")
    ap.add_argument("--unfused", action="store_true",
                    help="plan path: separate reshape_and_cache and attention launches instead of the fused one")
    ap.add_argument("--merge", default="auto", choices=["auto", "fused", "separate"],
                    help="where the attention's partial results are merged (auto: the library decides per call)")
    ap.add_argument("--value-skew", type=int, default=256,
                    help="bytes between the base of a V range and its first row (0 = the reference's placement)")
    ap.add_argument("--head-major", default="auto", choices=["auto", "on", "off"],
                    help="tile order of the decode kernel: (kv head, sequence, rows) or (sequence, kv head, rows)")
    ap.add_argument("--head-size", type=int, default=0,
                    help="run the chosen decode workload with another head size of the reference's list (64, 80, 96, 112, "
                         "256); an fp8 cache then takes reshape_and_cache + attention as two launches (its fused append "
                         "exists at 128)")
    ap.add_argument("--heads", default="", metavar="HQ,HKV", help="likewise with other head counts")
    ap.add_argument("--chunk-mib", type=int, default=2,
                    help="size of a physical chunk (the reference's granularity is 2 MiB; vtkv_pool_set_chunk_bytes)")
    ap.add_argument("--workgroup-trace", action="store_true",
                    help="with a library built by `python -m glake_amd.build --define VTKV_ATTN_TRACE --out X` "
                         "(VTKV_LIBRARY_PATH=X): when the workgroups of the decode kernel's last launch ended, by XCD")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", action="store_true",
                    help="with --config c2: leave out the other BASELINE configurations (c3, c4 and the growth-and-swap "
                         "protocol) that the default run appends under \"configs\"")
    ap.add_argument("--other-repeats", type=int, default=7, help="timed regions of each of those other configurations")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (nothing in the KV-cache hot path communicates); "
              "use --gpus 1", file=sys.stderr)
        return 2

    cfg = CONFIGS[args.config]
    if cfg.get("prefill"):
        if args.steps == 200 and args.warmup == 20:
            args.steps, args.warmup = 20, 3
        return prompt_run(args, cfg)
    if cfg.get("f32"):
        if args.steps == 200 and args.warmup == 20:
            args.steps, args.warmup = 50, 5
        return f32_run(args, cfg)
    from glake_amd import _C

    if args.chunk_mib != 2:
        from glake_amd import vmm_allocator as vmm

        vmm.set_chunk_bytes(args.chunk_mib << 20)
    _C.check(_C.lib().vtkv_set_fused_merge({"auto": -1, "fused": 1, "separate": 0}[args.merge]))
    _C.check(_C.lib().vtkv_set_head_major({"auto": -1, "on": 1, "off": 0}[args.head_major]))
    R = args.repeats if args.repeats > 0 else (21 if args.steps <= 50 else 3)
    result = decode_run(args, args.config, R, with_swap=args.host_path != "backend", with_cpu=not args.no_cpu_baseline)
    # The other BASELINE configurations in the same line (the headline stays configs[1]): configs[2] and [3] as
    # plain decode workloads with fewer regions, configs[4] as BASELINE.json writes it, swap events included.
    if (args.config == "c2" and args.host_path == "plan" and args.partition_tokens == 0 and not args.only
            and not args.head_size and not args.heads):
        keep = ("value", "unit", "ms_per_step", "pct_of_hbm_peak", "tokens_per_s", "repeats", "regions_gbps",
                "algorithmic_bytes_per_step", "host_issue_ms_per_step", "dtype", "roofline", "mfma_util")
        others = {}
        for name in ("c3", "c4"):
            r = decode_run(args, name, args.other_repeats, with_swap=False, with_cpu=False)
            others[name] = {"workload": r["config"]["workload"], **{k: r[k] for k in keep}}
        others["c5"] = growth_and_swap_protocol(args)
        result["configs"] = others
    print(json.dumps(result))
    return 0


def decode_run(args, config: str, R: int, with_swap: bool, with_cpu: bool) -> dict:
    """W warm-up steps, R timed regions of exactly K decode steps, the per-kernel event pass, optionally the swap
    figures and the CPU baseline, for one workload of CONFIGS; returns the JSON object of that workload."""
    import torch

    from glake_amd import _C, _custom_ops as ops, vmm_allocator as vmm
    from glake_amd.worker.cache_engine import CacheEngine

    cfg = dict(CONFIGS[config])
    if args.head_size:
        cfg["d"] = args.head_size
        cfg["name"] = cfg["name"].replace("D=128", f"D={args.head_size}")
    if args.heads:
        cfg["hq"], cfg["hkv"] = (int(x) for x in args.heads.split(","))
        cfg["name"] += f" (Hq={cfg['hq']} Hkv={cfg['hkv']})"
    B, Hq, Hkv, D = cfg["batch"], cfg["hq"], cfg["hkv"], cfg["d"]
    K, W = args.steps, args.warmup
    backend_path = args.host_path == "backend"
    L = args.layers if backend_path else 1
    torch.cuda.set_device(0)
    dev = torch.device("cuda", 0)
    gen = torch.Generator().manual_seed(cfg["seed"])
    ctx0 = torch.randint(cfg["lo"], cfg["hi"] + 1, (B,), generator=gen).tolist()
    event_steps = max(1, min(K, 1024 // L))          # the library keeps the events of 1024 attention calls
    total_steps = (W + R * K) + (W + event_steps) + 4  # timed regions + kernel-timing pass, each with warm-up
    fp8 = cfg["kv"] == "fp8"
    eb = 1 if fp8 else 2            # bytes per KV element
    kv_dtype = "fp8" if fp8 else "auto"
    row = Hkv * D * eb
    max_tokens = max(ctx0) + total_steps + 1
    chunk = vmm.chunkBytes()
    chunks_per_range = (max_tokens * row + args.value_skew + chunk - 1) // chunk
    ensure_pool(2 * L * B * chunks_per_range + 16)
    engine = CacheEngine(num_layers=L, num_kv_heads=Hkv, head_size=D, dtype=torch.uint8 if fp8 else torch.bfloat16,
                         max_num_seqs=B, max_num_batched_tokens=max_tokens,
                         swap_space_bytes=0 if backend_path else 1 << 30, value_skew=args.value_skew)
    segs = engine.vmm_kvcache_segment

    # ---- resident synthetic KV: N(0,1) -> bf16, written straight into the mapped ranges
    ggen = torch.Generator(device=dev).manual_seed(cfg["seed"])
    # fp8: one scale per tensor; N(0,1) over ~1e8 draws peaks near 5.7, use amax = 6 -> scale = 6/448
    k_scale = v_scale = 6.0 / 448.0 if fp8 else 1.0
    for b in range(B):
        nbytes = ctx0[b] * row
        # (counts the V offset; the engine's accounting, which the backend path follows, maps 100 rows ahead)
        segs[b].ensure_mapped(nbytes + (100 * row if backend_path else 0))
        for l in range(L):
            for base in (segs[b].getKeyDevicePtr(l), segs[b].getValueDevicePtr(l)):
                t = torch.randn(ctx0[b], Hkv, D, generator=ggen, device=dev, dtype=torch.float32).to(torch.bfloat16)
                if fp8:
                    codes = torch.empty(t.shape, dtype=torch.uint8, device=dev)
                    ops.convert_fp8(codes, t, k_scale)
                    t = codes
                ops.swap_ranges([t.data_ptr()], [base], [nbytes], "d2d")
                torch.cuda.synchronize()
        segs[b].set_used_size(nbytes)
    q = torch.randn(B, Hq * D, generator=ggen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    new_k = torch.randn(B, Hkv * D, generator=ggen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    new_v = torch.randn(B, Hkv * D, generator=ggen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    out = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=dev)
    slot_ids = list(range(B))
    slot_t = torch.arange(B, dtype=torch.int64, device=dev)
    scale = float(D) ** -0.5
    kv_size = row

    # A plain copy of known size (256 MiB read, 256 MiB written: 1024 blocks of 128 KiB for K and for V)
    # outside the timed region: under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` its `copy_blocks_kernel`
    # dispatch calibrates the counters.
    cal = [torch.zeros(2048, 128 << 10, dtype=torch.uint8, device=dev) for _ in range(2)]
    pairs = torch.stack([torch.arange(1024), torch.arange(1024) + 1024], dim=1).to(device=dev, dtype=torch.int64)
    ops.copy_blocks([cal[0]], [cal[1]], pairs)
    torch.cuda.synchronize()
    del cal, pairs

    # Step metadata goes up in ONE async copy: B int64 byte offsets followed by B int32 lengths.  Pinned
    # staging rows, one per step, so an upload never races the next step's host writes.
    stage = torch.empty(total_steps, 3 * B, dtype=torch.int32).pin_memory()
    stage_np = stage.numpy()
    meta_t = torch.empty(3 * B, dtype=torch.int32, device=dev)
    slot_m_t = meta_t[:2 * B].view(torch.int64)
    lens_t = meta_t[2 * B:]
    state = {"step": 0, "lens": list(ctx0)}
    zeros = [0] * B
    tok_bytes = [kv_size] * B

    from glake_amd.worker.step import DecodeStepPlan, prepare_step
    plan = DecodeStepPlan(segs, slot_ids, engine.k_cache_ptr[0], engine.v_cache_ptr[0], Hq, Hkv, D, scale,
                          kv_cache_dtype=kv_dtype, k_scale=k_scale, v_scale=v_scale, device=dev,
                          fused=not args.unfused)
    q3 = q.view(B, Hq, D)

    def step_plan() -> int:
        plan.run(q3, new_k, new_v, out)
        return int(plan.seq_lens.sum())

    def step_ops() -> int:
        i = state["step"]
        # 1. range bookkeeping (maps a chunk on a 2 MiB boundary), llama.py:340
        slot_m = vmm.extend_kv_cache_batch(None, None, slot_ids, tok_bytes, segs, zeros, kv_size, True)
        lens = state["lens"] = [n + 1 for n in state["lens"]]
        stage_np[i, :2 * B].view(np.int64)[:] = slot_m
        stage_np[i, 2 * B:] = lens
        meta_t.copy_(stage[i], non_blocking=True)
        max_len = max(lens)
        # 2. append the new token's K/V rows
        ops.reshape_and_cache(new_k, new_v, engine.k_cache_ptr[0], engine.v_cache_ptr[0], slot_m_t, slot_t, None,
                              None, 1, Hkv, D, kv_dtype, k_scale, v_scale)
        # 3. decode attention over the whole context
        ops.paged_attention_v1(out, q.view(B, Hq, D), engine.k_cache_ptr[0], engine.v_cache_ptr[0], Hkv, scale,
                               lens_t, 1, max_len, None, kv_dtype, k_scale, slot_t, v_scale=v_scale,
                               partition_tokens=args.partition_tokens)
        state["step"] = i + 1
        return sum(lens)

    # The reference's own call sequence (llama.py:307-351): per step the metadata the model runner builds
    # (model_runner.py:595-622, with its host-to-device uploads), one prologue, then every layer's forward.
    from glake_amd.attention.backends.vtensor import VTensorBackend
    impl = VTensorBackend.get_impl_cls()(Hq, D, scale, Hkv, None, None, kv_dtype)
    impl.fuse_decode_append = not args.unfused
    no_extend = [-1] * B
    # the engine-side accounting claims every sequence's rows 100 ahead of what is written (sequence.py:343) and
    # names the slots whose claim crosses a chunk in a step (block_manager_v1.py:436-455): prepare_step hands
    # those to the map-ahead worker, so the chunk is there long before a row needs it
    from glake_amd.core import ChunkSpaceManager, SequenceChunks
    mgr = ChunkSpaceManager(B, 2 * B * chunks_per_range + 16, watermark=0.0)
    claims = []
    for b in range(B):
        c = SequenceChunks(row, chunk_bytes=chunk, value_skew=args.value_skew)
        c.append_tokens(ctx0[b])
        assert mgr.allocate(c)
        claims.append(c)

    def step_backend() -> int:
        lens = state["lens"] = [n + 1 for n in state["lens"]]
        max_len = max(lens)
        grow = []
        for c in claims:                                  # scheduler.py:1119-1150 _append_slots
            c.append_tokens(1)
            mgr.append_slots(c, grow)
        extend = [s if s in grow else -1 for s in slot_ids] if grow else no_extend
        meta = VTensorBackend.make_metadata(
            num_prefills=0, num_prefill_tokens=0, num_decode_tokens=B, slot_mapping=slot_t, seq_lens=lens,
            seq_lens_tensor=torch.tensor(lens, dtype=torch.int32, device=dev), max_query_len=None,
            max_prefill_seq_len=0, max_decode_seq_len=max_len, query_start_loc=None, seq_start_loc=None,
            context_lens_tensor=None, block_tables=None, is_extend=0, kv_batch_stride=engine.kv_batch_stride,
            kv_num_heads=Hkv, kv_head_size=D, max_seq_len=max_len, slot_mapping_list=slot_ids, set_used_size=zeros,
            extend_seq_list=extend, use_cuda_graph=False)
        meta.k_cache_segment_ptr_list = engine.k_cache_ptr          # model_runner.py:749-755
        meta.v_cache_segment_ptr_list = engine.v_cache_ptr
        meta.kvcache_segment = segs
        prepare_step(meta, engine.gpu_cache)
        for kc, vc in engine.gpu_cache:
            impl.forward(q, new_k, new_v, kc, vc, meta, k_scale, v_scale)
        return sum(lens)

    if backend_path:
        step = step_backend
    elif args.host_path == "plan" and args.partition_tokens == 0:
        step = step_plan
    else:
        step = step_ops

    def attn_bytes(sum_ctx: int) -> int:
        # K+V rows of every context token, plus q in and out out
        return sum_ctx * 2 * Hkv * D * eb + B * Hq * D * 2 + B * Hq * D * 2

    append_bytes = B * 2 * Hkv * D * (2 + eb)  # reshape_and_cache in/out

    # Everything below runs on a non-blocking stream of default priority, not on the null stream:
    # hipMemMap and hipMemUnmap wait for all work queued on the null stream, so a chunk mapped while
    # decode steps are queued there would drain the pipeline every time a sequence crosses 2 MiB.
    torch.cuda.synchronize()
    torch.cuda.set_stream(bench_stream(dev))

    # ---- timed regions: each exactly K steps, synchronised on both sides.  A region of few steps carries the
    # fixed cost of its two ends (the host work before the first launch reaches the GPU, the wake-up after
    # the last kernel) and whatever state the clocks are in; R regions are timed and the median one is
    # reported, all of them listed.
    for _ in range(W):
        step()
    regions = []
    for _ in range(R):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        nbytes = 0
        for _ in range(K):
            nbytes += L * (attn_bytes(step()) + append_bytes)
        host_dt = time.perf_counter() - t0  # all K steps issued; the GPU may still be running
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        regions.append((nbytes / dt / 1e9, dt, host_dt, nbytes))
    gbps, dt, host_dt, region_bytes = sorted(regions)[len(regions) // 2]
    ms_per_step = dt / K * 1e3
    tokens_per_s = B * K / dt

    # ---- per-kernel pass: HIP events around each kernel on the stream it runs on, steps queued back to
    # back as in the timed region (the events are read after the pass)
    lib = _C.lib()
    for _ in range(W):
        step()
    _C.check(lib.vtkv_set_kernel_timing(1))
    kbytes = []
    for _ in range(event_steps):
        kbytes += [attn_bytes(step())] * L
    _C.check(lib.vtkv_set_kernel_timing(0))
    t_stream = (C.c_float * len(kbytes))()
    t_reduce = (C.c_float * len(kbytes))()
    got = _C.check(lib.vtkv_attention_kernel_times(t_stream, t_reduce, len(kbytes)))
    assert got == len(kbytes), (got, len(kbytes))
    part_ms, red_ms = list(t_stream), list(t_reduce)
    avg_part_ms = float(np.mean(part_ms))
    achieved = float(np.mean(kbytes)) / (avg_part_ms * 1e-3) / 1e9
    ratio, mfma_busy, source = (None, None, None) if (args.head_size or args.heads) else measured_traffic(config)
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": None if ratio is None else int(ratio * float(np.mean(kbytes))),
                "traffic_unit": "bytes per launch", "traffic_over_algorithmic": ratio, "traffic_source": source,
                # (the ratio was measured in a separate rocprofv3 --pmc run of this workload, not in this run)
                "traffic_replayed_from_profile": ratio is not None,
                "kernel": "decode_attn_stream_kernel", "avg_kernel_us": round(avg_part_ms * 1e3, 2),
                "avg_reduce_kernel_us": round(float(np.mean(red_ms)) * 1e3, 2),
                "algorithmic_bytes_per_launch": int(np.mean(kbytes))}

    final_lens = [s.get_used_slot() // row for s in segs]

    trace = None
    if args.workgroup_trace:
        # the tracing build keeps {XCC id, start, span, end, tiles} of every workgroup of the last launch (100 MHz clock)
        torch.cuda.synchronize()
        step()
        torch.cuda.synchronize()
        buf = (C.c_ulonglong * (1024 * 6))()
        fn = lib.vtkv_debug_attn_trace
        fn.argtypes = [C.c_void_p, C.c_int]
        _C.check(fn(buf, 1024))
        t = np.array(list(buf), dtype=np.int64).reshape(1024, 6)
        t = t[t[:, 1] > t[:, 1].max() - 5000]   # the last launch only (a workgroup without tiles keeps an older record)
        t0 = t[:, 1].min()
        end = (t[:, 3] - t0) / 100.0
        trace = {"workgroups": int(len(t)), "end_us": {"min": round(float(end.min()), 1), "mean": round(float(end.mean()), 1),
                                                        "p90": round(float(np.percentile(end, 90)), 1),
                                                        "max": round(float(end.max()), 1)},
                 "start_spread_us": round(float((t[:, 1].max() - t0) / 100.0), 1),
                 "end_us_mean_by_xcc": [round(float(end[t[:, 0] == x].mean()), 1) for x in range(8)],
                 "end_us_by_dispatch_third": [round(float(end[(t[:, 2] % (len(t) // 8)) * 3 // (len(t) // 8) == k].mean()), 1)
                                              for k in range(3)]}

    # ---- swap: 25 % of the sequences out to pinned host memory and back.  Unmapping is lazy, so a
    # sequence swapped back in before its chunks were needed elsewhere finds them still mapped ("warm");
    # the second round trip forces the unmapping in between ("cold": swap-in has to map every chunk).
    swap = None
    if with_swap:
        nswap = max(1, B // 4)
        swap_slots = list(range(nswap))
        engine.swap_out(swap_slots)  # untimed: first use of the pinned arena and of the copy streams
        engine.swap_in(swap_slots)
        torch.cuda.synchronize()
        rounds = []
        for _ in range(5):   # single transfers of a few milliseconds scatter: five rounds, the median of each figure
            t0 = time.perf_counter()
            moved = engine.swap_out(swap_slots)
            t1 = time.perf_counter()
            engine.swap_in(swap_slots)
            t2 = time.perf_counter()
            engine.swap_out(swap_slots)
            t3 = time.perf_counter()
            trimmed = vmm.trim()
            t4 = time.perf_counter()
            engine.swap_in(swap_slots)
            t5 = time.perf_counter()
            rounds.append((moved / (t1 - t0) / 1e9, moved / (t2 - t1) / 1e9, moved / (t5 - t4) / 1e9,
                           (t4 - t3) / max(trimmed, 1) * 1e6))
        med = [sorted(r[k] for r in rounds)[len(rounds) // 2] for k in range(4)]
        swap = {"bytes_per_direction": moved, "out_gbps": round(med[0], 2), "in_gbps": round(med[1], 2),
                "in_cold_gbps": round(med[2], 2), "unmap_us_per_chunk": round(med[3], 1), "chunks": trimmed,
                "sequences": nswap, "rounds": len(rounds)}

    G = Hq // Hkv
    result = {
        "metric": "decode-attn HBM GB/s (% peak) + tokens/s @ Llama-3-8B shape B=64; swap GB/s",
        "value": round(gbps, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 (fp8-e4m3 KV)" if fp8 else "bf16", "data": "synthetic",
        "config": {"workload": cfg["name"], "layers": L, "new_tokens_per_step": B, "kv_chunk": f"{chunk >> 20}MiB VMM",
                   "mean_ctx": round(float(np.mean(final_lens)), 1), "host_path": args.host_path,
                   "fused_append": (bool(plan.fused) and step is step_plan) or (backend_path and not args.unfused),
                   "value_skew_bytes": engine.value_skew},
        "repeats": R,
        "regions_gbps": [round(r[0], 1) for r in regions],
        # attention + cache-write bytes of one step of the median region (value = this / ms_per_step)
        "algorithmic_bytes_per_step": int(region_bytes // K),
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "tokens_per_s": round(tokens_per_s, 1),
        "ms_per_layer": round(ms_per_step / L, 4),
        "host_issue_ms_per_step": round(host_dt / K * 1e3, 4),
        "swap": swap,
        "workgroup_trace": trace,
        "roofline": roofline,
        # matrix pipe of the dominant kernel, from the same counter runs as `traffic`: the share of SIMD
        # cycles with an MFMA executing, and the part of it that is real work (G of the 16 head columns)
        "mfma_util": None if mfma_busy is None else {"busy_frac": mfma_busy, "useful_frac": round(mfma_busy * G / 16, 4),
                                                      "source": source},
    }

    if with_cpu:
        result["cpu_baseline"] = cpu_baseline(cfg, engine, final_lens, q, scale, args.cpu_seconds, k_scale, v_scale)
        result["cpu_baseline_c1"] = cpu_baseline_c1(max(2.0, args.cpu_seconds / 3))

    engine.close()
    torch.cuda.synchronize()
    return result


_STREAM = {}


def bench_stream(dev):
    """The one non-blocking stream of default priority that every workload of this process runs on."""
    import torch

    if dev not in _STREAM:
        _STREAM[dev] = torch.cuda.Stream(device=dev)
    return _STREAM[dev]


def ensure_pool(chunks: int) -> None:
    """Have at least `chunks` free physical chunks in the pool (chunks of a workload that has ended are free again)."""
    from glake_amd import vmm_allocator as vmm

    have = vmm.showFreeBlocks() if vmm.totalBlocks() > 0 else 0
    if have < chunks:
        vmm.init_physical_handle(chunks - have, 0)




def growth_and_swap_protocol(args) -> dict:
    """BASELINE.json configs[4] as written: 256 sequences (bf16, Hq=32, Hkv=8, D=128, initial context
    U[256,2048], seed 1004), 64 decode steps that append one token each and map a 2 MiB chunk where a range
    crosses a boundary; after steps 16, 32, 48 and 64 a seeded random 25 % of the sequences is swapped out to
    pinned host memory and back in.  Reported: attention GB/s over the decode steps (each block of 16 steps timed
    between two synchronisations; algorithmic bytes as everywhere), host-link GB/s of every swap-out and swap-in
    (bytes of the swapped ranges over the wall time of the call, which ends with the copies done and the chunks
    given back or mapped), the chunks mapped while the sequences grew, and a bit-exact check: every byte of
    every swapped range is copied aside on the device before the swap-out and again after the swap-in (outside the
    timed calls) and the two copies are compared, and the rows appended by the 64 steps are compared with the
    step's inputs."""
    import torch

    from glake_amd import _C, vmm_allocator as vmm
    from glake_amd.worker.cache_engine import CacheEngine
    from glake_amd.worker.step import DecodeStepPlan

    cfg = CONFIGS["c5"]
    B, Hq, Hkv, D = cfg["batch"], cfg["hq"], cfg["hkv"], cfg["d"]
    steps, every, W = 64, 16, max(args.warmup, 5)
    dev = torch.device("cuda", 0)
    gen = torch.Generator().manual_seed(cfg["seed"])
    ctx0 = torch.randint(cfg["lo"], cfg["hi"] + 1, (B,), generator=gen).tolist()
    row = Hkv * D * 2
    chunk = vmm.chunkBytes()
    max_tokens = max(ctx0) + steps + W + 1
    chunks_per_range = (max_tokens * row + args.value_skew + chunk - 1) // chunk
    ensure_pool(2 * B * chunks_per_range + 16)
    engine = CacheEngine(num_layers=1, num_kv_heads=Hkv, head_size=D, dtype=torch.bfloat16, max_num_seqs=B,
                         max_num_batched_tokens=max_tokens, swap_space_bytes=1 << 30, value_skew=args.value_skew)
    segs = engine.vmm_kvcache_segment
    from glake_amd import _custom_ops as ops

    ggen = torch.Generator(device=dev).manual_seed(cfg["seed"])
    for b in range(B):
        nbytes = ctx0[b] * row
        segs[b].ensure_mapped(nbytes)
        for base in (segs[b].getKeyDevicePtr(0), segs[b].getValueDevicePtr(0)):
            t = torch.randn(ctx0[b], Hkv, D, generator=ggen, device=dev, dtype=torch.float32).to(torch.bfloat16)
            ops.swap_ranges([t.data_ptr()], [base], [nbytes], "d2d")
            torch.cuda.synchronize()
        segs[b].set_used_size(nbytes)
    q = torch.randn(B, Hq, D, generator=ggen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    new_k = torch.randn(B, Hkv * D, generator=ggen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    new_v = torch.randn(B, Hkv * D, generator=ggen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    out = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=dev)
    plan = DecodeStepPlan(segs, list(range(B)), engine.k_cache_ptr[0], engine.v_cache_ptr[0], Hq, Hkv, D,
                          float(D) ** -0.5, device=dev)
    torch.cuda.synchronize()
    torch.cuda.set_stream(bench_stream(dev))

    def snapshot(slots):
        """The used bytes of the K and V ranges of `slots`, gathered into one device buffer with device-to-device
        copies (the comparison stays on the GPU: reading 0.6 GB back to the host around every event would leave the
        GPU idle for a tenth of a second, which the next steps' clocks would show)."""
        sizes = [segs[s_].used_size for s_ in slots]
        buf = torch.empty(2 * sum(sizes), dtype=torch.uint8, device=dev)
        src, dst, nb, at = [], [], [], buf.data_ptr()
        for s_, n in zip(slots, sizes):
            for base in (segs[s_].getKeyDevicePtr(0), segs[s_].getValueDevicePtr(0)):
                src.append(base)
                dst.append(at)
                nb.append(n)
                at += n
        ops.swap_ranges(src, dst, nb, "d2d")
        return buf

    # warm-up steps (they append rows too), one untimed swap round trip (first use of the pinned arena and the copy
    # streams), then the sequences are set back to their initial lengths: the 64 steps start from BASELINE's contexts
    for _ in range(W):
        plan.run(q, new_k, new_v, out)
    torch.cuda.synchronize()
    engine.swap_out([0, 1])
    engine.swap_in([0, 1])
    torch.cuda.synchronize()
    for b in range(B):
        segs[b].set_used_size(ctx0[b] * row)
    mapped0 = sum(s.actual_size for s in segs) // chunk

    blocks, events = [], []
    bit_exact, checked = True, 0
    step_bytes = step_time = 0.0
    debug_timing = os.environ.get("VTKV_BENCH_BLOCK_KERNEL_TIMES") == "1"   # (events on every launch: slows the steps)
    kernel_us = []
    for blk in range(steps // every):
        torch.cuda.synchronize()
        if debug_timing:
            _C.check(_C.lib().vtkv_set_kernel_timing(1))
        t0 = time.perf_counter()
        nbytes = 0
        for _ in range(every):
            plan.run(q, new_k, new_v, out)
            nbytes += int(plan.seq_lens.sum()) * 2 * row + 2 * B * Hq * D * 2 + B * 2 * row * 2
        host_dt = time.perf_counter() - t0
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if debug_timing:
            _C.check(_C.lib().vtkv_set_kernel_timing(0))
            ts, tr = (C.c_float * every)(), (C.c_float * every)()
            _C.check(_C.lib().vtkv_attention_kernel_times(ts, tr, every))
            kernel_us.append([round(x * 1e3, 1) for x in ts] + [round(host_dt * 1e6 / every, 1)])
        blocks.append(round(nbytes / dt / 1e9, 1))
        step_bytes += nbytes
        step_time += dt
        # the swap event: a seeded random quarter of the sequences out and back in
        chosen = sorted(torch.randperm(B, generator=gen)[:B // 4].tolist())
        before = snapshot(chosen)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        moved = engine.swap_out(chosen)
        t1 = time.perf_counter()
        engine.swap_in(chosen)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        after = snapshot(chosen)
        bit_exact = bit_exact and after.shape == before.shape and bool(torch.equal(after, before))
        checked += after.numel()
        del before, after
        events.append({"after_step": (blk + 1) * every, "sequences": len(chosen), "bytes_per_direction": moved,
                       "out_gbps": round(moved / (t1 - t0) / 1e9, 2), "in_gbps": round(moved / (t2 - t1) / 1e9, 2)})
    mapped1 = sum(s.actual_size for s in segs) // chunk
    # the rows the 64 steps appended: every sequence's last 64 K and V rows equal the step's input rows
    nk = new_k.view(torch.int16).cpu().numpy().view(np.uint16)
    nv = new_v.view(torch.int16).cpu().numpy().view(np.uint16)
    appended_exact = True
    for b in range(B):
        appended_exact = appended_exact and segs[b].used_size == (ctx0[b] + steps) * row
        tail = np.empty((2, steps, Hkv * D), np.uint16)
        off = ctx0[b] * row
        _C.check(_C.lib().vtkv_memcpy_d2h(tail[0].ctypes.data_as(C.c_void_p), segs[b].getKeyDevicePtr(0) + off, steps * row))
        _C.check(_C.lib().vtkv_memcpy_d2h(tail[1].ctypes.data_as(C.c_void_p), segs[b].getValueDevicePtr(0) + off, steps * row))
        appended_exact = appended_exact and bool(np.all(tail[0] == nk[b]) and np.all(tail[1] == nv[b]))
    engine.close()
    torch.cuda.synchronize()
    med = lambda xs: sorted(xs)[len(xs) // 2]
    gbps = step_bytes / step_time / 1e9
    return {
        "workload": "growth+swap bf16: 256 seqs Hq=32 Hkv=8 D=128 ctx0~U[256,2048], 64 steps, 25 % swapped out and in "
                    "after steps 16/32/48/64 (BASELINE.json configs[4])",
        "value": round(gbps, 1), "unit": "GB/s", "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "ms_per_step": round(step_time / steps * 1e3, 4), "tokens_per_s": round(B * steps / step_time, 1),
        "algorithmic_bytes_per_step": int(step_bytes // steps), "steps": steps, "blocks_gbps": blocks,
        "chunks_mapped_while_growing": int(mapped1 - mapped0),
        "swap_events": events,
        "swap_out_gbps": med([e["out_gbps"] for e in events]), "swap_in_gbps": med([e["in_gbps"] for e in events]),
        "bit_exact": bool(bit_exact and appended_exact), "swapped_bytes_checked": int(checked),
        "appended_rows_checked": B * steps * 2,
        **({"kernel_us_by_block_and_host_us_per_step": kernel_us} if debug_timing else {}),
    }

def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _time_calls(run, budget_s: float):
    run()  # warm-up (thread pool, page faults)
    t0 = time.perf_counter()
    iters = 0
    while True:
        run()
        iters += 1
        el = time.perf_counter() - t0
        if el >= budget_s or iters >= 20000:
            return el / iters, iters, el


def cpu_baseline_c1(budget_s: float):
    """BASELINE config 1 exactly, on this host's cores: fp32, B=8, Hq=32, Hkv=8, D=128, ctx U[128,1024]
    (seed 1000; draws in the order ctx, q, K, V), the reference's CPU paged_attention_v1 on the paged
    block-16 layout behind a random block table, and the C restatement on the contiguous [T,Hkv,D] layout."""
    import torch

    from oracle import oracle as O

    gen = torch.Generator().manual_seed(1000)
    B, Hq, Hkv, D, bs, x = 8, 32, 8, 128, 16, 4
    lens = torch.randint(128, 1025, (B,), generator=gen).tolist()
    q = torch.randn(B, Hq, D, generator=gen).numpy()
    ks = [torch.randn(n, Hkv, D, generator=gen).numpy() for n in lens]
    vs = [torch.randn(n, Hkv, D, generator=gen).numpy() for n in lens]
    nblk = [(n + bs - 1) // bs for n in lens]
    perm = torch.randperm(sum(nblk), generator=gen).numpy()
    k_cache = np.zeros((sum(nblk), Hkv, D // x, bs, x), np.float32)
    v_cache = np.zeros((sum(nblk), Hkv, D, bs), np.float32)
    block_tables = np.zeros((B, max(nblk)), np.int32)
    at = 0
    for b in range(B):
        ids = perm[at:at + nblk[b]]
        at += nblk[b]
        block_tables[b, :nblk[b]] = ids
        for rows, dst in ((ks[b], k_cache), (vs[b], v_cache)):
            pad = np.zeros((nblk[b] * bs, Hkv, D), np.float32)
            pad[:lens[b]] = rows
            blk = pad.reshape(nblk[b], bs, Hkv, D)
            if dst is k_cache:
                dst[ids] = blk.reshape(nblk[b], bs, Hkv, D // x, x).transpose(0, 2, 3, 1, 4)
            else:
                dst[ids] = blk.transpose(0, 2, 3, 1)
    sl = np.array(lens, np.int32)
    scale = float(D) ** -0.5
    nbytes = sum(lens) * 2 * Hkv * D * 4 + 2 * B * Hq * D * 4
    out = {"workload": f"fp32 B={B} Hq={Hq} Hkv={Hkv} D={D} ctx~U[128,1024] seed 1000 ({sum(lens)} context tokens)",
           "cpu_model": cpu_model(), "unit": "GB/s", "algorithmic_bytes_per_call": nbytes}
    if O.ref_available():
        per, iters, el = _time_calls(lambda: O.ref_paged_attention(1, q, k_cache, v_cache, block_tables, sl, scale),
                                     budget_s)
        out["paged_block16"] = {"value": round(nbytes / per / 1e9, 3), "kind": "reference", "ms_per_call": round(per * 1e3, 3),
                                "cores": int(O.ref().ref_num_threads()), "calls": iters}
    else:
        pc = O.PagedCache(k_cache, v_cache, block_tables)
        per, iters, el = _time_calls(lambda: O.paged_attention_v1(q, pc, scale, sl), budget_s)
        out["paged_block16"] = {"value": round(nbytes / per / 1e9, 3), "kind": "port", "ms_per_call": round(per * 1e3, 3),
                                "cores": O.num_threads(), "calls": iters}
    vc = O.VTensorCache(ks, vs, np.arange(B), Hkv, D)
    per, iters, el = _time_calls(lambda: O.paged_attention_v1(q, vc, scale, sl), budget_s)
    out["contiguous"] = {"value": round(nbytes / per / 1e9, 3), "kind": "port", "ms_per_call": round(per * 1e3, 3),
                         "cores": O.num_threads(), "calls": iters}
    out["omp_max_threads"] = O.num_threads()
    return out


def cpu_baseline(cfg, engine, lens, q, scale, budget_s: float, k_scale: float = 1.0, v_scale: float = 1.0):
    """The reference's CPU paged attention v1 (compiled from the reference sources when that
    build is present, otherwise the C restatement) on the first sequences of the same batch, in the
    paged block-16 layout it requires.  An fp8 cache is first converted back to bf16 with its scale, the
    reference's own protocol for fp8 (tests/kernels/test_attention.py:233-252): its CPU kernels have no fp8."""
    import torch

    from glake_amd import _C
    from oracle import oracle as O

    B, Hq, Hkv, D = cfg["batch"], cfg["hq"], cfg["hkv"], cfg["d"]
    fp8 = cfg["kv"] == "fp8"
    nsample = min(B, 16)
    bs, x = 16, 8
    lens = lens[:nsample]
    nblk = [(n + bs - 1) // bs for n in lens]
    k_cache = np.zeros((sum(nblk), Hkv, D // x, bs, x), np.uint16)
    v_cache = np.zeros((sum(nblk), Hkv, D, bs), np.uint16)
    block_tables = np.zeros((nsample, max(nblk)), np.int32)
    blk0 = 0
    for b in range(nsample):
        seg = engine.vmm_kvcache_segment[b]
        n = lens[b]
        rows = np.zeros((nblk[b] * bs, Hkv, D), np.uint16)
        for which, dst in ((0, k_cache), (1, v_cache)):
            src = seg.getKeyDevicePtr(0) if which == 0 else seg.getValueDevicePtr(0)
            if fp8:
                codes = np.zeros((n, Hkv, D), np.uint8)
                _C.check(_C.lib().vtkv_memcpy_d2h(codes.ctypes.data_as(C.c_void_p), src, n * Hkv * D))
                rows[:n] = O.fp8_decode(codes, k_scale if which == 0 else v_scale, to_bf16=True)
            else:
                _C.check(_C.lib().vtkv_memcpy_d2h(rows.ctypes.data_as(C.c_void_p), src, n * Hkv * D * 2))
            blk = rows.reshape(nblk[b], bs, Hkv, D)
            if which == 0:  # [blk, bs, H, D/x, x] -> [blk, H, D/x, bs, x]
                dst[blk0:blk0 + nblk[b]] = blk.reshape(nblk[b], bs, Hkv, D // x, x).transpose(0, 2, 3, 1, 4)
            else:           # [blk, bs, H, D] -> [blk, H, D, bs]
                dst[blk0:blk0 + nblk[b]] = blk.transpose(0, 2, 3, 1)
        block_tables[b, :nblk[b]] = np.arange(blk0, blk0 + nblk[b])
        blk0 += nblk[b]
    q_np = q.view(B, Hq, D)[:nsample].contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    sl = np.array(lens, np.int32)
    if O.ref_available():
        kind = "reference"
        run = lambda: O.ref_paged_attention(1, q_np, k_cache, v_cache, block_tables, sl, scale)
        cores = int(O.ref().ref_num_threads())
    else:
        kind = "port"
        pc = O.PagedCache(k_cache, v_cache, block_tables)
        run = lambda: O.paged_attention_v1(q_np, pc, scale, sl)
        cores = O.num_threads()
    # contexts beyond 8192 rows: upstream's rule would take the split-K kernel there (vllm/attention/ops/
    # paged_attn.py:116-117; the fork forces v1, :118), so that one is timed beside v1 with half the budget
    v2 = None
    if max(lens) > 8192:
        budget_s /= 2
        if kind == "reference":
            run2 = lambda: O.ref_paged_attention(2, q_np, k_cache, v_cache, block_tables, sl, scale)
        else:
            run2 = lambda: O.paged_attention_v2(q_np, pc, scale, sl)
        v2 = _time_calls(run2, budget_s)
    per_call, iters, el = _time_calls(run, budget_s)
    # the bytes the CPU kernel reads: bf16 rows (also for an fp8 cache, which it sees dequantised)
    nbytes = sum(lens) * 2 * Hkv * D * 2 + 2 * nsample * Hq * D * 2
    extra = {} if v2 is None else {"v2": {"value": round(nbytes / v2[0] / 1e9, 3), "ms_per_call": round(v2[0] * 1e3, 3),
                                          "calls": v2[1], "what": "paged_attention_v2 (512-row partitions), same inputs"}}
    return {**extra, "value": round(nbytes / per_call / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": kind,
            "cpu_model": cpu_model(),
            "tokens_per_s": round(nsample / per_call, 1), "ms_per_call": round(per_call * 1e3, 3),
            "sample": f"paged_attention_v1 (block 16, bf16{' from the fp8 cache' if fp8 else ''}) on the first "
                      f"{nsample} of {B} sequences ({sum(lens)} context tokens), {iters} calls in {el:.1f} s"}


if __name__ == "__main__":
    sys.exit(main())
