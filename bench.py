#!/usr/bin/env python3
"""Routed tokens/s through the MoE dispatch + expert + combine hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config mixtral] [--no-cpu-baseline]

A "step" is one pass of rank 0's share of the path over one batch of synthetic tokens (see
iris_testing_amd/pipeline.py): route + count + pack as a source, unpack + grouped expert MLP + return
pack as a destination, combine as a source.  Inputs are resident in HBM when the timed region starts.
Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"hbm": 8000.0, "mfma_bf16": 2500.0, "mfma_fp8": 5000.0, "fp32": 157.3}  # GB/s, TFLOP/s


def cpu_baseline(cfg, world_np, budget_tokens: int):
    """The CPU oracle timed on a bounded sample of the same workload: the first `budget_tokens`
    tokens of shard 0 through route + count + pack, their routed rows through rank 0's expert MLP,
    and the combine.  Returns (tokens/s, seconds, threads, description)."""
    import numpy as np
    from oracle import moe_oracle as O

    x, router, bias, weights = world_np
    Ts = min(budget_tokens, x.shape[0])
    xs = x[:Ts]
    t0 = time.perf_counter()
    idx, gate, _ = O.route(xs, router, cfg.topk, bias)
    counts = O.send_counts(idx, cfg.world, cfg.experts)
    sizes, offs = O.dst_sizes_offsets(counts)
    pos, row_token = O.payload_positions(idx, cfg.experts)
    payload = O.send_payload(xs, row_token)
    M = O.pair_capacity(sizes)
    send = O.pack_fixed_m(payload, offs, sizes, M)
    # destination side on the same number of routed rows: all rows through the local experts of rank 0,
    # spread over them in proportion (the sample keeps rows-per-token = k)
    rows = payload
    E_l = cfg.e_local
    cnt = np.full(E_l, rows.shape[0] // E_l, np.int32)
    cnt[: rows.shape[0] - int(cnt.sum())] += 1
    if cfg.quant == "fp8":
        y = O.expert_mlp_fp8(rows, cnt, *weights)
    elif cfg.act == "swiglu":
        y = O.expert_mlp(rows, cnt, weights[0], weights[2], "swiglu", cfg.dtype, w_up=weights[1])
    else:
        y = O.expert_mlp(rows, cnt, weights[0], weights[1], cfg.act, cfg.dtype)
    ret = O.pack_fixed_m(y, offs, sizes, M)
    out = O.combine(ret, idx, pos, gate, offs, E_l, cfg.dtype)
    dt = time.perf_counter() - t0
    assert out.shape == xs.shape and send.shape[1] == M
    return Ts / dt, dt, blas_threads(), f"first {Ts} tokens of shard 0 ({rows.shape[0]} routed rows), all stages, numpy/C oracle"


def blas_threads() -> int:
    """Threads the BLAS behind numpy's matmul actually runs (where the CPU baseline spends its time)."""
    try:
        from threadpoolctl import threadpool_info
        n = [int(p["num_threads"]) for p in threadpool_info() if p.get("user_api") == "blas"]
        if n:
            return max(n)
    except Exception:
        pass
    return 1


def per_element_loop_baseline():
    """The reference's own host algorithm, one Python iteration per routed slot (utils.py:213-219), on the
    CPU-runnable plumbing workload (256 tokens, top-2): timed for the record, one thread."""
    from iris_testing_amd.configs import CONFIGS, gen_router, gen_shard_tokens
    from oracle import moe_oracle as O
    cfg = CONFIGS["plumbing"]
    x, router = gen_shard_tokens(cfg, 0).numpy(), gen_router(cfg).numpy()
    t0 = time.perf_counter()
    idx = O.route(x, router, cfg.topk)[0]
    payload, counts, offs, sizes = O.bucket_loop_pack(x, idx, cfg.world, cfg.experts)
    dt = time.perf_counter() - t0
    assert payload.shape[0] == cfg.tokens * cfg.topk
    return {"value": round(cfg.tokens / dt, 1), "unit": "tokens/s", "cores": 1, "seconds": round(dt, 4),
            "sample": "plumbing workload, route + per-slot Python bucket loop + payload (the reference's host routine)"}


def profiled_traffic(workload: str, stage: str):
    """HBM bytes per launch of a stage's kernel as summarised under profiles/ from separate rocprofv3 --pmc runs
    (FETCH_SIZE, WRITE_SIZE): the line `TRAFFIC_BYTES <stage> <bytes>` of profiles/<workload>_hbm_traffic.txt.
    (None, None) when no such summary exists: this run itself measures no counters."""
    path = os.path.join(ROOT, "profiles", f"{workload}_hbm_traffic.txt")
    try:
        with open(path) as f:
            for line in f:
                p = line.split()
                if len(p) >= 3 and p[0] == "TRAFFIC_BYTES" and p[1] == stage:
                    return float(p[2]), f"profiles/{workload}_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, separate runs)"
    except OSError:
        pass
    return None, None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="mixtral")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay timing")
    ap.add_argument("--bf16-dispatch", action="store_true",
                    help="fp8 workloads: send the tokens as bf16 and quantise them at the destination (default: quantise "
                         "them where they are packed and send fp8 codes and scales)")
    ap.add_argument("--unfused", action="store_true",
                    help="run the destination side as unpack + MLP + return pack (the reference's operator split) "
                         "instead of gathering / scattering inside the GEMMs")
    ap.add_argument("--cpu-sample-tokens", type=int, default=0, help="0 = sized for roughly 10-30 s")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs rank 0's share of the path on ONE GPU; "
              "no collectives or multi-GPU sharding exist, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from iris_testing_amd import harness
    from iris_testing_amd.configs import CONFIGS
    from iris_testing_amd.pipeline import STAGES, DispatchPipeline

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    cfg = CONFIGS[args.config]
    dev = "cuda"
    torch.cuda.set_device(0)

    # ---- untimed set-up: W seeded shards routed and packed, rank 0's receive buffer assembled
    world = harness.build_world(cfg, dev)
    ew, raw, qs = harness.expert_weights(cfg, 0, dev)
    pipe = DispatchPipeline(world, ew, fused=False if args.unfused else None,
                            fp8_dispatch=False if (args.unfused or args.bf16_dispatch) else None)
    # the returned buffer: slot 0 is rank 0's own return slot; the other slots stand in for what the
    # other ranks' experts would send back (same shape and dtype, arbitrary finite contents)
    pipe.step()
    torch.cuda.synchronize()
    g = torch.Generator(device="cpu").manual_seed(cfg.seed + 4242)
    pipe.returned.copy_(torch.randn(pipe.returned.shape, generator=g, dtype=torch.float32).to(cfg.torch_dtype))
    pipe.returned[0].copy_(pipe.ret[0])
    assert int(pipe.status.item()) == 0

    for _ in range(args.warmup):
        pipe.step()
    torch.cuda.synchronize()

    events = []
    t_start, t_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    wall0 = time.perf_counter()
    t_start.record()
    for _ in range(args.steps):
        pipe.step(events)
    t_end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall0
    ms_total = t_start.elapsed_time(t_end)
    ms_per_step = ms_total / args.steps

    # the same K steps replayed as one HIP graph per step (launch overhead removed); the headline value is
    # the faster of the two ways of launching, and says which
    launch = "stream"
    if not args.no_graph:
        graph = pipe.capture()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        g0.record()
        for _ in range(args.steps):
            graph.replay()
        g1.record()
        torch.cuda.synchronize()
        ms_graph = g0.elapsed_time(g1) / args.steps
        stream_ms_per_step = ms_per_step
        if ms_graph < ms_per_step:
            ms_per_step, launch = ms_graph, "hipGraph"
    else:
        ms_graph, stream_ms_per_step = None, ms_per_step

    per_stage = {n: sorted(e[n][0].elapsed_time(e[n][1]) for e in events) for n in STAGES}
    stage_ms = {n: sum(v) / len(v) for n, v in per_stage.items()}
    stage_spread = {n: (v[0], v[len(v) // 2]) for n, v in per_stage.items()}  # (min, median) over the timed steps
    work = pipe.work()
    stages = {}
    for n, wk in work.items():
        ms = stage_ms[n]
        if ms <= 0:
            continue
        if wk["bound"] == "latency":
            # a few KB or a few rows: no roofline applies, the time is launch + dependency latency
            stages[n] = {"ms": round(ms, 4), "bound": "latency", "bytes": wk["amount"]}
            continue
        if wk["bound"] == "hbm":
            ach, peak, unit = wk["amount"] / (ms * 1e-3) / 1e9, PEAK["hbm"], "GB/s"
        else:
            ach = wk["amount"] / (ms * 1e-3) / 1e12
            peak = PEAK["mfma_fp8"] if cfg.quant == "fp8" else (PEAK["fp32"] if cfg.dtype == "f32" else PEAK["mfma_bf16"])
            unit = "TFLOP/s"
        stages[n] = {"ms": round(ms, 4), "ms_min": round(stage_spread[n][0], 4), "ms_median": round(stage_spread[n][1], 4),
                     "bound": wk["bound"], "achieved": round(ach, 2), "peak": peak, "unit": unit, "frac": round(ach / peak, 4)}
    dom = "mlp_up"  # the gate/up grouped GEMM: most of the flops of a step
    traffic, traffic_source = profiled_traffic(cfg.name, dom + "_fp8_dispatch" if pipe.fp8_dispatch else dom)
    if cfg.quant == "fp8":
        kname = ("moe_grouped_mlp_fp8_q (gate/up GEMM + SwiGLU + re-quantisation + down GEMM; the tokens arrive quantised)"
                 if pipe.fp8_dispatch else
                 "moe_grouped_mlp_fp8 (row quantisation + gate/up GEMM + SwiGLU + re-quantisation + down GEMM)")
    elif cfg.dtype == "f32":
        kname = "moe_grouped_mlp fp32 (both GEMMs)"
    else:
        kname = "grouped_gemm_kernel (gate/up + SwiGLU epilogue)" if cfg.act == "swiglu" else "grouped_gemm_kernel (up + activation)"
    roofline = {"kernel": kname,
                "bound": "mfma", "achieved": stages[dom]["achieved"], "peak": stages[dom]["peak"], "unit": "TFLOP/s",
                "frac": stages[dom]["frac"], "traffic": traffic, "traffic_source": traffic_source,
                "avg_launch_ms": stages[dom]["ms"], "flops_per_launch": work[dom]["amount"]}

    out = {
        "metric": "routed tokens/sec (dispatch+expert+combine) at 1 MI355X",
        "value": round(cfg.tokens / (ms_per_step * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8" if cfg.quant == "fp8" else cfg.dtype,
        "data": "synthetic (seeded N(0,1) tokens, random-init router and expert weights)",
        "config": {"workload": cfg.name, "tokens": cfg.tokens, "hidden": cfg.hidden, "experts": cfg.experts,
                   "topk": cfg.topk, "world": cfg.world, "ffn": cfg.ffn, "act": cfg.act, "M": world.M, "CAP": world.CAP,
                   "rows_received": world.S},
        "routed_rows_per_s": round(cfg.tokens * cfg.topk / (ms_per_step * 1e-3), 1),
        "host_wall_ms_per_step": round(wall * 1e3 / args.steps, 4),
        "launch": launch,
        "destination_side": "gather/scatter inside the GEMMs" if pipe.fused else "unpack + MLP + return pack",
        "dispatch": "fp8 codes + row scales (quantised while packing)" if pipe.fp8_dispatch else cfg.dtype,
        "ms_per_step_stream": round(stream_ms_per_step, 4),
        "ms_per_step_graph": None if ms_graph is None else round(ms_graph, 4),
        "roofline": roofline,
        "stages": stages,
    }

    if not args.no_cpu_baseline:
        def to_np(t):
            t = t.detach().cpu()
            return t.float().numpy() if t.dtype == torch.bfloat16 else t.numpy()

        x_np = to_np(world.x0)
        router_np = to_np(world.router)
        bias_np = None if world.bias is None else to_np(world.bias)
        if qs is not None:
            w_np = tuple(to_np(t) for pair in qs for t in pair)
        else:
            w_np = tuple(to_np(t) for t in raw)
        flops_per_token = 2 * cfg.hidden * cfg.ffn * cfg.n_mat * cfg.topk
        sample = args.cpu_sample_tokens or max(64, min(cfg.tokens, int(1.2e13 / flops_per_token)))
        v, secs, threads, desc = cpu_baseline(cfg, (x_np, router_np, bias_np, w_np), sample)
        out["cpu_baseline"] = {"value": round(v, 1), "unit": "tokens/s", "cores": threads, "kind": "port",
                               "sample": desc, "seconds": round(secs, 2), "host_cpus": os.cpu_count(),
                               "per_element_loop_plumbing": per_element_loop_baseline()}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
