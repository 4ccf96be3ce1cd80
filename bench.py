#!/usr/bin/env python3
"""Routed tokens/s through the MoE dispatch + expert + combine hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config mixtral] [--no-cpu-baseline]
                    [--unfused | --gated | --padding-free] [--backward] [--stream-ceiling] [--mfma-ceiling]

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


def cpu_baseline(cfg, router, bias, weights, budget_tokens: int):
    """The CPU oracle timed on the same step as the GPU leg, on a bounded sample of the same workload: the simulated
    world made of the first ``budget_tokens`` tokens of EVERY source shard (the whole workload when the budget covers
    it).  Untimed, as on the GPU: routing and packing the other shards to assemble rank 0's receive buffer and its
    real, skewed recv_counts.  Timed: rank 0 as a source (route + count + pack), as a destination (expert-major unpack
    of what it received, grouped expert MLP over the real per-expert row counts, return pack), as a source again
    (combine).  Returns (tokens/s, seconds, threads, description)."""
    import numpy as np
    from iris_testing_amd.configs import gen_shard_tokens
    from oracle import moe_oracle as O

    W, E, E_l, k = cfg.world, cfg.experts, cfg.e_local, cfg.topk
    Ts = min(budget_tokens, cfg.tokens)
    f32 = lambda t: t.float().numpy() if t.dtype != __import__("torch").float32 else t.numpy()  # noqa: E731
    xs = [f32(gen_shard_tokens(cfg, s)[:Ts]) for s in range(W)]

    def source_side(x):
        idx, gate, _ = O.route(x, router, k, bias)
        counts = O.send_counts(idx, W, E)
        sizes, offs = O.dst_sizes_offsets(counts)
        pos, row_token = O.payload_positions(idx, E)
        return idx, gate, counts, sizes, offs, pos, O.send_payload(x, row_token)

    # ---- untimed: what the other ranks send to rank 0
    others = [source_side(x) for x in xs]
    M = O.pair_capacity(np.stack([o[3] for o in others]))
    recv = np.stack([O.pack_fixed_m(o[6], o[4], o[3], M)[0] for o in others])
    rc = np.stack([o[2][0] for o in others]).astype(np.int32)
    S = int(rc.sum())
    rng = np.random.default_rng(cfg.seed + 4242)
    returned = O.round_to(rng.standard_normal((W, M, cfg.hidden)).astype(np.float32), cfg.dtype)
    del others

    # ---- timed: one step of rank 0
    t0 = time.perf_counter()
    idx, gate, counts, sizes, offs, pos, payload = source_side(xs[0])
    assert O.pair_capacity(sizes) <= M
    send = O.pack_fixed_m(payload, offs, sizes, M)
    rows = O.unpack_expert_major(recv, rc)
    cnt = O.expert_row_counts(rc.T)
    if cfg.quant == "fp8":
        y = O.expert_mlp_fp8(rows, cnt, *weights)
    elif cfg.act == "swiglu":
        y = O.expert_mlp(rows, cnt, weights[0], weights[2], "swiglu", cfg.dtype, w_up=weights[1])
    else:
        y = O.expert_mlp(rows, cnt, weights[0], weights[1], cfg.act, cfg.dtype)
    ret = O.return_pack(y, rc, M)
    returned[0] = ret[0]
    out = O.combine(returned, idx, pos, gate, offs, E_l, cfg.dtype)
    dt = time.perf_counter() - t0
    assert out.shape == xs[0].shape and send.shape == (W, M, cfg.hidden) and rows.shape[0] == S
    whole = "the whole workload" if Ts == cfg.tokens else f"the first {Ts} of {cfg.tokens} tokens of every source shard"
    return Ts / dt, dt, blas_threads(), (f"{whole}: rank 0 routes and packs {Ts} tokens, runs its {E_l} local experts on the "
                                         f"{S} rows it receives (real per-expert counts, {int(cnt.min())}..{int(cnt.max())}), "
                                         f"returns them and combines; numpy/C oracle")


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


def _timed(fn, n, torch):
    """Average milliseconds of n calls of fn on the current stream (one untimed call first)."""
    fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(n):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / n


def backward_leg(cfg, world, raw, steps):
    """Forward and backward of rank 0's expert MLP at the workload's shape (the S rows it receives, its real per-expert
    counts), through the autograd operators of the host layer: gradients with respect to the rows and to every weight
    matrix.  bf16 / fp32 experts only.  Flops: forward 2 S H F n_mat, backward twice that (one product for the
    gradient of the input and one for the gradient of the weights per forward product)."""
    import torch
    from iris_testing_amd import ops
    from iris_testing_amd.layers import ExpertWeights, expert_mlp
    from iris_testing_amd.layers.expert import _packed_weights_t, _part_ws
    dev = world.recv.device
    S, H, F = world.S, cfg.hidden, cfg.ffn
    rows, cnt = ops.unpack_expert_major(world.recv, world.recv_counts, S)
    rows.requires_grad_(True)
    ws = [w.to(dev).requires_grad_(True) for w in raw]
    ew = ExpertWeights.prepare(cfg.act, ws[0], ws[2], ws[1]) if cfg.act == "swiglu" else ExpertWeights.prepare(cfg.act, ws[0], ws[1])
    gy = torch.randn((S, H), generator=torch.Generator(device="cpu").manual_seed(cfg.seed + 77), dtype=torch.float32).to(cfg.torch_dtype).to(dev)

    def fwd():
        with torch.no_grad():
            expert_mlp(rows, ew, cnt)

    def fwd_bwd():
        rows.grad = None
        for w in ws:
            w.grad = None
        expert_mlp(rows, ew, cnt).backward(gy)

    f_ms = _timed(fwd, steps, torch)
    fb_ms = _timed(fwd_bwd, steps, torch)
    # the forward inside fwd_bwd also keeps the pre-activations (one more store per value): time it on its own
    def fwd_keep():
        expert_mlp(rows, ew, cnt)
    fk_ms = _timed(fwd_keep, steps, torch)
    b_ms = fb_ms - fk_ms
    fl_f = 2 * S * H * F * cfg.n_mat
    peak = PEAK["fp32"] if cfg.dtype == "f32" else PEAK["mfma_bf16"]
    # the pieces of the backward pass one by one (same calls as ExpertMLP.backward makes)
    pieces = {}
    if cfg.dtype == "bf16":
        swiglu = cfg.act == "swiglu"
        NP = 2 * F if swiglu else F
        pws = _part_ws(dev)
        with torch.no_grad():
            hidden = torch.empty((S, F), dtype=rows.dtype, device=dev)
            a1 = torch.empty((S, NP), dtype=rows.dtype, device=dev)
            ops.grouped_gemm_act_keep(rows, ew.w1, cnt, S, F, ew.act, hidden, a1, part_ws=pws)
            dh = torch.zeros((S, F), dtype=rows.dtype, device=dev)
            dx = torch.zeros((S, H), dtype=rows.dtype, device=dev)
            w1r, w2r, wur = ew.raw
            w2t, w1t = _packed_weights_t(w2r), _packed_weights_t(w1r, wur)
            da1 = ops.mlp_act_backward(a1, dh, ew.act)
            pieces["d_hidden = dy @ W2^T"] = (_timed(lambda: ops.grouped_gemm_mapped(gy, None, w2t, cnt, S, F, "none", dh, part_ws=pws), steps, torch), 2 * S * H * F)
            pieces["d_W2 = hidden^T @ dy (ragged K)"] = (_timed(lambda: ops.grouped_gemm_dw(hidden, gy, cnt), steps, torch), 2 * S * H * F)
            pieces["activation gradient"] = (_timed(lambda: ops.mlp_act_backward(a1, dh, ew.act), steps, torch), 0)
            pieces["d_x = d_a1 @ W1^T"] = (_timed(lambda: ops.grouped_gemm_mapped(da1, None, w1t, cnt, S, H, "none", dx, part_ws=pws), steps, torch), 2 * S * H * NP)
            pieces["d_W1 = x^T @ d_a1 (ragged K)"] = (_timed(lambda: ops.grouped_gemm_dw(rows, da1, cnt, split_F=F if swiglu else 0), steps, torch), 2 * S * H * NP)
    return {
        "what": "expert MLP of rank 0 on the rows it receives: forward, then gradients of the rows and of every weight matrix",
        "rows": S, "forward_ms": round(f_ms, 4), "forward_keeping_preactivations_ms": round(fk_ms, 4),
        "backward_ms": round(b_ms, 4), "backward_over_forward": round(b_ms / f_ms, 3),
        "forward_tflops": round(fl_f / f_ms / 1e9, 1), "backward_tflops": round(2 * fl_f / b_ms / 1e9, 1),
        "backward_frac_of_peak": round(2 * fl_f / b_ms / 1e9 / peak, 4), "peak_tflops": peak,
        "pieces": {n: {"ms": round(ms, 4), **({"tflops": round(fl / ms / 1e9, 1), "frac": round(fl / ms / 1e9 / peak, 4)} if fl else {})}
                   for n, (ms, fl) in pieces.items()},
    }


def mfma_ceiling_leg(steps):
    """What the matrix cores sustain from registers (moe_diag_mfma_loop: the grouped GEMM's wave layout, no LDS, no memory),
    on all-zero operands and on operands drawn like N(0,1): the chip runs against a power limit, so the second figure, not the
    published peak, is what a GEMM on the workload's data can approach."""
    import torch
    L_ = __import__("iris_testing_amd._lib", fromlist=["x"])
    lib = L_.lib()
    sink = torch.empty(lib.moe_diag_mfma_loop_sink_floats(), dtype=torch.float32, device="cuda")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = {"what": "register-only MFMA loop, 4 waves per compute unit, 128 x 128 outputs per wave (bf16: 16x16x32, fp8: 32x32x64)",
           "workgroups": cus}
    for fp8, name, peak in ((0, "bf16", PEAK["mfma_bf16"]), (1, "fp8", PEAK["mfma_fp8"])):
        for rnd, dname in ((0, "zeros"), (1, "normal")):
            iters = 100000  # (about 50 ms per launch, several launches back to back: the power limit acts on sustained load)
            fl = lib.moe_diag_mfma_loop_flops(fp8, iters, cus)
            ms = _timed(lambda: L_.check(lib.moe_diag_mfma_loop(fp8, rnd, iters, cus, L_.ptr(sink), L_.stream_ptr())), max(steps, 3), torch)
            out[f"{name}_{dname}"] = {"ms": round(ms, 3), "TFLOP/s": round(fl / ms / 1e9, 1), "frac_of_published_peak": round(fl / ms / 1e9 / peak, 4)}
    return out


def stream_ceiling_leg(cfg, steps, world=None):
    """What the memory system sustains for the three traffic mixes of the row-moving stages, measured with the product's own
    kernels on buffers of 1 GiB: a plain row copy (moe_pack_payload with the identity map: one byte read per byte written),
    a pure write (moe_zero_padding_rows over a buffer that is all padding) and read-mostly sums (moe_combine with unit gates
    and k rows read per row written).  From the first two, the read rate R and write rate W of the model
    time = read bytes / R + written bytes / W.  Then the same three at the sizes of this workload's own stages (the copy on
    as many rows as the unpack moves, the sums on as many tokens as the combine, slots in sequence): a launch's start-up
    and drain do not shrink with the buffer, so the rates of a 0.4 GB launch are lower than those of a 2 GB one."""
    import torch
    from iris_testing_amd import ops
    dev = "cuda"
    H = cfg.hidden
    B = 2
    rows = (1 << 30) // (H * B)
    src = torch.randn((rows, H), device=dev, dtype=torch.float32).to(torch.bfloat16)
    ident = torch.arange(rows, dtype=torch.int32, device=dev)
    dst = torch.empty_like(src)
    L_ = __import__("iris_testing_amd._lib", fromlist=["x"])
    lib, p, st = L_.lib(), L_.ptr, L_.stream_ptr

    def copy():
        L_.check(lib.moe_pack_payload(p(src), 1, rows, H, p(ident), rows, p(dst), st()))
    ms_copy = _timed(copy, steps, torch)
    zero_counts = torch.zeros((1, 1), dtype=torch.int32, device=dev)

    def write():
        L_.check(lib.moe_zero_padding_rows(p(dst), 1, 1, rows, H, p(zero_counts), 1, st()))
    ms_write = _timed(write, steps, torch)
    n_bytes = rows * H * B
    copy_rate = 2 * n_bytes / ms_copy / 1e6   # GB/s
    write_rate = n_bytes / ms_write / 1e6
    read_rate = n_bytes / (ms_copy - ms_write) / 1e6 if ms_copy > ms_write else float("nan")
    out = {"buffer_rows": rows, "row_bytes": H * B,
           "copy": {"kernel": "gather_rows_kernel (moe_pack_payload, identity map)", "ms": round(ms_copy, 4), "GB/s": round(copy_rate, 1)},
           "write": {"kernel": "zero_padding_rows_kernel (every row padding)", "ms": round(ms_write, 4), "GB/s": round(write_rate, 1)},
           "model": {"read_GB/s": round(read_rate, 1), "write_GB/s": round(write_rate, 1),
                     "formula": "time = bytes read / read rate + bytes written / write rate; read rate from copy time - write time"},
           "combine_unit_gates": {}}
    for k in (1, 2, 8):
        T = rows // k
        idx = torch.zeros((T, k), dtype=torch.int32, device=dev)
        # slot of (t, kk): rows spread over the whole buffer, every row read exactly once
        pos = (torch.arange(T, device=dev, dtype=torch.int32)[:, None] + T * torch.arange(k, device=dev, dtype=torch.int32)[None, :]).contiguous()
        zero = torch.zeros(1, dtype=torch.int32, device=dev)
        o = torch.empty((T, H), dtype=torch.bfloat16, device=dev)

        def comb():
            L_.check(lib.moe_combine(p(src), 1, 1, rows, H, p(idx), p(pos), None, p(zero), T, k, 1, p(o), None, st()))
        ms = _timed(comb, steps, torch)
        rd, wr = T * k * H * B, T * H * B
        model_ms = (rd / read_rate + wr / write_rate) / 1e6
        out["combine_unit_gates"][f"k={k}"] = {"ms": round(ms, 4), "GB/s": round((rd + wr) / ms / 1e6, 1), "read_share": round(rd / (rd + wr), 3),
                                                "model_GB/s": round((rd + wr) / model_ms / 1e6, 1)}
    if world is not None and cfg.dtype == "bf16":
        # the same kernels at this workload's sizes
        S, T, k = world.S, cfg.tokens, cfg.topk
        n_copy = min(S, rows)

        def copy_w():
            L_.check(lib.moe_pack_payload(p(src), 1, rows, H, p(ident), n_copy, p(dst), st()))
        ms_c = _timed(copy_w, steps, torch)
        n_slots = min(T * k, rows)
        Tw = n_slots // k
        idx = torch.zeros((Tw, k), dtype=torch.int32, device=dev)
        pos = (torch.arange(Tw, device=dev, dtype=torch.int32)[:, None] + Tw * torch.arange(k, device=dev, dtype=torch.int32)[None, :]).contiguous()
        zero = torch.zeros(1, dtype=torch.int32, device=dev)
        o = torch.empty((Tw, H), dtype=torch.bfloat16, device=dev)

        def comb_w():
            L_.check(lib.moe_combine(p(src), 1, 1, rows, H, p(idx), p(pos), None, p(zero), Tw, k, 1, p(o), None, st()))
        ms_s = _timed(comb_w, steps, torch)
        out["at_workload_size"] = {
            "copy": {"rows": n_copy, "MB": round(2 * n_copy * H * B / 1e6, 1), "ms": round(ms_c, 4), "GB/s": round(2 * n_copy * H * B / ms_c / 1e6, 1)},
            "combine_unit_gates": {"tokens": Tw, "k": k, "MB": round((Tw * k + Tw) * H * B / 1e6, 1), "ms": round(ms_s, 4),
                                   "GB/s": round((Tw * k + Tw) * H * B / ms_s / 1e6, 1)}}
    return out


def gemm_phases_leg(cfg, pipe, steps):
    """Where time goes inside the grouped GEMMs of this workload (moe_diag_gemm_trace: the same kernels with wall-clock stamps):
    per tile the K loop, the epilogue and the gap to the next K loop, averaged over all workgroups and tiles but each
    workgroup's first; the duration of one MFMA block (64 bytes of K of a 256 x 256 tile) of workgroup 0 early and late in the
    launch (the clock falls under sustained load); and the same launch with the epilogue's stores suppressed."""
    import numpy as np
    import torch
    L_ = __import__("iris_testing_amd._lib", fromlist=["x"])
    lib = L_.lib()
    words = lib.moe_diag_gemm_trace_words()
    TW = 256  # words per workgroup
    n_wg = (words - 4096) // TW
    buf = torch.zeros(words, dtype=torch.int64, device="cuda")
    fp8 = cfg.quant == "fp8"
    s = L_.stream_ptr()
    out = {"clock": "100 MHz wall clock, times in microseconds", "workgroups": n_wg}
    for name, sel, fn in (("gate_up", 0x200, pipe.mlp_up), ("down", 0x100, pipe.mlp_up if fp8 else pipe.mlp_down)):
        out[name] = {}
        variants = (("with_stores", 0), ("stores_suppressed", 1))
        call_ms = {label: [] for label, _ in variants}
        stamps = {}
        for rep in range(3):  # (the two variants in turn: what the clock does under sustained load then weighs on both alike)
            for label, bit in variants:
                L_.check(lib.moe_diag_gemm_trace(buf.data_ptr(), words, sel | bit))
                try:
                    call_ms[label].append(_timed(lambda: fn(s), max(steps // 2, 2), torch))
                    if rep == 2:
                        buf.zero_()
                        fn(s)
                        torch.cuda.synchronize()
                        stamps[label] = buf.cpu().numpy()
                finally:
                    L_.check(lib.moe_diag_gemm_trace(None, 0, 0))
        for label, bit in variants:
            ms = sum(call_ms[label]) / len(call_ms[label])
            h = stamps[label]
            tiles = h[:n_wg * TW].reshape(n_wg, TW)
            kl, ep, gap = [], [], []
            per_wg = []
            for w in range(n_wg):
                ev = tiles[w][tiles[w] > 0]
                n = len(ev) // 3
                per_wg.append(n)
                if n < 2:
                    continue
                e = ev[:3 * n].reshape(n, 3).astype(np.float64) / 100.0
                kl += list(e[1:, 1] - e[1:, 0])
                ep += list(e[1:, 2] - e[1:, 1])
                gap += list(e[1:, 0] - e[:-1, 1])
            blk = h[n_wg * TW:]
            # workgroup 0: from the start of a tile's K loop to the end of its first MFMA block (the hand-over at the end of that
            # block waits, in issue order, behind the stores of the epilogue before it)
            ev0 = tiles[0][tiles[0] > 0]
            b0 = blk[blk > 0]
            first = []
            for ti in range(1, len(ev0) // 3):
                after = b0[b0 > ev0[3 * ti]]
                if len(after) and after[0] <= ev0[3 * ti + 1]:
                    first.append((after[0] - ev0[3 * ti]) / 100.0)
            d = np.diff(blk[blk > 0].astype(np.float64)) / 100.0
            med = float(np.median(d)) if len(d) else float("nan")
            body = d[d < 2.0 * med] if len(d) else d   # (blocks inside a K loop: the stamps across a tile boundary hold the epilogue)
            q = max(len(body) // 4, 1)
            stamped = h[h > 0]
            out[name][label] = {
                "call_ms": round(ms, 4), "tiles_per_workgroup": [int(min(per_wg)), int(max(per_wg))],
                "k_loop_us": round(float(np.mean(kl)), 2), "epilogue_us": round(float(np.mean(ep)), 2),
                "k_loop_end_to_next_k_loop_us": round(float(np.mean(gap)), 2),
                "block_us_first_quarter": round(float(np.median(body[:q])), 3), "block_us_last_quarter": round(float(np.median(body[-q:])), 3),
                "first_block_of_a_tile_us": round(float(np.median(first)), 2) if first else None,
                "blocks_stamped": int(len(d) + 1), "launch_span_us": round(float(stamped.max() - stamped.min()) / 100.0, 1)}
    if fp8:
        out["note"] = "fp8: one call runs both GEMMs (call_ms is the call; the stamps are of the GEMM named)"
    pipe.step()
    torch.cuda.synchronize()
    return out


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
    ap.add_argument("--gated", action="store_true",
                    help="ship the top-k gates with the rows, weight the result rows in the down projection's epilogue, "
                         "combine by plain sum (bf16 experts)")
    ap.add_argument("--padding-free", action="store_true",
                    help="rows cross as the padding-free payload instead of fixed-M slots: the GEMMs gather from / scatter "
                         "into flat buffers through a row map over the payload")
    ap.add_argument("--backward", action="store_true", help="also time forward + backward of rank 0's expert MLP")
    ap.add_argument("--stream-ceiling", action="store_true",
                    help="also measure copy / write / read-mostly rates of the row-moving kernels on 1 GiB buffers")
    ap.add_argument("--gemm-phases", action="store_true",
                    help="also trace the phases of the grouped GEMMs' tiles (moe_diag_gemm_trace), with and without the epilogue's stores")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="also measure what the matrix cores sustain from registers, on all-zero and on N(0,1)-like operands")
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
                            fp8_dispatch=False if (args.unfused or args.bf16_dispatch or args.padding_free) else None,
                            gated=args.gated, padding_free=args.padding_free,
                            recv_gate=harness.recv_gates(world) if args.gated else None,
                            recv_flat=harness.recv_flat(world) if args.padding_free else None)
    # the returned buffer: slot 0 is rank 0's own return slot; the other slots stand in for what the
    # other ranks' experts would send back (same shape and dtype, arbitrary finite contents)
    pipe.step()
    torch.cuda.synchronize()
    g = torch.Generator(device="cpu").manual_seed(cfg.seed + 4242)
    pipe.returned.copy_(torch.randn(pipe.returned.shape, generator=g, dtype=torch.float32).to(cfg.torch_dtype))
    if not args.padding_free:
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
        bound = wk["bound"]
        if bound == "hbm" and wk.get("flops", 0) / (PEAK["fp32"] * 1e12) > wk["amount"] / (PEAK["hbm"] * 1e9):
            # more fp32 matrix work than memory traffic (the router logits of a workload with many experts): the fp32 rate binds
            bound = "fp32"
            ach, peak, unit = wk["flops"] / (ms * 1e-3) / 1e12, PEAK["fp32"], "TFLOP/s"
        elif bound == "hbm":
            ach, peak, unit = wk["amount"] / (ms * 1e-3) / 1e9, PEAK["hbm"], "GB/s"
        else:
            ach = wk["amount"] / (ms * 1e-3) / 1e12
            peak = PEAK["mfma_fp8"] if cfg.quant == "fp8" else (PEAK["fp32"] if cfg.dtype == "f32" else PEAK["mfma_bf16"])
            unit = "TFLOP/s"
        stages[n] = {"ms": round(ms, 4), "ms_min": round(stage_spread[n][0], 4), "ms_median": round(stage_spread[n][1], 4),
                     "bound": bound, "achieved": round(ach, 2), "peak": peak, "unit": unit, "frac": round(ach / peak, 4)}
    dom = "mlp_up"  # the gate/up grouped GEMM: most of the flops of a step
    traffic, traffic_source = profiled_traffic(cfg.name, dom + "_fp8_dispatch" if pipe.fp8_dispatch else dom)
    if cfg.quant == "fp8":
        kname = ("moe_grouped_mlp_fp8_q (gate/up GEMM + SwiGLU + block quantisation in its epilogue, down GEMM on block-scaled "
                 "MFMAs; the tokens arrive quantised)" if pipe.fp8_dispatch else
                 "moe_grouped_mlp_fp8 (row quantisation + gate/up GEMM + SwiGLU + block quantisation in its epilogue, down GEMM "
                 "on block-scaled MFMAs)")
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
        "destination_side": ("gather/scatter inside the GEMMs over the padding-free payload" if pipe.padding_free else
                             "gather/scatter inside the GEMMs, result rows weighted by their gates, combine by plain sum" if pipe.gated
                             else "gather/scatter inside the GEMMs" if pipe.fused else "unpack + MLP + return pack"),
        "dispatch": "fp8 codes + row scales (quantised while packing)" if pipe.fp8_dispatch else cfg.dtype,
        "ms_per_step_stream": round(stream_ms_per_step, 4),
        "ms_per_step_graph": None if ms_graph is None else round(ms_graph, 4),
        "roofline": roofline,
        "stages": stages,
    }

    if args.backward:
        if cfg.quant == "fp8":
            out["backward"] = {"skipped": "the fp8 expert has no backward pass"}
        else:
            out["backward"] = backward_leg(cfg, world, raw, max(args.steps // 4, 2))
    if args.stream_ceiling:
        out["stream_ceiling"] = stream_ceiling_leg(cfg, max(args.steps // 2, 3), world)
    if args.mfma_ceiling:
        out["mfma_ceiling"] = mfma_ceiling_leg(max(args.steps // 4, 3))
    if args.gemm_phases:
        if cfg.dtype == "f32":
            out["gemm_phases"] = {"skipped": "the fp32 expert runs the plain LDS-tiled kernel"}
        else:
            out["gemm_phases"] = gemm_phases_leg(cfg, pipe, max(args.steps // 2, 3))

    if not args.no_cpu_baseline:
        def to_np(t):
            t = t.detach().cpu()
            return t.float().numpy() if t.dtype == torch.bfloat16 else t.numpy()

        router_np = to_np(world.router)
        bias_np = None if world.bias is None else to_np(world.bias)
        if qs is not None:
            w_np = tuple(to_np(t) for pair in qs for t in pair)
        else:
            w_np = tuple(to_np(t) for t in raw)
        flops_per_token = 2 * cfg.hidden * cfg.ffn * cfg.n_mat * cfg.topk
        sample = args.cpu_sample_tokens or max(64, min(cfg.tokens, int(1.2e13 / flops_per_token)))
        v, secs, threads, desc = cpu_baseline(cfg, router_np, bias_np, w_np, sample)
        out["cpu_baseline"] = {"value": round(v, 1), "unit": "tokens/s", "cores": threads, "kind": "port",
                               "sample": desc, "seconds": round(secs, 2), "host_cpus": os.cpu_count(),
                               "per_element_loop_plumbing": per_element_loop_baseline()}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
