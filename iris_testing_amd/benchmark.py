"""Dispatch benchmark / sweep driver with the reference's environment-variable interface.

    WORLD_SIZE=8 BATCH=4 SEQ=2048 HIDDEN=4096 TOPK=2 E_LOCAL=4 python -m iris_testing_amd.benchmark
    SWEEP=topk python -m iris_testing_amd.benchmark          # batch | seq | e_local | topk | all

Same knobs and defaults as the reference's benchmark entry (benchmark.py:17-22, 446-453): WORLD_SIZE,
BATCH, SEQ, HIDDEN, TOPK, E_LOCAL, CAPACITY, SEED, WARMUP, ITERS, CHECK, CLEAR_TOKEN_BUF,
SKIP_ON_OVERFLOW; SWEEP walks one of the four axes of the reference's figures (batch, seq, experts per
rank, top-k) and prints one table row per point.

What is timed differs from the reference by construction: the reference times the inter-GPU exchange on
8 GPUs; this build has one GPU and no transfer, so it times rank 0's share of the work on either side of
the exchange -- route + count + pack into the fixed [W,M,H] layout as a source, and the receive buffer
-> token_buf [E_l,W,CAP,H] -> expert-major rows as a destination -- with the receive buffer assembled
(untimed) from all W seeded shards.  CHECK=1 prints a correctness report in the reference's form
(benchmark.py:431-440): the token_buf filled from the fixed-M receive buffer against the token_buf filled
from the padding-free flat payload by ``reorder_flat_to_token_buf``, two independent device routes to the
same layout, compared over the valid region only (benchmark.py:52-79).

A sweep ends with a table in the layout of the reference's figures (figures/all2all_{batch,seq,expert,topk}_change.png:
per axis value the time of ten iterations in seconds for the custom kernels and for the library baseline, and the
speedup printed above the bars).  The figures compare the custom exchange with torch's all_to_all_single; with no
exchange on one GPU, the pair compared here is the data movement on both sides of it -- the pack into [W,M,H] and the
expert-major unpack -- by this library's kernels and by PyTorch's own indexing operators on the same device
(``torch_dispatch_baseline``, the stand-in for the reference's run_baseline_ref, baseline.py:227-305).
"""
from __future__ import annotations

import os
import sys

import torch

from . import harness, ops
from .baseline import reorder_flat_to_token_buf
from .configs import MoEConfig

WARMUP = int(os.getenv("WARMUP", "5"))
ITERS = int(os.getenv("ITERS", "20"))
CHECK = int(os.getenv("CHECK", "1"))
CLEAR_TOKEN_BUF = int(os.getenv("CLEAR_TOKEN_BUF", "0"))
SKIP_ON_OVERFLOW = int(os.getenv("SKIP_ON_OVERFLOW", "1"))

SWEEPS = {
    "batch": ("BATCH", [1, 2, 4, 8, 16]),
    "seq": ("SEQ", [512, 1024, 2048, 4096, 8192]),
    "e_local": ("E_LOCAL", [1, 2, 4, 8, 16]),
    "topk": ("TOPK", [1, 2, 4, 8]),
}


def _env(name: str, default: int, override=None) -> int:
    if override and name in override:
        return int(override[name])
    return int(os.getenv(name, str(default)))


def _timed(fn, warmup: int, iters: int) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def _masked_stats(a: torch.Tensor, b: torch.Tensor, pca: torch.Tensor):
    """max|a-b| and the two sums over the valid rows only (j < pca[e,src]); cf. reference benchmark.py:52-79."""
    E_l, W, CAP, _ = a.shape
    valid = torch.arange(CAP, device=a.device)[None, None, :] < pca[:, :, None]
    af, bf = a.float() * valid[..., None], b.float() * valid[..., None]
    return (af - bf).abs().max(), af.sum(), bf.sum()


def torch_dispatch_baseline(x, row_token, dst_sizes, dst_offsets, M, recv, recv_counts, S):
    """The same two row movements with PyTorch's indexing operators (the library baseline of the sweep tables):
    returns (pack, unpack) closures producing send [W,M,H] and the expert-major rows [S,H]."""
    dev = x.device
    W = dst_sizes.numel()
    H = x.shape[1]
    E_l = recv_counts.shape[1]
    # index tables built once, untimed (the reference's baseline also prepares its split sizes outside the loop)
    m = torch.arange(M, device=dev)[None, :]
    valid = m < dst_sizes[:, None].long()
    src = torch.where(valid, row_token.long()[(dst_offsets[:, None].long() + m).clamp(max=max(row_token.numel() - 1, 0))],
                      torch.zeros((), dtype=torch.long, device=dev))
    rc = recv_counts.long()
    src_off = torch.cumsum(rc, 1) - rc                       # [W,E_l] row inside slot s where expert e starts
    rows_idx = []
    for e in range(E_l):
        for s in range(W):
            c = int(rc[s, e].item())
            if c:
                rows_idx.append(s * M + int(src_off[s, e].item()) + torch.arange(c, device=dev))
    rows_idx = torch.cat(rows_idx) if rows_idx else torch.zeros((0,), dtype=torch.long, device=dev)
    flat_src, flat_valid = src.reshape(-1), valid.reshape(-1, 1)

    def pack():
        return (x.index_select(0, flat_src) * flat_valid).view(W, M, H)

    def unpack():
        return recv.view(W * M, H).index_select(0, rows_idx)

    return pack, unpack


def run_point(override=None, report=True, keep=False):
    world_size = _env("WORLD_SIZE", 8, override)
    batch, seq = _env("BATCH", 4, override), _env("SEQ", 2048, override)
    hidden, topk = _env("HIDDEN", 4096, override), _env("TOPK", 2, override)
    e_local, seed = _env("E_LOCAL", 4, override), _env("SEED", 42, override)
    capacity = _env("CAPACITY", 1024, override)
    dev = "cuda"
    cfg = MoEConfig("env", seed, batch * seq, hidden, "bf16", world_size * e_local, topk, world_size, 0, "silu")
    world = harness.build_world(cfg, dev)
    r0 = world.routes[0]
    M, S, E_l, W, H = world.M, world.S, cfg.e_local, cfg.world, cfg.hidden
    skipped = world.CAP > capacity
    if skipped and SKIP_ON_OVERFLOW and report:
        print(f"[SKIP] max_recv_count={world.CAP} > CAPACITY={capacity}. Timing with CAPACITY={world.CAP} instead.")
    cap = max(capacity, world.CAP)

    send = torch.empty((W, M, H), dtype=cfg.torch_dtype, device=dev)
    token_buf = torch.zeros((E_l, W, cap, H), dtype=cfg.torch_dtype, device=dev)
    pca = torch.zeros((E_l, W), dtype=torch.int32, device=dev)
    rows = torch.empty((S, H), dtype=cfg.torch_dtype, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)

    def source_side():
        idx, _, _ = ops.route_topk(world.x0, world.router, topk, world.bias)
        c = ops.count_and_offsets(idx, cfg.experts, W)
        ops.pack_tokens(world.x0, idx, c.pos, c.dst_sizes, c.dst_offsets, E_l, M, out=send, status=status)

    def destination_side():
        if CLEAR_TOKEN_BUF:
            token_buf.zero_()
        ops.unpack_token_buf(world.recv, world.recv_counts, cap, token_buf=token_buf, pca=pca, status=status)
        ops.shuffle_rows(token_buf, pca, S, out=rows)

    def destination_direct():
        ops.unpack_expert_major(world.recv, world.recv_counts, S, out=rows)

    c0 = r0.counts

    def move_custom():
        ops.pack_tokens(world.x0, r0.idx, c0.pos, c0.dst_sizes, c0.dst_offsets, E_l, M, out=send, status=status)
        ops.unpack_expert_major(world.recv, world.recv_counts, S, out=rows)

    t_pack, t_unpack = torch_dispatch_baseline(world.x0, c0.row_token, c0.dst_sizes, c0.dst_offsets, M, world.recv,
                                               world.recv_counts, S)

    def move_torch():
        t_pack()
        t_unpack()

    src_ms = _timed(source_side, WARMUP, ITERS)
    dst_ms = _timed(destination_side, WARMUP, ITERS)
    direct_ms = _timed(destination_direct, WARMUP, ITERS)
    move_ms = _timed(move_custom, WARMUP, ITERS)
    move_torch_ms = _timed(move_torch, WARMUP, ITERS)
    same = torch.equal(t_pack(), send) and torch.equal(t_unpack(), rows)
    B = 2
    src_gbs = (cfg.tokens * H * B + W * M * H * B) / src_ms / 1e6
    direct_gbs = 2 * S * H * B / direct_ms / 1e6
    res = dict(world=W, e_local=E_l, cap=cap, hidden=H, batch=batch, seq=seq, topk=topk, M=M, S=S,
               source_ms=src_ms, dest_ms=dst_ms, dest_direct_ms=direct_ms, source_gbs=src_gbs, direct_gbs=direct_gbs,
               move_ms=move_ms, move_torch_ms=move_torch_ms, baseline_agrees=same)
    if report:
        print("=== Dispatch Perf (one GPU = rank 0's share on either side of the exchange; no transfer) ===")
        print(f"world={W} E_local={E_l} CAP={cap} H={H} batch={batch} seq={seq} topk={topk}  (M={M}, rows received={S})")
        print(f"source_ms      route+count+pack [W,M,H]:            {src_ms:.3f}   ({src_gbs:.0f} GB/s of pack bytes)")
        print(f"dest_ms        recv -> token_buf -> expert-major:   {dst_ms:.3f}")
        print(f"dest_direct_ms recv -> expert-major (one copy):     {direct_ms:.3f}   ({direct_gbs:.0f} GB/s)")
        print(f"speedup (token_buf route / direct):                 {dst_ms / direct_ms:.3f}x")

    if CHECK and report:
        # the padding-free flat payload rank 0 would receive: source-major, expert-minor blocks
        flat_parts = []
        for s in range(W):
            rs = world.routes[s]
            x = world.x0 if s == 0 else harness.gen_shard_tokens(cfg, s).to(dev)
            payload = ops.pack_payload(x, rs.counts.row_token)
            o, n = int(rs.counts.dst_offsets[0].item()), int(rs.counts.dst_sizes[0].item())
            flat_parts.append(payload[o:o + n])
        flat = torch.cat(flat_parts).contiguous()
        base = torch.zeros_like(token_buf)
        reorder_flat_to_token_buf(flat, world.recv_counts, cap, base)
        token_buf.zero_()
        ops.unpack_token_buf(world.recv, world.recv_counts, cap, token_buf=token_buf, pca=pca, status=status)
        torch.cuda.synchronize()
        expected_pca = world.recv_counts.t().contiguous()
        pca_diff = (pca - expected_pca).abs().max().item()
        max_diff, sum_a, sum_b = _masked_stats(token_buf, base, expected_pca)
        print("=== Correctness Report ===")
        print(f"PCA max|diff|: {pca_diff:.6g}")
        print(f"TOKEN_BUF max|diff| valid: {max_diff.item():.6g}")
        print(f"TOKEN_BUF sum(valid) fixed-M route:      {sum_a.item():.6g}")
        print(f"TOKEN_BUF sum(valid) padding-free route: {sum_b.item():.6g}")
        ok = pca_diff == 0 and max_diff.item() == 0.0 and abs(sum_a.item() - sum_b.item()) < 1e-3 and \
            torch.equal(token_buf, base) and int(status.item()) == 0
        ok = ok and same  # and the library baseline moved the same bytes
        print("PASS" if ok else "FAIL")
        res["ok"] = ok
        if keep:
            res.update(token_buf=token_buf, pca=pca, recv=world.recv, recv_counts=world.recv_counts, world_obj=world)
    return res


AXIS_FIGURE = {"batch": "all2all_batch_change", "seq": "all2all_seq_change", "e_local": "all2all_expert_change",
               "topk": "all2all_topk_change"}


def run_sweep(sweep: str, values=None):
    """One axis of the reference's figures; returns the rows and prints the detailed table and the figure-style one."""
    var, default_values = SWEEPS[sweep]
    values = list(values or default_values)
    print(f"sweep over {var}: {values}  (other knobs from the environment / reference defaults)")
    print(f"{var:>8s} {'tokens':>8s} {'M':>7s} {'rows_in':>8s} {'source_ms':>10s} {'pack GB/s':>10s} {'dest_ms':>9s} "
          f"{'direct_ms':>10s} {'copy GB/s':>10s}")
    rows = []
    for v in values:
        r = run_point({var: v}, report=False)
        rows.append((v, r))
        print(f"{v:8d} {r['batch'] * r['seq']:8d} {r['M']:7d} {r['S']:8d} {r['source_ms']:10.3f} {r['source_gbs']:10.0f} "
              f"{r['dest_ms']:9.3f} {r['dest_direct_ms']:10.3f} {r['direct_gbs']:10.0f}", flush=True)
    # the reference's figure for this axis, as text: seconds per ten iterations, custom against library, speedup
    print(f"=== {AXIS_FIGURE[sweep]} (pack + expert-major unpack, seconds per 10 iterations) ===")
    print(f"{var:>8s} {'custom_s':>12s} {'torch_s':>12s} {'speedup':>9s} {'same_bytes':>11s}")
    for v, r in rows:
        print(f"{v:8d} {r['move_ms'] * 1e-2:12.6f} {r['move_torch_ms'] * 1e-2:12.6f} {r['move_torch_ms'] / r['move_ms']:8.2f}x "
              f"{'yes' if r['baseline_agrees'] else 'NO':>11s}", flush=True)
    return rows


def main() -> int:
    if not torch.cuda.is_available():
        print("iris_testing_amd.benchmark: no GPU visible", file=sys.stderr)
        return 1
    sweep = os.getenv("SWEEP", "").lower()
    if not sweep:
        res = run_point()
        return 0 if res.get("ok", True) else 1
    if sweep != "all" and sweep not in SWEEPS:
        print(f"SWEEP must be one of {sorted(SWEEPS)} or all", file=sys.stderr)
        return 2
    ok = True
    for axis in (SWEEPS if sweep == "all" else [sweep]):
        ok = all(r["baseline_agrees"] for _, r in run_sweep(axis)) and ok
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main())
