"""One GPU acting as rank 0 of a simulated W-rank expert-parallel group.

The inter-GPU transfer is not part of this build: what rank 0 would receive is assembled here
from W seeded source shards, each routed and packed with the same HIP kernels (untimed set-up
work for the benchmark, and the multi-rank scaffolding for the parity tests).  Nothing in this
module computes on the CPU.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import torch

from . import ops
from .configs import MoEConfig, gen_expert_weights, gen_router, gen_router_bias, gen_shard_tokens
from .layers.expert import ExpertWeights


@dataclass
class ShardRoute:
    idx: torch.Tensor    # [T,k] i32
    gate: torch.Tensor   # [T,k] f32
    logits: torch.Tensor  # [T,E] f32
    counts: ops.Counts


@dataclass
class World:
    cfg: MoEConfig
    router: torch.Tensor
    bias: Optional[torch.Tensor]
    x0: torch.Tensor                 # shard 0 tokens (rank 0 as a source)
    routes: List[ShardRoute]         # one per source shard
    M: int                           # pair capacity (max rows between any device pair)
    CAP: int                         # per-(src,dst,expert) capacity
    recv: torch.Tensor               # [W,M,H] what rank 0 receives
    recv_counts: torch.Tensor        # [W,E_l] i32: recv_counts[s,e] rows from source s for local expert e
    S: int                           # rows received by rank 0
    # fp8 workloads: the same receive buffer as the sources send it when they quantise their tokens while packing
    # (ops.pack_tokens_fp8): per-row codes [W,M,H] and scales [W,M]
    recv_q: Optional[torch.Tensor] = None
    recv_scale: Optional[torch.Tensor] = None


def route_shard(cfg: MoEConfig, x: torch.Tensor, router: torch.Tensor, bias: Optional[torch.Tensor]) -> ShardRoute:
    idx, gate, logits = ops.route_topk(x, router, cfg.topk, bias)
    return ShardRoute(idx, gate, logits, ops.count_and_offsets(idx, cfg.experts, cfg.world))


def pack_for_dst(x: torch.Tensor, r: ShardRoute, dst: int, M: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The [M,H] slot a source sends to one destination (the fixed-M pack restricted to that dst)."""
    c = r.counts
    o = ops.pack_fixed_m(x, c.row_token, c.dst_sizes[dst:dst + 1].contiguous(), c.dst_offsets[dst:dst + 1].contiguous(),
                         M, out=None if out is None else out.view(1, M, -1))
    return o.view(M, -1)


def build_world(cfg: MoEConfig, device="cuda", dst_rank: int = 0, keep_shards: bool = False):
    """Route all W shards, derive M / CAP, and assemble rank ``dst_rank``'s receive buffer."""
    router = gen_router(cfg).to(device)
    bias = gen_router_bias(cfg)
    bias = None if bias is None else bias.to(device)
    routes, shards = [], []
    for s in range(cfg.world):
        x = gen_shard_tokens(cfg, s).to(device)
        routes.append(route_shard(cfg, x, router, bias))
        shards.append(x if (keep_shards or s == 0) else None)
    caps = torch.stack([r.counts.caps for r in routes])  # [W,2]
    M = int(ops.max_floor1(caps[:, 0].contiguous()).item())
    CAP = int(ops.max_floor1(caps[:, 1].contiguous()).item())
    recv = torch.empty((cfg.world, M, cfg.hidden), dtype=cfg.torch_dtype, device=device)
    recv_counts = torch.empty((cfg.world, cfg.e_local), dtype=torch.int32, device=device)
    for s in range(cfg.world):
        x = shards[s] if shards[s] is not None else gen_shard_tokens(cfg, s).to(device)
        pack_for_dst(x, routes[s], dst_rank, M, out=recv[s])
        recv_counts[s] = routes[s].counts.send_counts[dst_rank]
    S = int(recv_counts.sum().item())
    w = World(cfg, router, bias, shards[0], routes, M, CAP, recv, recv_counts, S)
    if cfg.quant == "fp8":
        # (per-row quantisation commutes with moving rows: quantising the assembled buffer row by row gives what W
        # quantise-and-pack launches would have sent)
        q, sc = ops.quantize_rows_fp8(recv.view(cfg.world * M, cfg.hidden))
        w.recv_q, w.recv_scale = q.view(cfg.world, M, cfg.hidden), sc.view(cfg.world, M)
    return (w, shards) if keep_shards else w


def expert_weights(cfg: MoEConfig, rank: int, device="cuda"):
    """(ExpertWeights prepared for the kernels, raw CPU tensors) for one rank."""
    raw = gen_expert_weights(cfg, rank)
    if cfg.quant == "fp8":
        wg, wu, wd = raw
        qs = [quantize_weight_fp8(w.to(device)) for w in (wg, wu, wd)]
        ew = ExpertWeights.prepare_fp8(qs[0][0], qs[0][1], qs[1][0], qs[1][1], qs[2][0], qs[2][1])
        return ew, raw, qs
    if cfg.act == "swiglu":
        wg, wu, wd = raw
        return ExpertWeights.prepare("swiglu", wg.to(device), wd.to(device), wu.to(device)), raw, None
    w1, w2 = raw
    return ExpertWeights.prepare(cfg.act, w1.to(device), w2.to(device)), raw, None


def quantize_weight_fp8(w: torch.Tensor):
    """One-time weight preparation (not on the per-step path): per-output-channel e4m3 codes and
    fp32 scales, amax/448, with torch's own float8_e4m3fn cast.  w [E_l,K,N] -> (uint8 [E_l,K,N], f32 [E_l,N])."""
    wf = w.float()
    amax = wf.abs().amax(dim=1)  # [E_l,N]
    zero = amax == 0
    safe = torch.where(zero, torch.ones_like(amax), amax)
    scale = torch.where(zero, torch.ones_like(amax), safe / 448.0)
    inv = torch.where(zero, torch.ones_like(amax), 448.0 / safe)
    q = (wf * inv[:, None, :]).to(torch.float8_e4m3fn).view(torch.uint8)
    return q.contiguous(), scale.contiguous()


def recv_gates(world: World, dst_rank: int = 0) -> torch.Tensor:
    """[W,M] fp32: the gates that arrive with rank ``dst_rank``'s rows when the sources ship them (ops.pack_tokens with
    ``gate``): slot s = what source s wrote beside its rows, zero in the padding."""
    cfg = world.cfg
    out = torch.empty((cfg.world, world.M), dtype=torch.float32, device=world.recv.device)
    send = torch.empty((cfg.world, world.M, cfg.hidden), dtype=cfg.torch_dtype, device=world.recv.device)
    for s, r in enumerate(world.routes):
        x = world.x0 if s == 0 else gen_shard_tokens(cfg, s).to(world.recv.device)
        c = r.counts
        _, g = ops.pack_tokens(x, r.idx, c.pos, c.dst_sizes, c.dst_offsets, cfg.e_local, world.M, out=send, gate=r.gate)
        out[s] = g[dst_rank]
    return out


def recv_flat(world: World, dst_rank: int = 0) -> torch.Tensor:
    """[S,H]: what rank ``dst_rank`` receives when the sources send their padding-free payload (reference utils.py:235-246)
    instead of fixed-M slots: every source's block for this rank, concatenated in source order."""
    cfg = world.cfg
    blocks = []
    for s, r in enumerate(world.routes):
        x = world.x0 if s == 0 else gen_shard_tokens(cfg, s).to(world.recv.device)
        c = r.counts
        o, n = int(c.dst_offsets[dst_rank].item()), int(c.dst_sizes[dst_rank].item())
        blocks.append(ops.pack_payload(x, c.row_token[o:o + n].contiguous()))
    return torch.cat(blocks) if blocks else torch.empty((0, cfg.hidden), dtype=cfg.torch_dtype, device=world.recv.device)
