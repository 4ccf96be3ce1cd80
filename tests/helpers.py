"""Shared helpers for the tests: tensor <-> numpy conversion and oracle-side world assembly."""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import moe_oracle as O  # noqa: E402


def to_np(t: torch.Tensor) -> np.ndarray:
    """Any tensor -> numpy (bf16 widened exactly to fp32)."""
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
        return t.float().numpy()
    return t.numpy()


def bits(a) -> np.ndarray:
    """Bit pattern view for exact comparisons (works for fp32 arrays and tensors)."""
    if isinstance(a, torch.Tensor):
        a = to_np(a)
    a = np.ascontiguousarray(a)
    if a.dtype == np.float32:
        return a.view(np.uint32)
    return a


def assert_bits_equal(got, want, what=""):
    g, w = bits(got), bits(want)
    assert g.shape == w.shape, f"{what}: shape {g.shape} != {w.shape}"
    if not np.array_equal(g, w):
        bad = np.argwhere(g != w)
        raise AssertionError(f"{what}: {len(bad)} of {g.size} elements differ; first at {bad[0].tolist()}: "
                             f"got {np.asarray(got if not isinstance(got, torch.Tensor) else to_np(got))[tuple(bad[0])]} "
                             f"want {np.asarray(want)[tuple(bad[0])]}")


def err_stats(got: np.ndarray, want: np.ndarray):
    """(max abs error, max abs error / rms(want), max elementwise relative error where |want| > rms/8)."""
    got = got.astype(np.float64)
    want = want.astype(np.float64)
    d = np.abs(got - want)
    rms = float(np.sqrt(np.mean(want ** 2))) if want.size else 0.0
    big = np.abs(want) > rms / 8 if rms > 0 else np.zeros_like(want, bool)
    rel = float(np.max(d[big] / np.abs(want[big]))) if big.any() else 0.0
    return float(d.max()) if d.size else 0.0, (float(d.max()) / rms if rms > 0 else 0.0), rel


def oracle_world(cfg, xs, router, bias):
    """Oracle view of all W shards: per-shard (idx, gate, counts, sizes, offsets, pos, row_token), M, CAP."""
    shards = []
    for x in xs:
        idx, gate, logits = O.route(x, router, cfg.topk, bias)
        counts = O.send_counts(idx, cfg.world, cfg.experts)
        sizes, offs = O.dst_sizes_offsets(counts)
        pos, row_token = O.payload_positions(idx, cfg.experts)
        shards.append(dict(idx=idx, gate=gate, logits=logits, counts=counts, sizes=sizes, offs=offs, pos=pos,
                           row_token=row_token))
    M = O.pair_capacity(np.stack([s["sizes"] for s in shards]))
    CAP = max(O.compute_capacity_from_pca(s["counts"]) for s in shards)
    return shards, M, CAP


def oracle_recv(cfg, xs, shards, M, dst):
    """What rank ``dst`` receives: recv [W,M,H], recv_counts [W,E_l]."""
    recv = np.stack([O.pack_fixed_m(O.send_payload(x, s["row_token"]), s["offs"], s["sizes"], M)[dst]
                     for x, s in zip(xs, shards)])
    rc = np.stack([s["counts"][dst] for s in shards]).astype(np.int32)
    return recv, rc
