"""Host-side mirror of the layout helper of the reference's ``baseline.py``.

Only ``reorder_flat_to_token_buf`` (reference baseline.py:178-222) is on the dispatch path; the
torch.distributed all-to-all around it is a collective and is not part of a one-GPU build.
"""
from __future__ import annotations

import torch

from . import ops


def _assert_cuda(x: torch.Tensor, name: str) -> None:  # reference baseline.py:10-12
    if not x.is_cuda:
        raise ValueError(f"{name} must be a CUDA tensor")


def _assert_int32(x: torch.Tensor, name: str) -> None:  # reference baseline.py:14-16
    if x.dtype != torch.int32:
        raise ValueError(f"{name} must be int32")


def reorder_flat_to_token_buf(recv_payload_flat: torch.Tensor, recv_counts: torch.Tensor, capacity: int,
                              token_buf_out: torch.Tensor) -> torch.Tensor:
    """token_buf_out[e, src, :c] = the next c rows of the flat payload (src-major, expert-minor
    blocks), zero padding; same checks and exceptions as the reference (baseline.py:199-201,
    215-216, 220-221).  One kernel instead of a Python double loop."""
    _assert_cuda(recv_payload_flat, "recv_payload_flat")
    _assert_cuda(recv_counts, "recv_counts")
    _assert_int32(recv_counts, "recv_counts")
    world_size, e_local = recv_counts.shape
    hidden_dim = recv_payload_flat.shape[1]
    if tuple(token_buf_out.shape) != (e_local, world_size, capacity, hidden_dim):
        raise ValueError(f"token_buf_out shape {tuple(token_buf_out.shape)} mismatch expected "
                         f"({e_local},{world_size},{capacity},{hidden_dim}).")
    counts_host = recv_counts.cpu()
    over = (counts_host > capacity).nonzero()
    if over.numel():
        src, e = over[0].tolist()
        raise ValueError(f"[reorder] recv_count src={src},e={e} is {int(counts_host[src, e])} > capacity={capacity}")
    total = int(counts_host.sum())
    if total != recv_payload_flat.shape[0]:
        raise RuntimeError(f"[reorder] consumed rows={total} != total_recv={recv_payload_flat.shape[0]}")
    ops.reorder_flat(recv_payload_flat.contiguous(), recv_counts.contiguous(), capacity, token_buf_out)
    return token_buf_out
