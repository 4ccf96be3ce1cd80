"""Single-GPU stand-in for the reference's ``custom_a2a`` (layers/all_to_all.py:10-125).

The reference's operator moves rows between GPUs with Iris puts (kernels.py:21-146).  The
inter-GPU transfer is not part of a one-GPU build; what is kept is the operator's contract: the
10-argument signature, the in-place fill of ``local_pca`` / ``token_buf`` / the two completion
counters, and the returned ``token_buf``.  The sends of the other simulated ranks are supplied
through a ``SimulatedWorld``; placing the rows ([E_local, world, CAP, H], zero padded) is done by
the HIP reorder kernel.
"""
from __future__ import annotations

import contextlib
from typing import Dict, Optional, Tuple

import torch

from .. import ops
from ..utils import _assert_cuda_int32


class SimulatedWorld:
    """What every simulated source rank would send: (payload, dest_counts [W,E_l], dst_offsets [W])."""

    def __init__(self, world_size: int, rank: int = 0):
        self.world_size = int(world_size)
        self.rank = int(rank)
        self.sends: Dict[int, Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = {}

    def post(self, src: int, tokens: torch.Tensor, dest_counts: torch.Tensor, dst_offsets: torch.Tensor) -> None:
        assert 0 <= src < self.world_size
        self.sends[int(src)] = (tokens, dest_counts, dst_offsets)


_current: Optional[SimulatedWorld] = None


@contextlib.contextmanager
def simulated_world(world: SimulatedWorld):
    global _current
    prev, _current = _current, world
    try:
        yield world
    finally:
        _current = prev


class AllToAllOp(torch.autograd.Function):

    @staticmethod
    def forward(ctx, tokens, dest_counts, dst_offsets, local_pca, token_buf, counts_ready, token_sync, heap_bases,
                experts, capacity):
        """Same arguments as the reference (layers/all_to_all.py:13-46).  ``heap_bases`` is ignored."""
        _assert_cuda_int32(dest_counts, "dest_counts")
        _assert_cuda_int32(dst_offsets, "dst_offsets")
        _assert_cuda_int32(local_pca, "local_pca")
        world_size = local_pca.shape[1]
        world = _current if _current is not None else SimulatedWorld(world_size, 0)
        assert world.world_size == world_size, "simulated world size does not match local_pca"
        # the reference's assert is inverted (all_to_all.py:80); the intent is divisibility
        assert experts % world_size == 0, "EP-group size unevenly calculated."
        e_local = experts // world_size
        rank = world.rank
        world.post(rank, tokens, dest_counts, dst_offsets)

        # what each source sends to `rank`: rows [dst_offsets[rank], +sum(dest_counts[rank,:]))
        parts, counts = [], torch.zeros((world_size, e_local), dtype=torch.int32, device=tokens.device)
        for src in range(world_size):
            if src not in world.sends:
                continue
            p, dc, do = world.sends[src]
            n = int(dc[rank].sum().item())
            o = int(do[rank].item())
            parts.append(p[o:o + n])
            counts[src] = dc[rank]
        flat = torch.cat(parts, dim=0) if parts else tokens[:0]
        over = int(counts.max().item()) if counts.numel() else 0
        if over > capacity:
            raise ValueError(f"capacity overflow: a (src, expert) pair sends {over} rows > CAP={capacity}")
        if tuple(token_buf.shape) != (e_local, world_size, capacity, tokens.shape[-1]):
            raise ValueError(f"token_buf shape {tuple(token_buf.shape)} mismatch expected "
                             f"({e_local},{world_size},{capacity},{tokens.shape[-1]}).")
        ops.reorder_flat(flat.contiguous(), counts, capacity, token_buf)
        local_pca.copy_(counts.t())
        # completion counters in their final state: every source has signalled (all_to_all.py:59-69)
        counts_ready.fill_(world_size)
        token_sync.fill_(world_size)
        return token_buf

    @staticmethod
    def backward(ctx, *grad_outputs):
        raise NotImplementedError("Backward pass not implemented yet.")


custom_a2a = AllToAllOp.apply
