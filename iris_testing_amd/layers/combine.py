"""Top-k-weighted combine back to token order (no counterpart in the reference, which has no
return path and drops the gate values at utils.py:202)."""
from __future__ import annotations

import torch

from .. import ops


def combine(returned: torch.Tensor, topk_idx: torch.Tensor, pos: torch.Tensor, gate: torch.Tensor,
            dst_offsets: torch.Tensor, e_local: int) -> torch.Tensor:
    """out[t] = sum_kk gate[t,kk] * returned[dst, pos[t,kk] - dst_offsets[dst]], dst = idx[t,kk] // E_local.

    ``returned`` [W,M,H] holds the expert outputs in the slots the send buffer used.
    """
    return ops.combine(returned.contiguous(), topk_idx, pos, gate, dst_offsets, e_local)
