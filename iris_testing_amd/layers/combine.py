"""Top-k-weighted combine back to token order, and the fixed-M pack as a differentiable operator (no counterpart in the
reference, which has no return path, drops the gate values at utils.py:202 and leaves every backward empty)."""
from __future__ import annotations

import torch

from .. import ops


def _dst_sizes(dst_offsets: torch.Tensor, routed_rows: int) -> torch.Tensor:
    """Rows per destination from their exclusive prefix (the last one runs to the routed total)."""
    end = torch.full((1,), routed_rows, dtype=dst_offsets.dtype, device=dst_offsets.device)
    return torch.diff(dst_offsets, append=end).contiguous()


class Combine(torch.autograd.Function):

    @staticmethod
    def forward(ctx, returned, gate, topk_idx, pos, dst_offsets, e_local):
        returned = returned.contiguous()
        ctx.save_for_backward(returned, gate, topk_idx, pos, dst_offsets)
        ctx.e_local = e_local
        return ops.combine(returned, topk_idx, pos, gate.contiguous(), dst_offsets, e_local)

    @staticmethod
    def backward(ctx, d_out):
        """d returned[slot(t,kk)] = gate[t,kk] * d out[t] (zeros in the padding); d gate[t,kk] = <d out[t], returned[slot(t,kk)]>."""
        returned, gate, idx, pos, dst_offsets = ctx.saved_tensors
        sizes = _dst_sizes(dst_offsets, idx.numel())
        d_ret, d_gate = ops.combine_backward(d_out.contiguous(), returned, idx, pos, gate.contiguous(), sizes, dst_offsets, ctx.e_local)
        return d_ret, d_gate, None, None, None, None


def combine(returned: torch.Tensor, topk_idx: torch.Tensor, pos: torch.Tensor, gate: torch.Tensor,
            dst_offsets: torch.Tensor, e_local: int) -> torch.Tensor:
    """out[t] = sum_kk gate[t,kk] * returned[dst, pos[t,kk] - dst_offsets[dst]], dst = idx[t,kk] // E_local.

    ``returned`` [W,M,H] holds the expert outputs in the slots the send buffer used.  Differentiable with respect
    to ``returned`` and ``gate``.
    """
    return Combine.apply(returned, gate, topk_idx, pos, dst_offsets, e_local)


class PackFixedM(torch.autograd.Function):

    @staticmethod
    def forward(ctx, tokens, topk_idx, pos, dst_sizes, dst_offsets, e_local, M):
        ctx.save_for_backward(topk_idx, pos, dst_offsets)
        ctx.e_local = e_local
        return ops.pack_tokens(tokens.contiguous(), topk_idx, pos, dst_sizes, dst_offsets, e_local, M)

    @staticmethod
    def backward(ctx, d_send):
        """Every token row was copied to its k slots: its gradient is the sum of the k slot gradients, i.e. the combine
        with unit gates (fp32 sum in slot order, one rounding)."""
        idx, pos, dst_offsets = ctx.saved_tensors
        ones = torch.ones(idx.shape, dtype=torch.float32, device=idx.device)
        return ops.combine(d_send.contiguous(), idx, pos, ones, dst_offsets, ctx.e_local), None, None, None, None, None, None


def pack_fixed_m(tokens: torch.Tensor, topk_idx: torch.Tensor, pos: torch.Tensor, dst_sizes: torch.Tensor,
                 dst_offsets: torch.Tensor, e_local: int, M: int) -> torch.Tensor:
    """send [W,M,H] (README.md:5-7 layout) from token rows; differentiable with respect to ``tokens``."""
    return PackFixedM.apply(tokens, topk_idx, pos, dst_sizes, dst_offsets, e_local, M)
