"""Expert compute with the reference's ``expert`` signature (layers/expert.py:6-66), plus the full
expert MLP the workloads define (Linear-act-Linear, SwiGLU, fp8) which the reference lacks.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .. import ops
from ..utils import _assert_cuda_int32


# Re-tiled copies of weight tensors the operator has seen, keyed on the tensor's storage and version counter, so that
# a weight that did not change between calls is re-tiled once, not on every forward (the re-tiling reads and writes the
# whole tensor).  Entries die with their tensors (weak references); an in-place update bumps the version and re-tiles.
_PACKED = {}
_PART_WS = {}


def _packed_weights(w: torch.Tensor) -> torch.Tensor:
    import weakref
    key = (w.data_ptr(), w._version, tuple(w.shape), w.dtype, w.device)
    hit = _PACKED.get(key)
    if hit is not None and hit[0]() is w:
        return hit[1]
    for k in [k for k, v in _PACKED.items() if v[0]() is None or (v[0]() is w and k != key)]:
        del _PACKED[k]
    packed = ops.prepack_weights(w)
    _PACKED[key] = (weakref.ref(w), packed)
    return packed


def _part_ws(device) -> torch.Tensor:
    """One partial-sum workspace per device for the K split of an under-filled last round of GEMM tiles."""
    ws = _PART_WS.get(device)
    if ws is None:
        ws = _PART_WS[device] = ops.gemm_part_workspace(device)
    return ws


def _grouped_gemm(tokens: torch.Tensor, weights: torch.Tensor, cnt: torch.Tensor) -> torch.Tensor:
    """out[rows of g] = tokens[rows of g] @ weights[g]; rows past sum(cnt) are zero."""
    if tokens.dtype != torch.bfloat16 or weights.shape[1] % 64 or weights.shape[2] % 8:
        return ops.grouped_gemm(tokens, weights, cnt)
    S, N = tokens.shape[0], weights.shape[2]
    out = torch.zeros((S, N), dtype=tokens.dtype, device=tokens.device)
    if S:
        ops.grouped_gemm_mapped(tokens, None, _packed_weights(weights), cnt, S, N, "none", out,
                                part_ws=_part_ws(tokens.device))
    return out


class Expert(torch.autograd.Function):

    @staticmethod
    def forward(ctx, tokens, weights, local_expert_cnt, aggregrate_exp_cnt):
        """tokens [S,H], weights [E_local,H,F], local_expert_cnt [E_local] int32, total expert count
        (unused by the math, kept for the signature) -> [S,F] (layers/expert.py:20-29,43,60)."""
        assert tokens.is_cuda, "tokens must be CUDA"
        _assert_cuda_int32(local_expert_cnt, "local_expert_cnt")
        assert weights.shape[0] == local_expert_cnt.numel(), "one row count per local expert"
        ctx.save_for_backward(tokens, weights, local_expert_cnt)
        return _grouped_gemm(tokens.contiguous(), weights.contiguous(), local_expert_cnt.contiguous())

    @staticmethod
    def backward(ctx, do):
        """Gradients of out[rows of g] = tokens[rows of g] @ weights[g] (not implemented in the reference,
        layers/expert.py:62-64), both on the grouped GEMM kernel:
          d tokens[rows of g] = do[rows of g] @ weights[g]^T        one grouped launch over the transposed weights
          d weights[g]        = tokens[rows of g]^T @ do[rows of g]  one launch per expert: the reduction runs over
                                                                      the expert's rows, zero padded to 64
        Rows past the counted total get a zero gradient."""
        tokens, weights, cnt = ctx.saved_tensors
        do = do.contiguous()
        E_l, H, F = weights.shape
        d_tokens = ops.grouped_gemm(do, weights.transpose(1, 2).contiguous(), cnt.contiguous())
        counts = [max(int(c), 0) for c in cnt.cpu().tolist()]
        total = min(sum(counts), tokens.shape[0])
        if total < tokens.shape[0]:
            d_tokens[total:].zero_()
        d_weights = torch.zeros_like(weights)
        h_rows = torch.full((1,), H, dtype=torch.int32, device=tokens.device)
        row0 = 0
        for g, c in enumerate(counts):
            c = min(c, tokens.shape[0] - row0)
            if c > 0:
                pad = (c + 63) // 64 * 64
                xt = torch.zeros((H, pad), dtype=tokens.dtype, device=tokens.device)
                xt[:, :c] = tokens[row0:row0 + c].t()
                dy = torch.zeros((1, pad, F), dtype=do.dtype, device=do.device)
                dy[0, :c] = do[row0:row0 + c]
                d_weights[g] = ops.grouped_gemm(xt, dy, h_rows)
            row0 += c
        return d_tokens, d_weights, None, None


expert = Expert.apply


@dataclass
class ExpertWeights:
    """Weights of the local experts, prepared once for the kernels.

    act in {"gelu","silu"}: y = act(x W1) W2.  act == "swiglu": y = (silu(x Wg) * (x Wu)) Wd.
    bf16: re-tiled for the MFMA kernels; fp32: reference layout; fp8: e4m3 codes + per-channel scales.
    """
    act: str
    hidden: int
    ffn: int
    e_local: int
    dtype: torch.dtype
    w1: torch.Tensor
    w2: torch.Tensor
    w_up: Optional[torch.Tensor] = None
    scales: Optional[tuple] = None  # fp8: (sg, su, sd)

    @classmethod
    def prepare(cls, act: str, w1: torch.Tensor, w2: torch.Tensor, w_up: Optional[torch.Tensor] = None):
        e_l, H, F = w1.shape
        if w1.dtype == torch.float32:
            return cls(act, H, F, e_l, w1.dtype, w1.contiguous(), w2.contiguous(),
                       None if w_up is None else w_up.contiguous())
        p1 = ops.prepack_weights(w1.contiguous(), None if w_up is None else w_up.contiguous())
        p2 = ops.prepack_weights(w2.contiguous())
        return cls(act, H, F, e_l, w1.dtype, p1, p2)

    @classmethod
    def prepare_fp8(cls, wg_q, sg, wu_q, su, wd_q, sd):
        """e4m3 codes (uint8) [E_l,H,F] x2 and [E_l,F,H] with fp32 per-output-channel scales."""
        e_l, H, F = wg_q.shape
        p1 = ops.prepack_weights_fp8(wg_q.contiguous(), wu_q.contiguous())
        p2 = ops.prepack_weights_fp8(wd_q.contiguous())
        return cls("swiglu", H, F, e_l, torch.uint8, p1, p2, None, (sg.contiguous(), su.contiguous(), sd.contiguous()))


def expert_mlp(tokens: torch.Tensor, weights: ExpertWeights, local_expert_cnt: torch.Tensor) -> torch.Tensor:
    """Full expert MLP on expert-major rows -> [S,H]."""
    assert tokens.is_cuda, "tokens must be CUDA"
    _assert_cuda_int32(local_expert_cnt, "local_expert_cnt")
    if weights.dtype == torch.uint8:
        sg, su, sd = weights.scales
        return ops.grouped_mlp_fp8(tokens.contiguous(), local_expert_cnt, weights.ffn, weights.w1, sg, su, weights.w2, sd)
    return ops.grouped_mlp(tokens.contiguous(), local_expert_cnt, weights.act, weights.w1, weights.w2, weights.w_up,
                           F=weights.ffn)
