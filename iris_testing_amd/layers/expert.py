"""Expert compute with the reference's ``expert`` signature (layers/expert.py:6-66), plus the full
expert MLP the workloads define (Linear-act-Linear, SwiGLU, fp8) which the reference lacks.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch

from .. import ops
from ..utils import _assert_cuda_int32


# Re-tiled copies of weight tensors the operator has seen, keyed on the tensor's storage and version counter, so that
# a weight that did not change between calls is re-tiled once, not on every call (the re-tiling reads and writes the
# whole tensor).  Entries die with their tensors (weak references); an in-place update bumps the version and re-tiles.
_PACKED = {}
_PART_WS = {}


def _cached_pack(kind: str, w: torch.Tensor, w_up: Optional[torch.Tensor], build) -> torch.Tensor:
    import weakref
    key = (kind, w.data_ptr(), w._version, None if w_up is None else (w_up.data_ptr(), w_up._version), tuple(w.shape), w.dtype,
           w.device)
    hit = _PACKED.get(key)
    if hit is not None and hit[0]() is w:
        return hit[1]
    for k in [k for k, v in _PACKED.items() if v[0]() is None or (v[0]() is w and k[0] == kind)]:
        del _PACKED[k]
    packed = build(w, w_up)
    _PACKED[key] = (weakref.ref(w), packed)
    return packed


def _packed_weights(w: torch.Tensor, w_up: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Re-tiled w (with w_up: the fused gate/up pair) for the forward GEMM."""
    return _cached_pack("N", w, w_up, ops.prepack_weights)


def _packed_weights_t(w: torch.Tensor, w_up: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Re-tiled w^T (with w_up: of the pair, in the fused gate/up column order) for d tokens = d out @ w^T."""
    return _cached_pack("T", w, w_up, ops.prepack_weights_transposed)


def _grouped_gemm_t(do: torch.Tensor, weights: torch.Tensor, cnt: torch.Tensor) -> torch.Tensor:
    """d tokens[rows of g] = do[rows of g] @ weights[g]^T; rows past sum(cnt) are zero."""
    E_l, K, N = weights.shape
    S = do.shape[0]
    if do.dtype == torch.float32:
        return ops.grouped_gemm(do, ops.transpose_weights_f32(weights.contiguous()), cnt)
    out = torch.zeros((S, K), dtype=do.dtype, device=do.device)
    if S:
        ops.grouped_gemm_mapped(do, None, _packed_weights_t(weights), cnt, S, K, "none", out, part_ws=_part_ws(do.device))
    return out


def _part_ws(device) -> torch.Tensor:
    """One partial-sum workspace per device for the K split of an under-filled last round of GEMM tiles."""
    ws = _PART_WS.get(device)
    if ws is None:
        ws = _PART_WS[device] = ops.gemm_part_workspace(device)
    return ws


def _grouped_gemm(tokens: torch.Tensor, weights: torch.Tensor, cnt: torch.Tensor) -> torch.Tensor:
    """out[rows of g] = tokens[rows of g] @ weights[g]; rows past sum(cnt) are zero."""
    if tokens.dtype != torch.bfloat16 or weights.shape[1] % 64 or weights.shape[2] % 8:  # (what the MFMA kernel covers)
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
        layers/expert.py:62-64), both as grouped launches over all experts:
          d tokens[rows of g] = do[rows of g] @ weights[g]^T        the grouped GEMM over the transposed, re-tiled weights
          d weights[g]        = tokens[rows of g]^T @ do[rows of g]  the grouped GEMM in its weight-gradient mode: the
                                                                      reduction runs over the expert's (ragged) rows
        Rows past the counted total get a zero gradient, experts without rows a zero weight gradient."""
        tokens, weights, cnt = ctx.saved_tensors
        do = do.contiguous()
        cnt = cnt.contiguous()
        d_tokens = _grouped_gemm_t(do, weights, cnt)
        d_weights = ops.grouped_gemm_dw(tokens.contiguous(), do, cnt)
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
    # the tensors prepare() was given, in the reference layout: (w1, w2, w_up); the backward pass differentiates with
    # respect to them and re-tiles their transposes on first use
    raw: Optional[tuple] = field(default=None, repr=False)
    # version counters of the raw tensors when w1 / w2 / w_up were last derived from them (refresh() compares)
    raw_versions: Optional[tuple] = field(default=None, repr=False)

    @staticmethod
    def _derive(raw):
        """(w1, w2, w_up) as the kernels take them, from the tensors in the reference layout."""
        w1, w2, w_up = raw
        if w1.dtype == torch.float32:
            return w1.contiguous(), w2.contiguous(), None if w_up is None else w_up.contiguous()
        return (ops.prepack_weights(w1.contiguous(), None if w_up is None else w_up.contiguous()),
                ops.prepack_weights(w2.contiguous()), None)

    @staticmethod
    def _versions(raw):
        return tuple(None if t is None else t._version for t in raw)

    @classmethod
    def prepare(cls, act: str, w1: torch.Tensor, w2: torch.Tensor, w_up: Optional[torch.Tensor] = None):
        e_l, H, F = w1.shape
        raw = (w1, w2, w_up)
        p1, p2, pu = cls._derive(raw)
        return cls(act, H, F, e_l, w1.dtype, p1, p2, pu, raw=raw, raw_versions=cls._versions(raw))

    def refresh(self) -> "ExpertWeights":
        """Derive the kernels' copies again if a tensor prepare() was given has been updated in place since (an optimizer
        step): the forward pass would otherwise multiply with the weights of before the update while the backward pass,
        which re-tiles the transposes by tensor version, uses the new ones."""
        if self.raw is not None and self._versions(self.raw) != self.raw_versions:
            self.w1, self.w2, self.w_up = self._derive(self.raw)
            self.raw_versions = self._versions(self.raw)
        return self

    @classmethod
    def prepare_fp8(cls, wg_q, sg, wu_q, su, wd_q, sd):
        """e4m3 codes (uint8) [E_l,H,F] x2 and [E_l,F,H] with fp32 per-output-channel scales."""
        e_l, H, F = wg_q.shape
        p1 = ops.prepack_weights_fp8(wg_q.contiguous(), wu_q.contiguous())
        p2 = ops.prepack_weights_fp8(wd_q.contiguous())
        return cls("swiglu", H, F, e_l, torch.uint8, p1, p2, None, (sg.contiguous(), su.contiguous(), sd.contiguous()))


class ExpertMLP(torch.autograd.Function):
    """y = act(x W1) W2, or (silu(x Wg) * (x Wu)) Wd, on expert-major rows, with its gradients (the reference defines
    neither the MLP nor a backward).  Inputs that autograd sees: tokens and the weight tensors ``prepare`` was given."""

    @staticmethod
    def forward(ctx, tokens, cnt, ew, w1, w2, w_up):
        tokens = tokens.contiguous()
        S, F = tokens.shape[0], ew.ffn
        hidden = torch.empty((S, F), dtype=tokens.dtype, device=tokens.device)
        a1 = None
        if tokens.dtype == torch.bfloat16 and ew.act != "none" and S:
            # the first GEMM also keeps what it feeds to the activation: the backward pass would otherwise run it again
            ws = _part_ws(tokens.device)
            a1 = torch.empty((S, 2 * F if ew.act == "swiglu" else F), dtype=tokens.dtype, device=tokens.device)
            ops.grouped_gemm_act_keep(tokens, ew.w1, cnt, S, F, ew.act, hidden, a1, part_ws=ws)
            out = torch.zeros((S, ew.hidden), dtype=tokens.dtype, device=tokens.device)  # (rows past the counted total stay zero)
            ops.grouped_gemm_mapped(hidden, None, ew.w2, cnt, S, ew.hidden, "none", out, part_ws=ws)
        else:
            out = ops.grouped_mlp(tokens, cnt, ew.act, ew.w1, ew.w2, ew.w_up, F=F, hidden_ws=hidden)
        ctx.save_for_backward(tokens, hidden, cnt, w1, w2, w_up, a1)
        ctx.ew = ew
        return out

    @staticmethod
    def backward(ctx, dy):
        """With a1 the pre-activations (bf16: kept by the forward's first GEMM; fp32: recomputed):
          d h  = dy @ W2^T          d W2 = h^T @ dy            (per expert, ragged rows as the reduction dimension)
          d a1 = d h * act'(a1)     (SwiGLU: d g = d h * u * silu'(g), d u = d h * silu(g))
          d x  = d a1 @ W1^T        d W1 = x^T @ d a1          (SwiGLU: both halves in one launch each)"""
        tokens, hidden, cnt, w1, w2, w_up, a1 = ctx.saved_tensors
        ew = ctx.ew
        dy = dy.contiguous()
        S, H, F = tokens.shape[0], ew.hidden, ew.ffn
        swiglu = ew.act == "swiglu"
        if tokens.dtype == torch.float32:
            if swiglu:
                raise NotImplementedError("expert_mlp backward: fp32 SwiGLU (the fp32 path serves the GELU / SiLU plumbing workload)")
            dh = ops.grouped_gemm(dy, ops.transpose_weights_f32(w2.contiguous()), cnt)
            dw2 = ops.grouped_gemm_dw(hidden, dy, cnt)
            a1 = ops.grouped_gemm(tokens, w1.contiguous(), cnt)
            da1 = ops.mlp_act_backward(a1, dh, ew.act)
            dx = ops.grouped_gemm(da1, ops.transpose_weights_f32(w1.contiguous()), cnt)
            dw1 = ops.grouped_gemm_dw(tokens, da1, cnt)
            return dx, None, None, dw1, dw2, None
        ws = _part_ws(tokens.device)
        NP = 2 * F if swiglu else F
        dh = torch.zeros((S, F), dtype=dy.dtype, device=dy.device)
        dx = torch.zeros((S, H), dtype=dy.dtype, device=dy.device)
        if S:
            ops.grouped_gemm_mapped(dy, None, _packed_weights_t(w2), cnt, S, F, "none", dh, part_ws=ws)
        if a1 is None:  # (no rows, or an MLP without an activation)
            a1 = torch.zeros((S, NP), dtype=dy.dtype, device=dy.device)
            if S:
                ops.grouped_gemm_mapped(tokens, None, ew.w1, cnt, S, NP, "none", a1, part_ws=ws)
        dw2 = ops.grouped_gemm_dw(hidden, dy, cnt)
        da1 = ops.mlp_act_backward(a1, dh, ew.act)
        if S:
            ops.grouped_gemm_mapped(da1, None, _packed_weights_t(w1, w_up), cnt, S, H, "none", dx, part_ws=ws)
        dw1 = ops.grouped_gemm_dw(tokens, da1, cnt, split_F=F if swiglu else 0)
        if swiglu:
            return dx, None, None, dw1[..., :F], dw2, dw1[..., F:]
        return dx, None, None, dw1, dw2, None


def expert_mlp(tokens: torch.Tensor, weights: ExpertWeights, local_expert_cnt: torch.Tensor) -> torch.Tensor:
    """Full expert MLP on expert-major rows -> [S,H]."""
    assert tokens.is_cuda, "tokens must be CUDA"
    _assert_cuda_int32(local_expert_cnt, "local_expert_cnt")
    if weights.dtype == torch.uint8:
        sg, su, sd = weights.scales
        return ops.grouped_mlp_fp8(tokens.contiguous(), local_expert_cnt, weights.ffn, weights.w1, sg, su, weights.w2, sd)
    raw = weights.refresh().raw
    if torch.is_grad_enabled() and raw is not None and (tokens.requires_grad or any(t is not None and t.requires_grad for t in raw)):
        return ExpertMLP.apply(tokens, local_expert_cnt.contiguous(), weights, raw[0], raw[1], raw[2])
    return ops.grouped_mlp(tokens.contiguous(), local_expert_cnt, weights.act, weights.w1, weights.w2, weights.w_up,
                           F=weights.ffn)
