"""Tensor-level wrappers over the C ABI (one function per entry point of include/moe_gfx950.h).

PyTorch is used for device memory and the current stream only; every computation happens in
the HIP kernels.  Outputs and workspaces are allocated here (the C ABI itself allocates nothing)
unless the caller passes them in.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib as L


def _req_cuda(t: torch.Tensor, name: str) -> None:
    assert t.is_cuda, f"{name} must be CUDA"
    assert t.is_contiguous(), f"{name} must be contiguous"


def _req_i32(t: torch.Tensor, name: str) -> None:
    _req_cuda(t, name)
    assert t.dtype == torch.int32, f"{name} must be int32"


def _i32(n, device) -> torch.Tensor:
    return torch.empty(n, dtype=torch.int32, device=device)


# ---- a1 -------------------------------------------------------------------------------------
def route_topk(x: torch.Tensor, router: torch.Tensor, topk: int, bias: Optional[torch.Tensor] = None
               ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(topk_idx int32 [T,k], topk_gate fp32 [T,k], logits fp32 [T,E])."""
    _req_cuda(x, "tokens")
    _req_cuda(router, "router")
    assert x.dtype == router.dtype, "tokens and router must share a dtype"
    T, H = x.shape
    H2, E = router.shape
    assert H == H2, "router must be [H, E]"
    if bias is not None:
        _req_cuda(bias, "bias")
        assert bias.dtype == torch.float32 and bias.shape == (E,)
    dev = x.device
    logits = torch.empty((T, E), dtype=torch.float32, device=dev)
    idx = torch.empty((T, topk), dtype=torch.int32, device=dev)
    gate = torch.empty((T, topk), dtype=torch.float32, device=dev)
    nbytes = L.lib().moe_route_workspace_bytes(T, E)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
    L.check(L.lib().moe_route_topk(L.ptr(x), L.ptr(router), L.ptr(bias), L.dtype_code(x.dtype), T, H, E, topk,
                                   L.ptr(logits), L.ptr(idx), L.ptr(gate), L.ptr(ws), nbytes, L.stream_ptr()))
    return idx, gate, logits


# ---- a2/a4/a5/a6/a7 -------------------------------------------------------------------------
@dataclass
class Counts:
    send_counts: torch.Tensor   # [W,E_l] i32
    expert_offs: torch.Tensor   # [W,E_l] i32
    dst_sizes: torch.Tensor     # [W] i32
    dst_offsets: torch.Tensor   # [W] i32
    caps: torch.Tensor          # [2] i32: max(1,max dst_sizes), max(1,max send_counts)
    pos: torch.Tensor           # [T,k] i32 payload row of slot (t,kk)
    row_token: torch.Tensor     # [T*k] i32 token of payload row


def count_and_offsets(topk_idx: torch.Tensor, num_experts_total: int, world_size: int) -> Counts:
    _req_i32(topk_idx, "topk_idx")
    assert num_experts_total % world_size == 0, "num_experts_total must be divisible by world_size"
    T, k = topk_idx.shape
    E, W = num_experts_total, world_size
    dev = topk_idx.device
    e_l = E // W
    out = Counts(_i32((W, e_l), dev), _i32((W, e_l), dev), _i32((W,), dev), _i32((W,), dev), _i32((2,), dev),
                 _i32((T, k), dev), _i32((T * k,), dev))
    nbytes = L.lib().moe_count_workspace_bytes(T, k, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    L.check(L.lib().moe_count_and_offsets(L.ptr(topk_idx), T, k, E, W, L.ptr(out.send_counts), L.ptr(out.expert_offs),
                                          L.ptr(out.dst_sizes), L.ptr(out.dst_offsets), L.ptr(out.caps), L.ptr(out.pos),
                                          L.ptr(out.row_token), L.ptr(ws), nbytes, L.stream_ptr()))
    return out


def max_floor1(values: torch.Tensor) -> torch.Tensor:
    _req_i32(values, "values")
    out = _i32((1,), values.device)
    L.check(L.lib().moe_max_floor1(L.ptr(values), values.numel(), L.ptr(out), L.stream_ptr()))
    return out


# ---- a3 / a8 --------------------------------------------------------------------------------
def pack_payload(x: torch.Tensor, row_token: torch.Tensor) -> torch.Tensor:
    _req_cuda(x, "tokens")
    _req_i32(row_token, "row_token")
    T, H = x.shape
    R = row_token.numel()
    out = torch.empty((R, H), dtype=x.dtype, device=x.device)
    L.check(L.lib().moe_pack_payload(L.ptr(x), L.dtype_code(x.dtype), T, H, L.ptr(row_token), R, L.ptr(out),
                                     L.stream_ptr()))
    return out


def pack_fixed_m(x: torch.Tensor, row_token: torch.Tensor, dst_sizes: torch.Tensor, dst_offsets: torch.Tensor,
                 M: int, out: Optional[torch.Tensor] = None, map_ws: Optional[torch.Tensor] = None,
                 status: Optional[torch.Tensor] = None) -> torch.Tensor:
    """send [W,M,H]: rows of every destination in (el, token) order, zero padded to M."""
    _req_cuda(x, "tokens")
    _req_i32(row_token, "row_token")
    _req_i32(dst_sizes, "dst_sizes")
    _req_i32(dst_offsets, "dst_offsets")
    T, H = x.shape
    W = dst_sizes.numel()
    if out is None:
        out = torch.empty((W, M, H), dtype=x.dtype, device=x.device)
    assert out.shape == (W, M, H) and out.dtype == x.dtype and out.is_contiguous()
    L.check(L.lib().moe_pack(L.ptr(x), L.dtype_code(x.dtype), T, H, L.ptr(row_token), L.ptr(dst_sizes),
                             L.ptr(dst_offsets), W, M, L.ptr(out), L.ptr(map_ws), L.ptr(status), L.stream_ptr()))
    return out


def pack_tokens(x: torch.Tensor, topk_idx: torch.Tensor, pos: torch.Tensor, dst_sizes: torch.Tensor,
                dst_offsets: torch.Tensor, e_local: int, M: int, out: Optional[torch.Tensor] = None,
                status: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                out_gate: Optional[torch.Tensor] = None):
    """The send buffer of pack_fixed_m written token by token (every token row read once, stored k times).
    With ``gate`` [T,k] the slots' gates travel too: returns (send [W,M,H], send_gate [W,M] fp32, zero in the padding)."""
    _req_cuda(x, "tokens")
    _req_i32(topk_idx, "topk_idx")
    _req_i32(pos, "pos")
    _req_i32(dst_sizes, "dst_sizes")
    _req_i32(dst_offsets, "dst_offsets")
    T, H = x.shape
    W = dst_sizes.numel()
    k = topk_idx.shape[1] if topk_idx.dim() == 2 else 1
    assert topk_idx.numel() == T * k and pos.numel() == T * k
    if out is None:
        out = torch.empty((W, M, H), dtype=x.dtype, device=x.device)
    assert out.shape == (W, M, H) and out.dtype == x.dtype and out.is_contiguous()
    if gate is not None:
        _req_cuda(gate, "gate")
        assert gate.dtype == torch.float32 and gate.numel() == T * k and gate.is_contiguous()
        if out_gate is None:
            out_gate = torch.empty((W, M), dtype=torch.float32, device=x.device)
        assert out_gate.shape == (W, M) and out_gate.dtype == torch.float32 and out_gate.is_contiguous()
        L.check(L.lib().moe_pack_tokens_gated(L.ptr(x), L.dtype_code(x.dtype), T, H, L.ptr(topk_idx), L.ptr(pos), L.ptr(gate), k,
                                              e_local, L.ptr(dst_sizes), L.ptr(dst_offsets), W, M, L.ptr(out), L.ptr(out_gate),
                                              L.ptr(status), L.stream_ptr()))
        return out, out_gate
    L.check(L.lib().moe_pack_tokens(L.ptr(x), L.dtype_code(x.dtype), T, H, L.ptr(topk_idx), L.ptr(pos), k, e_local,
                                    L.ptr(dst_sizes), L.ptr(dst_offsets), W, M, L.ptr(out), L.ptr(status), L.stream_ptr()))
    return out


def pack_tokens_fp8(x: torch.Tensor, topk_idx: torch.Tensor, pos: torch.Tensor, dst_sizes: torch.Tensor,
                    dst_offsets: torch.Tensor, e_local: int, M: int, out_q: Optional[torch.Tensor] = None,
                    out_scale: Optional[torch.Tensor] = None, status: Optional[torch.Tensor] = None,
                    gate: Optional[torch.Tensor] = None, out_gate: Optional[torch.Tensor] = None):
    """pack_tokens with the per-token fp8 quantisation done on the way: ([W,M,H] uint8 codes, [W,M] fp32 scales) -- slot for
    slot what quantize_rows_fp8 makes of pack_tokens' bf16 buffer."""
    _req_cuda(x, "tokens")
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    for t, n in ((topk_idx, "topk_idx"), (pos, "pos"), (dst_sizes, "dst_sizes"), (dst_offsets, "dst_offsets")):
        _req_i32(t, n)
    T, H = x.shape
    W = dst_sizes.numel()
    k = topk_idx.shape[1] if topk_idx.dim() == 2 else 1
    assert topk_idx.numel() == T * k and pos.numel() == T * k
    if out_q is None:
        out_q = torch.empty((W, M, H), dtype=torch.uint8, device=x.device)
    if out_scale is None:
        out_scale = torch.empty((W, M), dtype=torch.float32, device=x.device)
    assert out_q.shape == (W, M, H) and out_q.dtype == torch.uint8 and out_q.is_contiguous()
    assert out_scale.shape == (W, M) and out_scale.dtype == torch.float32 and out_scale.is_contiguous()
    if gate is not None:  # (the slots' gates travel too: a third result, [W,M] fp32, zero in the padding)
        _req_cuda(gate, "gate")
        assert gate.dtype == torch.float32 and gate.numel() == T * k and gate.is_contiguous()
        if out_gate is None:
            out_gate = torch.empty((W, M), dtype=torch.float32, device=x.device)
        assert out_gate.shape == (W, M) and out_gate.dtype == torch.float32 and out_gate.is_contiguous()
        L.check(L.lib().moe_pack_tokens_fp8_gated(L.ptr(x), T, H, L.ptr(topk_idx), L.ptr(pos), L.ptr(gate), k, e_local,
                                                  L.ptr(dst_sizes), L.ptr(dst_offsets), W, M, L.ptr(out_q), L.ptr(out_scale),
                                                  L.ptr(out_gate), L.ptr(status), L.stream_ptr()))
        return out_q, out_scale, out_gate
    L.check(L.lib().moe_pack_tokens_fp8(L.ptr(x), T, H, L.ptr(topk_idx), L.ptr(pos), k, e_local, L.ptr(dst_sizes),
                                        L.ptr(dst_offsets), W, M, L.ptr(out_q), L.ptr(out_scale), L.ptr(status), L.stream_ptr()))
    return out_q, out_scale


# ---- a9 / a10 -------------------------------------------------------------------------------
def _map_ws(W, E_l, n_out, device, map_ws=None):
    need = L.lib().moe_recv_map_ints(W, E_l, n_out)
    if map_ws is None:
        return _i32((need,), device)
    assert map_ws.dtype == torch.int32 and map_ws.numel() >= need and map_ws.is_cuda
    return map_ws


def unpack_token_buf(recv: torch.Tensor, recv_counts: torch.Tensor, capacity: int,
                     token_buf: Optional[torch.Tensor] = None, pca: Optional[torch.Tensor] = None,
                     status: Optional[torch.Tensor] = None, map_ws=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """recv [W,M,H] + recv_counts [W,E_l] -> (token_buf [E_l,W,CAP,H] zero padded, pca [E_l,W])."""
    _req_cuda(recv, "recv")
    _req_i32(recv_counts, "recv_counts")
    W, M, H = recv.shape
    W2, E_l = recv_counts.shape
    assert W == W2
    dev = recv.device
    if token_buf is None:
        token_buf = torch.empty((E_l, W, capacity, H), dtype=recv.dtype, device=dev)
    if tuple(token_buf.shape) != (E_l, W, capacity, H):
        raise ValueError(f"token_buf shape {tuple(token_buf.shape)} mismatch expected ({E_l},{W},{capacity},{H}).")
    if pca is None:
        pca = _i32((E_l, W), dev)
    ws = _map_ws(W, E_l, E_l * W * capacity, dev, map_ws)
    L.check(L.lib().moe_unpack_token_buf(L.ptr(recv), L.dtype_code(recv.dtype), W, M, H, L.ptr(recv_counts), E_l,
                                         capacity, L.ptr(token_buf), L.ptr(pca), L.ptr(ws), L.ptr(status),
                                         L.stream_ptr()))
    return token_buf, pca


def reorder_flat(flat: torch.Tensor, recv_counts: torch.Tensor, capacity: int, token_buf: torch.Tensor,
                 status: Optional[torch.Tensor] = None) -> torch.Tensor:
    _req_cuda(flat, "recv_payload_flat")
    _req_i32(recv_counts, "recv_counts")
    R, H = flat.shape
    W, E_l = recv_counts.shape
    ws = _map_ws(W, E_l, E_l * W * capacity, flat.device)
    L.check(L.lib().moe_reorder_flat_to_token_buf(L.ptr(flat), L.dtype_code(flat.dtype), R, H, L.ptr(recv_counts), W,
                                                  E_l, capacity, L.ptr(token_buf), L.ptr(ws), L.ptr(status),
                                                  L.stream_ptr()))
    return token_buf


def shuffle_rows(token_buf: torch.Tensor, pca: torch.Tensor, S_rows: int, out: Optional[torch.Tensor] = None,
                 expert_cnt: Optional[torch.Tensor] = None, map_ws=None) -> Tuple[torch.Tensor, torch.Tensor]:
    _req_cuda(token_buf, "dispatched_tokens")
    _req_i32(pca, "pca")
    E_l, W, CAP, H = token_buf.shape
    assert pca.shape == (E_l, W)
    dev = token_buf.device
    if out is None:
        out = torch.empty((S_rows, H), dtype=token_buf.dtype, device=dev)
    if expert_cnt is None:
        expert_cnt = _i32((E_l,), dev)
    ws = _map_ws(W, E_l, S_rows, dev, map_ws)
    L.check(L.lib().moe_shuffle(L.ptr(token_buf), L.dtype_code(token_buf.dtype), E_l, W, CAP, H, L.ptr(pca), L.ptr(out),
                                S_rows, L.ptr(expert_cnt), L.ptr(ws), L.stream_ptr()))
    return out, expert_cnt


def shuffle_rows_backward(grad_rows: torch.Tensor, pca: torch.Tensor, capacity: int) -> torch.Tensor:
    """Gradient of shuffle_rows: [S,H] expert-major rows back into the zero-padded [E_l,W,CAP,H] layout."""
    _req_cuda(grad_rows, "grad_rows")
    _req_i32(pca, "pca")
    E_l, W = pca.shape
    H = grad_rows.shape[1]
    out = torch.empty((E_l, W, capacity, H), dtype=grad_rows.dtype, device=grad_rows.device)
    ws = _map_ws(W, E_l, 0, grad_rows.device)
    L.check(L.lib().moe_shuffle_backward(L.ptr(grad_rows), L.dtype_code(grad_rows.dtype), E_l, W, capacity, H, L.ptr(pca),
                                         L.ptr(out), L.ptr(ws), L.stream_ptr()))
    return out


def unpack_expert_major(recv: torch.Tensor, recv_counts: torch.Tensor, S_rows: int,
                        out: Optional[torch.Tensor] = None, expert_cnt: Optional[torch.Tensor] = None,
                        map_ws=None) -> Tuple[torch.Tensor, torch.Tensor]:
    _req_cuda(recv, "recv")
    _req_i32(recv_counts, "recv_counts")
    W, M, H = recv.shape
    E_l = recv_counts.shape[1]
    dev = recv.device
    if out is None:
        out = torch.empty((S_rows, H), dtype=recv.dtype, device=dev)
    if expert_cnt is None:
        expert_cnt = _i32((E_l,), dev)
    ws = _map_ws(W, E_l, S_rows, dev, map_ws)
    L.check(L.lib().moe_unpack_expert_major(L.ptr(recv), L.dtype_code(recv.dtype), W, M, H, L.ptr(recv_counts), E_l,
                                            L.ptr(out), S_rows, L.ptr(expert_cnt), L.ptr(ws), L.stream_ptr()))
    return out, expert_cnt


# ---- a11 / a12 ------------------------------------------------------------------------------
def prepack_weights(w: torch.Tensor, w_up: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[E_l,K,N] (reference layout) -> the MFMA kernels' K-contiguous layout (one-time, per weight)."""
    _req_cuda(w, "weights")
    assert w.dtype == torch.bfloat16, "prepack is for bf16 weights (fp32 uses the reference layout as is)"
    E_l, K, N = w.shape
    if w_up is not None:
        _req_cuda(w_up, "w_up")
        assert w_up.shape == w.shape and w_up.dtype == w.dtype
    n_eff = N * (2 if w_up is not None else 1)
    nbytes = L.lib().moe_prepack_bytes(L.MOE_BF16, E_l, K, n_eff)
    out = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    L.check(L.lib().moe_prepack_weights(L.ptr(w), L.ptr(w_up), L.MOE_BF16, E_l, K, N, L.ptr(out), L.stream_ptr()))
    return out


def grouped_gemm(tokens: torch.Tensor, weights: torch.Tensor, expert_cnt: torch.Tensor,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[rows of e] = tokens[rows of e] @ weights[e] (weights in the reference [E_l,K,N] layout)."""
    _req_cuda(tokens, "tokens")
    _req_cuda(weights, "weights")
    _req_i32(expert_cnt, "local_expert_cnt")
    assert tokens.dtype == weights.dtype
    S, K = tokens.shape
    E_l, K2, N = weights.shape
    assert K == K2 and expert_cnt.numel() == E_l
    if out is None:
        out = torch.zeros((S, N), dtype=tokens.dtype, device=tokens.device)
    code = L.dtype_code(tokens.dtype)
    nbytes = L.lib().moe_prepack_bytes(code, E_l, K, N)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=tokens.device)
    L.check(L.lib().moe_grouped_gemm(L.ptr(tokens), L.ptr(weights), L.ptr(expert_cnt), code, S, K, N, E_l, L.ptr(out),
                                     L.ptr(ws), nbytes, L.stream_ptr()))
    return out


def grouped_mlp(tokens: torch.Tensor, expert_cnt: torch.Tensor, act: str, w1, w2, w_up=None, F: Optional[int] = None,
                hidden_ws: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Expert MLP on expert-major rows.

    bf16: ``w1``/``w2`` are prepack_weights() results (``w1`` = prepack(Wg, Wu) for swiglu), ``F`` is
    required.  fp32: ``w1`` [E_l,H,F], ``w_up`` (swiglu only) [E_l,H,F], ``w2`` [E_l,F,H] in the
    reference layout.
    """
    _req_cuda(tokens, "tokens")
    _req_i32(expert_cnt, "local_expert_cnt")
    S, H = tokens.shape
    E_l = expert_cnt.numel()
    if tokens.dtype == torch.float32:
        F = w1.shape[2]
    assert F is not None
    dev = tokens.device
    if hidden_ws is None:
        hidden_ws = torch.empty((S, F), dtype=tokens.dtype, device=dev)
    if out is None:
        out = torch.zeros((S, H), dtype=tokens.dtype, device=dev)
    L.check(L.lib().moe_grouped_mlp(L.ptr(tokens), L.ptr(expert_cnt), L.dtype_code(tokens.dtype), S, H, F, E_l,
                                    L.ACT[act], L.ptr(w1), L.ptr(w_up), L.ptr(w2), L.ptr(hidden_ws), L.ptr(out),
                                    L.stream_ptr()))
    return out


def prepack_weights_fp8(w: torch.Tensor, w_up: Optional[torch.Tensor] = None) -> torch.Tensor:
    """uint8 e4m3 codes [E_l,K,N] -> packed layout (1 byte per element)."""
    _req_cuda(w, "weights")
    assert w.dtype == torch.uint8
    E_l, K, N = w.shape
    n_eff = N * (2 if w_up is not None else 1)
    nbytes = L.lib().moe_prepack_bytes(2, E_l, K, n_eff)
    out = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    L.check(L.lib().moe_prepack_weights_fp8(L.ptr(w), L.ptr(w_up), E_l, K, N, L.ptr(out), L.stream_ptr()))
    return out


def quantize_rows_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    _req_cuda(x, "x")
    assert x.dtype == torch.bfloat16
    R, C = x.shape
    q = torch.empty((R, C), dtype=torch.uint8, device=x.device)
    s = torch.empty((R,), dtype=torch.float32, device=x.device)
    L.check(L.lib().moe_quantize_rows_fp8(L.ptr(x), R, C, L.ptr(q), L.ptr(s), None, L.stream_ptr()))
    return q, s


def grouped_mlp_fp8(tokens: torch.Tensor, expert_cnt: torch.Tensor, F: int, wgu_packed, sg, su, wd_packed, sd,
                    ws: Optional[dict] = None, out: Optional[torch.Tensor] = None,
                    part_ws: Optional[torch.Tensor] = None, row_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp8 SwiGLU expert MLP on bf16 rows.  ws (fp8_workspace) receives the intermediates: "xq" / "xs" the rows quantised per
    row, "hq" / "hsc" the hidden activation as e4m3 codes with one power-of-two scale byte per row and 32 columns."""
    _req_cuda(tokens, "tokens")
    assert tokens.dtype == torch.bfloat16
    S, H = tokens.shape
    E_l = expert_cnt.numel()
    dev = tokens.device
    if ws is None:
        ws = fp8_workspace(S, H, F, dev)
    if out is None:
        out = torch.zeros((S, H), dtype=torch.bfloat16, device=dev)
    L.check(L.lib().moe_grouped_mlp_fp8_mapped(L.ptr(tokens), S, None, L.ptr(expert_cnt), S, H, F, E_l, L.ptr(wgu_packed),
                                               L.ptr(sg), L.ptr(su), L.ptr(wd_packed), L.ptr(sd), L.ptr(ws["xq"]),
                                               L.ptr(ws["xs"]), L.ptr(ws["hq"]), L.ptr(ws["hsc"]), L.ptr(row_gate), L.ptr(out), S,
                                               None, L.ptr(part_ws), 0 if part_ws is None else part_ws.numel() * part_ws.element_size(),
                                               L.stream_ptr()))
    return out


def grouped_mlp_fp8_q(a_q: torch.Tensor, a_scale: torch.Tensor, a_row_map: Optional[torch.Tensor], expert_cnt: torch.Tensor,
                      S_rows: int, F: int, wgu_packed, sg, su, wd_packed, sd, ws: dict, out: torch.Tensor,
                      c_row_map: Optional[torch.Tensor] = None, part_ws: Optional[torch.Tensor] = None,
                      row_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """grouped_mlp_fp8 for rows that arrive as fp8 codes and scales (pack_tokens_fp8): a_q [rows,H] uint8, a_scale [rows];
    ws as from fp8_workspace (its "xq" is not used, "xs" receives the scales in row order)."""
    _req_cuda(a_q, "a_q")
    _req_i32(expert_cnt, "expert_cnt")
    assert a_q.dtype == torch.uint8 and a_q.dim() == 2 and a_q.is_contiguous() and a_scale.dtype == torch.float32
    assert a_scale.numel() == a_q.shape[0] and out.dtype == torch.bfloat16 and out.dim() == 2 and out.is_contiguous()
    H = a_q.shape[1]
    assert out.shape[1] == H
    L.check(L.lib().moe_grouped_mlp_fp8_q_mapped(L.ptr(a_q), L.ptr(a_scale), a_q.shape[0], L.ptr(a_row_map), L.ptr(expert_cnt),
                                                 S_rows, H, F, expert_cnt.numel(), L.ptr(wgu_packed), L.ptr(sg), L.ptr(su),
                                                 L.ptr(wd_packed), L.ptr(sd), L.ptr(ws["xs"]), L.ptr(ws["hq"]), L.ptr(ws["hsc"]),
                                                 L.ptr(row_gate), L.ptr(out), out.shape[0], L.ptr(c_row_map), L.ptr(part_ws),
                                                 0 if part_ws is None else part_ws.numel() * part_ws.element_size(),
                                                 L.stream_ptr()))
    return out


def fp8_workspace(S: int, H: int, F: int, dev) -> dict:
    return {
        "xq": torch.empty((S, H), dtype=torch.uint8, device=dev),
        "xs": torch.empty((S,), dtype=torch.float32, device=dev),
        "hq": torch.empty((S, F), dtype=torch.uint8, device=dev),      # hidden activation: e4m3 codes ...
        "hsc": torch.empty((S, F // 32), dtype=torch.uint8, device=dev),  # ... and their block scales (E8M0 bytes)
    }


def dequantize_hidden_fp8(hq: torch.Tensor, hsc: torch.Tensor) -> torch.Tensor:
    """The hidden activation an fp8 MLP call left in its workspace, as fp32: code value x 2^(scale byte - 127) per block of 32."""
    vals = hq.view(torch.float8_e4m3fn).float()
    scale = torch.exp2(hsc.float() - 127.0)
    return (vals.view(hq.shape[0], -1, 32) * scale[:, :, None]).view(hq.shape)


# ---- a13 ------------------------------------------------------------------------------------
def return_pack(y: torch.Tensor, recv_counts: torch.Tensor, M: int, out: Optional[torch.Tensor] = None,
                map_ws=None) -> torch.Tensor:
    _req_cuda(y, "y")
    _req_i32(recv_counts, "recv_counts")
    S, H = y.shape
    W, E_l = recv_counts.shape
    if out is None:
        out = torch.empty((W, M, H), dtype=y.dtype, device=y.device)
    ws = _map_ws(W, E_l, W * M, y.device, map_ws)
    L.check(L.lib().moe_return_pack(L.ptr(y), L.dtype_code(y.dtype), S, H, L.ptr(recv_counts), W, E_l, M, L.ptr(out),
                                    L.ptr(ws), L.stream_ptr()))
    return out


# ---- destination side without the two row copies ------------------------------------------------
def recv_row_map(recv_counts: torch.Tensor, M: int, n_rows: int, row_map: Optional[torch.Tensor] = None,
                 expert_cnt: Optional[torch.Tensor] = None, map_ws=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """row_map[r] = row of the flattened [W*M,H] receive buffer holding expert-major row r, and the
    per-expert row counts (what unpack_expert_major returns beside the rows)."""
    _req_i32(recv_counts, "recv_counts")
    W, E_l = recv_counts.shape
    dev = recv_counts.device
    if row_map is None:
        row_map = _i32((max(n_rows, 1),), dev)
    if expert_cnt is None:
        expert_cnt = _i32((E_l,), dev)
    ws = _map_ws(W, E_l, n_rows, dev, map_ws)
    L.check(L.lib().moe_recv_row_map(L.ptr(recv_counts), W, E_l, M, n_rows, L.ptr(row_map), L.ptr(expert_cnt), L.ptr(ws),
                                     L.stream_ptr()))
    return row_map, expert_cnt


def recv_row_map_gated(recv_counts: torch.Tensor, M: int, n_rows: int, recv_gate: Optional[torch.Tensor] = None,
                       row_map: Optional[torch.Tensor] = None, expert_cnt: Optional[torch.Tensor] = None,
                       row_gate: Optional[torch.Tensor] = None):
    """recv_row_map that, given the gates that arrived with the rows (recv_gate, one per row of the receive buffer), also
    returns them in the GEMM's row order; M == 0: the receive buffer is a padding-free flat payload (see recv_row_map_flat).
    -> (row_map, expert_cnt, row_gate or None)."""
    _req_i32(recv_counts, "recv_counts")
    W, E_l = recv_counts.shape
    dev = recv_counts.device
    if row_map is None:
        row_map = _i32((max(n_rows, 1),), dev)
    if expert_cnt is None:
        expert_cnt = _i32((E_l,), dev)
    if recv_gate is not None:
        _req_cuda(recv_gate, "recv_gate")
        assert recv_gate.dtype == torch.float32 and recv_gate.is_contiguous()
        if row_gate is None:
            row_gate = torch.empty((max(n_rows, 1),), dtype=torch.float32, device=dev)
    L.check(L.lib().moe_recv_row_map_gated(L.ptr(recv_counts), W, E_l, M, n_rows, L.ptr(recv_gate), L.ptr(row_map), L.ptr(row_gate),
                                           L.ptr(expert_cnt), L.stream_ptr()))
    return row_map, expert_cnt, row_gate


def recv_row_map_flat(recv_counts: torch.Tensor, n_rows: int, row_map: Optional[torch.Tensor] = None,
                      expert_cnt: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """row_map[r] = row of a padding-free flat receive payload (source-major, expert-minor blocks: what
    reorder_flat_to_token_buf reads) holding expert-major row r, and the per-expert row counts."""
    _req_i32(recv_counts, "recv_counts")
    W, E_l = recv_counts.shape
    dev = recv_counts.device
    if row_map is None:
        row_map = _i32((max(n_rows, 1),), dev)
    if expert_cnt is None:
        expert_cnt = _i32((E_l,), dev)
    L.check(L.lib().moe_recv_row_map_flat(L.ptr(recv_counts), W, E_l, n_rows, L.ptr(row_map), L.ptr(expert_cnt), L.stream_ptr()))
    return row_map, expert_cnt


def grouped_gemm_mapped_gated(a_base: torch.Tensor, a_row_map: Optional[torch.Tensor], packed: torch.Tensor,
                              expert_cnt: torch.Tensor, S_rows: int, N: int, row_gate: torch.Tensor, out: torch.Tensor,
                              c_row_map: Optional[torch.Tensor] = None, part_ws: Optional[torch.Tensor] = None) -> torch.Tensor:
    """grouped_gemm_mapped without activation whose result row r is multiplied by row_gate[r] (fp32, before the rounding)."""
    assert a_base.dim() == 2 and out.dim() == 2 and a_base.is_contiguous() and out.is_contiguous()
    assert a_base.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and out.shape[1] == N
    assert row_gate.dtype == torch.float32 and row_gate.numel() >= S_rows and row_gate.is_contiguous()
    _req_i32(expert_cnt, "expert_cnt")
    K = a_base.shape[1]
    L.check(L.lib().moe_grouped_gemm_mapped_gated(L.ptr(a_base), a_base.shape[0], L.ptr(a_row_map), L.ptr(packed), L.ptr(expert_cnt),
                                                  S_rows, K, N, expert_cnt.numel(), L.ptr(row_gate), L.ptr(out), out.shape[0],
                                                  L.ptr(c_row_map), L.ptr(part_ws),
                                                  0 if part_ws is None else part_ws.numel() * part_ws.element_size(),
                                                  L.stream_ptr()))
    return out


def grouped_gemm_mapped(a_base: torch.Tensor, a_row_map: Optional[torch.Tensor], packed: torch.Tensor,
                        expert_cnt: torch.Tensor, S_rows: int, N: int, act: str, out: torch.Tensor,
                        c_row_map: Optional[torch.Tensor] = None, part_ws: Optional[torch.Tensor] = None) -> torch.Tensor:
    """grouped_gemm_packed with row indirection on the way in (a_base rows a_row_map[r]) and / or on the
    way out (out rows c_row_map[r]).  a_base and out are 2-D views [rows, K] / [rows, N].  part_ws: optional
    scratch (gemm_part_workspace) that lets an under-filled last round of tiles be split along K."""
    _req_cuda(a_base, "a_base")
    _req_i32(expert_cnt, "expert_cnt")
    assert a_base.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and a_base.dim() == 2 and out.dim() == 2
    assert a_base.is_contiguous() and out.is_contiguous() and out.shape[1] == N
    for m, name in ((a_row_map, "a_row_map"), (c_row_map, "c_row_map")):
        if m is not None:
            _req_i32(m, name)
            assert m.numel() >= S_rows, f"{name} must cover S_rows"
    L.check(L.lib().moe_grouped_gemm_mapped(L.ptr(a_base), a_base.shape[0], L.ptr(a_row_map) if a_row_map is not None else None,
                                            L.ptr(packed), L.ptr(expert_cnt), S_rows, a_base.shape[1], N, expert_cnt.numel(),
                                            L.ACT[act], L.ptr(out), out.shape[0],
                                            L.ptr(c_row_map) if c_row_map is not None else None,
                                            L.ptr(part_ws) if part_ws is not None else None,
                                            part_ws.numel() * part_ws.element_size() if part_ws is not None else 0,
                                            L.stream_ptr()))
    return out


def grouped_gemm_act_keep(a_base: torch.Tensor, packed: torch.Tensor, expert_cnt: torch.Tensor, S_rows: int, N: int, act: str,
                          out: torch.Tensor, pre_act: torch.Tensor, part_ws: Optional[torch.Tensor] = None) -> torch.Tensor:
    """grouped_gemm_mapped with an activation that also keeps the values before it (for the backward pass):
    pre_act [S_rows, N], for SwiGLU [S_rows, 2N] in the fused gate / up column order (what mlp_act_backward takes)."""
    _req_cuda(a_base, "a_base")
    _req_i32(expert_cnt, "expert_cnt")
    assert act in ("gelu", "silu", "swiglu"), "an activation to keep the input of"
    assert a_base.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and pre_act.dtype == torch.bfloat16
    assert a_base.is_contiguous() and out.is_contiguous() and pre_act.is_contiguous()
    assert out.shape == (S_rows, N) and pre_act.shape == (S_rows, 2 * N if act == "swiglu" else N)
    L.check(L.lib().moe_grouped_gemm_act_keep(L.ptr(a_base), a_base.shape[0], None, L.ptr(packed), L.ptr(expert_cnt), S_rows,
                                              a_base.shape[1], N, expert_cnt.numel(), L.ACT[act], L.ptr(out), L.ptr(pre_act),
                                              L.ptr(part_ws) if part_ws is not None else None,
                                              part_ws.numel() * part_ws.element_size() if part_ws is not None else 0,
                                              L.stream_ptr()))
    return out


def gemm_part_workspace(device) -> torch.Tensor:
    """fp32 scratch for the K-split of grouped_gemm_mapped, sized for any launch."""
    return torch.empty(L.lib().moe_gemm_part_workspace_bytes() // 4, dtype=torch.float32, device=device)


def zero_padding_rows(buf: torch.Tensor, recv_counts: torch.Tensor) -> torch.Tensor:
    """Zero the rows of a [W,M,H] buffer that lie past what each slot received."""
    _req_cuda(buf, "buf")
    _req_i32(recv_counts, "recv_counts")
    W, M, H = buf.shape
    L.check(L.lib().moe_zero_padding_rows(L.ptr(buf), L.dtype_code(buf.dtype), W, M, H, L.ptr(recv_counts),
                                          recv_counts.shape[1], L.stream_ptr()))
    return buf


def combine(ret: torch.Tensor, topk_idx: torch.Tensor, pos: torch.Tensor, gate: Optional[torch.Tensor],
            dst_offsets: torch.Tensor, e_local: int, out: Optional[torch.Tensor] = None,
            status: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = sum_kk gate[t,kk] * ret[slot of (t,kk)].  Slots the pack dropped (row at or past M) are skipped
    and raise ``status`` (int32 [1], optional).  gate None: the rows arrive weighted and are only added."""
    _req_cuda(ret, "ret")
    _req_i32(topk_idx, "topk_idx")
    _req_i32(pos, "pos")
    _req_i32(dst_offsets, "dst_offsets")
    if gate is not None:
        _req_cuda(gate, "gate")
        assert gate.dtype == torch.float32
    W, M, H = ret.shape
    T, k = topk_idx.shape
    if out is None:
        out = torch.empty((T, H), dtype=ret.dtype, device=ret.device)
    L.check(L.lib().moe_combine(L.ptr(ret), L.dtype_code(ret.dtype), W, M, H, L.ptr(topk_idx), L.ptr(pos), L.ptr(gate),
                                L.ptr(dst_offsets), T, k, e_local, L.ptr(out), L.ptr(status), L.stream_ptr()))
    return out


def build_expert_offsets(send_counts: torch.Tensor, with_dst: bool = False):
    """expert_offs [W,E_l] (and, with_dst, dst_sizes [W], dst_offsets [W]) for a counts matrix."""
    _req_i32(send_counts, "send_counts")
    W, E_l = send_counts.shape
    dev = send_counts.device
    offs = _i32((W, E_l), dev)
    sizes = _i32((W,), dev) if with_dst else None
    doffs = _i32((W,), dev) if with_dst else None
    L.check(L.lib().moe_build_expert_offsets(L.ptr(send_counts), W, E_l, L.ptr(offs), L.ptr(sizes), L.ptr(doffs),
                                             L.stream_ptr()))
    return (offs, sizes, doffs) if with_dst else offs


# ---- gradients ----------------------------------------------------------------------------------
def prepack_weights_transposed(w: torch.Tensor, w_up: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[E_l,K,N] bf16 -> the kernels' layout of w^T (weights of d tokens = d out @ w^T); with ``w_up`` the pair is
    transposed together in the fused gate/up column order."""
    _req_cuda(w, "weights")
    assert w.dtype == torch.bfloat16
    E_l, K, N = w.shape
    if w_up is not None:
        _req_cuda(w_up, "w_up")
        assert w_up.shape == w.shape and w_up.dtype == w.dtype
    n_tot = N * (2 if w_up is not None else 1)
    nbytes = L.lib().moe_prepack_bytes(L.MOE_BF16, E_l, n_tot, K)
    out = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    L.check(L.lib().moe_prepack_weights_transposed(L.ptr(w), L.ptr(w_up), L.MOE_BF16, E_l, K, N, L.ptr(out), L.stream_ptr()))
    return out


def transpose_weights_f32(w: torch.Tensor) -> torch.Tensor:
    """[E_l,K,N] fp32 -> [E_l,N,K]."""
    _req_cuda(w, "weights")
    assert w.dtype == torch.float32
    E_l, K, N = w.shape
    out = torch.empty((E_l, N, K), dtype=w.dtype, device=w.device)
    L.check(L.lib().moe_transpose_weights_f32(L.ptr(w), E_l, K, N, L.ptr(out), L.stream_ptr()))
    return out


def grouped_gemm_dw(x: torch.Tensor, dy: torch.Tensor, expert_cnt: torch.Tensor, split_F: int = 0) -> torch.Tensor:
    """d w[g] = x[rows of g]^T @ dy[rows of g] for all groups in one launch -> [E_l,K,N] (zeros for empty groups).
    ``split_F`` > 0: dy is [S, 2 split_F] in the fused gate/up column order, the result [E_l,K,2 split_F] holds
    [d w_gate | d w_up] side by side."""
    _req_cuda(x, "x")
    _req_cuda(dy, "dy")
    _req_i32(expert_cnt, "expert_cnt")
    assert x.dtype == dy.dtype and x.shape[0] == dy.shape[0]
    S, K = x.shape
    N = dy.shape[1]
    E_l = expert_cnt.numel()
    code = L.dtype_code(x.dtype)
    dw = torch.empty((E_l, K, N), dtype=x.dtype, device=x.device)
    nbytes = L.lib().moe_dw_workspace_bytes(S, E_l, K, N) if x.dtype == torch.bfloat16 else 0
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
    L.check(L.lib().moe_grouped_gemm_dw(L.ptr(x), L.ptr(dy), L.ptr(expert_cnt), code, S, K, N, E_l, split_F, L.ptr(dw), L.ptr(ws),
                                        nbytes, L.stream_ptr()))
    return dw


def mlp_act_backward(a1: torch.Tensor, dh: torch.Tensor, act: str) -> torch.Tensor:
    """Gradient of the pre-activations a1 ([S,F]; swiglu: [S,2F] in the fused gate/up column order) from d hidden [S,F]."""
    _req_cuda(a1, "a1")
    _req_cuda(dh, "dh")
    assert a1.dtype == dh.dtype
    S, F = dh.shape
    out = torch.empty_like(a1)
    L.check(L.lib().moe_mlp_act_backward(L.ptr(a1), L.ptr(dh), L.dtype_code(a1.dtype), S, F, L.ACT[act], L.ptr(out), L.stream_ptr()))
    return out


def combine_backward(d_out: torch.Tensor, ret: torch.Tensor, topk_idx: torch.Tensor, pos: torch.Tensor, gate: torch.Tensor,
                     dst_sizes: torch.Tensor, dst_offsets: torch.Tensor, e_local: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(d ret [W,M,H], d gate [T,k]) of out = combine(ret, ...)."""
    _req_cuda(d_out, "d_out")
    _req_cuda(ret, "ret")
    _req_i32(topk_idx, "topk_idx")
    _req_i32(pos, "pos")
    _req_i32(dst_sizes, "dst_sizes")
    _req_i32(dst_offsets, "dst_offsets")
    W, M, H = ret.shape
    T, k = topk_idx.shape
    d_ret = torch.empty_like(ret)
    d_gate = torch.empty((T, k), dtype=torch.float32, device=ret.device)
    L.check(L.lib().moe_combine_backward(L.ptr(d_out), L.ptr(ret), L.dtype_code(ret.dtype), W, M, H, L.ptr(topk_idx), L.ptr(pos),
                                         L.ptr(gate), L.ptr(dst_sizes), L.ptr(dst_offsets), T, k, e_local, L.ptr(d_ret),
                                         L.ptr(d_gate), L.stream_ptr()))
    return d_ret, d_gate
