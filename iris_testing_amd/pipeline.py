"""The whole hot path of one step on rank 0, with every buffer allocated once up front.

A step = what rank 0 does for one batch:
  as a source       route + top-k  ->  counts / offsets / positions  ->  pack into [W,M,H]
  as a destination  expert-major unpack of its receive buffer  ->  grouped expert MLP  ->  return pack
  as a source       top-k-weighted combine of the returned buffer into token order
With ``fused=True`` (bf16 or fp8 experts) the destination side skips the two row copies: "unpack" only builds the
row map, the first GEMM gathers its input rows from the receive buffer, the second scatters its result rows
into the returned layout, and "return_pack" only zeroes the padding rows.
With ``fp8_dispatch=True`` (fp8 experts, fused) the tokens are quantised per row where they are packed: the send and
receive buffers hold fp8 codes and one scale per row, and the destination runs no quantisation pass over its input.
With ``gated=True`` (fused) the top-k gates travel with the rows ([W,M] fp32 beside the send buffer), the down projection
multiplies every result row by its gate before rounding it, and the combine only adds the returned rows.
With ``padding_free=True`` (fused) the rows cross as the reference's padding-free payload (utils.py:235-246) instead of
fixed-M slots: "pack" gathers the payload, the GEMMs gather from / scatter into flat [S,H] buffers through a row map over
the payload's source-major blocks, nothing is zero-filled, and the combine reads the returned payload by position.
The two transfers in between are not part of a one-GPU build: the receive buffer and the returned
buffer are assembled beforehand (harness.build_world) and stay fixed.  Each stage is one C-ABI call
on the current stream; no stage synchronises or allocates.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from . import _lib as L
from .harness import World
from .layers.expert import ExpertWeights

STAGES = ["route", "count", "pack", "unpack", "mlp_up", "mlp_down", "return_pack", "combine"]


class DispatchPipeline:
    def __init__(self, world: World, weights: ExpertWeights, returned: Optional[torch.Tensor] = None,
                 fused: Optional[bool] = None, fp8_dispatch: Optional[bool] = None, gated: bool = False,
                 padding_free: bool = False, recv_gate: Optional[torch.Tensor] = None,
                 recv_flat: Optional[torch.Tensor] = None):
        cfg = world.cfg
        # gather / scatter inside the GEMMs needs the bf16 MFMA path and a receive buffer under 4 GiB
        can_fuse = weights.dtype in (torch.bfloat16, torch.uint8) and \
            world.recv.numel() * world.recv.element_size() < (1 << 32)
        self.fused = can_fuse if fused is None else bool(fused)
        if self.fused and not can_fuse:
            raise ValueError("the fused destination path needs bf16 or fp8 expert weights and a receive buffer under 4 GiB")
        self.gated, self.padding_free = bool(gated), bool(padding_free)
        if (self.gated or self.padding_free) and not self.fused:
            raise ValueError("gated / padding_free are forms of the fused destination side")
        if self.gated and self.padding_free:
            raise ValueError("gated and padding_free are separate modes")
        if self.gated and weights.dtype == torch.float32:
            raise ValueError("the gated return needs bf16 or fp8 experts")
        if self.gated and recv_gate is None:
            raise ValueError("gated: pass the gates that arrive with the rows (harness.recv_gates)")
        if self.padding_free and recv_flat is None:
            raise ValueError("padding_free: pass the flat receive payload (harness.recv_flat)")
        self.recv_gate, self.recv_flat = recv_gate, recv_flat
        can_q = self.fused and weights.dtype == torch.uint8 and world.recv_q is not None and cfg.torch_dtype == torch.bfloat16 \
            and not self.padding_free
        self.fp8_dispatch = can_q if fp8_dispatch is None else bool(fp8_dispatch)
        if self.fp8_dispatch and not can_q:
            raise ValueError("fp8 dispatch needs fp8 experts, bf16 tokens, the fused destination side and a quantised receive buffer")
        self.world, self.cfg, self.weights = world, cfg, weights
        dev = world.x0.device
        T, H, E, k, W, E_l, F = cfg.tokens, cfg.hidden, cfg.experts, cfg.topk, cfg.world, cfg.e_local, cfg.ffn
        M, S = world.M, world.S
        self.S = S
        dt = cfg.torch_dtype
        i32 = lambda *s: torch.empty(s, dtype=torch.int32, device=dev)  # noqa: E731
        lib = L.lib()
        self.code = L.dtype_code(dt)
        # source side
        self.logits = torch.empty((T, E), dtype=torch.float32, device=dev)
        self.route_ws_bytes = lib.moe_route_workspace_bytes(T, E)
        self.route_ws = torch.empty(max(self.route_ws_bytes, 16), dtype=torch.uint8, device=dev)
        self.idx, self.gate = i32(T, k), torch.empty((T, k), dtype=torch.float32, device=dev)
        self.send_counts, self.expert_offs = i32(W, E_l), i32(W, E_l)
        self.dst_sizes, self.dst_offsets, self.caps = i32(W), i32(W), i32(2)
        self.pos, self.row_token = i32(T, k), i32(T * k)
        self.count_ws_bytes = lib.moe_count_workspace_bytes(T, k, E)
        self.count_ws = torch.empty(self.count_ws_bytes, dtype=torch.uint8, device=dev)
        self.send = torch.empty((W, M, H), dtype=dt, device=dev) if not self.padding_free else None
        if self.gated:
            self.send_gate = torch.empty((W, M), dtype=torch.float32, device=dev)
            self.row_gate = torch.empty((max(S, 1),), dtype=torch.float32, device=dev)
        if self.padding_free:
            self.payload = torch.empty((T * k, H), dtype=dt, device=dev)   # what this rank sends: [R,H], (dst, el, token) order
            self.ret_flat = torch.empty((max(S, 1), H), dtype=dt, device=dev)  # what it sends back: one row per received row
            self.zero_off = torch.zeros(1, dtype=torch.int32, device=dev)
        if self.fp8_dispatch:
            self.send_q = torch.empty((W, M, H), dtype=torch.uint8, device=dev)
            self.send_scale = torch.empty((W, M), dtype=torch.float32, device=dev)
        self.status = torch.zeros(1, dtype=torch.int32, device=dev)
        # destination side
        self.rows = torch.empty((S, H), dtype=dt, device=dev)
        self.expert_cnt = i32(E_l)
        self.unpack_map = i32(lib.moe_recv_map_ints(W, E_l, S))
        self.hidden = torch.empty((S, F), dtype=dt, device=dev) if weights.dtype != torch.uint8 else None
        self.y = torch.zeros((S, H), dtype=dt, device=dev)
        self.ret = torch.empty((W, M, H), dtype=dt, device=dev) if not self.padding_free else None
        self.ret_map = i32(lib.moe_recv_map_ints(W, E_l, W * M))
        self.row_map = i32(max(S, 1))
        # scratch for the K-split of an under-filled last round of GEMM tiles (bf16 and fp8 experts)
        self.part_ws_bytes = lib.moe_gemm_part_workspace_bytes() if weights.dtype in (torch.bfloat16, torch.uint8) else 0
        self.part_ws = torch.empty(self.part_ws_bytes // 4, dtype=torch.float32, device=dev) if self.part_ws_bytes else None
        if weights.dtype == torch.uint8:
            self.xq = torch.empty((S, H), dtype=torch.uint8, device=dev)
            self.xs = torch.empty((S,), dtype=torch.float32, device=dev)
            self.hq = torch.empty((S, F), dtype=torch.uint8, device=dev)          # hidden activation: e4m3 codes
            self.hsc = torch.empty((S, F // 32), dtype=torch.uint8, device=dev)   # and one scale byte per row and 32 columns
        # source side again: what comes back ([W,M,H], same slots as `send`) and the combined output
        if self.padding_free:  # the returned payload: [R,H], row pos[t,kk] is the result of slot (t,kk)
            self.returned = returned if returned is not None else torch.zeros((T * k, H), dtype=dt, device=dev)
        else:
            self.returned = returned if returned is not None else torch.zeros((W, M, H), dtype=dt, device=dev)
        self.out = torch.empty((T, H), dtype=dt, device=dev)
        self._p = L.ptr

    # each stage is a closure-free method so that callers can time them one by one
    def route(self, s):
        c, w = self.cfg, self.world
        L.check(L.lib().moe_route_topk(self._p(w.x0), self._p(w.router), self._p(w.bias), self.code, c.tokens, c.hidden,
                                       c.experts, c.topk, self._p(self.logits), self._p(self.idx), self._p(self.gate),
                                       self._p(self.route_ws), self.route_ws_bytes, s))

    def count(self, s):
        c = self.cfg
        L.check(L.lib().moe_count_and_offsets(self._p(self.idx), c.tokens, c.topk, c.experts, c.world,
                                              self._p(self.send_counts), self._p(self.expert_offs), self._p(self.dst_sizes),
                                              self._p(self.dst_offsets), self._p(self.caps), self._p(self.pos),
                                              self._p(self.row_token), self._p(self.count_ws), self.count_ws_bytes, s))

    def pack(self, s):
        c, w = self.cfg, self.world
        if self.fp8_dispatch:
            L.check(L.lib().moe_pack_tokens_fp8_gated(self._p(w.x0), c.tokens, c.hidden, self._p(self.idx), self._p(self.pos),
                                                      self._p(self.gate) if self.gated else None, c.topk, c.e_local,
                                                      self._p(self.dst_sizes), self._p(self.dst_offsets), c.world, w.M,
                                                      self._p(self.send_q), self._p(self.send_scale),
                                                      self._p(self.send_gate) if self.gated else None, self._p(self.status), s))
            return
        if self.padding_free:
            L.check(L.lib().moe_pack_payload(self._p(w.x0), self.code, c.tokens, c.hidden, self._p(self.row_token),
                                             c.tokens * c.topk, self._p(self.payload), s))
            return
        if self.gated:
            L.check(L.lib().moe_pack_tokens_gated(self._p(w.x0), self.code, c.tokens, c.hidden, self._p(self.idx), self._p(self.pos),
                                                  self._p(self.gate), c.topk, c.e_local, self._p(self.dst_sizes),
                                                  self._p(self.dst_offsets), c.world, w.M, self._p(self.send),
                                                  self._p(self.send_gate), self._p(self.status), s))
            return
        L.check(L.lib().moe_pack_tokens(self._p(w.x0), self.code, c.tokens, c.hidden, self._p(self.idx), self._p(self.pos),
                                        c.topk, c.e_local, self._p(self.dst_sizes), self._p(self.dst_offsets), c.world, w.M,
                                        self._p(self.send), self._p(self.status), s))

    def unpack(self, s):
        c, w = self.cfg, self.world
        if self.padding_free:
            L.check(L.lib().moe_recv_row_map_flat(self._p(w.recv_counts), c.world, c.e_local, self.S, self._p(self.row_map),
                                                  self._p(self.expert_cnt), s))
            return
        if self.gated:
            L.check(L.lib().moe_recv_row_map_gated(self._p(w.recv_counts), c.world, c.e_local, w.M, self.S, self._p(self.recv_gate),
                                                   self._p(self.row_map), self._p(self.row_gate), self._p(self.expert_cnt), s))
            return
        if self.fused:
            L.check(L.lib().moe_recv_row_map(self._p(w.recv_counts), c.world, c.e_local, w.M, self.S, self._p(self.row_map),
                                             self._p(self.expert_cnt), self._p(self.unpack_map), s))
            return
        L.check(L.lib().moe_unpack_expert_major(self._p(w.recv), self.code, c.world, w.M, c.hidden, self._p(w.recv_counts),
                                                c.e_local, self._p(self.rows), self.S, self._p(self.expert_cnt),
                                                self._p(self.unpack_map), s))

    def mlp_up(self, s):
        c, ew = self.cfg, self.weights
        lib = L.lib()
        if ew.dtype == torch.uint8:
            sg, su, sd = ew.scales
            # the fp8 entry point runs quantise + gate/up + quantise + down in one call; fused: input rows gathered from
            # the receive buffer, result rows scattered into the returned layout
            w = self.world
            if self.fp8_dispatch:
                L.check(lib.moe_grouped_mlp_fp8_q_mapped(self._p(w.recv_q), self._p(w.recv_scale), c.world * w.M,
                                                         self._p(self.row_map), self._p(self.expert_cnt), self.S, c.hidden, c.ffn,
                                                         c.e_local, self._p(ew.w1), self._p(sg), self._p(su), self._p(ew.w2),
                                                         self._p(sd), self._p(self.xs), self._p(self.hq), self._p(self.hsc),
                                                         self._p(self.row_gate) if self.gated else None, self._p(self.ret),
                                                         c.world * w.M, self._p(self.row_map),
                                                         self._p(self.part_ws), self.part_ws_bytes, s))
                return
            src, n_src, a_map = (w.recv, c.world * w.M, self.row_map) if self.fused else (self.rows, self.S, None)
            dst, n_dst, c_map = (self.ret, c.world * w.M, self.row_map) if self.fused else (self.y, self.S, None)
            if self.padding_free:
                src, n_src, dst, n_dst = self.recv_flat, self.S, self.ret_flat, self.S
            L.check(lib.moe_grouped_mlp_fp8_mapped(self._p(src), n_src, self._p(a_map), self._p(self.expert_cnt), self.S, c.hidden,
                                                   c.ffn, c.e_local, self._p(ew.w1), self._p(sg), self._p(su), self._p(ew.w2),
                                                   self._p(sd), self._p(self.xq), self._p(self.xs), self._p(self.hq),
                                                   self._p(self.hsc), self._p(self.row_gate) if self.gated else None,
                                                   self._p(dst), n_dst, self._p(c_map),
                                                   self._p(self.part_ws), self.part_ws_bytes, s))
        elif ew.dtype == torch.float32:
            L.check(lib.moe_grouped_mlp(self._p(self.rows), self._p(self.expert_cnt), self.code, self.S, c.hidden, c.ffn,
                                        c.e_local, L.ACT[ew.act], self._p(ew.w1), self._p(ew.w_up), self._p(ew.w2),
                                        self._p(self.hidden), self._p(self.y), s))
        elif self.fused:
            w = self.world
            src, n_src = (self.recv_flat, self.S) if self.padding_free else (w.recv, c.world * w.M)
            L.check(lib.moe_grouped_gemm_mapped(self._p(src), n_src, self._p(self.row_map), self._p(ew.w1),
                                                self._p(self.expert_cnt), self.S, c.hidden, c.ffn, c.e_local, L.ACT[ew.act],
                                                self._p(self.hidden), self.S, None, self._p(self.part_ws), self.part_ws_bytes, s))
        else:
            L.check(lib.moe_grouped_gemm_mapped(self._p(self.rows), self.S, None, self._p(ew.w1), self._p(self.expert_cnt),
                                                self.S, c.hidden, c.ffn, c.e_local, L.ACT[ew.act], self._p(self.hidden),
                                                self.S, None, self._p(self.part_ws), self.part_ws_bytes, s))

    def mlp_down(self, s):
        c, ew = self.cfg, self.weights
        if ew.dtype == torch.bfloat16 and self.gated:
            w = self.world
            L.check(L.lib().moe_grouped_gemm_mapped_gated(self._p(self.hidden), self.S, None, self._p(ew.w2), self._p(self.expert_cnt),
                                                          self.S, c.ffn, c.hidden, c.e_local, self._p(self.row_gate),
                                                          self._p(self.ret), c.world * w.M, self._p(self.row_map),
                                                          self._p(self.part_ws), self.part_ws_bytes, s))
        elif ew.dtype == torch.bfloat16 and self.fused:
            w = self.world
            dst, n_dst = (self.ret_flat, self.S) if self.padding_free else (self.ret, c.world * w.M)
            L.check(L.lib().moe_grouped_gemm_mapped(self._p(self.hidden), self.S, None, self._p(ew.w2), self._p(self.expert_cnt),
                                                    self.S, c.ffn, c.hidden, c.e_local, 0, self._p(dst), n_dst,
                                                    self._p(self.row_map), self._p(self.part_ws), self.part_ws_bytes, s))
        elif ew.dtype == torch.bfloat16:
            L.check(L.lib().moe_grouped_gemm_mapped(self._p(self.hidden), self.S, None, self._p(ew.w2), self._p(self.expert_cnt),
                                                    self.S, c.ffn, c.hidden, c.e_local, 0, self._p(self.y), self.S, None,
                                                    self._p(self.part_ws), self.part_ws_bytes, s))

    def return_pack(self, s):
        c, w = self.cfg, self.world
        if self.padding_free:
            return  # (a flat returned payload has no padding rows)
        if self.fused:
            L.check(L.lib().moe_zero_padding_rows(self._p(self.ret), self.code, c.world, w.M, c.hidden, self._p(w.recv_counts),
                                                  c.e_local, s))
            return
        L.check(L.lib().moe_return_pack(self._p(self.y), self.code, self.S, c.hidden, self._p(w.recv_counts), c.world,
                                        c.e_local, w.M, self._p(self.ret), self._p(self.ret_map), s))

    def combine(self, s):
        c, w = self.cfg, self.world
        if self.padding_free:
            # the returned payload is indexed by position: one "destination" that holds all experts, offset 0
            L.check(L.lib().moe_combine(self._p(self.returned), self.code, 1, c.tokens * c.topk, c.hidden, self._p(self.idx),
                                        self._p(self.pos), self._p(self.gate), self._p(self.zero_off), c.tokens, c.topk,
                                        c.experts, self._p(self.out), self._p(self.status), s))
            return
        L.check(L.lib().moe_combine(self._p(self.returned), self.code, c.world, w.M, c.hidden, self._p(self.idx),
                                    self._p(self.pos), None if self.gated else self._p(self.gate), self._p(self.dst_offsets),
                                    c.tokens, c.topk, c.e_local, self._p(self.out), self._p(self.status), s))

    def step(self, events: Optional[List[Dict[str, tuple]]] = None):
        """One pass of the hot path.  With ``events`` (a list), per-stage (start, end) torch.cuda.Event
        pairs of this step are appended to it."""
        s = L.stream_ptr()
        rec = {} if events is not None else None
        for name in STAGES:
            if rec is not None:
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
            getattr(self, name)(s)
            if rec is not None:
                b.record()
                rec[name] = (a, b)
        if events is not None:
            events.append(rec)

    def capture(self):
        """The whole step as one HIP graph (every stage only enqueues kernels: no allocation, no memset,
        no synchronisation, so the capture is a plain kernel chain).  Returns a torch.cuda.CUDAGraph whose
        replay() runs one step on the capturing stream's successor."""
        self.step()  # warm every kernel before capture
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self.step()
        return g

    # ---- algorithmic work per stage (bytes for the HBM-bound ones, flops for the GEMMs) ---------
    def work(self) -> Dict[str, dict]:
        c, w = self.cfg, self.world
        T, H, E, k, W, F = c.tokens, c.hidden, c.experts, c.topk, c.world, c.ffn
        B = 4 if c.dtype == "f32" else 2
        S, M = self.S, w.M
        up_mats = 2 if c.act == "swiglu" else 1
        if self.weights.dtype != torch.bfloat16:
            # fp8 and fp32 run both GEMMs (and the fp8 quantisation passes) inside one entry point
            mlp = {"mlp_up": dict(bound="mfma", amount=2 * S * H * F * (up_mats + 1))}
        else:
            mlp = {"mlp_up": dict(bound="mfma", amount=2 * S * H * F * up_mats),
                   "mlp_down": dict(bound="mfma", amount=2 * S * F * H)}
        if self.fused:
            # the row copies are gone: what is left of the two stages is the row map and the padding rows
            unpack = dict(bound="latency", amount=S * 4 + W * c.e_local * 4)
            ret = dict(bound="latency", amount=0 if self.padding_free else max(W * M - S, 0) * H * B)
        else:
            unpack = dict(bound="hbm", amount=2 * S * H * B)
            ret = dict(bound="hbm", amount=S * H * B + W * M * H * B)
        return {
            # (the logits are also 2 T H E fp32 flops on the matrix cores: with many experts that rate, not the memory, binds)
            "route": dict(bound="hbm", amount=T * H * B + H * E * B + T * k * 8, flops=2 * T * H * E),
            "pack": dict(bound="hbm", amount=T * H * B + W * M * (H + 4) if self.fp8_dispatch else
                         (T * H * B + T * k * H * B if self.padding_free else T * H * B + W * M * H * B)),
            "unpack": unpack,
            **mlp,
            "return_pack": ret,
            "combine": dict(bound="hbm", amount=T * k * H * B + T * H * B + T * k * 8),
        }
