"""The two wider forms of the copy-free destination side, through the C ABI, against the oracle:
  * gated return -- the top-k gates travel with the rows, the down projection multiplies every result row by its gate
    before the one rounding, the combine only adds (oracle: pack_gates, expert_mlp(row_gate), combine(pre_weighted));
  * padding-free payload -- the rows cross as the reference's send_payload blocks (utils.py:235-246), the GEMMs gather from
    and scatter into flat buffers through flat_recv_row_map, the combine reads the returned payload by position;
    results bit-equal to the fixed-M route."""
import numpy as np
import pytest
import torch

from helpers import O, assert_bits_equal, err_stats, oracle_recv, oracle_world, to_np

pytestmark = pytest.mark.gpu

from iris_testing_amd import harness, ops  # noqa: E402
from iris_testing_amd.configs import CONFIGS, gen_shard_tokens  # noqa: E402
from iris_testing_amd.pipeline import DispatchPipeline  # noqa: E402

DEV = "cuda"


def _shrunk(name, tokens):
    from dataclasses import replace
    cfg = CONFIGS[name]
    return cfg if tokens is None else replace(cfg, tokens=tokens)


@pytest.mark.parametrize("name,tokens", [("small", None), ("mixtral", 2048), ("finegrained", 512), ("zipf_k4", 1024)])
def test_gated_return_against_oracle(name, tokens):
    cfg = _shrunk(name, tokens)
    print(f"case {cfg}", flush=True)
    W, E_l, k, H = cfg.world, cfg.e_local, cfg.topk, cfg.hidden
    world = harness.build_world(cfg, DEV)
    M, S = world.M, world.S
    ew, raw, qs = harness.expert_weights(cfg, 0, DEV)
    recv_gate = harness.recv_gates(world)
    pipe = DispatchPipeline(world, ew, gated=True, recv_gate=recv_gate)
    pipe.step()
    torch.cuda.synchronize()
    assert int(pipe.status.item()) == 0
    # oracle view of all shards
    xs = [to_np(gen_shard_tokens(cfg, s)) for s in range(W)]
    bias = None if world.bias is None else to_np(world.bias)
    shards, oM, _ = oracle_world(cfg, xs, to_np(world.router), bias)
    assert oM == M
    s0 = shards[0]
    # source side: the same send buffer as without gates, and the gates in their slots
    o_send = O.pack_fixed_m(O.send_payload(xs[0], s0["row_token"]), s0["offs"], s0["sizes"], M)
    if pipe.fp8_dispatch:
        o_q, o_sc = O.pack_fixed_m_fp8(O.send_payload(xs[0], s0["row_token"]), s0["offs"], s0["sizes"], M)
        assert_bits_equal(pipe.send_q, o_q, "send codes")
        assert_bits_equal(pipe.send_scale, o_sc, "send scales")
    else:
        assert_bits_equal(pipe.send, o_send, "send")
    assert_bits_equal(pipe.send_gate, O.pack_gates(to_np(pipe.gate), s0["idx"], s0["pos"], s0["offs"], E_l, W, M), "send_gate")
    # what arrives at rank 0: source s's gates for destination 0 (the harness assembled them with the same kernel)
    o_rg = np.stack([O.pack_gates(sh["gate"], sh["idx"], sh["pos"], sh["offs"], E_l, W, M)[0] for sh in shards])
    np.testing.assert_allclose(to_np(recv_gate), o_rg, rtol=1e-5, atol=0)  # (gates: expf differs in the last bits)
    # destination side
    o_recv, o_rc = oracle_recv(cfg, xs, shards, M, 0)
    o_map = to_np(pipe.row_map)[:S]
    g_rows = to_np(recv_gate).reshape(-1)[o_map]
    assert_bits_equal(pipe.row_gate[:S], g_rows, "row gates in the GEMM's row order")
    rows = O.unpack_expert_major(o_recv, o_rc)
    cnt = O.expert_row_counts(o_rc.T)
    f = to_np
    if cfg.quant == "fp8":
        # the down projection on the GPU's own block-quantised hidden activation (the first GEMM is held to the oracle elsewhere)
        (_, _), (_, _), (dq, ds) = [(f(q), f(s_)) for q, s_ in qs]
        y = O.expert_down_fp8(f(pipe.hq), f(pipe.hsc), cnt, dq, ds, row_gate=g_rows)
    elif cfg.act == "swiglu":
        y = O.expert_mlp(rows, cnt, f(raw[0]), f(raw[2]), "swiglu", cfg.dtype, w_up=f(raw[1]), row_gate=g_rows)
    else:
        y = O.expert_mlp(rows, cnt, f(raw[0]), f(raw[1]), cfg.act, cfg.dtype, row_gate=g_rows)
    want_ret = O.return_pack(y, o_rc, M)
    got_ret = to_np(pipe.ret)
    mx, mx_rms, _ = err_stats(got_ret, want_ret)
    print(f"{name}: weighted return buffer max-abs {mx:.3e} ({mx_rms:.3e} of rms)", flush=True)
    assert mx <= 2.0 ** -7 * float(np.abs(want_ret).max()) + 1e-6
    valid = np.arange(M)[None, :] < o_rc.sum(1)[:, None]
    assert (np.abs(got_ret).sum(-1)[~valid] == 0).all(), "padding rows of the return buffer must be zero"
    # the combine only adds: bit-exact against the oracle on an arbitrary returned buffer, gates ignored
    rng = np.random.default_rng(3)
    returned = O.bf16_round(rng.standard_normal((W, M, H)).astype(np.float32))
    pipe.returned.copy_(torch.from_numpy(returned).to(cfg.torch_dtype))
    pipe.combine(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert_bits_equal(pipe.out, O.combine(returned, s0["idx"], s0["pos"], None, s0["offs"], E_l, cfg.dtype, pre_weighted=True),
                      "combine of weighted rows")
    # against the ungated pipeline: weighting at the destination instead of the source moves the result by bf16 roundings only
    plain = DispatchPipeline(world, ew)
    plain.step()
    torch.cuda.synchronize()
    gate_slots = torch.from_numpy(o_rg).to(DEV)[:, :, None]
    d = (pipe.ret.float() - plain.ret.float() * gate_slots).abs().max().item()
    assert d <= 2.0 ** -7 * plain.ret.float().abs().max().item()


@pytest.mark.parametrize("name", ["plumbing_bf16", "small"])
def test_gated_pipeline_end_to_end_matches_dense(name):
    """Every simulated rank's experts in turn, gates applied at the destinations, plain sum at the source: against the dense
    closed form  out[t] = sum_kk p[t, idx[t,kk]] * MLP_{idx[t,kk]}(x[t])."""
    from dataclasses import replace
    from iris_testing_amd.layers.expert import _part_ws
    cfg = CONFIGS["small"] if name == "small" else replace(CONFIGS["small"], tokens=300, topk=2, seed=9)
    W, E_l = cfg.world, cfg.e_local
    world, shards = harness.build_world(cfg, DEV, keep_shards=True)
    M, r0 = world.M, world.routes[0]
    returned = torch.zeros((W, M, cfg.hidden), dtype=cfg.torch_dtype, device=DEV)
    raw_weights = []
    for d in range(W):
        recv = torch.stack([harness.pack_for_dst(shards[s], world.routes[s], d, M) for s in range(W)])
        rc = torch.stack([world.routes[s].counts.send_counts[d] for s in range(W)]).contiguous()
        gates = harness.recv_gates(world, d)
        S = int(rc.sum().item())
        row_map, cnt, row_gate = ops.recv_row_map_gated(rc, M, S, gates.view(-1))
        ew, raw, _ = harness.expert_weights(cfg, d, DEV)
        raw_weights.append(raw)
        hidden = torch.empty((max(S, 1), cfg.ffn), dtype=cfg.torch_dtype, device=DEV)
        ret = torch.zeros((W * M, cfg.hidden), dtype=cfg.torch_dtype, device=DEV)
        if S:
            ops.grouped_gemm_mapped(recv.view(W * M, -1), row_map, ew.w1, cnt, S, cfg.ffn, ew.act, hidden, part_ws=_part_ws(DEV))
            ops.grouped_gemm_mapped_gated(hidden, None, ew.w2, cnt, S, cfg.hidden, row_gate, ret, c_row_map=row_map,
                                          part_ws=_part_ws(DEV))
        returned[d] = ret.view(W, M, -1)[0]
    out = ops.combine(returned, r0.idx, r0.counts.pos, None, r0.counts.dst_offsets, E_l)
    x = to_np(shards[0])
    o_idx, o_gate, _ = O.route(x, to_np(world.router), cfg.topk, None)
    assert_bits_equal(r0.idx, o_idx, "indices")
    want = np.zeros((cfg.tokens, cfg.hidden), dtype=np.float64)
    for ex in range(cfg.experts):
        d, el = divmod(ex, E_l)
        t_sel, k_sel = np.nonzero(o_idx == ex)
        if len(t_sel) == 0:
            continue
        w1, w2 = (to_np(w[el:el + 1]) for w in raw_weights[d])
        y = O.expert_mlp(x[t_sel], np.array([len(t_sel)]), w1, w2, cfg.act, cfg.dtype)
        want[t_sel] += o_gate[t_sel, k_sel][:, None].astype(np.float64) * y
    mx, mx_rms, rel = err_stats(to_np(out), want)
    print(f"{name}: gated end-to-end max-abs {mx:.3e}, max-abs/rms {mx_rms:.3e}", flush=True)
    assert mx_rms < 2.0 ** -6 * 4


@pytest.mark.parametrize("name,tokens", [("small", None), ("mixtral", 2048), ("finegrained", 512), ("zipf_k4", 1024)])
def test_padding_free_route_equals_fixed_m_route(name, tokens):
    cfg = _shrunk(name, tokens)
    print(f"case {cfg}", flush=True)
    W, E_l, k, H = cfg.world, cfg.e_local, cfg.topk, cfg.hidden
    world = harness.build_world(cfg, DEV)
    M, S = world.M, world.S
    ew, raw, _ = harness.expert_weights(cfg, 0, DEV)
    flat = harness.recv_flat(world)
    assert flat.shape == (S, H)
    # the flat payload and its row map against the oracle
    xs = [to_np(gen_shard_tokens(cfg, s)) for s in range(W)]
    bias = None if world.bias is None else to_np(world.bias)
    shards, _, _ = oracle_world(cfg, xs, to_np(world.router), bias)
    o_flat = np.concatenate([O.send_payload(x, sh["row_token"])[sh["offs"][0]:sh["offs"][0] + sh["sizes"][0]]
                             for x, sh in zip(xs, shards)])
    assert_bits_equal(flat, o_flat, "flat receive payload")
    o_rc = np.stack([sh["counts"][0] for sh in shards]).astype(np.int32)
    pf = DispatchPipeline(world, ew, padding_free=True, recv_flat=flat,
                          fp8_dispatch=False if ew.dtype == torch.uint8 else None)
    fm = DispatchPipeline(world, ew, fp8_dispatch=False if ew.dtype == torch.uint8 else None)
    pf.step()
    fm.step()
    torch.cuda.synchronize()
    assert_bits_equal(pf.row_map[:S], O.flat_recv_row_map(o_rc), "row map over the flat payload")
    assert torch.equal(pf.expert_cnt, fm.expert_cnt)
    # source side: the payload the reference's route_and_pack_padding_free returns
    assert_bits_equal(pf.payload, O.send_payload(xs[0], shards[0]["row_token"]), "send_payload")
    # destination side: the same expert-major rows went through the same GEMMs -> the same result rows, in flat order
    # (fixed-M: result row r sits in slot row_map_fm[r]; flat: in row row_map_pf[r])
    got = torch.empty((S, H), dtype=cfg.torch_dtype, device=DEV)
    got[:] = pf.ret_flat[pf.row_map[:S].long()]
    want = fm.ret.view(W * M, H)[fm.row_map[:S].long()]
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "padding-free and fixed-M result rows differ"
    # combine over a returned payload, by position, against the oracle (one destination holding all experts)
    rng = np.random.default_rng(5)
    returned = O.bf16_round(rng.standard_normal((cfg.tokens * k, H)).astype(np.float32))
    pf.returned.copy_(torch.from_numpy(returned).to(cfg.torch_dtype))
    pf.combine(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    s0 = shards[0]
    want_out = O.combine(returned[None], s0["idx"], s0["pos"], to_np(pf.gate), np.zeros(1, np.int32), cfg.experts, cfg.dtype)
    assert_bits_equal(pf.out, want_out, "combine over the returned payload")
    # ... which is what the fixed-M combine gives when the same rows sit in their slots
    slots = torch.zeros((W, M, H), dtype=cfg.torch_dtype, device=DEV)
    idx_t, pos_t = fm.idx.long(), fm.pos.long()
    d = idx_t // E_l
    m = pos_t - fm.dst_offsets.long()[d]
    slots[d.reshape(-1), m.reshape(-1)] = pf.returned[pos_t.reshape(-1)]
    fm.returned.copy_(slots)
    fm.combine(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(fm.out.view(torch.int16), pf.out.view(torch.int16))


def test_flat_row_map_with_empty_blocks_and_rows_past_the_total():
    rng = np.random.default_rng(6)
    W, E_l = 8, 32
    rc = rng.integers(0, 5, (W, E_l)).astype(np.int32)
    rc[rng.random((W, E_l)) < 0.5] = 0
    rc[3] = 0
    S = int(rc.sum())
    row_map, cnt = ops.recv_row_map_flat(torch.from_numpy(rc).to(DEV), S + 7)
    want = O.flat_recv_row_map(rc)
    assert_bits_equal(row_map[:S], want, "flat row map")
    assert (to_np(row_map)[S:] == 0).all()
    assert_bits_equal(cnt, rc.sum(0).astype(np.int32), "expert counts")


@pytest.mark.parametrize("name,mode", [("small", "gated"), ("small", "padding_free"), ("zipf_k1", "gated"), ("zipf_k1", "padding_free")])
def test_graph_replay_of_the_wider_forms_equals_eager(name, mode):
    """The gated and the padding-free step captured as one HIP graph: every replay (outputs cleared before it, eager work and
    synchronisation between replays) reproduces the eager step bit for bit."""
    cfg = CONFIGS[name]
    world = harness.build_world(cfg, DEV)
    ew, _, _ = harness.expert_weights(cfg, 0, DEV)
    gated, flat = mode == "gated", mode == "padding_free"
    pipe = DispatchPipeline(world, ew, gated=gated, padding_free=flat,
                            fp8_dispatch=False if flat else None,
                            recv_gate=harness.recv_gates(world) if gated else None,
                            recv_flat=harness.recv_flat(world) if flat else None)
    pipe.returned.copy_(torch.randn(pipe.returned.shape, device=DEV).to(pipe.returned.dtype))
    pipe.step()
    torch.cuda.synchronize()
    assert int(pipe.status.item()) == 0
    names = ["idx", "gate", "send_counts", "pos", "row_map", "out"] + (["ret_flat"] if flat else ["ret"]) + (["row_gate"] if gated else [])
    eager = {n: getattr(pipe, n).clone() for n in names}
    graph = pipe.capture()
    for rep in range(3):
        for n in names:
            getattr(pipe, n).zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for n in names:
            assert torch.equal(getattr(pipe, n), eager[n]), f"{mode} replay {rep}: {n} differs from the eager step"
        pipe.step()  # eager work between replays
        torch.cuda.synchronize()
