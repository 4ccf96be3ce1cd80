"""Pins the oracle's integer/layout functions (a2-a10, a13) against a literal pure-Python restatement
of the reference's bucket loop (utils.py:204-246), brute force, round trips and the reference's own
uniform placement pattern (unit_tests.py:137-150,211-218).  CPU only."""
import numpy as np
import pytest

from helpers import O


def reference_bucket_loop(x, top_idxs, world_size, num_experts_total):
    """The reference's host algorithm, line by line (utils.py:204-246), on numpy arrays."""
    e_local = num_experts_total // world_size
    buckets = [[[] for _ in range(e_local)] for _ in range(world_size)]
    for ti in range(x.shape[0]):
        for kk in range(top_idxs.shape[1]):
            ex = int(top_idxs[ti, kk])
            dst = ex // e_local
            el = ex - dst * e_local
            buckets[dst][el].append(x[ti])
    send_counts = np.zeros((world_size, e_local), np.int32)
    chunks, dst_offsets, dst_sizes, running = [], np.zeros(world_size, np.int32), np.zeros(world_size, np.int32), 0
    for dst in range(world_size):
        dst_offsets[dst] = running
        rows = 0
        for el in range(e_local):
            n = len(buckets[dst][el])
            send_counts[dst, el] = n
            if n:
                chunks.append(np.stack(buckets[dst][el]))
            rows += n
        dst_sizes[dst] = rows
        running += rows
    payload = np.concatenate(chunks) if running else np.empty((0, x.shape[1]), x.dtype)
    return payload, send_counts, dst_offsets, dst_sizes


def coded_rows(T, H):
    """x[t,h] = t*H + h in fp32: every row identifiable (the reference's bf16 codes collide)."""
    return (np.arange(T)[:, None] * H + np.arange(H)[None, :]).astype(np.float32)


@pytest.mark.parametrize("T,E,k,W,seed", [(37, 8, 2, 4, 0), (64, 16, 1, 8, 1), (50, 12, 4, 3, 2), (9, 6, 6, 2, 3),
                                          (0, 8, 2, 4, 4)])
def test_counts_offsets_payload_against_bucket_loop(T, E, k, W, seed):
    rng = np.random.default_rng(seed)
    H = 5
    x = coded_rows(T, H)
    idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32) if T else np.zeros((0, k), np.int32)
    payload, counts, offs, sizes = reference_bucket_loop(x, idx, W, E)
    o_counts = O.send_counts(idx, W, E)
    o_sizes, o_offs = O.dst_sizes_offsets(o_counts)
    pos, row_token = O.payload_positions(idx, E)
    assert np.array_equal(o_counts, counts) and o_counts.dtype == np.int32
    assert np.array_equal(o_sizes, sizes) and np.array_equal(o_offs, offs)
    assert np.array_equal(O.send_payload(x, row_token), payload)
    lp, lc, lo, ls = O.bucket_loop_pack(x, idx, W, E)  # the per-slot loop the benchmark times for the record
    assert np.array_equal(lp, payload) and np.array_equal(lc, counts) and np.array_equal(lo, offs) and np.array_equal(ls, sizes)
    # brute-force count cube and invariants
    cube = np.zeros(E, np.int64)
    np.add.at(cube, idx.reshape(-1), 1)
    assert np.array_equal(cube.reshape(W, E // W), counts)
    assert counts.sum() == T * k and (o_offs[-1] + o_sizes[-1] == T * k)
    eo = O.build_expert_offsets(counts)
    for d in range(W):
        for e in range(E // W):
            assert eo[d, e] == counts[d, :e].sum()
    # pos is the inverse of row_token and points at the token's own row
    for t in range(T):
        for kk in range(k):
            assert row_token[pos[t, kk]] == t
    # capacities, floor of 1 (utils.py:121)
    assert O.compute_capacity_from_pca(counts) == max(1, counts.max(initial=0))
    assert O.pair_capacity(sizes) == max(1, sizes.max(initial=0))


def test_route_and_pack_padding_free_end_to_end():
    rng = np.random.default_rng(5)
    T, H, E, k, W = 70, 32, 8, 2, 4
    x = rng.standard_normal((T, H)).astype(np.float32)
    w = rng.standard_normal((H, E)).astype(np.float32)
    payload, counts, offs, sizes = O.route_and_pack_padding_free(x, w, k, W, E)
    idx = O.route(x, w, k)[0]
    p2, c2, o2, s2 = reference_bucket_loop(x, idx, W, E)
    assert np.array_equal(payload, p2) and np.array_equal(counts, c2) and np.array_equal(offs, o2) and np.array_equal(sizes, s2)
    with pytest.raises(AssertionError):
        O.send_counts(idx, 3, E)  # utils.py:197


def test_fixed_m_layout_and_receive_side_round_trip():
    rng = np.random.default_rng(6)
    W, E_l, T, k, H = 4, 3, 45, 3, 6
    E = W * E_l
    xs = [coded_rows(T, H) + s * 10000 for s in range(W)]
    routes = []
    for s in range(W):
        idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        counts = O.send_counts(idx, W, E)
        sizes, offs = O.dst_sizes_offsets(counts)
        pos, rt = O.payload_positions(idx, E)
        routes.append(dict(idx=idx, counts=counts, sizes=sizes, offs=offs, pos=pos, rt=rt))
    M = O.pair_capacity(np.stack([r["sizes"] for r in routes]))
    CAP = max(O.compute_capacity_from_pca(r["counts"]) for r in routes)
    sends = [O.pack_fixed_m(O.send_payload(x, r["rt"]), r["offs"], r["sizes"], M) for x, r in zip(xs, routes)]
    for s, (send, r) in enumerate(zip(sends, routes)):
        assert send.shape == (W, M, H)
        for d in range(W):
            n = r["sizes"][d]
            assert (send[d, n:] == 0).all()  # padding rows are all-zero
            # rows of dst d are the stable sort by local expert of the tokens routed there
            want = [xs[s][t] for el in range(E_l) for t in range(T) if (r["idx"][t] == d * E_l + el).any()]
            assert np.array_equal(send[d, :n], np.stack(want) if want else np.empty((0, H), np.float32))
    with pytest.raises(ValueError):
        O.pack_fixed_m(O.send_payload(xs[0], routes[0]["rt"]), routes[0]["offs"], routes[0]["sizes"], M - 1 if
                       routes[0]["sizes"].max() == M else routes[0]["sizes"].max() - 1)
    for d in range(W):
        recv = np.stack([sends[s][d] for s in range(W)])
        rc = np.stack([routes[s]["counts"][d] for s in range(W)])
        tb, pca = O.recv_to_token_buf(recv, rc, CAP)
        assert np.array_equal(pca, rc.T)
        # same placement as the reference's reorder loop fed with the padding-free concatenation
        flat = np.concatenate([recv[s, :rc[s].sum()] for s in range(W)])
        tb2 = O.reorder_flat_to_token_buf(flat, rc, CAP, np.full((E_l, W, CAP, H), 9.0, np.float32))
        assert np.array_equal(tb, tb2)
        sh = O.shuffle(tb, pca)
        assert np.array_equal(sh, O.unpack_expert_major(recv, rc))
        # every routed row arrives exactly once, grouped by expert, in (src, token) order
        want = [xs[s][t] for el in range(E_l) for s in range(W) for t in range(T)
                if (routes[s]["idx"][t] == d * E_l + el).any()]
        assert np.array_equal(sh, np.stack(want))
        assert np.array_equal(O.expert_row_counts(pca), [sum((routes[s]["idx"] == d * E_l + el).sum() for s in range(W))
                                                         for el in range(E_l)])
        # return path inverts the unpack exactly
        assert np.array_equal(O.return_pack(sh, rc, M), recv)


def test_reorder_error_cases():
    rc = np.array([[2, 1], [0, 3]], np.int32)
    flat = np.zeros((6, 4), np.float32)
    with pytest.raises(ValueError):
        O.reorder_flat_to_token_buf(flat, rc, 3, np.zeros((2, 2, 4, 4), np.float32))  # wrong shape (baseline.py:199-201)
    with pytest.raises(ValueError):
        O.reorder_flat_to_token_buf(flat, rc, 2, np.zeros((2, 2, 2, 4), np.float32))  # count > capacity (:215-216)
    with pytest.raises(RuntimeError):
        O.reorder_flat_to_token_buf(np.zeros((7, 4), np.float32), rc, 3, np.zeros((2, 2, 3, 4), np.float32))  # rows consumed (:220-221)


def test_uniform_pattern_of_the_reference_unit_test():
    # every src sends exactly cap rows to every (dst, expert): dst_offsets = arange(W)*E_l*cap (unit_tests.py:138-139)
    W, E_l, cap, H = 8, 2, 32, 4
    counts = np.full((W, E_l), cap, np.int32)
    sizes, offs = O.dst_sizes_offsets(counts)
    assert np.array_equal(offs, np.arange(W) * E_l * cap) and (sizes == E_l * cap).all()
    assert np.array_equal(O.build_expert_offsets(counts), np.tile(np.arange(E_l) * cap, (W, 1)))
    rank = 5
    payloads = [(s * 1_000_000 + np.arange(W * E_l * cap))[:, None].repeat(H, 1).astype(np.float32) for s in range(W)]
    flat = np.concatenate([p[offs[rank]:offs[rank] + sizes[rank]] for p in payloads])
    tb = O.reorder_flat_to_token_buf(flat, counts, cap, np.empty((E_l, W, cap, H), np.float32))
    for e in range(E_l):
        for s in range(W):
            start = offs[rank] + e * cap
            assert np.array_equal(tb[e, s], payloads[s][start:start + cap])  # unit_tests.py:211-218


def test_combine_closed_forms():
    rng = np.random.default_rng(8)
    T, H, E, k, W = 30, 8, 8, 3, 4
    E_l = E // W
    x = O.bf16_round(rng.standard_normal((T, H)).astype(np.float32))
    w = rng.standard_normal((H, E)).astype(np.float32)
    idx, gate, _ = O.route(x, w, k)
    counts = O.send_counts(idx, W, E)
    sizes, offs = O.dst_sizes_offsets(counts)
    pos, rt = O.payload_positions(idx, E)
    M = O.pair_capacity(sizes)
    send = O.pack_fixed_m(O.send_payload(x, rt), offs, sizes, M)
    # identity experts: out[t] = (sum_kk gate) * x[t]
    out = O.combine(send, idx, pos, gate, offs, E_l, "f32")
    np.testing.assert_allclose(out, gate.sum(1, keepdims=True) * x, rtol=1e-6, atol=1e-7)
    # brute force per token
    for t in range(T):
        acc = np.zeros(H, np.float32)
        for kk in range(k):
            d = idx[t, kk] // E_l
            acc = acc + gate[t, kk] * send[d, pos[t, kk] - offs[d]]
        assert np.array_equal(O.combine(send, idx, pos, gate, offs, E_l, "bf16")[t], O.bf16_round(acc))


def test_oracle_reproduces_the_frozen_dispatch_vectors():
    """tests/golden/dispatch_small.npz freezes every intermediate of the dispatch path on a tiny seeded case;
    regenerating it from the oracle must give the same bits (a change of the oracle shows up here first)."""
    import importlib.util
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(here, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    frozen = np.load(os.path.join(here, "dispatch_small.npz"))
    fresh = mod.build()
    assert sorted(frozen.keys()) == sorted(fresh.keys())
    for k in frozen.keys():
        a, b = np.asarray(frozen[k]), np.asarray(fresh[k])
        assert a.dtype == b.dtype and a.shape == b.shape, k
        assert np.array_equal(a.view(np.uint8) if a.dtype.kind == "f" and a.ndim else a,
                              b.view(np.uint8) if b.dtype.kind == "f" and b.ndim else b), f"{k} drifted"
    # a few facts that must hold for the vectors to mean anything
    assert int(frozen["M"]) == max(int(frozen[f"counts{s}"].sum(1).max()) for s in range(3))
    assert int(frozen["recv_counts"].sum()) == frozen["rows"].shape[0] and (frozen["pca"] == frozen["recv_counts"].T).all()


def test_capacity_overflow_drops_the_same_rows_everywhere():
    """With M below the largest pair size the pack drops the rows at and past M of a slot; the receive side then
    sees zero rows where they were counted, the way back has no slot for them, and the combine skips them.
    Pinned per element against the definition (a routed slot survives iff its row inside the slot is < M)."""
    rng = np.random.default_rng(11)
    T, H, E, k, W = 40, 4, 6, 2, 3
    E_l = E // W
    xs = [coded_rows(T, H) + 1000.0 * s for s in range(W)]
    idxs = [np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32) for _ in range(W)]
    parts = []
    for x, idx in zip(xs, idxs):
        counts = O.send_counts(idx, W, E)
        sizes, offs = O.dst_sizes_offsets(counts)
        pos, row_token = O.payload_positions(idx, E)
        parts.append(dict(counts=counts, sizes=sizes, offs=offs, pos=pos, row_token=row_token))
    M_full = O.pair_capacity(np.stack([p["sizes"] for p in parts]))
    M = M_full - 6
    assert any((p["sizes"] > M).any() for p in parts)
    with pytest.raises(ValueError):
        O.pack_fixed_m(O.send_payload(xs[0], parts[0]["row_token"]), parts[0]["offs"], parts[0]["sizes"], M)
    sends = [O.pack_fixed_m(O.send_payload(x, p["row_token"]), p["offs"], p["sizes"], M, drop=True) for x, p in zip(xs, parts)]
    # the pack, per element
    for x, idx, p, send in zip(xs, idxs, parts, sends):
        seen = np.zeros((W, M), bool)
        for t in range(T):
            for kk in range(k):
                d = idx[t, kk] // E_l
                m = p["pos"][t, kk] - p["offs"][d]
                if m < M:
                    assert np.array_equal(send[d, m], x[t])
                    seen[d, m] = True
        assert (send[~seen] == 0).all()
    # the receive side of rank 0
    recv = np.stack([s[0] for s in sends])
    rc = np.stack([p["counts"][0] for p in parts]).astype(np.int32)
    rows = O.unpack_expert_major(recv, rc)
    assert rows.shape[0] == rc.sum()
    eo = O.build_expert_offsets(rc)
    r = 0
    n_dropped = 0
    for e in range(E_l):
        for s in range(W):
            for j in range(rc[s, e]):
                m = eo[s, e] + j
                if m < M:
                    assert np.array_equal(rows[r], recv[s, m])
                else:
                    assert (rows[r] == 0).all()
                    n_dropped += 1
                r += 1
    assert n_dropped > 0
    CAP = int(rc.max())
    tb, _ = O.recv_to_token_buf(recv, rc, CAP)
    assert np.array_equal(O.shuffle(tb, rc.T), rows)
    # the way back: the surviving rows return to their slots, the dropped ones have none
    back = O.return_pack(rows * 2, rc, M)
    assert np.array_equal(back, recv * 2)
    # combine on shard 0: dropped slots contribute nothing
    p0, gate = parts[0], rng.random((T, k)).astype(np.float32)
    out = O.combine(sends[0], idxs[0], p0["pos"], gate, p0["offs"], E_l, "f32")
    for t in range(T):
        acc = np.zeros(H, np.float32)
        for kk in range(k):
            d = idxs[0][t, kk] // E_l
            m = p0["pos"][t, kk] - p0["offs"][d]
            if m < M:
                acc = (acc + gate[t, kk] * xs[0][t]).astype(np.float32)
        assert np.array_equal(out[t], acc)


def test_quantising_rows_commutes_with_packing_them():
    """pack_fixed_m_fp8 (tokens quantised to fp8 where they are packed) against the other order: quantise every token row
    first -- with torch's own e4m3 cast, as test_oracle_expert pins quantize_rows_fp8 -- then move the codes and the
    scales as payload.  Padding slots are all-zero rows: codes 0, scale 1.  Includes an all-zero token."""
    import torch
    rng = np.random.default_rng(8)
    T, H, E, k, W = 70, 48, 12, 3, 4
    x = O.bf16_round((rng.standard_normal((T, H)) * rng.uniform(0.1, 4.0, (T, 1))).astype(np.float32))
    x[5] = 0.0
    idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    counts = O.send_counts(idx, W, E)
    sizes, offs = O.dst_sizes_offsets(counts)
    pos, row_token = O.payload_positions(idx, E)
    M = O.pair_capacity(sizes) + 3
    q, sc = O.pack_fixed_m_fp8(O.send_payload(x, row_token), offs, sizes, M)
    # the other order, with torch's cast
    xt = torch.from_numpy(x)
    amax = xt.abs().amax(dim=1)
    zero = amax == 0
    safe = torch.where(zero, torch.ones_like(amax), amax)
    scale_t = torch.where(zero, torch.ones_like(amax), safe / 448.0).numpy()
    codes_t = (xt * torch.where(zero, torch.ones_like(amax), 448.0 / safe)[:, None]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    want_q = np.zeros((W, M, H), np.uint8)
    want_s = np.ones((W, M), np.float32)
    for t in range(T):
        for j in range(k):
            d = idx[t, j] // (E // W)
            m = pos[t, j] - offs[d]
            want_q[d, m], want_s[d, m] = codes_t[t], scale_t[t]
    assert np.array_equal(q, want_q) and np.array_equal(sc, want_s)
    assert (sc[0, sizes[0]:] == 1.0).all() and (q[0, sizes[0]:] == 0).all()


def _routed(rng, T, H, E, k, W):
    x = (rng.standard_normal((T, H)) * 4).round().astype(np.float32)
    idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    counts = O.send_counts(idx, W, E)
    sizes, offs = O.dst_sizes_offsets(counts)
    pos, row_token = O.payload_positions(idx, E)
    return x, idx, counts, sizes, offs, pos, row_token


def test_flat_receive_row_map_against_the_reference_reorder():
    """A padding-free receive payload (every source's send_payload block for this rank, concatenated in source order,
    utils.py:235-246) read through flat_recv_row_map gives the expert-major rows that the reference's own route gives:
    reorder_flat_to_token_buf (baseline.py:204-218) followed by the token shuffle; and the same rows as the fixed-M
    route (unpack_expert_major of the [W,M,H] buffer)."""
    rng = np.random.default_rng(21)
    T, H, E, k, W = 60, 8, 12, 3, 4
    E_l, dst = E // W, 1
    flats, slots, rcs = [], [], []
    parts = [_routed(rng, T, H, E, k, W) for _ in range(W)]
    M = O.pair_capacity(np.stack([p[3] for p in parts]))
    for s, (x, idx, counts, sizes, offs, pos, row_token) in enumerate(parts):
        x += 1000.0 * s  # rows of different sources differ
        payload = O.send_payload(x, row_token)
        flats.append(payload[offs[dst]:offs[dst] + sizes[dst]])
        slots.append(O.pack_fixed_m(payload, offs, sizes, M)[dst])
        rcs.append(counts[dst])
    flat, recv, rc = np.concatenate(flats), np.stack(slots), np.stack(rcs).astype(np.int32)
    rm = O.flat_recv_row_map(rc)
    assert rm.shape == (int(rc.sum()),) and sorted(rm.tolist()) == list(range(int(rc.sum())))  # a permutation
    CAP = int(rc.max())
    tb = O.reorder_flat_to_token_buf(flat, rc, CAP, np.empty((E_l, W, CAP, H), np.float32))
    assert np.array_equal(flat[rm], O.shuffle(tb, rc.T))
    assert np.array_equal(flat[rm], O.unpack_expert_major(recv, rc))
    # brute force: row (e, s, j) of the expert-major order sits at (rows of earlier sources) + (rows of s for earlier experts) + j
    r = 0
    for e in range(E_l):
        for s in range(W):
            for j in range(rc[s, e]):
                assert rm[r] == rc[:s].sum() + rc[s, :e].sum() + j
                r += 1


def test_gates_shipped_with_the_rows():
    """pack_gates puts a slot's gate where pack_fixed_m puts its row: packing a one-column payload of gates (in payload
    order) gives the same [W,M] array; padding slots hold zero; slots past an undersized M are dropped with their rows."""
    rng = np.random.default_rng(22)
    T, H, E, k, W = 50, 4, 8, 2, 4
    x, idx, counts, sizes, offs, pos, row_token = _routed(rng, T, H, E, k, W)
    gate = rng.random((T, k)).astype(np.float32) + 0.25
    g_payload = np.zeros((T * k, 1), np.float32)
    g_payload[pos.reshape(-1), 0] = gate.reshape(-1)
    for M in (O.pair_capacity(sizes) + 2, O.pair_capacity(sizes) - 3):
        sg = O.pack_gates(gate, idx, pos, offs, E // W, W, M)
        assert np.array_equal(sg, O.pack_fixed_m(g_payload, offs, sizes, M, drop=True)[:, :, 0])
        for d in range(W):
            assert (sg[d, min(sizes[d], M):] == 0).all() and (sg[d, :min(sizes[d], M)] > 0).all()


def test_pre_weighted_combine():
    """Gates applied at the destination instead of the source.  In fp32 nothing is rounded between the expert output and
    the combine, so both orders give the same bits: combine(pre_weighted) of rows multiplied by their gates ==
    combine(gate) of the plain rows.  In bf16 the weighted rows are rounded once (round(fp32 * gate), pinned against
    torch's bf16 cast) and the combine only adds: against a per-token evaluation."""
    import torch
    rng = np.random.default_rng(23)
    T, H, E, k, W = 40, 16, 8, 3, 4
    E_l = E // W
    x, idx, counts, sizes, offs, pos, row_token = _routed(rng, T, H, E, k, W)
    x = rng.standard_normal((T, H)).astype(np.float32)
    gate = rng.random((T, k)).astype(np.float32)
    M = O.pair_capacity(sizes) + 1
    send = O.pack_fixed_m(O.send_payload(x, row_token), offs, sizes, M)
    sg = O.pack_gates(gate, idx, pos, offs, E_l, W, M)
    # identity experts: the destination returns round(row * gate)
    cnt_all = np.array([W * M], np.int32)
    eye = np.eye(H, dtype=np.float32)[None]
    w32 = O.grouped_gemm(send.reshape(W * M, H), eye, cnt_all, "f32", row_gate=sg.reshape(-1)).reshape(W, M, H)
    assert np.array_equal(w32, (send * sg[:, :, None]).astype(np.float32))
    a = O.combine(w32, idx, pos, gate, offs, E_l, "f32", pre_weighted=True)
    b = O.combine(send, idx, pos, gate, offs, E_l, "f32")
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    # bf16
    xb = O.bf16_round(x)
    sendb = O.pack_fixed_m(O.send_payload(xb, row_token), offs, sizes, M)
    wb = O.grouped_gemm(sendb.reshape(W * M, H), eye, cnt_all, "bf16", row_gate=sg.reshape(-1)).reshape(W, M, H)
    want_rows = torch.from_numpy((sendb * sg[:, :, None]).astype(np.float32)).bfloat16().float().numpy()
    assert np.array_equal(wb, want_rows)
    out = O.combine(wb, idx, pos, None, offs, E_l, "bf16", pre_weighted=True)
    for t in range(T):
        acc = np.zeros(H, np.float32)
        for kk in range(k):
            acc = (acc + torch.from_numpy((gate[t, kk] * xb[t]).astype(np.float32)).bfloat16().float().numpy()).astype(np.float32)
        assert np.array_equal(out[t], torch.from_numpy(acc).bfloat16().float().numpy())
    # the MLP form: expert_mlp(row_gate) is round(fp32 result * gate), i.e. within one bf16 step of gate * round(result)
    cnt = np.array([30, 10], np.int32)
    rows = O.bf16_round(rng.standard_normal((40, H)).astype(np.float32))
    w1 = O.bf16_round(rng.standard_normal((2, H, 32)).astype(np.float32) * 0.25)
    w2 = O.bf16_round(rng.standard_normal((2, 32, H)).astype(np.float32) * 0.2)
    g = rng.random(40).astype(np.float32)
    yw = O.expert_mlp(rows, cnt, w1, w2, "silu", "bf16", row_gate=g)
    y = O.expert_mlp(rows, cnt, w1, w2, "silu", "bf16")
    assert np.abs(yw - g[:, None] * y).max() <= 2.0 ** -7 * np.abs(y).max()
    assert not np.array_equal(yw, O.bf16_round(g[:, None] * y))  # (the rounding order is a different one)
