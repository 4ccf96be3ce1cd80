"""Pins the oracle's router (a1) against things the oracle did not write: torch's own softmax/topk
(the routines the reference calls, utils.py:201-202), float64 dot products, hand-built ties and
closed forms.  CPU only."""
import numpy as np
import pytest
import torch

from helpers import O


def _rand(T, H, E, seed=0, scale=1.0):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((T, H)).astype(np.float32), (rng.standard_normal((H, E)) * scale).astype(np.float32))


def test_logits_match_float64_dot():
    x, w = _rand(64, 300, 24, 1, 0.1)
    b = np.random.default_rng(2).standard_normal(24).astype(np.float32)
    lg = O.router_logits(x, w, b)
    ref = x.astype(np.float64) @ w.astype(np.float64) + b
    # an fp32 fma chain of length 300 stays within ~H * eps * sum|x w| of the exact value
    bound = 300 * 2.0 ** -24 * (np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64)) + 1e-6
    assert (np.abs(lg - ref) <= bound).all()


def _segmented_chain(x, w, t, e, fma):
    """The specified order spelled out in Python: eight contiguous segments of ceil(H/8) rounded up to a
    multiple of 8, a chain per segment from +0, the chains added in segment order."""
    H = x.shape[1]
    L = (-(-H // 8) + 7) // 8 * 8
    total = None
    for p in range(8):
        acc = np.float32(0)
        for h in range(min(p * L, H), min((p + 1) * L, H)):
            acc = fma(x[t, h], w[h, e], acc)
        total = acc if total is None else np.float32(total + acc)
    return total


@pytest.mark.parametrize("H", [37, 8, 64, 100, 130])
def test_logits_fixed_order_is_eight_fma_chains(H):
    # brute force in Python emulating fmaf: float32(x*w + acc) with the product and the sum exact in
    # float64 (operands are small integers over 4 and 8, sums stay far below 2^53) -> catches a swapped or
    # dropped term, a non-fused multiply, a wrong segment boundary or a wrong order of the final additions
    rng = np.random.default_rng(3 + H)
    x = rng.integers(-8, 9, size=(5, H)).astype(np.float32) / 4
    w = rng.integers(-8, 9, size=(H, 6)).astype(np.float32) / 8
    lg = O.router_logits(x, w)
    fma = lambda a, b, c: np.float32(np.float64(a) * np.float64(b) + np.float64(c))  # noqa: E731
    want = np.array([[_segmented_chain(x, w, t, e, fma) for e in range(6)] for t in range(5)], np.float32)
    assert np.array_equal(lg.view(np.uint32), want.view(np.uint32))


def test_segment_sums_are_added_in_segment_order_with_fp32_rounding():
    # H = 64 -> eight segments of 8.  Segment sums 2^24, 1, 1, -2^24, 0...: in fp32, in segment order,
    # ((2^24 + 1) + 1) - 2^24 = 0 (each +1 is rounded away); any other association, or a wider accumulator,
    # gives 1 or 2.  A single chain over all of H would give 0 + ... as well only by accident: it is
    # excluded by the next case, where the order inside a segment matters instead.
    x = np.zeros((1, 64), np.float32)
    w = np.ones((64, 1), np.float32)
    x[0, 0], x[0, 8], x[0, 16], x[0, 24] = 2.0 ** 24, 1.0, 1.0, -2.0 ** 24
    assert O.router_logits(x, w)[0, 0] == 0.0
    # the same four values inside ONE segment in the order 2^24, -2^24, 1, 1 give 2: chains run in ascending h
    x = np.zeros((1, 64), np.float32)
    x[0, 0], x[0, 1], x[0, 2], x[0, 3] = 2.0 ** 24, -2.0 ** 24, 1.0, 1.0
    assert O.router_logits(x, w)[0, 0] == 2.0
    # segments 1 and 2 hold 1 and 1, segment 0 holds 2^24 and segment 3 -2^24, bias 0.5 last: (0 + 0.5)
    x = np.zeros((1, 64), np.float32)
    x[0, 7], x[0, 15], x[0, 23], x[0, 31] = 2.0 ** 24, 1.0, 1.0, -2.0 ** 24
    assert O.router_logits(x, w, np.array([0.5], np.float32))[0, 0] == 0.5
    # boundaries: with H = 100 the segments are 16 long (ceil(100/8) = 13 -> 16): h = 15 and h = 16 lie in
    # different segments, h = 96..99 form the seventh, the eighth is empty
    x = np.zeros((1, 100), np.float32)
    w = np.ones((100, 1), np.float32)
    x[0, 15], x[0, 16], x[0, 17] = 2.0 ** 24, 1.0, -2.0 ** 24   # (2^24) + (1 - 2^24 -> -2^24 + 1 = exact) ...
    # segment 0 sum = 2^24; segment 1 chain: fma(1,1,0) = 1, then fma(-2^24,1,1) = -2^24 + 1 = -16777215 (exact)
    # total = 2^24 + (-16777215) = 1; a single chain would give (2^24 + 1 -> 2^24) - 2^24 = 0
    assert O.router_logits(x, w)[0, 0] == 1.0


def test_fma_is_fused():
    # (1+2^-12)^2 = 1 + 2^-11 + 2^-24: a separate multiply rounds the 2^-24 away, an fma keeps it
    a = np.float32(1 + 2.0 ** -12)
    x = np.array([[1.0, a]], np.float32)   # chain: fma(1,-1,0) = -1, then fma(a,a,-1) = a*a - 1 exactly
    w = np.array([[-1.0], [a]], np.float32)
    lg = O.router_logits(x, w)
    assert lg[0, 0] == np.float32(2.0 ** -11 + 2.0 ** -24)


def test_bf16_entry_point_equals_widened_f32():
    x, w = _rand(33, 130, 9, 4)
    xb, wb = O.bf16_round(x), O.bf16_round(w)
    import ctypes
    out = np.empty((33, 9), np.float32)
    u16p, fp = ctypes.POINTER(ctypes.c_uint16), ctypes.POINTER(ctypes.c_float)
    xbits, wbits = O.bf16_bits(xb), O.bf16_bits(wb)
    rc = O._lib().oracle_router_logits_bf16(xbits.ctypes.data_as(u16p), wbits.ctypes.data_as(u16p), None, 33, 130, 9,
                                            out.ctypes.data_as(fp))
    assert rc == 0 and np.array_equal(out, O.router_logits(xb, wb))
    assert np.array_equal(O.bf16_from_bits(xbits), xb)


@pytest.mark.parametrize("E,k", [(8, 2), (16, 1), (60, 8), (256, 8)])
def test_topk_matches_torch_on_softmax(E, k):
    x, w = _rand(512, 96, E, E, 0.3)
    idx, gate, lg = O.route(x, w, k)
    p = torch.softmax(torch.from_numpy(lg), dim=-1)
    tv, ti = torch.topk(p, k, dim=-1)
    # untied rows: identical ordered indices; gates equal torch's probabilities
    vals = np.take_along_axis(lg, idx.astype(np.int64), 1)
    kth = vals[:, -1]
    nxt = np.sort(lg, axis=1)[:, ::-1][:, k] if k < E else np.full(len(lg), -np.inf, np.float32)
    untied = (np.diff(vals, axis=1) != 0).all(axis=1) & (kth != nxt)
    assert untied.mean() > 0.95
    assert np.array_equal(ti.numpy()[untied], idx[untied])
    np.testing.assert_allclose(gate, tv.numpy(), rtol=2e-6)
    # C selection == numpy stable argsort selection
    import ctypes
    cidx = np.empty_like(idx)
    O._lib().oracle_topk_select(lg.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), len(lg), E, k,
                                cidx.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)))
    assert np.array_equal(cidx, idx)


def test_ties_break_to_lower_index():
    lg = np.array([[1.0, 3.0, 3.0, 2.0, 3.0, 0.5], [0.0, 0.0, 0.0, 0.0, 0.0, 0.0]], np.float32)
    assert O.topk_select(lg, 4).tolist() == [[1, 2, 4, 3], [0, 1, 2, 3]]


def test_closed_forms():
    T, H, E = 40, 16, 8
    rng = np.random.default_rng(7)
    x = np.abs(rng.standard_normal((T, H))).astype(np.float32) + 0.1
    # one-hot router: expert e sees only feature e -> argmax over the first E features
    w = np.zeros((H, E), np.float32)
    w[np.arange(E), np.arange(E)] = 1.0
    idx, gate, lg = O.route(x, w, 1)
    assert np.array_equal(idx[:, 0], np.argmax(x[:, :E], axis=1))
    # softmax sums to one; shifting all logits changes neither order nor gates
    allg = O.softmax_gates(lg, np.tile(np.arange(E, dtype=np.int32), (T, 1)))
    np.testing.assert_allclose(allg.sum(1), 1.0, rtol=1e-6)
    idx2, gate2, _ = O.route(x, w, 3, bias=np.full(E, 5.0, np.float32))
    idx3, gate3, _ = O.route(x, w, 3)
    assert np.array_equal(idx2, idx3)
    np.testing.assert_allclose(gate2, gate3, rtol=1e-5)
    # a huge bias forces an expert to the front
    b = np.zeros(E, np.float32)
    b[5] = 1e30
    assert (O.route(x, w, 2, bias=b)[0][:, 0] == 5).all()
    # identical rows route identically
    xx = np.repeat(x[:1], 7, axis=0)
    r = O.route(xx, rng.standard_normal((H, E)).astype(np.float32), 3)[0]
    assert (r == r[0]).all()


def test_bf16_round_matches_torch():
    rng = np.random.default_rng(0)
    a = (rng.standard_normal(200000) * np.exp(rng.uniform(-30, 30, 200000))).astype(np.float32)
    a[:4] = [0.0, -0.0, np.float32(1 + 2.0 ** -8), np.float32(1 + 3 * 2.0 ** -9)]
    want = torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    assert np.array_equal(O.bf16_round(a).view(np.uint32), want.view(np.uint32))


def test_fp8_codec_matches_torch():
    rng = np.random.default_rng(1)
    a = np.clip((rng.standard_normal(300000) * np.exp(rng.uniform(-12, 6, 300000))).astype(np.float32), -448, 448)
    a[:6] = [0.0, 448.0, -448.0, 2.0 ** -9, 2.0 ** -10, 0.0009765625 * 1.5]
    want = torch.from_numpy(a).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = O.fp8_e4m3_encode(a)
    # +-0 may differ in sign bit handling only if torch flushes -0; compare values
    assert np.array_equal(O.fp8_e4m3_decode(got), O.fp8_e4m3_decode(want))
    codes = np.arange(256, dtype=np.uint8)
    tdec = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.nan_to_num(O.fp8_e4m3_decode(codes), nan=7e7), np.nan_to_num(tdec, nan=7e7))
    # per-row quantisation: dequantised values within half an fp8 step of the input, max maps to +-448
    x = O.bf16_round(rng.standard_normal((50, 256)).astype(np.float32))
    q, s = O.quantize_rows_fp8(x)
    deq = O.fp8_e4m3_decode(q) * s[:, None]
    assert (np.abs(deq - x) <= np.abs(x) * 2.0 ** -4 + s[:, None] * 2.0 ** -10).all()
    assert (np.abs(O.fp8_e4m3_decode(q)).max(axis=1) == 448).all()
