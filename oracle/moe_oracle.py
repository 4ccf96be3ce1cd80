"""CPU oracle for the MoE dispatch / expert hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under ``iris_testing_amd/`` imports this module.  It may be imported by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py`` -- as the checker or as the timed CPU baseline, never as a fallback
for the HIP path.

It is a clean numpy restatement of what the reference computes (or, where the
reference holds only a sketch, of the layouts it documents).  Every function
cites the reference lines it follows.  bf16 data is carried as float32 arrays
whose values are bf16-representable; ``bf16_round`` is the only place rounding
to bf16 happens.

Pinning status (what, other than this file's own formulas, fixes each function;
the checks live in tests/test_oracle_*.py):

* router_logits / topk_select / softmax_gates: the library routines the
  reference itself calls (torch.softmax / torch.topk on CPU), float64 dot
  products, hand-built ties, closed forms (one-hot router, +inf bias, shift
  invariance).
* counts / offsets / payload order / pack: a literal pure-Python restatement of
  the reference's bucket loop, np.add.at brute force, the reference's uniform
  "cap rows to every (dst, expert)" pattern.
* token_buf / shuffle: the reference's reorder loop restated per element,
  round trips, multiset equality.
* grouped_gemm: per-group float64 matmul (the check the reference intended,
  unit_tests.py:231-237), identity / one-hot weights.
* expert_mlp (activation, SwiGLU gate order, GELU variant, fp8 quantisation)
  and combine (no renormalisation of the top-k gates): **parity unpinned** by
  the reference -- it defines none of these; they are fixed here and checked
  against torch.nn.functional on CPU and dense per-token closed forms.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def _lib():
    """Load the C restatement of the fixed-order router dot product (oracle/router_ref.c)."""
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle_router.so")
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is not built; run `make -C oracle` (or __graft_entry__.build())")
        lib = ctypes.CDLL(path)
        fp = ctypes.POINTER(ctypes.c_float)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        i32p = ctypes.POINTER(ctypes.c_int32)
        lib.oracle_router_logits_f32.argtypes = [fp, fp, fp, ctypes.c_int, ctypes.c_int, ctypes.c_int, fp]
        lib.oracle_router_logits_f32.restype = ctypes.c_int
        lib.oracle_router_logits_bf16.argtypes = [u16p, u16p, fp, ctypes.c_int, ctypes.c_int, ctypes.c_int, fp]
        lib.oracle_router_logits_bf16.restype = ctypes.c_int
        lib.oracle_topk_select.argtypes = [fp, ctypes.c_int, ctypes.c_int, ctypes.c_int, i32p]
        lib.oracle_topk_select.restype = ctypes.c_int
        _LIB = lib
    return _LIB


# --------------------------------------------------------------------------------------
# number formats
# --------------------------------------------------------------------------------------
def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round fp32 to the nearest bf16 (ties to even), returned as fp32.  NaN stays NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32).reshape(x.shape)
    nan = np.isnan(x)
    if nan.any():
        out = out.copy()
        out[nan] = np.float32("nan")
    return out


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 holding bf16-representable values -> uint16 bit patterns."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return (x.view(np.uint32) >> 16).astype(np.uint16).reshape(x.shape)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32).reshape(b.shape)


def round_to(x: np.ndarray, dtype: str) -> np.ndarray:
    if dtype == "bf16":
        return bf16_round(x)
    if dtype == "f32":
        return np.asarray(x, dtype=np.float32)
    raise ValueError(dtype)


FP8_MAX = 448.0  # largest finite OCP e4m3fn value


def fp8_e4m3_decode(b: np.ndarray) -> np.ndarray:
    """OCP fp8 e4m3fn bit patterns (uint8) -> fp32.  bias 7, no inf, 0x7f/0xff = NaN."""
    b = np.asarray(b, dtype=np.uint8)
    s = (b >> 7).astype(np.int32)
    e = ((b >> 3) & 0xF).astype(np.int32)
    m = (b & 7).astype(np.int32)
    sub = (m.astype(np.float32) / 8.0) * np.float32(2.0 ** -6)
    nor = (1.0 + m.astype(np.float32) / 8.0) * np.exp2((e - 7).astype(np.float32))
    v = np.where(e == 0, sub, nor).astype(np.float32)
    v = np.where((e == 15) & (m == 7), np.float32("nan"), v)
    return np.where(s == 1, -v, v).astype(np.float32)


_FP8_TABLE = None


def fp8_e4m3_encode(x: np.ndarray) -> np.ndarray:
    """fp32 -> OCP e4m3fn bit patterns, round to nearest even, saturating at +-448."""
    global _FP8_TABLE
    if _FP8_TABLE is None:
        _FP8_TABLE = fp8_e4m3_decode(np.arange(0, 127, dtype=np.uint8)).astype(np.float64)  # 0..448 ascending
    x = np.asarray(x, dtype=np.float32)
    a = np.minimum(np.abs(x.astype(np.float64)), FP8_MAX)
    tab = _FP8_TABLE
    hi = np.searchsorted(tab, a, side="left")
    hi = np.clip(hi, 0, 126)
    lo = np.clip(hi - 1, 0, 126)
    dlo = a - tab[lo]
    dhi = tab[hi] - a
    pick_hi = (dhi < dlo) | ((dhi == dlo) & ((hi & 1) == 0))
    code = np.where(pick_hi, hi, lo).astype(np.uint8)
    code = np.where(tab[hi] == a, hi.astype(np.uint8), code)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    out = (code | sign).astype(np.uint8)
    return np.where(np.isnan(x), np.uint8(0x7F), out)


def quantize_rows_fp8(x: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """Per-row (per-token) symmetric fp8 quantisation.

    amax = max|x[r,:]|;  scale[r] = amax/448 (1.0 for an all-zero row);
    q[r,:] = e4m3(x[r,:] * (448/amax)).  Returns (uint8 codes [R,C], fp32 scales [R]).
    Not in the reference (defined by the workload description only).
    """
    x = np.asarray(x, dtype=np.float32)
    amax = np.max(np.abs(x), axis=1) if x.shape[1] else np.zeros(x.shape[0], np.float32)
    amax = amax.astype(np.float32)
    zero = amax == 0
    safe = np.where(zero, np.float32(1.0), amax)
    inv = (np.float32(FP8_MAX) / safe).astype(np.float32)
    scale = np.where(zero, np.float32(1.0), (safe / np.float32(FP8_MAX)).astype(np.float32)).astype(np.float32)
    inv = np.where(zero, np.float32(1.0), inv).astype(np.float32)
    q = fp8_e4m3_encode((x * inv[:, None]).astype(np.float32))
    return q, scale


FP8_BLOCK = 32  # columns per block scale of the fp8 hidden activation


def quantize_blocks_fp8(x: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """Block quantisation of the fp8 expert's hidden activation: one power-of-two scale per row and 32 columns.

    For every block: amax = max|x|; scale byte b = the smallest b >= 0 with amax / 2^(b-127) <= 448 (an E8M0 exponent:
    from the bits of amax = m 2^p, b = p + 127 - 8, one more when m > 1.75; the integer expression below is the one the
    kernels evaluate); codes = e4m3(x / 2^(b-127)), the division being exact.  Returns (uint8 codes [R,C], uint8 scale
    bytes [R, C/32]).  Not in the reference (the workload description only says "fp8 MFMA grouped GEMM")."""
    x = np.asarray(x, dtype=np.float32)
    R, C = x.shape
    assert C % FP8_BLOCK == 0
    xb = x.reshape(R, C // FP8_BLOCK, FP8_BLOCK)
    amax = np.max(np.abs(xb), axis=2).astype(np.float32)
    bits = amax.view(np.uint32).astype(np.int64)
    b = np.maximum(((bits + 0x1FFFFF) >> 23) - 8, 0)
    inv = ((254 - b).astype(np.uint32) << np.uint32(23)).view(np.float32)  # 2^(127-b), exact
    q = fp8_e4m3_encode((xb * inv[:, :, None]).astype(np.float32)).reshape(R, C)
    return q, b.astype(np.uint8)


def dequantize_blocks_fp8(q: np.ndarray, b: np.ndarray) -> np.ndarray:
    """codes [R,C] and scale bytes [R,C/32] -> fp32 values (exact: a power of two times an e4m3 value)."""
    R, C = q.shape
    v = fp8_e4m3_decode(q).reshape(R, C // FP8_BLOCK, FP8_BLOCK)
    return (v * np.exp2(b.astype(np.float32) - 127.0)[:, :, None]).astype(np.float32).reshape(R, C)


def quantize_cols_fp8(w: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """Per-output-channel fp8 weights: w [..., K, N] -> (codes [..., K, N], scales [..., N])."""
    w = np.asarray(w, dtype=np.float32)
    amax = np.max(np.abs(w), axis=-2).astype(np.float32)
    zero = amax == 0
    safe = np.where(zero, np.float32(1.0), amax)
    scale = np.where(zero, np.float32(1.0), safe / np.float32(FP8_MAX)).astype(np.float32)
    inv = np.where(zero, np.float32(1.0), np.float32(FP8_MAX) / safe).astype(np.float32)
    q = fp8_e4m3_encode((w * inv[..., None, :]).astype(np.float32))
    return q, scale


# --------------------------------------------------------------------------------------
# a1: router  (reference utils.py:200-202)
# --------------------------------------------------------------------------------------
def router_logits(x: np.ndarray, w: np.ndarray, bias: Optional[np.ndarray] = None) -> np.ndarray:
    """logits[t,e] = bias[e] + sum_h x[t,h] w[h,e] in pinned fp32 arithmetic: h in eight contiguous
    segments of ceil(H/8) rounded up to a multiple of 8, one fmaf chain per segment in ascending h from
    +0, the eight chains added in segment order, the bias last (see oracle/router_ref.c).

    Restates ``torch.einsum('th,he->te', tokens, router)`` (utils.py:201), whose own order is
    unspecified.  ``bias`` (per-expert, added to the logits) is the load-skew term of the fine-grained /
    Zipf workloads.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    T, H = x.shape
    H2, E = w.shape
    assert H == H2
    out = np.empty((T, E), dtype=np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    b = None
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32)
        assert bias.shape == (E,)
        b = bias.ctypes.data_as(fp)
    rc = _lib().oracle_router_logits_f32(x.ctypes.data_as(fp), w.ctypes.data_as(fp), b, T, H, E,
                                         out.ctypes.data_as(fp))
    if rc != 0:
        raise RuntimeError(f"oracle_router_logits_f32 -> {rc}")
    return out


def topk_select(logits: np.ndarray, k: int) -> np.ndarray:
    """Top-k expert ids per token, descending logit, ties -> lower expert id.  int32 [T,k].

    Restates ``torch.topk(softmax(logits), k).indices`` (utils.py:202): softmax is
    strictly increasing, so ordering logits orders the probabilities; torch leaves ties
    unspecified, this fixes them.
    """
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    T, E = logits.shape
    if not 0 <= k <= E:
        raise ValueError("topk out of range")
    # stable argsort of -logit: equal logits keep ascending expert order
    order = np.argsort(-logits, axis=1, kind="stable")
    return np.ascontiguousarray(order[:, :k]).astype(np.int32)


def softmax_gates(logits: np.ndarray, idx: np.ndarray) -> np.ndarray:
    """p[t, idx[t,kk]] with p = softmax(logits, -1) (utils.py:201); fp32 [T,k].

    The reference discards the values (``_`` at utils.py:202); the combine needs them.
    Raw softmax probabilities, NOT renormalised over the selected k.
    """
    l = np.asarray(logits, dtype=np.float32)
    m = l.max(axis=1, keepdims=True)
    ex = np.exp((l - m).astype(np.float32)).astype(np.float32)
    s = ex.sum(axis=1, keepdims=True, dtype=np.float32)
    p = (ex / s).astype(np.float32)
    return np.take_along_axis(p, idx.astype(np.int64), axis=1).astype(np.float32)


def route(x, w, k, bias=None):
    """(idx int32 [T,k], gate fp32 [T,k], logits fp32 [T,E])."""
    lg = router_logits(x, w, bias)
    idx = topk_select(lg, k)
    return idx, softmax_gates(lg, idx), lg


# --------------------------------------------------------------------------------------
# a2, a4, a5: counts and offsets  (reference utils.py:204-238, utils.py:20-31, benchmark.py:44-49)
# --------------------------------------------------------------------------------------
def send_counts(idx: np.ndarray, world_size: int, num_experts_total: int) -> np.ndarray:
    """send_counts[dst, el] = #{(t,kk): idx[t,kk] == dst*E_l + el}; int32 [W, E_l].

    Expert ex lives on rank ex // E_l as local expert ex % E_l (utils.py:217-218).
    """
    if num_experts_total % world_size != 0:
        raise AssertionError("num_experts_total must be divisible by world_size")  # utils.py:197
    e_local = num_experts_total // world_size
    c = np.bincount(np.asarray(idx).reshape(-1).astype(np.int64), minlength=num_experts_total)
    return c.reshape(world_size, e_local).astype(np.int32)


def build_expert_offsets(counts: np.ndarray) -> np.ndarray:
    """expert_offs[dst, e] = sum_{e'<e} counts[dst, e'] (utils.py:20-31): int64 cumsum - self -> int32."""
    sc = np.asarray(counts).astype(np.int64)
    return (np.cumsum(sc, axis=1) - sc).astype(np.int32)


def dst_sizes_offsets(counts: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """(dst_sizes [W], dst_offsets [W]) int32: row totals and their exclusive prefix
    (utils.py:229,237; benchmark.py:44-49)."""
    sizes = np.asarray(counts).astype(np.int64).sum(axis=1)
    offs = np.cumsum(sizes) - sizes
    return sizes.astype(np.int32), offs.astype(np.int32)


# --------------------------------------------------------------------------------------
# a3: payload order  (reference utils.py:204-246)
# --------------------------------------------------------------------------------------
def payload_positions(idx: np.ndarray, num_experts_total: int) -> Tuple[np.ndarray, np.ndarray]:
    """Row of every routed (t,kk) in the padding-free payload, and its inverse.

    The reference appends token rows to bucket[dst][el] in increasing token index, then
    increasing top-k slot (utils.py:210-219), and concatenates buckets in (dst, el) order
    (utils.py:226-244).  (dst, el) order is global-expert order, so the payload is the
    stable sort of the (t,kk)-ordered list by expert id.

    returns pos int32 [T,k] (payload row of slot (t,kk)), row_token int32 [T*k] (token of
    payload row r).
    """
    idx = np.asarray(idx)
    T, k = idx.shape
    flat = idx.reshape(-1).astype(np.int64)
    order = np.argsort(flat, kind="stable")  # payload row r holds flattened slot order[r]
    pos = np.empty(T * k, dtype=np.int32)
    pos[order] = np.arange(T * k, dtype=np.int32)
    row_token = (order // max(k, 1)).astype(np.int32)
    return pos.reshape(T, k), row_token


def send_payload(x: np.ndarray, row_token: np.ndarray) -> np.ndarray:
    """send_payload [T*k, H] (utils.py:235-246); empty [0,H] when nothing is routed (utils.py:240-242)."""
    x = np.asarray(x)
    if row_token.size == 0:
        return np.empty((0, x.shape[1]), dtype=x.dtype)
    return x[row_token.astype(np.int64)]


def bucket_loop_pack(x: np.ndarray, top_idxs: np.ndarray, world_size: int, num_experts_total: int):
    """The reference's host algorithm as it is written, one Python iteration per routed slot (utils.py:204-246):
    append each token row to bucket[dst][el] in (token, slot) order, then concatenate the buckets in (dst, el)
    order.  Returns (send_payload, send_counts, dst_offsets, dst_sizes).  Slow by construction; the vectorised
    functions above are held to it in the tests, and the benchmark times it on the smallest workload."""
    e_local = num_experts_total // world_size
    buckets = [[[] for _ in range(e_local)] for _ in range(world_size)]
    for ti in range(x.shape[0]):
        for kk in range(top_idxs.shape[1]):
            ex = int(top_idxs[ti, kk])
            dst = ex // e_local
            buckets[dst][ex - dst * e_local].append(x[ti])
    counts = np.zeros((world_size, e_local), np.int32)
    offs, sizes = np.zeros(world_size, np.int32), np.zeros(world_size, np.int32)
    chunks, running = [], 0
    for dst in range(world_size):
        offs[dst] = running
        for el in range(e_local):
            n = len(buckets[dst][el])
            counts[dst, el] = n
            if n:
                chunks.append(np.stack(buckets[dst][el]))
            sizes[dst] += n
        running += int(sizes[dst])
    payload = np.concatenate(chunks) if running else np.empty((0, x.shape[1]), x.dtype)
    return payload, counts, offs, sizes


def route_and_pack_padding_free(x, w, topk, world_size, num_experts_total, bias=None):
    """The reference's host routine end to end (utils.py:176-246).

    returns (send_payload [R,H], send_counts [W,E_l] i32, dst_offsets [W] i32, dst_sizes [W] i32).
    """
    idx, _, _ = route(x, w, topk, bias)
    counts = send_counts(idx, world_size, num_experts_total)
    sizes, offs = dst_sizes_offsets(counts)
    _, row_token = payload_positions(idx, num_experts_total)
    return send_payload(x, row_token), counts, offs, sizes


# --------------------------------------------------------------------------------------
# a6, a7: capacities  (reference utils.py:118-121, benchmark.py:134-135, README.md:4-7)
# --------------------------------------------------------------------------------------
def compute_capacity_from_pca(pca: np.ndarray) -> int:
    """CAP = max(1, max(pca)) (utils.py:118-121); the all-reduce MAX over ranks is the
    caller's max over the per-rank values."""
    pca = np.asarray(pca)
    return max(int(pca.max()) if pca.size else 0, 1)


def pair_capacity(dst_sizes_all: np.ndarray) -> int:
    """M = max over (src, dst) of rows sent between the pair (README.md:4-7), floored at 1
    like CAP (utils.py:121)."""
    a = np.asarray(dst_sizes_all)
    return max(int(a.max()) if a.size else 0, 1)


# --------------------------------------------------------------------------------------
# a8: fixed [W, M, H] send layout  (reference README.md:5-7)
# --------------------------------------------------------------------------------------
def pack_fixed_m(payload: np.ndarray, dst_offsets: np.ndarray, dst_sizes: np.ndarray, M: int,
                 drop: bool = False) -> np.ndarray:
    """send[dst, m, :] = payload[dst_offsets[dst] + m] for m < dst_sizes[dst], else zeros.

    A destination with more than M rows is an error, unless ``drop``: then its rows at and past M are
    dropped (the capacity-overflow behaviour of the kernels, which also raise a status word; the reference
    skips the whole exchange instead, benchmark.py:137-142)."""
    W = len(dst_sizes)
    H = payload.shape[1]
    if int(np.max(dst_sizes, initial=0)) > M and not drop:
        raise ValueError(f"pair capacity M={M} < max dst size {int(np.max(dst_sizes))}")
    out = np.zeros((W, M, H), dtype=payload.dtype)
    for d in range(W):
        n = min(int(dst_sizes[d]), M)
        o = int(dst_offsets[d])
        out[d, :n] = payload[o:o + n]
    return out


# --------------------------------------------------------------------------------------
# a9: receive layout  (reference baseline.py:178-222; kernels.py:100-102,124-125)
# --------------------------------------------------------------------------------------

def pack_fixed_m_fp8(payload: np.ndarray, dst_offsets: np.ndarray, dst_sizes: np.ndarray, M: int,
                     drop: bool = False) -> Tuple[np.ndarray, np.ndarray]:
    """The fixed [W,M,H] send layout (README.md:5-7 of the reference) of tokens quantised per row to fp8 before they are
    sent: (codes [W,M,H] uint8, scales [W,M] fp32) = quantize_rows_fp8 of every row of pack_fixed_m's buffer; a padding
    slot is an all-zero row (codes 0, scale 1).  Not in the reference, which sends the token dtype: the workload
    description asks for per-token fp8 activations, and per-row quantisation commutes with moving rows (checked in
    tests/test_oracle_dispatch.py), so quantising at the source changes no result."""
    send = pack_fixed_m(payload, dst_offsets, dst_sizes, M, drop=drop)
    W, _, H = send.shape
    q, sc = quantize_rows_fp8(send.reshape(W * M, H))
    return q.reshape(W, M, H), sc.reshape(W, M)

def reorder_flat_to_token_buf(flat: np.ndarray, recv_counts: np.ndarray, capacity: int,
                              token_buf_out: np.ndarray) -> np.ndarray:
    """token_buf[e, src, :c] = next c rows of ``flat`` for src-major, expert-minor blocks;
    padding zero; same error cases as baseline.py:199-201,215-216,220-221."""
    W, e_local = recv_counts.shape
    H = flat.shape[1]
    if token_buf_out.shape != (e_local, W, capacity, H):
        raise ValueError("token_buf_out shape mismatch")
    token_buf_out[...] = 0
    off = 0
    for src in range(W):
        for e in range(e_local):
            c = int(recv_counts[src, e])
            if c == 0:
                continue
            if c > capacity:
                raise ValueError(f"[reorder] recv_count src={src},e={e} is {c} > capacity={capacity}")
            token_buf_out[e, src, :c] = flat[off:off + c]
            off += c
    if off != flat.shape[0]:
        raise RuntimeError(f"[reorder] consumed rows={off} != total_recv={flat.shape[0]}")
    return token_buf_out


def recv_to_token_buf(recv: np.ndarray, recv_counts: np.ndarray, capacity: int) -> Tuple[np.ndarray, np.ndarray]:
    """Fixed-M receive buffer -> (token_buf [E_l, W, CAP, H], pca [E_l, W]).

    recv[s] is what source s wrote into its [M,H] slot for this rank: its rows for this
    rank's experts in (el, token) order, then zeros.  pca[e, s] = recv_counts[s, e]
    (kernels.py:46-47; benchmark.py:131).  token_buf[e, s, j] = recv[s, expert_offs_s[e] + j]
    for j < pca[e,s] (kernels.py:93-102,124-125), zero elsewhere (baseline.py:204).
    """
    W, M, H = recv.shape
    e_local = recv_counts.shape[1]
    if int(np.max(recv_counts, initial=0)) > capacity:
        raise ValueError("capacity overflow")
    offs = build_expert_offsets(recv_counts)
    tb = np.zeros((e_local, W, capacity, H), dtype=recv.dtype)
    for s in range(W):
        for e in range(e_local):
            c = int(recv_counts[s, e])
            o = int(offs[s, e])
            c = max(min(c, M - o), 0)  # rows at or past M never reached the slot (dropped by the sender's pack): zeros
            tb[e, s, :c] = recv[s, o:o + c]
    return tb, np.ascontiguousarray(recv_counts.T).astype(np.int32)


# --------------------------------------------------------------------------------------
# a10: expert-major unpack  (reference layers/token_shuffle.py:31-41; kernels.py:179-205)
# --------------------------------------------------------------------------------------
def shuffle(token_buf: np.ndarray, pca: np.ndarray) -> np.ndarray:
    """shuffled[off[e,s] + j] = token_buf[e, s, j], off = exclusive prefix over flattened
    (e, s) of pca (token_shuffle.py:35-37); S = sum(pca) rows (token_shuffle.py:40-41)."""
    e_local, W, CAP, H = token_buf.shape
    S = int(np.asarray(pca).astype(np.int64).sum())
    out = np.zeros((S, H), dtype=token_buf.dtype)
    r = 0
    for e in range(e_local):
        for s in range(W):
            c = int(pca[e, s])
            out[r:r + c] = token_buf[e, s, :c]
            r += c
    return out


def unpack_expert_major(recv: np.ndarray, recv_counts: np.ndarray) -> np.ndarray:
    """recv [W,M,H] -> shuffled [S,H] without materialising token_buf (same result as
    shuffle(recv_to_token_buf(...)))."""
    W, M, H = recv.shape
    e_local = recv_counts.shape[1]
    offs = build_expert_offsets(recv_counts)
    parts = []
    for e in range(e_local):
        for s in range(W):
            c = int(recv_counts[s, e])
            o = int(offs[s, e])
            have = max(min(c, M - o), 0)  # counted rows at or past M were dropped by the sender's pack: zero rows
            parts.append(recv[s, o:o + have])
            if have < c:
                parts.append(np.zeros((c - have, H), dtype=recv.dtype))
    return np.concatenate(parts, axis=0) if parts else np.zeros((0, H), dtype=recv.dtype)


def expert_row_counts(pca: np.ndarray) -> np.ndarray:
    """cnt[e] = sum_s pca[e,s] (layers/expert.py:26-27)."""
    return np.asarray(pca).astype(np.int64).sum(axis=1).astype(np.int32)


# --------------------------------------------------------------------------------------
# a11: grouped GEMM  (reference layers/expert.py:20-43; kernels.py:240-289)
# --------------------------------------------------------------------------------------
def grouped_gemm(tokens: np.ndarray, weights: np.ndarray, cnt: np.ndarray, dtype: str = "f32",
                 row_gate: Optional[np.ndarray] = None) -> np.ndarray:
    """out[rows of e] = tokens[rows of e] @ weights[e]; fp32 accumulate (kernels.py:265),
    cast to the token dtype (kernels.py:276); rows of e = [sum cnt[:e], + cnt[e]).
    row_gate [S] (not in the reference, which has no return path): every fp32 result row is multiplied by its
    gate -- one fp32 multiplication -- before the one rounding to ``dtype``."""
    S, K = tokens.shape
    E_l, K2, N = weights.shape
    assert K == K2 and len(cnt) == E_l
    out = np.zeros((S, N), dtype=np.float32)
    r = 0
    for e in range(E_l):
        c = int(cnt[e])
        if c:
            out[r:r + c] = tokens[r:r + c].astype(np.float32) @ weights[e].astype(np.float32)
        r += c
    assert r <= S
    if row_gate is not None:
        out = (out * np.asarray(row_gate, dtype=np.float32)[:S, None]).astype(np.float32)
    return round_to(out, dtype)


# --------------------------------------------------------------------------------------
# a12: expert MLP  (NOT in the reference; shape from the workload descriptions)
# --------------------------------------------------------------------------------------
def _erf(x):
    try:
        from scipy.special import erf
        return erf(x)
    except ImportError:  # pragma: no cover
        from math import erf
        return np.vectorize(erf, otypes=[np.float64])(x)


def act_gelu(x: np.ndarray) -> np.ndarray:
    """erf GELU (torch.nn.functional.gelu default)."""
    x64 = x.astype(np.float64)
    return (0.5 * x64 * (1.0 + _erf(x64 / np.sqrt(2.0)))).astype(np.float32)


def act_silu(x: np.ndarray) -> np.ndarray:
    x64 = x.astype(np.float64)
    return (x64 / (1.0 + np.exp(-x64))).astype(np.float32)


def expert_mlp(tokens, cnt, w1, w2, act: str, dtype: str = "bf16", w_up=None, row_gate=None):
    """Per-expert MLP on expert-major rows.

    row_gate [S] (optional): the result rows leave weighted, round(fp32 result * gate) -- see grouped_gemm.

    act in {"gelu","silu"}:  y = act(x W1_e) W2_e              (w1 [E_l,H,F], w2 [E_l,F,H])
    act == "swiglu":         y = (silu(x Wg_e) * (x Wu_e)) Wd_e (w1 = Wg, w_up = Wu, w2 = Wd)
    fp32 accumulation in both GEMMs; the hidden activation is rounded once to ``dtype``
    before the second GEMM; the output is rounded to ``dtype``.
    """
    S, H = tokens.shape
    E_l = w1.shape[0]
    y = np.zeros((S, w2.shape[2]), dtype=np.float32)
    r = 0
    for e in range(E_l):
        c = int(cnt[e])
        if c:
            xe = tokens[r:r + c].astype(np.float32)
            a = xe @ w1[e].astype(np.float32)
            if act == "gelu":
                h = act_gelu(a)
            elif act == "silu":
                h = act_silu(a)
            elif act == "swiglu":
                u = xe @ w_up[e].astype(np.float32)
                h = (act_silu(a).astype(np.float32) * u).astype(np.float32)
            elif act == "none":
                h = a
            else:
                raise ValueError(act)
            h = round_to(h, dtype)
            y[r:r + c] = h @ w2[e].astype(np.float32)
        r += c
    if row_gate is not None:
        y = (y * np.asarray(row_gate, dtype=np.float32)[:S, None]).astype(np.float32)
    return round_to(y, dtype)


def expert_up_fp8(tokens, cnt, wg_q, wg_s, wu_q, wu_s):
    """First half of the fp8 SwiGLU expert: bf16 rows quantised per token to e4m3, e4m3 weights with
    per-output-channel fp32 scales, fp32 accumulation, epilogue acc * s_tok[m] * s_ch[n], then
    h = silu(g) * u in fp32, block-quantised (quantize_blocks_fp8) without a rounding to bf16 in between.
    [S,H] -> (codes [S,F] uint8, scale bytes [S,F/32] uint8)."""
    S, H = tokens.shape
    E_l = wg_q.shape[0]
    h = np.zeros((S, wg_q.shape[2]), dtype=np.float32)
    xq, xs = quantize_rows_fp8(tokens)
    xf = fp8_e4m3_decode(xq)
    r = 0
    for e in range(E_l):
        c = int(cnt[e])
        if c:
            xe = xf[r:r + c]
            sx = xs[r:r + c, None]
            g = ((xe @ fp8_e4m3_decode(wg_q[e])) * sx).astype(np.float32) * wg_s[e][None, :]
            u = ((xe @ fp8_e4m3_decode(wu_q[e])) * sx).astype(np.float32) * wu_s[e][None, :]
            h[r:r + c] = (act_silu(g.astype(np.float32)) * u.astype(np.float32)).astype(np.float32)
        r += c
    return quantize_blocks_fp8(h)


def expert_down_fp8(hq, hsc, cnt, wd_q, wd_s, row_gate=None):
    """Second half: the block-quantised hidden activation (codes, scale bytes) times the e4m3 down projection -- every
    block of 32 k enters the sum with its power-of-two scale, fp32 accumulation -- then the channel scale (and the row's
    gate where given: one more fp32 multiplication, of the channel scale), rounded to bf16.  -> [S,H]."""
    E_l = wd_q.shape[0]
    hf = dequantize_blocks_fp8(hq, hsc)
    y = np.zeros((hf.shape[0], wd_q.shape[2]), dtype=np.float32)
    r = 0
    for e in range(E_l):
        c = int(cnt[e])
        if c:
            acc = (hf[r:r + c] @ fp8_e4m3_decode(wd_q[e])).astype(np.float32)
            if row_gate is None:
                y[r:r + c] = acc * wd_s[e][None, :]
            else:
                y[r:r + c] = acc * (wd_s[e][None, :] * np.asarray(row_gate, np.float32)[r:r + c, None]).astype(np.float32)
        r += c
    return bf16_round(y)


def expert_mlp_fp8(tokens, cnt, wg_q, wg_s, wu_q, wu_s, wd_q, wd_s, row_gate=None):
    """fp8 SwiGLU expert = expert_down_fp8(expert_up_fp8(x)).  Not in the reference."""
    hq, hsc = expert_up_fp8(tokens, cnt, wg_q, wg_s, wu_q, wu_s)
    return expert_down_fp8(hq, hsc, cnt, wd_q, wd_s, row_gate)


# --------------------------------------------------------------------------------------
# a13: return path and combine  (NOT in the reference; defined by the task statement)
# --------------------------------------------------------------------------------------
def return_pack(y: np.ndarray, recv_counts: np.ndarray, M: int) -> np.ndarray:
    """Inverse of unpack_expert_major: ret[s, expert_offs_s[e] + j] = y[off[e,s] + j]; zero padding.

    ret[s] is the [M,H] slot this rank sends back to source s, rows in the order s sent them.
    """
    W, e_local = recv_counts.shape
    H = y.shape[1]
    offs = build_expert_offsets(recv_counts)
    ret = np.zeros((W, M, H), dtype=y.dtype)
    r = 0
    for e in range(e_local):
        for s in range(W):
            c = int(recv_counts[s, e])
            o = int(offs[s, e])
            have = max(min(c, M - o), 0)  # rows at or past M have no slot on the way back
            ret[s, o:o + have] = y[r:r + have]
            r += c
    return ret


def pack_gates(gate: np.ndarray, idx: np.ndarray, pos: np.ndarray, dst_offsets: np.ndarray, e_local: int,
               W: int, M: int) -> np.ndarray:
    """send_gate[dst, m] = gate[t,kk] for the slot (dst, m) of (t,kk), zero in the padding: the gates shipped with the
    rows of the fixed [W,M,H] layout (README.md:5-7) when the destination is to apply them.  Slots past M are dropped
    like their rows."""
    T, k = idx.shape
    out = np.zeros((W, M), dtype=np.float32)
    for t in range(T):
        for kk in range(k):
            d = int(idx[t, kk]) // e_local
            if 0 <= d < W:
                m = int(pos[t, kk]) - int(dst_offsets[d])
                if 0 <= m < M:
                    out[d, m] = gate[t, kk]
    return out


def flat_recv_row_map(recv_counts: np.ndarray) -> np.ndarray:
    """Expert-major row r = (e, s, j) -> row of a padding-free flat receive payload laid out in source-major,
    expert-minor blocks (what every source's send_payload holds for this rank, utils.py:235-246, concatenated in source
    order; the layout reorder_flat_to_token_buf reads, baseline.py:204-218)."""
    W, e_local = recv_counts.shape
    flat_off = np.concatenate([[0], np.cumsum(recv_counts.reshape(-1).astype(np.int64))])
    rows = []
    for e in range(e_local):
        for s in range(W):
            c = int(recv_counts[s, e])
            rows.append(flat_off[s * e_local + e] + np.arange(c, dtype=np.int64))
    return np.concatenate(rows).astype(np.int32) if rows else np.zeros(0, np.int32)


def combine(ret: np.ndarray, idx: np.ndarray, pos: np.ndarray, gate: np.ndarray,
            dst_offsets: np.ndarray, e_local: int, dtype: str = "bf16", pre_weighted: bool = False) -> np.ndarray:
    """out[t] = sum_kk gate[t,kk] * ret[dst, pos[t,kk] - dst_offsets[dst]],  dst = idx[t,kk] // E_l.

    pre_weighted: the returned rows were multiplied by their gates where they were computed (grouped_gemm /
    expert_mlp with row_gate: the multiplication happens in fp32 BEFORE the expert output is rounded to ``dtype``,
    instead of after it); the combine then only adds them, fp32, ascending kk, one rounding.  ``gate`` is ignored.

    ret [W,M,H] is the returned buffer in the same slots the send buffer used.  fp32
    accumulate in ascending kk, one fp32 multiply and one fp32 add per term (no fused
    multiply-add), then one rounding to ``dtype``.  A slot whose row lies outside [0, M) (dropped by a pack
    that ran over the pair capacity) or whose dst lies outside [0, W) has no returned row and is skipped.
    """
    T, k = idx.shape
    W, M, H = ret.shape
    out = np.zeros((T, H), dtype=np.float32)
    for kk in range(k):
        d = (idx[:, kk] // e_local).astype(np.int64)
        d_ok = (d >= 0) & (d < W)
        m = pos[:, kk].astype(np.int64) - dst_offsets.astype(np.int64)[np.where(d_ok, d, 0)]
        have = d_ok & (m >= 0) & (m < M)
        rows = ret[np.where(have, d, 0), np.where(have, m, 0)].astype(np.float32)
        weighted = rows if pre_weighted else (gate[:, kk:kk + 1].astype(np.float32) * rows).astype(np.float32)
        term = (out + weighted).astype(np.float32)
        out = np.where(have[:, None], term, out)
    return round_to(out, dtype)
