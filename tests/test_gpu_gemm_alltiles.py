"""Every output tile of the grouped GEMMs at the full published sizes.

The CPU cannot redo a 33 000 x 4096 x 28 672 product in test time, so two checks stand in for it, both over ALL
rows and columns of the kernels' outputs:

* a randomised projection in float64 (Freivalds): for a +-1 matrix R with one column per 256-column block of the
  output, (Y R) computed from the kernel's output must equal X (W R) computed from the inputs.  It costs
  O(S K + K N) per block instead of O(S K N), involves no GEMM library on the reference side beyond thin
  float64 products, and a wrong tile, a tile that missed one K stage, or a tile written to the wrong place moves
  its block's projection by many times the bf16 rounding noise;
* a plain fp32 PyTorch GEMM of the same operands, compared element by element (this is what pins the fused
  SwiGLU epilogue, which is not linear, and the fp8 path).

Both run with and without the partial-sum workspace (the K split of the last round of tiles).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from iris_testing_amd import harness, ops  # noqa: E402
from iris_testing_amd.configs import CONFIGS  # noqa: E402

DEV = "cuda"
BLK = 256


def _block_signs(n_cols, seed):
    """R [n_cols, ceil(n_cols / 256)] float64: column j holds random +-1 on output columns [256 j, 256 j + 256)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    nb = (n_cols + BLK - 1) // BLK
    signs = (torch.randint(0, 2, (n_cols,), generator=g, dtype=torch.int64) * 2 - 1).double()
    R = torch.zeros((n_cols, nb), dtype=torch.float64)
    R[torch.arange(n_cols), torch.arange(n_cols) // BLK] = signs
    return R.to(DEV)


def _freivalds(Y, X, Wfull, cnt, what, col_scale=None, row_scale=None):
    """Y [S,N] (kernel output, bf16), X [S,K] and Wfull [E_l,K,N] (exact operand values as float tensors);
    optional fp8 scales: Y = (X W) * row_scale[:,None] * col_scale[e][None,:]."""
    S, N = Y.shape
    R = _block_signs(N, 1234 + N)
    lhs = Y.double() @ R                                                # [S, nb]
    norm = torch.sqrt((Y.double() ** 2) @ R.abs())                      # per-row, per-block 2-norm of the output
    rhs = torch.empty_like(lhs)
    r0 = 0
    for e, c in enumerate(cnt):
        if c == 0:
            continue
        We = Wfull[e].double()
        if col_scale is not None:
            We = We * col_scale[e].double()[None, :]
        rhs[r0:r0 + c] = X[r0:r0 + c].double() @ (We @ R)
        r0 += c
    assert r0 == S
    if row_scale is not None:
        rhs = rhs * row_scale.double()[:, None]
    # rounding each output to bf16 moves it by at most 2^-8 of its value; under random signs the block sum of these
    # errors has a standard deviation below 2^-8 / sqrt(3) of the block's 2-norm: 2^-6 is seven of those.
    # One K stage (32 values of K) missing from a tile moves the sum by about sqrt(32 / K) of the norm (2^-4.4 at
    # K = 14 336), a wrong tile by about sqrt(2) of it.
    excess = (lhs - rhs).abs() - (2.0 ** -6 * norm + 1e-6 * norm.max())
    worst = float(excess.max())
    ratio = float(((lhs - rhs).abs() / (norm + 1e-30))[norm > 0].max()) if bool((norm > 0).any()) else 0.0
    print(f"{what}: projection of {S} rows x {lhs.shape[1]} column blocks, worst |Y R - X W R| / ||Y_block|| = {ratio:.3e}",
          flush=True)
    if worst > 0:
        bad = torch.nonzero(excess > 0)
        raise AssertionError(f"{what}: {bad.shape[0]} (row, column block) projections off; first {bad[0].tolist()}")


def _close(got, ref, what, rtol=2.0 ** -7, atol=2.0 ** -7):
    """Element by element against an fp32 reference: |err| <= rtol |ref| + atol rms(ref) (one bf16 rounding step
    either way plus the hidden rounding that an accumulation-order difference can flip)."""
    got, ref = got.float(), ref.float()
    rms = float(torch.sqrt((ref.double() ** 2).mean()))
    err = (got - ref).abs()
    bad = err > rtol * ref.abs() + atol * rms
    print(f"{what}: {got.numel()} elements, max-abs {float(err.max()):.3e}, rms {rms:.3e}", flush=True)
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} elements outside tolerance"


def _close_fp8_hidden(hq, hsc, ref, what):
    """The block-quantised hidden activation of the fp8 expert (codes, scale bytes) against an fp32 evaluation of what was
    quantised: every dequantised value within one e4m3 step of the reference (2^-3 of its magnitude) or within 2^-11 of its
    block's maximum (the fp32 summation noise of values that nearly cancel, and the block's smallest steps), and every block scale the
    smallest power of two that fits the reference's block maximum, give or take one where that maximum sits on a boundary."""
    got = ops.dequantize_hidden_fp8(hq, hsc)
    S, F = ref.shape
    amax = ref.abs().view(S, F // 32, 32).amax(dim=2)
    floor = (amax * 2.0 ** -11).repeat_interleave(32, dim=1)  # (2^-12 of the largest value the block's scale admits: sums that nearly cancel)
    err = (got - ref).abs()
    bad = err > 2.0 ** -3 * ref.abs() + floor + 1e-30
    print(f"{what}: {got.numel()} elements, max-abs {float(err.max()):.3e}, {float((err <= 2.0 ** -4 * 1.01 * ref.abs() + floor).float().mean()):.6f} "
          f"within half a step", flush=True)
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} of {bad.numel()} hidden activations further than an e4m3 step from the fp32 value"
    want_b = torch.ceil(torch.log2(torch.clamp(amax.double(), min=1e-300) / 448.0)).clamp(min=-127.0) + 127.0
    off = (hsc.double() - want_b).abs()
    assert float(off.max()) <= 1 and float((off == 0).double().mean()) > 0.999, f"{what}: block scales"


def _ref_gemm(X, W, cnt):
    """Per-expert fp32 PyTorch GEMM (vendor BLAS), the reference the reference itself intended
    (unit_tests.py:231-235)."""
    out = torch.empty((X.shape[0], W.shape[2]), dtype=torch.float32, device=X.device)
    r0 = 0
    for e, c in enumerate(cnt):
        if c:
            out[r0:r0 + c] = X[r0:r0 + c].float() @ W[e].float()
        r0 += c
    return out


@pytest.mark.parametrize("split", [False, True], ids=["whole_tiles", "k_split"])
@pytest.mark.parametrize("name", ["mixtral", "finegrained"])
def test_bf16_gemms_every_tile_at_full_size(name, split):
    cfg = CONFIGS[name]
    print(f"case {cfg} split={split}", flush=True)
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        world = harness.build_world(cfg, DEV)
        ew, raw, _ = harness.expert_weights(cfg, 0, DEV)
        wg, wu, wd = (w.to(DEV) for w in raw)
        S, H, F = world.S, cfg.hidden, cfg.ffn
        rows, cnt_t = ops.unpack_expert_major(world.recv, world.recv_counts, S)
        cnt = [int(c) for c in cnt_t.cpu().tolist()]
        ws = ops.gemm_part_workspace(DEV) if split else None
        if ws is not None:
            ws.fill_(float("nan"))
        # gate projection alone, no activation: linear, so the projection check applies to it as it stands
        G = torch.full((S, F), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.grouped_gemm_mapped(rows, None, ops.prepack_weights(wg), cnt_t, S, F, "none", G, part_ws=ws)
        _freivalds(G, rows, wg, cnt, f"{name} gate GEMM (no activation)")
        g_ref = _ref_gemm(rows, wg, cnt)
        _close(G, g_ref, f"{name} gate GEMM vs fp32 GEMM")
        # the fused gate/up kernel with its SwiGLU epilogue, every element
        u_ref = _ref_gemm(rows, wu, cnt)
        h_ref = torch.nn.functional.silu(g_ref) * u_ref
        del g_ref, u_ref
        hid = torch.full((S, F), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.grouped_gemm_mapped(rows, None, ew.w1, cnt_t, S, F, "swiglu", hid, part_ws=ws)
        _close(hid, h_ref, f"{name} gate/up GEMM + SwiGLU vs fp32")
        del h_ref
        # down projection on the kernel's own hidden activation
        Y = torch.full((S, H), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.grouped_gemm_mapped(hid, None, ew.w2, cnt_t, S, H, "none", Y, part_ws=ws)
        _freivalds(Y, hid, wd, cnt, f"{name} down GEMM")
        _close(Y, _ref_gemm(hid, wd, cnt), f"{name} down GEMM vs fp32 GEMM")
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev


def _dec(codes):
    return codes.view(torch.float8_e4m3fn).float()


@pytest.mark.parametrize("name", ["zipf_k8", "zipf_k1"])
def test_fp8_gemms_every_tile_at_full_size(name):
    cfg = CONFIGS[name]
    print(f"case {cfg}", flush=True)
    world = harness.build_world(cfg, DEV)
    ew, _, qs = harness.expert_weights(cfg, 0, DEV)
    (gq, gs), (uq, us), (dq, ds) = qs
    S, H, F = world.S, cfg.hidden, cfg.ffn
    rows, cnt_t = ops.unpack_expert_major(world.recv, world.recv_counts, S)
    cnt = [int(c) for c in cnt_t.cpu().tolist()]
    ws = ops.fp8_workspace(S, H, F, DEV)
    sg, su, sd = ew.scales
    y = ops.grouped_mlp_fp8(rows, cnt_t, F, ew.w1, sg, su, ew.w2, sd, ws=ws)
    # gate/up + SwiGLU from the kernel's own row codes and scales (those are bit-exact against the oracle in
    # test_quantize_rows_fp8_bit_exact): e4m3 products are exact in fp32, only the summation order differs
    xd = _dec(ws["xq"])
    h_ref = torch.empty((S, F), dtype=torch.float32, device=DEV)
    r0 = 0
    for e, c in enumerate(cnt):
        if c:
            sx = ws["xs"][r0:r0 + c, None]
            g = (xd[r0:r0 + c] @ _dec(gq[e])) * sx * gs[e][None, :]
            u = (xd[r0:r0 + c] @ _dec(uq[e])) * sx * us[e][None, :]
            h_ref[r0:r0 + c] = torch.nn.functional.silu(g) * u
        r0 += c
    _close_fp8_hidden(ws["hq"], ws["hsc"], h_ref, f"{name} fp8 gate/up GEMM + SwiGLU + block quantisation vs fp32")
    del h_ref, xd
    hd = ops.dequantize_hidden_fp8(ws["hq"], ws["hsc"])  # the operand values of the down projection, exactly
    _freivalds(y, hd, _dec(dq), cnt, f"{name} fp8 down GEMM", col_scale=ds)
    y_ref = torch.empty((S, H), dtype=torch.float32, device=DEV)
    r0 = 0
    for e, c in enumerate(cnt):
        if c:
            y_ref[r0:r0 + c] = (hd[r0:r0 + c] @ _dec(dq[e])) * ds[e][None, :]
        r0 += c
    _close(y, y_ref, f"{name} fp8 down GEMM vs fp32")


def test_projection_check_sees_a_wrong_tile():
    """The check itself: one 256 x 256 tile of a correct product replaced by a neighbouring tile's values, and one tile
    that misses 32 of its K values, must both fail it; the untouched product must pass."""
    torch.manual_seed(0)
    S, K, N = 1024, 2048, 1024
    X = torch.randn((S, K), device=DEV).bfloat16()
    W = (torch.randn((1, K, N), device=DEV) * K ** -0.5).bfloat16()
    Y = (X.float() @ W[0].float()).bfloat16()
    _freivalds(Y, X, W, [S], "intact product")
    swapped = Y.clone()
    swapped[256:512, 512:768] = Y[512:768, 512:768]
    with pytest.raises(AssertionError):
        _freivalds(swapped, X, W, [S], "one tile from the wrong rows")
    short = Y.clone()
    short[0:256, 0:256] = (X[0:256, 32:].float() @ W[0, 32:, 0:256].float()).bfloat16()
    with pytest.raises(AssertionError):
        _freivalds(short, X, W, [S], "one tile short of a K stage")


def test_more_rounds_than_the_tile_table_holds():
    """A workgroup decodes its tiles 256 rounds at a time into a table; a launch of more than 256 rounds (66 048 tiles
    here: 258 row tiles x 256 column tiles on 256 workgroups, K = 64 to keep it cheap) must refill it.  The output rows are
    mapped away (negative map entries store nothing) except a sample that holds every row of the rounds past the first
    table, which is compared with a plain fp32 product."""
    torch.manual_seed(5)
    S, K, N = 66000, 64, 65536
    x = torch.randn((S, K), device=DEV).bfloat16()
    w = (torch.randn((1, K, N), device=DEV) * K ** -0.5).bfloat16()
    cnt = torch.tensor([S], dtype=torch.int32, device=DEV)
    keep = torch.cat([torch.arange(0, 300), torch.arange(30000, 30300), torch.arange(65536 - 200, S)]).to(DEV)
    c_map = torch.full((S,), -1, dtype=torch.int32, device=DEV)
    c_map[keep] = torch.arange(keep.numel(), dtype=torch.int32, device=DEV)
    out = torch.full((keep.numel(), N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops.grouped_gemm_mapped(x, None, ops.prepack_weights(w), cnt, S, N, "none", out, c_row_map=c_map)
    torch.cuda.synchronize()
    ref = x[keep].float() @ w[0].float()
    _close(out, ref, "rows of the first, a middle and the last rounds")


def test_bf16_gemm_over_random_shapes_and_maps():
    """Thirty seeded launches over the corners of the kernel's shape space -- K from two ring stages up, column counts that
    are no multiple of a tile or of a 32-column group, empty and one-row groups, more tiles than workgroups or fewer, row
    maps on either side with dropped (negative) rows, every epilogue, with and without the K-split workspace -- each
    compared element by element with a plain fp32 product of the same operands."""
    rng = np.random.default_rng(2024)
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    ws = ops.gemm_part_workspace(DEV)
    try:
        for case in range(30):
            E_l = int(rng.integers(1, 7))
            K = 64 * int(rng.choice([1, 2, 3, 4, 5, 8, 11, 16]))
            act = str(rng.choice(["none", "none", "swiglu", "gelu", "silu"]))
            N = int(rng.choice([32, 96, 264, 1024, 2080, 4096])) if act != "swiglu" else int(rng.choice([32, 96, 512, 1504, 4096]))
            big = rng.random() < 0.4
            cnt = rng.integers(0, 4000 if big else 300, size=E_l).astype(np.int32)
            cnt[rng.integers(0, E_l)] = int(rng.choice([0, 1, 255, 256, 257]))
            S = int(cnt.sum())
            if S == 0:
                cnt[0] = 5
                S = 5
            n_in, n_out = S + 37, S + 11
            use_amap, use_cmap, split = rng.random() < 0.6, rng.random() < 0.6, rng.random() < 0.5
            print(f"case {case}: E_l={E_l} K={K} N={N} act={act} cnt={cnt.tolist()} a_map={use_amap} c_map={use_cmap} split={split}", flush=True)
            base = torch.from_numpy(rng.standard_normal((n_in, K)).astype(np.float32)).to(DEV).bfloat16()
            w = torch.from_numpy((rng.standard_normal((E_l, K, N)) * K ** -0.5).astype(np.float32)).to(DEV).bfloat16()
            wu = torch.from_numpy((rng.standard_normal((E_l, K, N)) * K ** -0.5).astype(np.float32)).to(DEV).bfloat16() if act == "swiglu" else None
            a_map = rng.permutation(n_in)[:S].astype(np.int32) if use_amap else np.arange(S, dtype=np.int32)
            c_map = rng.permutation(n_out)[:S].astype(np.int32) if use_cmap else np.arange(S, dtype=np.int32)
            dropped = rng.random(S) < 0.02 if use_cmap else np.zeros(S, bool)
            c_map_dev = np.where(dropped, -1, c_map).astype(np.int32)
            out = torch.full((n_out, N), -7.0, dtype=torch.bfloat16, device=DEV)
            ops.grouped_gemm_mapped(base, torch.from_numpy(a_map).to(DEV) if use_amap else None, ops.prepack_weights(w, wu),
                                    torch.from_numpy(cnt).to(DEV), S, N, act, out,
                                    torch.from_numpy(c_map_dev).to(DEV) if use_cmap else None, part_ws=ws if split else None)
            torch.cuda.synchronize()
            x = base[torch.from_numpy(a_map).long().to(DEV)].float()
            ref = torch.empty((S, N), dtype=torch.float32, device=DEV)
            r0 = 0
            for e, c in enumerate(cnt.tolist()):
                if c:
                    g = x[r0:r0 + c] @ w[e].float()
                    if act == "swiglu":
                        g = torch.nn.functional.silu(g) * (x[r0:r0 + c] @ wu[e].float())
                    elif act == "gelu":
                        g = torch.nn.functional.gelu(g)
                    elif act == "silu":
                        g = torch.nn.functional.silu(g)
                    ref[r0:r0 + c] = g
                r0 += c
            kept = torch.from_numpy(~dropped).to(DEV)
            got = out[torch.from_numpy(c_map).long().to(DEV)]
            _close(got[kept], ref[kept], f"case {case}")
            written = np.zeros(n_out, bool)
            written[c_map[~dropped]] = True
            assert bool((out[torch.from_numpy(~written).to(DEV)] == -7.0).all()), f"case {case}: a row outside the map (or a dropped one) was written"
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev


def test_fp8_mlp_over_random_shapes():
    """Twelve seeded fp8 expert MLPs (H, F multiples of 128 from the shortest K up; empty, tiny and large groups; more tiles
    than workgroups or fewer; with and without the K-split workspace), each GEMM compared element by element with an fp32
    product of the decoded codes and scales the kernels themselves used."""
    from helpers import O
    rng = np.random.default_rng(77)
    part = ops.gemm_part_workspace(DEV)
    for case in range(12):
        E_l = int(rng.integers(1, 6))
        H = 128 * int(rng.choice([1, 2, 3, 5, 8, 16]))
        F = 128 * int(rng.choice([1, 2, 3, 11, 16]))
        big = rng.random() < 0.4
        cnt = rng.integers(0, 5000 if big else 300, size=E_l).astype(np.int32)
        cnt[rng.integers(0, E_l)] = int(rng.choice([0, 1, 255, 257]))
        if int(cnt.sum()) == 0:
            cnt[0] = 9
        S = int(cnt.sum())
        split = rng.random() < 0.5
        print(f"case {case}: E_l={E_l} H={H} F={F} cnt={cnt.tolist()} split={split}", flush=True)
        x = torch.from_numpy((rng.standard_normal((S, H)) * rng.uniform(0.3, 3.0, (S, 1))).astype(np.float32)).to(DEV).bfloat16()
        qs = [O.quantize_cols_fp8((rng.standard_normal(sh) * sc).astype(np.float32))
              for sh, sc in (((E_l, H, F), H ** -0.5), ((E_l, H, F), H ** -0.5), ((E_l, F, H), F ** -0.5))]
        (gq, gs), (uq, us), (dq, ds) = [(torch.from_numpy(q).to(DEV), torch.from_numpy(s).to(DEV)) for q, s in qs]
        p1, p2 = ops.prepack_weights_fp8(gq, uq), ops.prepack_weights_fp8(dq)
        ws = ops.fp8_workspace(S, H, F, DEV)
        y = ops.grouped_mlp_fp8(x, torch.from_numpy(cnt).to(DEV), F, p1, gs, us, p2, ds, ws=ws, part_ws=part if split else None)
        torch.cuda.synchronize()
        xd, hd = _dec(ws["xq"]), ops.dequantize_hidden_fp8(ws["hq"], ws["hsc"])
        h_ref = torch.empty((S, F), dtype=torch.float32, device=DEV)
        y_ref = torch.empty((S, H), dtype=torch.float32, device=DEV)
        r0 = 0
        for e, c in enumerate(cnt.tolist()):
            if c:
                sx = ws["xs"][r0:r0 + c, None]
                g = (xd[r0:r0 + c] @ _dec(gq[e])) * sx * gs[e][None, :]
                u = (xd[r0:r0 + c] @ _dec(uq[e])) * sx * us[e][None, :]
                h_ref[r0:r0 + c] = torch.nn.functional.silu(g) * u
                y_ref[r0:r0 + c] = (hd[r0:r0 + c] @ _dec(dq[e])) * ds[e][None, :]
            r0 += c
        _close_fp8_hidden(ws["hq"], ws["hsc"], h_ref, f"case {case} gate/up + SwiGLU + block quantisation")
        _close(y, y_ref, f"case {case} down")
