"""The diagnostic entry points: they must not change what the product kernels compute.

moe_diag_gemm_trace switches the forward grouped-GEMM launches of the process to an instantiation of the same kernel that
writes wall-clock stamps; the output must stay bit-identical, the stamps must be ordered, and switching it off must bring
the product instantiation back.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from iris_testing_amd import _lib as L, ops  # noqa: E402

DEV = "cuda"
TW = 256  # stamp words per workgroup


def _trace(buf, flags):
    L.check(L.lib().moe_diag_gemm_trace(None if buf is None else buf.data_ptr(), 0 if buf is None else buf.numel(), flags))


@pytest.mark.parametrize("act", ["none", "swiglu"])
def test_gemm_trace_keeps_the_result_and_orders_its_stamps(act):
    g = torch.Generator(device="cpu").manual_seed(7)
    # enough 256-row tiles that the launcher takes the 256-row kernel (31 row tiles x 8 column tiles, one round of the grid)
    E_l, K, N = 3, 256, 2048 if act == "none" else 1024
    rows = (256 * 11, 256 * 10 + 7, 256 * 8 + 249)
    S = sum(rows)
    x = torch.randn((S, K), generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn((E_l, K, N), generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    wu = (torch.randn((E_l, K, N), generator=g) * 0.05).to(torch.bfloat16).to(DEV) if act == "swiglu" else None
    packed = ops.prepack_weights(w, wu)
    cnt = torch.tensor(rows, dtype=torch.int32, device=DEV)
    want = torch.full((S, N), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.grouped_gemm_mapped(x, None, packed, cnt, S, N, act, want)

    words = L.lib().moe_diag_gemm_trace_words()
    n_wg = (words - 4096) // TW
    buf = torch.zeros(words, dtype=torch.int64, device=DEV)
    with pytest.raises(L.MoeLibraryError):
        _trace(buf[:100], 0)  # too small a buffer is refused
    got = torch.full((S, N), 7.0, dtype=torch.bfloat16, device=DEV)
    untouched = torch.full((S, N), 7.0, dtype=torch.bfloat16, device=DEV)
    try:
        _trace(buf, 0)
        ops.grouped_gemm_mapped(x, None, packed, cnt, S, N, act, got)
        torch.cuda.synchronize()
        h = buf.cpu().numpy()
        buf.zero_()
        _trace(buf, 1)  # the epilogue stores nothing
        ops.grouped_gemm_mapped(x, None, packed, cnt, S, N, act, untouched)
        # launches the selection leaves out are not traced: this one is the product kernel
        _trace(buf, 0x200 if act == "none" else 0x100)
        buf.zero_()
        again = torch.empty_like(want)
        ops.grouped_gemm_mapped(x, None, packed, cnt, S, N, act, again)
        torch.cuda.synchronize()
        assert int(buf.abs().sum().item()) == 0
        # a launch the time-stamping instantiation does not cover is refused, not run untraced
        _trace(buf, 0)
        few = torch.empty((300, N), dtype=torch.bfloat16, device=DEV)
        with pytest.raises(L.MoeLibraryError):
            ops.grouped_gemm_mapped(x, None, packed, torch.tensor([300, 0, 0], dtype=torch.int32, device=DEV), 300, N, act, few)
    finally:
        _trace(None, 0)
    assert torch.equal(got, want)
    assert torch.equal(again, want)
    assert bool((untouched == 7.0).all())
    # stamps: per workgroup 3 per tile, non-decreasing; all tiles accounted for
    n_col_tiles = (N * (2 if act == "swiglu" else 1)) // 256
    n_tiles = sum((r + 255) // 256 for r in rows) * n_col_tiles
    tiles = h[:n_wg * TW].reshape(n_wg, TW)
    seen = 0
    for wg in range(n_wg):
        ev = tiles[wg][tiles[wg] > 0]
        assert len(ev) % 3 == 0
        assert np.all(np.diff(ev) >= 0), f"workgroup {wg}: stamps out of order"
        seen += len(ev) // 3
    assert seen == n_tiles
    blocks = h[n_wg * TW:]
    blocks = blocks[blocks > 0]
    nk = K * 2 // 64
    assert len(blocks) == (len(tiles[0][tiles[0] > 0]) // 3) * nk and np.all(np.diff(blocks) >= 0)
    # and with the switch off the product kernel runs again
    after = torch.empty_like(want)
    ops.grouped_gemm_mapped(x, None, packed, cnt, S, N, act, after)
    assert torch.equal(after, want)


def test_mfma_loop_runs_and_counts_its_flops():
    lib = L.lib()
    sink = torch.empty(lib.moe_diag_mfma_loop_sink_floats(), dtype=torch.float32, device=DEV)
    for fp8 in (0, 1):
        for rnd in (0, 1):
            L.check(lib.moe_diag_mfma_loop(fp8, rnd, 10, 8, L.ptr(sink), L.stream_ptr()))
    torch.cuda.synchronize()
    # 4 waves x 128 x 128 outputs per workgroup, K = 32 (bf16) or 64 (fp8) per pass
    assert lib.moe_diag_mfma_loop_flops(0, 10, 8) == 2.0 * 4 * 128 * 128 * 32 * 10 * 8
    assert lib.moe_diag_mfma_loop_flops(1, 10, 8) == 2.0 * 4 * 128 * 128 * 64 * 10 * 8
