"""Pins the oracle's expert math (a11, a12) against float64 / torch.nn.functional on the CPU."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import O


@pytest.mark.parametrize("E_l,K,N", [(2, 24, 48), (5, 128, 128)])  # the reference's intended cases (unit_tests.py:247-248)
def test_grouped_gemm_against_per_group_einsum(E_l, K, N):
    rng = np.random.default_rng(K)
    cnt = rng.integers(0, 100, size=E_l).astype(np.int32)  # unit_tests.py:116
    cnt[0] = 0
    x = rng.standard_normal((int(cnt.sum()), K)).astype(np.float32)
    w = rng.standard_normal((E_l, K, N)).astype(np.float32)
    out = O.grouped_gemm(x, w, cnt, "f32")
    r = 0
    for e in range(E_l):
        c = cnt[e]
        want = np.einsum("sd,df->sf", x[r:r + c].astype(np.float64), w[e].astype(np.float64))  # unit_tests.py:233
        np.testing.assert_allclose(out[r:r + c], want, rtol=1e-2, atol=1e-4)  # reference rtol (unit_tests.py:237)
        np.testing.assert_allclose(out[r:r + c], want, rtol=1e-5, atol=1e-4)
        r += c
    # identity weights give exact copies
    eye = np.tile(np.eye(K, dtype=np.float32), (E_l, 1, 1))
    assert np.array_equal(O.grouped_gemm(x, eye, cnt, "f32"), x)
    # bf16 output is the rounded fp32 result
    assert np.array_equal(O.grouped_gemm(x, w, cnt, "bf16"), O.bf16_round(out))


@pytest.mark.parametrize("act", ["gelu", "silu", "swiglu"])
def test_expert_mlp_against_torch_functional(act):
    rng = np.random.default_rng(11)
    E_l, H, Fd = 3, 32, 48
    cnt = np.array([7, 0, 12], np.int32)
    x = rng.standard_normal((19, H)).astype(np.float32)
    w1 = rng.standard_normal((E_l, H, Fd)).astype(np.float32) / 6
    wu = rng.standard_normal((E_l, H, Fd)).astype(np.float32) / 6
    w2 = rng.standard_normal((E_l, Fd, H)).astype(np.float32) / 7
    out = O.expert_mlp(x, cnt, w1, w2, act, "f32", w_up=wu if act == "swiglu" else None)
    r = 0
    for e in range(E_l):
        c = cnt[e]
        xe = torch.from_numpy(x[r:r + c]).double()
        a = xe @ torch.from_numpy(w1[e]).double()
        if act == "gelu":
            h = F.gelu(a)  # erf form
        elif act == "silu":
            h = F.silu(a)
        else:
            h = F.silu(a) * (xe @ torch.from_numpy(wu[e]).double())
        want = (h @ torch.from_numpy(w2[e]).double()).numpy()
        np.testing.assert_allclose(out[r:r + c], want, rtol=2e-5, atol=2e-6)
        r += c


def test_fp8_mlp_is_the_dequantised_mlp():
    rng = np.random.default_rng(12)
    E_l, H, Fd = 2, 64, 32
    cnt = np.array([9, 5], np.int32)
    x = O.bf16_round(rng.standard_normal((14, H)).astype(np.float32))
    wg, wu = (rng.standard_normal((E_l, H, Fd)).astype(np.float32) / 8 for _ in range(2))
    wd = rng.standard_normal((E_l, Fd, H)).astype(np.float32) / 6
    (gq, gs), (uq, us), (dq, ds) = (O.quantize_cols_fp8(w) for w in (wg, wu, wd))
    # per-channel quantisation reproduces the weights to fp8 precision
    np.testing.assert_allclose(O.fp8_e4m3_decode(gq) * gs[:, None, :], wg, rtol=2.0 ** -4, atol=1e-4)
    out = O.expert_mlp_fp8(x, cnt, gq, gs, uq, us, dq, ds)
    ref = O.expert_mlp(x, cnt, wg, wd, "swiglu", "f32", w_up=wu)
    rms = np.sqrt((ref ** 2).mean())
    assert np.abs(out - ref).max() < 0.25 * rms  # fp8 noise, far below signal
