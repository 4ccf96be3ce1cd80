"""The allocation-free variant of the counting entry point (scratch in a fixed array inside the library) against the
workspace-taking one, through the C ABI: bit-identical outputs on two calls in a row, the second on a smaller input
(the array keeps the first call's contents), then the size limit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from iris_testing_amd import _lib as L  # noqa: E402

DEV = "cuda"
NAMES = ["send_counts", "expert_offs", "dst_sizes", "dst_offsets", "caps", "pos", "row_token"]


def _outputs(T, k, E, W):
    i32 = lambda *s: torch.full(s, -7, dtype=torch.int32, device=DEV)  # noqa: E731
    return [i32(W, E // W), i32(W, E // W), i32(W), i32(W), i32(2), i32(T, k), i32(T * k)]


def _idx(T, k, E, seed):
    rng = np.random.default_rng(seed)
    # distinct experts per token, skewed towards the low ids
    p = 1.0 / np.arange(1, E + 1)
    p /= p.sum()
    return torch.from_numpy(np.stack([rng.choice(E, size=k, replace=False, p=p) for _ in range(T)]).astype(np.int32)).to(DEV)


def _both(T, k, E, W, seed):
    lib = L.lib()
    idx = _idx(T, k, E, seed)
    s = L.stream_ptr()
    want = _outputs(T, k, E, W)
    nbytes = lib.moe_count_workspace_bytes(T, k, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    L.check(lib.moe_count_and_offsets(L.ptr(idx), T, k, E, W, *[L.ptr(t) for t in want], L.ptr(ws), nbytes, s))
    got = _outputs(T, k, E, W)
    before = torch.cuda.memory_allocated()
    L.check(lib.moe_count_and_offsets_static(L.ptr(idx), T, k, E, W, *[L.ptr(t) for t in got], s))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    for name, g, w in zip(NAMES, got, want):
        assert torch.equal(g, w), f"{name} differs between the static-scratch call and the workspace call (T={T} E={E} k={k})"
    assert int(want[0].sum().item()) == T * k


def test_static_scratch_count_matches_workspace_count_twice():
    print("case T=16384 E=256 k=8 W=8, then T=1500 E=60 k=4 W=4, then the small one-block path", flush=True)
    _both(16384, 8, 256, 8, 0)     # multi-kernel path, 256 x 256 histogram cells
    _both(1500, 4, 60, 4, 1)       # smaller input over the same array, stale contents around it
    _both(300, 2, 8, 4, 2)         # few tokens: the one-block kernel, which leaves the array alone
    _both(4096, 2, 8, 8, 3)


def test_static_scratch_rejects_sizes_beyond_the_array():
    lib = L.lib()
    cap = lib.moe_count_static_scratch_bytes()
    T, k, E, W = 1 << 17, 2, 512, 8
    assert lib.moe_count_workspace_bytes(T, k, E) > cap
    idx = torch.zeros((T, k), dtype=torch.int32, device=DEV)
    outs = _outputs(T, k, E, W)
    rc = lib.moe_count_and_offsets_static(L.ptr(idx), T, k, E, W, *[L.ptr(t) for t in outs], L.stream_ptr())
    assert rc == -3 and b"scratch" in lib.moe_last_error()
    torch.cuda.synchronize()
    assert all(bool((t == -7).all()) for t in outs), "a rejected call must not touch its outputs"
