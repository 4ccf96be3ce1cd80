"""Host-side mirror of the reference's ``utils.py`` for the dispatch path.

Same names, argument order, return types and assertion behaviour as the reference
(utils.py:14-31, 34-121, 125-261); the device work goes through the HIP kernels
(`iris_testing_amd.ops`) instead of Python loops and torch ops.  There is no Iris symmetric heap on
a single GPU: the ``shmem`` argument of the allocators may be ``None`` (plain device tensors) or
any object with a ``zeros(shape, dtype=..., device=...)`` method.
"""
from __future__ import annotations

import random
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import ops


def _assert_cuda_int32(x: torch.Tensor, name: str) -> None:  # reference utils.py:14-17
    assert x.is_cuda, f"{name} must be CUDA"
    assert x.dtype == torch.int32, f"{name} must be int32"


def build_expert_offsets(send_counts: torch.Tensor) -> torch.Tensor:
    """expert_offs[dst, e] = row offset of expert e inside the dst block (reference utils.py:20-31)."""
    _assert_cuda_int32(send_counts, "send_counts")
    return ops.build_expert_offsets(send_counts.contiguous())


@dataclass
class ShmemBuffers:  # reference utils.py:34-46
    pca: torch.Tensor           # [E, world] int32
    counts_ready: torch.Tensor  # [1] int32
    token_buf: torch.Tensor     # [E, world, CAP, H]
    token_sync: torch.Tensor    # [E] int32
    heap_bases: Optional[torch.Tensor]


@dataclass
class CountsBuffers:  # reference utils.py:81-84 (a dataclass here; the reference forgot the decorator)
    pca: torch.Tensor
    counts_ready: torch.Tensor
    heap_bases: Optional[torch.Tensor]


@dataclass
class TokenBuffers:  # reference utils.py:95-98
    token_buf: torch.Tensor
    token_sync: torch.Tensor


def _zeros(shmem, shape, dtype):
    if shmem is None:
        return torch.zeros(shape, dtype=dtype, device="cuda")
    return shmem.zeros(shape, dtype=dtype, device="cuda")


def _heap_bases(shmem):
    return shmem.get_heap_bases() if shmem is not None and hasattr(shmem, "get_heap_bases") else None


def alloc_shmem_buffers(shmem, world_size: int, e_local: int, capacity: int, hidden_dim: int,
                        token_dtype: torch.dtype) -> ShmemBuffers:  # reference utils.py:49-80
    return ShmemBuffers(
        pca=_zeros(shmem, (e_local, world_size), torch.int32),
        counts_ready=_zeros(shmem, (1,), torch.int32),
        token_buf=_zeros(shmem, (e_local, world_size, capacity, hidden_dim), token_dtype),
        token_sync=_zeros(shmem, (e_local,), torch.int32),
        heap_bases=_heap_bases(shmem),
    )


def alloc_counts_buffers(shmem, world_size: int, e_local: int) -> CountsBuffers:  # reference utils.py:100-104
    return CountsBuffers(pca=_zeros(shmem, (e_local, world_size), torch.int32),
                         counts_ready=_zeros(shmem, (1,), torch.int32), heap_bases=_heap_bases(shmem))


def alloc_token_buffers(shmem, world_size: int, e_local: int, capacity: int, hidden_dim: int,
                        token_dtype: torch.dtype) -> TokenBuffers:  # reference utils.py:106-116
    return TokenBuffers(token_buf=_zeros(shmem, (e_local, world_size, capacity, hidden_dim), token_dtype),
                        token_sync=_zeros(shmem, (e_local,), torch.int32))


def reset_counts_sync(cb: CountsBuffers) -> None:
    cb.counts_ready.zero_()


def reset_token_sync(tb: TokenBuffers) -> None:
    tb.token_sync.zero_()


def reset_token_buf_debug(tb: TokenBuffers) -> None:
    tb.token_buf.zero_()


def compute_capacity_from_pca(pca: torch.Tensor) -> int:
    """CAP = max(1, max over ranks of pca.max()) (reference utils.py:118-121).

    One GPU holds every simulated rank, so the all-reduce MAX of the reference becomes the max
    over whatever ``pca`` holds (pass the stacked per-rank arrays to get the global value).
    """
    _assert_cuda_int32(pca, "pca")
    return int(ops.max_floor1(pca.contiguous().view(-1)).item())


def pair_capacity(dst_sizes_all: torch.Tensor) -> int:
    """M = max over (src, dst) of the rows one device sends another, floored at 1 (reference README.md:4-7)."""
    _assert_cuda_int32(dst_sizes_all, "dst_sizes")
    return int(ops.max_floor1(dst_sizes_all.contiguous().view(-1)).item())


def set_seed(base_seed: int, rank: int) -> None:  # reference utils.py:125-139
    seed = int(base_seed) + int(rank)
    random.seed(seed)
    try:
        import numpy as np
        np.random.seed(seed)
    except Exception:
        pass
    torch.manual_seed(seed)


def gen_local_tokens(batch: int, seq: int, hidden_dim: int, dtype: torch.dtype, device, base_seed: int,
                     rank: int) -> torch.Tensor:
    """Uniform [0,1) tokens seeded base_seed + rank (reference utils.py:142-154); generated on the
    CPU generator and copied, so CPU and GPU consumers see identical bits."""
    g = torch.Generator(device="cpu")
    g.manual_seed(int(base_seed) + int(rank))
    return torch.rand(batch * seq, hidden_dim, generator=g, dtype=torch.float32).to(dtype).to(device)


def gen_router(hidden_dim: int, num_experts: int, dtype: torch.dtype, device, base_seed: int) -> torch.Tensor:
    """Router [H, E] ~ 0.001 * N(0,1), seeded base_seed + 777, same on every rank (reference utils.py:157-173)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(int(base_seed) + 777)
    return (torch.randn(hidden_dim, num_experts, generator=g, dtype=torch.float32) * 0.001).to(dtype).to(device)


def gen_local_weights(e_local: int, hidden_dim: int, out_dim: int, dtype: torch.dtype, device, base_seed: int,
                      rank: int) -> torch.Tensor:
    """Expert weights [E_local, H, F] ~ N(0, 0.02), seeded base_seed + 12345 + rank (reference utils.py:248-261)."""
    g = torch.Generator(device="cpu")
    g.manual_seed(int(base_seed) + 12345 + int(rank))
    return (torch.randn(e_local, hidden_dim, out_dim, generator=g, dtype=torch.float32) * 0.02).to(dtype).to(device)


def route_and_pack_padding_free(
    tokens: torch.Tensor,
    router: torch.Tensor,
    topk: int,
    world_size: int,
    num_experts_total: int,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Padding-free routing -> (send_payload, send_counts, send_dst_offsets, send_dst_sizes).

    Same contract as the reference (utils.py:176-246): send_payload is DEST-major then
    EXPERT-local-major, rows of a bucket in ascending token order; send_counts int32 [world, E_local];
    send_dst_offsets / send_dst_sizes int32 [world].  Empty [0, H] payload when nothing is routed.
    """
    assert tokens.is_cuda, "Expect CUDA tokens"
    assert num_experts_total % world_size == 0, "num_experts_total must be divisible by world_size"
    tokens = tokens.contiguous()
    router = router.contiguous()
    if tokens.shape[0] == 0:
        e_local = num_experts_total // world_size
        z = lambda *s: torch.zeros(s, dtype=torch.int32, device=tokens.device)  # noqa: E731
        return (torch.empty((0, tokens.shape[1]), dtype=tokens.dtype, device=tokens.device), z(world_size, e_local),
                z(world_size), z(world_size))
    idx, _, _ = ops.route_topk(tokens, router, topk)
    c = ops.count_and_offsets(idx, num_experts_total, world_size)
    payload = ops.pack_payload(tokens, c.row_token)
    return payload, c.send_counts, c.dst_offsets, c.dst_sizes
