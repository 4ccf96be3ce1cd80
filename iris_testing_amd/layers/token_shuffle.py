"""Expert-major unpack with the reference's ``shuffle`` signature (layers/token_shuffle.py:7-62).

shuffled[off[e,src] + j] = dispatched_tokens[e, src, j] for j < pca[e, src], off = exclusive prefix
of pca over flattened (e, src) (token_shuffle.py:35-41; kernels.py:179-205): zero padding removed,
rows grouped by local expert, then by source rank, then in arrival order.
"""
from __future__ import annotations

import torch

from .. import ops
from ..utils import _assert_cuda_int32


class TokenShuffle(torch.autograd.Function):

    @staticmethod
    def forward(ctx, dispatched_tokens, pca, token_sync):
        assert dispatched_tokens.is_cuda, "dispatched_tokens must be CUDA"
        _assert_cuda_int32(pca, "pca")
        e_local, world_size = pca.shape
        if token_sync is not None:
            # the reference kernel spins until token_sync[e] >= world_size (kernels.py:192); on one
            # GPU the data is either complete or never will be, so an incomplete counter is an error
            if int(token_sync.min().item()) < world_size:
                raise RuntimeError("token_sync shows an incomplete transfer (expected >= world_size)")
        total = int(pca.sum().item())
        out, _ = ops.shuffle_rows(dispatched_tokens.contiguous(), pca.contiguous(), total)
        ctx.save_for_backward(pca)
        ctx.capacity = dispatched_tokens.shape[2]
        return out

    @staticmethod
    def backward(ctx, grad_shuffled):
        """The shuffle is a row permutation that drops the padding, so its gradient puts row off[e,src] + j back
        at [e, src, j] and leaves zeros in the padding (empty in the reference, token_shuffle.py:58-60)."""
        (pca,) = ctx.saved_tensors
        grad = ops.shuffle_rows_backward(grad_shuffled.contiguous(), pca.contiguous(), ctx.capacity)
        return grad, None, None


shuffle = TokenShuffle.apply
