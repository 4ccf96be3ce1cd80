"""Writes tests/golden/dispatch_small.npz: the dispatch path on one tiny seeded case, frozen.

    python tests/golden/make_fixtures.py

The reference holds no data files for this path (its tests compute their expectations on 8 GPUs at run
time), so these vectors come from this repository's CPU oracle, after that oracle was pinned by the
independent checks of tests/test_oracle_*.py.  Their job is to keep the oracle, and through it the
kernels, from drifting: inputs and every intermediate of route -> count -> pack -> unpack -> return ->
combine for W = 3 simulated ranks, T = 40 tokens of H = 32 per shard, E = 12 experts, top-3, as
plain arrays.  Integer and index arrays and the packed buffers are exact; gates are fp32 values.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import moe_oracle as O  # noqa: E402

W, T, H, E, K = 3, 40, 32, 12, 3


def build():
    rng = np.random.default_rng(20240607)
    router = (rng.standard_normal((H, E)) / np.sqrt(H)).astype(np.float32)
    bias = rng.standard_normal(E).astype(np.float32)
    xs = [rng.standard_normal((T, H)).astype(np.float32) for _ in range(W)]
    out = {"router": router, "bias": bias}
    routes = []
    for s, x in enumerate(xs):
        idx, gate, logits = O.route(x, router, K, bias)
        counts = O.send_counts(idx, W, E)
        sizes, offs = O.dst_sizes_offsets(counts)
        pos, row_token = O.payload_positions(idx, E)
        routes.append((idx, gate, counts, sizes, offs, pos, row_token))
        out.update({f"x{s}": x, f"idx{s}": idx, f"gate{s}": gate, f"logits{s}": logits, f"counts{s}": counts,
                    f"pos{s}": pos, f"row_token{s}": row_token})
    M = O.pair_capacity(np.stack([r[3] for r in routes]))
    CAP = O.compute_capacity_from_pca(np.stack([r[2] for r in routes]))
    sends = [O.pack_fixed_m(O.send_payload(x, r[6]), r[4], r[3], M) for x, r in zip(xs, routes)]
    recv = np.stack([s[0] for s in sends])                      # what rank 0 receives
    rc = np.stack([r[2][0] for r in routes]).astype(np.int32)   # recv_counts[s, e]
    token_buf, pca = O.recv_to_token_buf(recv, rc, CAP)
    rows = O.unpack_expert_major(recv, rc)
    ret = O.return_pack(rows * 2.0, rc, M)                      # "expert" = doubling: exact in fp32
    # rank 0 as a source again: every rank applies the same doubling, so slot d of what comes back is 2 * send0[d]
    returned = 2.0 * sends[0]
    idx0, gate0, _, _, offs0, pos0, _ = routes[0]
    combined = O.combine(returned, idx0, pos0, gate0, offs0, E // W, "f32")
    out.update({"M": np.int32(M), "CAP": np.int32(CAP), "send0": sends[0], "recv": recv, "recv_counts": rc,
                "token_buf": token_buf, "pca": pca, "rows": rows, "ret": ret, "combined": combined})
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dispatch_small.npz")
    np.savez_compressed(path, **build())
    print("wrote", path, os.path.getsize(path), "bytes")
