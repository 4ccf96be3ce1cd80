"""CPU-side checks of the product: the C-ABI library loads and exports every symbol the header
declares, the host layer rejects CPU tensors the way the reference does, and nothing in the
package reaches for the oracle."""
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "moe_gfx950.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from iris_testing_amd import _lib as L
    lib = L.lib()
    declared = _declared()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/moe_gfx950.h but not exported"
    assert sorted(L.exported_symbols()) == declared, "ctypes table and header disagree"
    assert lib.moe_abi_version() == 3
    assert lib.moe_last_error() == b""


def test_argument_errors_are_reported_without_a_gpu():
    # calls that fail validation before any HIP call
    from iris_testing_amd import _lib as L
    lib = L.lib()
    rc = lib.moe_count_and_offsets(None, 4, 2, 9, 4, None, None, None, None, None, None, None, None, 0, None)
    assert rc == -1 and b"divisible" in lib.moe_last_error()
    rc = lib.moe_route_topk(None, None, None, 0, 4, 64, 8, 9, None, None, None, None, 0, None)
    assert rc == -1 and b"topk" in lib.moe_last_error()
    rc = lib.moe_route_topk(None, None, None, 1, 4, 60, 8, 2, None, None, None, None, 0, None)
    assert rc == -1 and b"16-byte" in lib.moe_last_error()
    with pytest.raises(L.MoeLibraryError):
        L.check(lib.moe_pack(None, 7, 1, 64, None, None, None, 4, 4, None, None, None, None))
    assert lib.moe_count_workspace_bytes(1000, 2, 8) == 4 * (2 * 8 * 16 + 2 * 8 + 1)


def test_argument_errors_of_the_fused_variants_and_diagnostics_without_a_gpu():
    """The gated / flat-payload / fp8 entry points and the diagnostics validate before they touch the GPU."""
    from iris_testing_amd import _lib as L
    lib = L.lib()
    # gates and their output buffer go together
    rc = lib.moe_pack_tokens_gated(None, 1, 4, 64, None, None, 1, 2, 2, None, None, 2, 4, None, None, None, None)
    assert rc == -1 and b"go together" in lib.moe_last_error()
    rc = lib.moe_recv_row_map_gated(None, 2, 2, 4, 8, 1, None, None, None, None)
    assert rc == -1
    rc = lib.moe_recv_row_map_flat(None, 0, 2, 8, None, None, None)
    assert rc == -1
    # the gated down projection needs its gates; bf16 GEMMs need K % 64 == 0
    rc = lib.moe_grouped_gemm_mapped_gated(1, 8, None, 1, 1, 8, 64, 64, 1, None, 1, 8, None, None, 0, None)
    assert rc == -1 and b"null pointer" in lib.moe_last_error()
    rc = lib.moe_grouped_gemm_mapped_gated(1, 8, None, 1, 1, 8, 48, 64, 1, 1, 1, 8, None, None, 0, None)
    assert rc == -2 and b"K %" in lib.moe_last_error()
    # fp8 expert: H and F in multiples of 128
    rc = lib.moe_grouped_mlp_fp8_q_mapped(1, 1, 8, None, 1, 8, 256, 96, 1, 1, 1, 1, 1, 1, 1, 1, 1, None, 1, 8, None, None, 0, None)
    assert rc == -2 and b"multiples of 128" in lib.moe_last_error()
    rc = lib.moe_grouped_mlp_fp8_mapped(1, 8, None, 1, 8, 200, 128, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, None, 1, 8, None, None, 0, None)
    assert rc == -2 and b"multiples of 128" in lib.moe_last_error()
    # time stamps need a buffer of the advertised size; switching them off needs none
    assert lib.moe_diag_gemm_trace_words() >= 128 + 4096
    rc = lib.moe_diag_gemm_trace(1, 16, 0)
    assert rc == -3 and b"words" in lib.moe_last_error()
    assert lib.moe_diag_gemm_trace(None, 0, 0) == 0
    assert lib.moe_diag_mfma_loop_flops(0, 1, 1) == 2.0 * 4 * 128 * 128 * 32


def test_static_scratch_count_rejects_oversized_inputs_without_a_gpu():
    """The allocation-free counting entry point checks its size limit before it touches the GPU."""
    from iris_testing_amd import _lib as L
    lib = L.lib()
    cap = lib.moe_count_static_scratch_bytes()
    assert cap == 4 << 20
    assert lib.moe_count_workspace_bytes(1 << 17, 2, 512) > cap
    rc = lib.moe_count_and_offsets_static(None, 1 << 17, 2, 512, 8, None, None, None, None, None, None, None, None)
    assert rc == -3 and b"scratch" in lib.moe_last_error()
    assert lib.moe_count_and_offsets_static(None, 64, 0, 8, 4, None, None, None, None, None, None, None, None) == -1


def test_host_layer_rejects_cpu_tensors_like_the_reference():
    from iris_testing_amd import utils
    from iris_testing_amd.baseline import reorder_flat_to_token_buf
    with pytest.raises(AssertionError, match="Expect CUDA tokens"):  # reference utils.py:193
        utils.route_and_pack_padding_free(torch.zeros(4, 8), torch.zeros(8, 4), 1, 2, 4)
    with pytest.raises(AssertionError, match="must be CUDA"):  # reference utils.py:16
        utils.build_expert_offsets(torch.zeros((2, 2), dtype=torch.int32))
    with pytest.raises(ValueError, match="CUDA"):  # reference baseline.py:10-12
        reorder_flat_to_token_buf(torch.zeros(2, 4), torch.zeros((1, 1), dtype=torch.int32), 2, torch.zeros(1, 1, 2, 4))


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "iris_testing_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "harness.py" and "moe_oracle" not in text, \
                    f"{f} mentions the oracle"


def test_configs_and_generators_are_deterministic():
    from iris_testing_amd.configs import CONFIGS, gen_router, gen_router_bias, gen_shard_tokens
    cfg = CONFIGS["plumbing"]
    a, b = gen_shard_tokens(cfg, 1), gen_shard_tokens(cfg, 1)
    assert torch.equal(a, b) and not torch.equal(a, gen_shard_tokens(cfg, 2))
    assert gen_router(cfg).shape == (256, 8)
    z = gen_router_bias(CONFIGS["zipf_k2"])
    assert z.shape == (60,) and torch.all(z[:-1] > z[1:])  # expert 0 hottest
    assert abs(float(torch.exp(z).sum()) - 1) < 1e-5
    for name, c in CONFIGS.items():
        assert c.experts % c.world == 0 and c.topk <= c.experts, name


def test_gemm_split_plan_covers_every_tile_and_every_k_stage_once():
    """The walk of a grouped-GEMM launch (whole tiles, then the tiles of an under-filled last round cut along K) is
    one host/device function; here its host side: every tile appears, the parts of a split tile tile its K range
    exactly, every part has an even, non-zero number of stages, and the part tiles fit the workspace."""
    import ctypes
    import random
    from iris_testing_amd import _lib as L
    lib = L.lib()
    out = (ctypes.c_int32 * 4)()
    rnd = random.Random(3)
    split_seen = 0
    for _ in range(3000):
        grid = rnd.choice([256, 256, 304, 64, 8])
        total = rnd.randint(0, 4 * grid + 5)
        nk = 2 * rnd.randint(1, 400)
        max_units = rnd.choice([grid, grid // 2, 3, 1, 0])
        assert lib.moe_gemm_split_plan(total, grid, nk, max_units, out) == 0
        full, P, nkp, units = out[0], out[1], out[2], out[3]
        tail = total - full
        assert 0 <= full <= total and P >= 1 and units == full + tail * P
        if P == 1:
            assert full == total
            continue
        split_seen += 1
        assert tail == total % grid and 4 * tail <= grid and tail * P <= min(grid, max_units) and P <= 16
        assert nkp % 2 == 0 and nkp >= 8
        stages = [min(nkp, nk - part * nkp) for part in range(P)]
        assert sum(stages) == nk and all(s >= 2 and s % 2 == 0 for s in stages)
    assert split_seen > 100
    # the shapes of the bench workloads: Mixtral-style down GEMM (2064 tiles, 448 stages) and the small config's GEMMs
    for total, nk, want in [(2064, 448, (2048, 16, 28)), (14448, 128, (14448, 1, 128)), (64, 64, (0, 4, 16)), (32, 128, (0, 8, 16))]:
        lib.moe_gemm_split_plan(total, 256, nk, 256, out)
        assert (out[0], out[1], out[2]) == want
    assert lib.moe_gemm_split_plan(10, 0, 8, 4, out) != 0 and lib.moe_gemm_split_plan(10, 8, 7, 4, out) != 0


def test_bench_refuses_more_than_one_gpu():
    """This build has no collectives: bench.py --gpus 2 must say so and exit non-zero without touching a GPU."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "--gpus must be 1" in r.stderr and r.stdout.strip() == ""


def test_ctypes_table_has_the_argument_count_of_every_declaration():
    """Every entry of the ctypes signature table has as many arguments as the header's declaration of that symbol."""
    from iris_testing_amd import _lib as L
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "moe_gfx950.h")).read(), flags=re.S)
    for name, (_, args) in L._SIGNATURES.items():
        m = re.search(r"\b" + name + r"\s*\(([^;]*?)\)\s*;", text, re.S)
        assert m, f"{name} is not declared"
        params = [x for x in m.group(1).split(",") if x.strip() and x.strip() != "void"]
        assert len(params) == len(args), f"{name}: header declares {len(params)} arguments, the ctypes table {len(args)}"
