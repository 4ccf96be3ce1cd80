"""ctypes binding of libmoe_gfx950.so (the C ABI declared in include/moe_gfx950.h).

There is no CPU fallback: if the library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_size_t, c_uint8, c_void_p, POINTER

import torch  # noqa: F401  (must be imported first: the library binds the HIP runtime torch loaded)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmoe_gfx950.so")

MOE_F32, MOE_BF16 = 0, 1
ACT = {"none": 0, "gelu": 1, "silu": 2, "swiglu": 3}
MOE_MAX_EXPERTS = 512
MOE_MAX_TOPK = 16


class MoeLibraryError(RuntimeError):
    """A C-ABI call returned an error code."""

    def __init__(self, code: int, text: str):
        super().__init__(f"libmoe_gfx950 error {code}: {text}")
        self.code = code
        self.text = text


P = c_void_p
_SIGNATURES = {
    "moe_abi_version": (c_int, []),
    "moe_last_error": (c_char_p, []),
    "moe_route_workspace_bytes": (c_size_t, [c_int, c_int]),
    "moe_route_topk": (c_int, [P, P, P, c_int, c_int, c_int, c_int, c_int, P, P, P, P, c_size_t, P]),
    "moe_count_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "moe_count_and_offsets": (c_int, [P, c_int, c_int, c_int, c_int, P, P, P, P, P, P, P, P, c_size_t, P]),
    "moe_count_static_scratch_bytes": (c_size_t, []),
    "moe_count_and_offsets_static": (c_int, [P, c_int, c_int, c_int, c_int, P, P, P, P, P, P, P, P]),
    "moe_build_expert_offsets": (c_int, [P, c_int, c_int, P, P, P, P]),
    "moe_max_floor1": (c_int, [P, c_int, P, P]),
    "moe_pack_payload": (c_int, [P, c_int, c_int, c_int, P, c_int, P, P]),
    "moe_pack": (c_int, [P, c_int, c_int, c_int, P, P, P, c_int, c_int, P, P, P, P]),
    "moe_pack_tokens": (c_int, [P, c_int, c_int, c_int, P, P, c_int, c_int, P, P, c_int, c_int, P, P, P]),
    "moe_pack_tokens_gated": (c_int, [P, c_int, c_int, c_int, P, P, P, c_int, c_int, P, P, c_int, c_int, P, P, P, P]),
    "moe_pack_tokens_fp8_gated": (c_int, [P, c_int, c_int, P, P, P, c_int, c_int, P, P, c_int, c_int, P, P, P, P, P]),
    "moe_recv_row_map_flat": (c_int, [P, c_int, c_int, c_int, P, P, P]),
    "moe_recv_row_map_gated": (c_int, [P, c_int, c_int, c_int, c_int, P, P, P, P, P]),
    "moe_grouped_gemm_mapped_gated": (c_int, [P, c_int, P, P, P, c_int, c_int, c_int, c_int, P, P, c_int, P, P, c_size_t, P]),
    "moe_recv_map_ints": (c_size_t, [c_int, c_int, c_int]),
    "moe_unpack_token_buf": (c_int, [P, c_int, c_int, c_int, c_int, P, c_int, c_int, P, P, P, P, P]),
    "moe_reorder_flat_to_token_buf": (c_int, [P, c_int, c_int, c_int, P, c_int, c_int, c_int, P, P, P, P]),
    "moe_shuffle": (c_int, [P, c_int, c_int, c_int, c_int, c_int, P, P, c_int, P, P, P]),
    "moe_shuffle_backward": (c_int, [P, c_int, c_int, c_int, c_int, c_int, P, P, P, P]),
    "moe_unpack_expert_major": (c_int, [P, c_int, c_int, c_int, c_int, P, c_int, P, c_int, P, P, P]),
    "moe_prepack_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "moe_prepack_weights": (c_int, [P, P, c_int, c_int, c_int, c_int, P, P]),
    "moe_grouped_gemm": (c_int, [P, P, P, c_int, c_int, c_int, c_int, c_int, P, P, c_size_t, P]),
    "moe_grouped_gemm_packed": (c_int, [P, P, P, c_int, c_int, c_int, c_int, c_int, P, P]),
    "moe_grouped_mlp": (c_int, [P, P, c_int, c_int, c_int, c_int, c_int, c_int, P, P, P, P, P, P]),
    "moe_prepack_weights_fp8": (c_int, [P, P, c_int, c_int, c_int, P, P]),
    "moe_quantize_rows_fp8": (c_int, [P, c_int, c_int, P, P, P, P]),
    "moe_grouped_mlp_fp8": (c_int, [P, P, c_int, c_int, c_int, c_int, P, P, P, P, P, P, P, P, P, P, P]),
    "moe_return_pack": (c_int, [P, c_int, c_int, c_int, P, c_int, c_int, c_int, P, P, P]),
    "moe_recv_row_map": (c_int, [P, c_int, c_int, c_int, c_int, P, P, P, P]),
    "moe_grouped_gemm_mapped": (c_int, [P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, P, c_int, P, P, c_size_t, P]),
    "moe_pack_tokens_fp8": (c_int, [P, c_int, c_int, P, P, c_int, c_int, P, P, c_int, c_int, P, P, P, P]),
    "moe_grouped_mlp_fp8_q_mapped": (c_int, [P, P, c_int, P, P, c_int, c_int, c_int, c_int, P, P, P, P, P, P, P, P, P, P, c_int,
                                             P, P, c_size_t, P]),  # (.., xs_ws, hq_ws, hscale_ws, row_gate, out, out_rows, ..)
    "moe_grouped_gemm_act_keep": (c_int, [P, c_int, P, P, P, c_int, c_int, c_int, c_int, c_int, P, P, P, c_size_t, P]),
    "moe_gemm_part_workspace_bytes": (c_size_t, []),
    "moe_prepack_weights_transposed": (c_int, [P, P, c_int, c_int, c_int, c_int, P, P]),
    "moe_dw_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "moe_grouped_gemm_dw": (c_int, [P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, P, P, c_size_t, P]),
    "moe_transpose_weights_f32": (c_int, [P, c_int, c_int, c_int, P, P]),
    "moe_mlp_act_backward": (c_int, [P, P, c_int, c_int, c_int, c_int, P, P]),
    "moe_combine_backward": (c_int, [P, P, c_int, c_int, c_int, c_int, P, P, P, P, P, c_int, c_int, c_int, P, P, P]),
    "moe_gemm_split_plan": (c_int, [c_int, c_int, c_int, c_int, P]),
    "moe_zero_padding_rows": (c_int, [P, c_int, c_int, c_int, c_int, P, c_int, P]),
    "moe_grouped_mlp_fp8_mapped": (c_int, [P, c_int, P, P, c_int, c_int, c_int, c_int, P, P, P, P, P, P, P, P, P, P, P, c_int, P, P,
                                           c_size_t, P]),  # (.., xq_ws, xs_ws, hq_ws, hscale_ws, row_gate, out, out_rows, ..)
    "moe_diag_mfma_loop_sink_floats": (c_size_t, []),
    "moe_diag_mfma_loop_flops": (ctypes.c_double, [c_int, c_int, c_int]),
    "moe_diag_mfma_loop": (c_int, [c_int, c_int, c_int, c_int, P, P]),
    "moe_diag_gemm_trace_words": (c_size_t, []),
    "moe_diag_gemm_trace": (c_int, [P, c_size_t, c_int]),
    "moe_combine": (c_int, [P, c_int, c_int, c_int, c_int, P, P, P, P, c_int, c_int, c_int, P, P, P]),
}

_lib = None


def exported_symbols():
    """Names the header declares (used by the load/export test)."""
    return sorted(_SIGNATURES)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m iris_testing_amd.csrc.build` "
                "(there is no CPU fallback for the HIP path)")
        l = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(l, name)  # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise MoeLibraryError(rc, lib().moe_last_error().decode("utf-8", "replace"))


def ptr(t) -> int:
    """Device pointer of a tensor (None -> NULL)."""
    if t is None:
        return None
    return t.data_ptr()


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return MOE_F32
    if dt == torch.bfloat16:
        return MOE_BF16
    raise TypeError(f"unsupported token dtype {dt}; expected float32 or bfloat16")
