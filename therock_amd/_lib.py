"""Loader and ctypes prototypes of libmi355_moe.so (the C ABI declared in include/mi355_moe.h).

The library is built in-tree by ``therock_amd.build`` (hipcc, gfx950).  There is no fallback: if
it is missing, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# MI355_MOE_LIB names another build of the same library (A/B timing of two builds in one process each)
LIB_PATH = os.environ.get("MI355_MOE_LIB") or os.path.join(_HERE, "libmi355_moe.so")

OK, E_UNSUPPORTED, E_INVALID, E_HIP, E_WORKSPACE = 0, -1, -2, -3, -4
DTYPES = {"bf16": 0, "fp8": 1, "int8": 2, "fp32": 3, "int32": 4, "fp16": 5}


class SortingArgs(C.Structure):
    _fields_ = [
        ("p_topk_ids", C.c_void_p), ("p_weights", C.c_void_p), ("p_local_expert_mask", C.c_void_p),
        ("p_local_tokens", C.c_void_p), ("p_sorted_token_ids", C.c_void_p), ("p_sorted_weights", C.c_void_p),
        ("p_sorted_expert_ids", C.c_void_p), ("p_total_tokens_post_pad", C.c_void_p), ("p_moe_buf", C.c_void_p),
        ("p_ws", C.c_void_p), ("tokens", C.c_int32), ("unit_size", C.c_int32), ("num_experts", C.c_int32),
        ("topk", C.c_int32), ("moe_buf_interm_dim", C.c_int32), ("moe_buf_elem_bytes", C.c_int32),
    ]


class SortingTraits(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "index_type", "weight_type", "local_expert_masking", "clear_workspace_inside_api", "dispatch_policy",
        "skip_experts_with_zero_tokens")]


class FusedMoeTraits(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "prec_i", "prec_w", "prec_o", "prec_st", "prec_sw", "prec_sq", "prec_kw", "block_m", "activation",
        "gate_only", "fused_quant", "local_expert_masking", "weight_permute")]


class FusedMoeGemmArgs(C.Structure):
    _fields_ = [
        ("a_ptr", C.c_void_p), ("a_scale_ptr", C.c_void_p), ("g_ptr", C.c_void_p), ("d_ptr", C.c_void_p),
        ("g_scale_ptr", C.c_void_p), ("d_scale_ptr", C.c_void_p), ("y_smooth_scale_ptr", C.c_void_p),
        ("o_ptr", C.c_void_p), ("sorted_token_ids_ptr", C.c_void_p), ("sorted_weight_ptr", C.c_void_p),
        ("sorted_expert_ids_ptr", C.c_void_p), ("num_sorted_tiles_ptr", C.c_void_p),
        ("hidden_size", C.c_int32), ("intermediate_size", C.c_int32),
        ("num_tokens", C.c_int32), ("num_experts", C.c_int32), ("topk", C.c_int32), ("stride_token", C.c_int32),
    ]


class FusedMoeArgs(C.Structure):
    _fields_ = [
        ("a_ptr", C.c_void_p), ("a_scale_ptr", C.c_void_p), ("g_ptr", C.c_void_p), ("d_ptr", C.c_void_p),
        ("g_scale_ptr", C.c_void_p), ("d_scale_ptr", C.c_void_p), ("y_smooth_scale_ptr", C.c_void_p),
        ("local_expert_mask_ptr", C.c_void_p), ("o_ptr", C.c_void_p), ("ws_ptr", C.c_void_p),
        ("topk_ids_ptr", C.c_void_p), ("topk_weight_ptr", C.c_void_p),
        ("sorted_token_ids_ptr", C.c_void_p), ("sorted_weight_ptr", C.c_void_p),
        ("sorted_expert_ids_ptr", C.c_void_p), ("num_sorted_tiles_ptr", C.c_void_p), ("block_m", C.c_int32),
        ("hidden_size", C.c_int32), ("intermediate_size", C.c_int32), ("num_tokens", C.c_int32),
        ("num_experts", C.c_int32), ("topk", C.c_int32), ("stride_token", C.c_int32),
    ]


class TopkSoftmaxArgs(C.Structure):
    _fields_ = [
        ("p_input", C.c_void_p), ("p_output", C.c_void_p), ("p_indices", C.c_void_p), ("num_rows", C.c_int32),
        ("num_experts", C.c_int32), ("topk", C.c_int32), ("stride_input", C.c_int32), ("stride_output", C.c_int32),
    ]


class TopkSoftmaxTraits(C.Structure):
    _fields_ = [
        ("input_type", C.c_int32), ("weight_type", C.c_int32), ("experts", C.c_int32), ("activation", C.c_int32),
        ("renormalize", C.c_int32),
    ]


class FlatmmArgs(C.Structure):
    _fields_ = [
        ("p_sorted_token_ids", C.c_void_p), ("p_sorted_expert_weights", C.c_void_p), ("p_sorted_expert_ids", C.c_void_p),
        ("p_max_token_id", C.c_void_p), ("a_ptr", C.c_void_p), ("b_ptr", C.c_void_p), ("c_ptr", C.c_void_p),
        ("NumTokens", C.c_int32), ("NumExperts", C.c_int32), ("TopK", C.c_int32), ("k_batch", C.c_int32),
        ("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("stride_A", C.c_int32), ("stride_B", C.c_int32),
        ("stride_C", C.c_int32), ("n_padded_zeros", C.c_int32), ("k_padded_zeros", C.c_int32),
        ("scale_m", C.c_void_p), ("scale_n", C.c_void_p), ("exp_bias", C.c_void_p), ("prec_a", C.c_int32),
        ("prec_b", C.c_int32), ("block_m", C.c_int32), ("activation", C.c_int32), ("swiglu_alpha", C.c_float),
        ("swiglu_limit", C.c_float), ("b_shuffle", C.c_int32),
    ]


class Workspace(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("bytes", C.c_size_t)]


class SmoothquantArgs(C.Structure):
    _fields_ = [
        ("p_x", C.c_void_p), ("p_smscale", C.c_void_p), ("p_topk_ids", C.c_void_p), ("p_yscale", C.c_void_p),
        ("p_qy", C.c_void_p), ("tokens", C.c_int32), ("hidden_size", C.c_int32), ("experts", C.c_int32),
        ("topk", C.c_int32), ("x_stride", C.c_int32), ("y_stride", C.c_int32),
    ]


# every symbol include/mi355_moe.h declares: name -> (restype, argtypes)
PROTOTYPES = {
    "mi355_moe_max_num_tokens_padded": (C.c_int64, [C.c_int32] * 4),
    "mi355_moe_sorting_workspace_size": (C.c_size_t, [C.c_int32] * 3),
    "mi355_moe_sorting_workspace_size2": (C.c_size_t, [C.c_int32] * 4),
    "mi355_moe_sorting": (C.c_int, [C.POINTER(SortingArgs), C.c_void_p]),
    "mi355_moe_sorting2": (C.c_int, [C.POINTER(SortingTraits), C.POINTER(SortingArgs), C.c_void_p]),
    "mi355_topk_softmax": (C.c_int, [C.POINTER(TopkSoftmaxTraits), C.POINTER(TopkSoftmaxArgs), C.c_void_p]),
    "mi355_fused_moe_supported": (C.c_int, [C.POINTER(FusedMoeTraits)]),
    "mi355_fused_moe_workspace_size": (C.c_size_t, [C.POINTER(FusedMoeTraits)] + [C.c_int32] * 5),
    "mi355_fused_moe_tile_rows": (C.c_int32, [C.POINTER(FusedMoeTraits)] + [C.c_int32] * 5),
    "mi355_fused_moe_chosen_tile_rows": (C.c_int32, [C.POINTER(FusedMoeTraits)] + [C.c_int32] * 5 + [C.POINTER(Workspace), C.c_void_p]),
    "mi355_fused_moegemm": (C.c_int, [C.POINTER(FusedMoeTraits), C.POINTER(FusedMoeGemmArgs), C.POINTER(Workspace),
                                      C.c_void_p]),
    "mi355_fused_moe": (C.c_int, [C.POINTER(FusedMoeTraits), C.POINTER(FusedMoeArgs), C.POINTER(Workspace), C.c_void_p]),
    "mi355_fused_moe_static_ws_capacity": (C.c_size_t, []),
    "mi355_fused_moe_static_ws": (C.c_int, [C.POINTER(FusedMoeTraits), C.POINTER(FusedMoeArgs), C.c_void_p]),
    "mi355_moe_flatmm_workspace_size": (C.c_size_t, [C.c_int32, C.POINTER(FlatmmArgs)]),
    "mi355_moe_flatmm": (C.c_int, [C.c_int32, C.POINTER(FlatmmArgs), C.POINTER(Workspace), C.c_void_p]),
    "mi355_moe_permute_weights": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_int32] * 8 + [C.c_void_p]),
    "mi355_moe_smoothquant": (C.c_int, [C.POINTER(SmoothquantArgs), C.c_int32, C.c_void_p]),
    "mi355_moe_rowwise_quant": (C.c_int, [C.c_void_p, C.c_int64, C.c_int32, C.c_int64, C.c_int32, C.c_void_p,
                                          C.c_void_p, C.c_void_p]),
    "mi355_moe_profile_start": (C.c_int, []),
    "mi355_moe_profile_start_kinds": (C.c_int, [C.c_uint32]),
    "mi355_moe_profile_stop": (C.c_int, [C.POINTER(C.c_double), C.POINTER(C.c_int32)]),
    "mi355_moe_kernel_name": (C.c_char_p, [C.c_int32]),
    "mi355_moe_mfma_sustained": (C.c_int, [C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_double), C.c_void_p]),
    "mi355_moe_last_error": (C.c_char_p, []),
    "mi355_moe_version": (C.c_int, []),
}

_lib = None


def header_version() -> int:
    """MI355_MOE_VERSION as include/mi355_moe.h defines it (what a freshly built library must report)."""
    import re

    text = open(os.path.join(os.path.dirname(_HERE), "include", "mi355_moe.h")).read()
    return int(re.search(r"^#define\s+MI355_MOE_VERSION\s+(\d+)", text, re.M).group(1))


def load():
    """dlopen the HIP library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m therock_amd.build` (needs hipcc); "
                "there is no CPU fallback")
        # PyTorch ships its own HIP runtime under the same soname as ROCm's.  Whichever is loaded first serves
        # the whole process, and initialising ROCm's copy from this library before torch initialises left the
        # process without a visible device.  torch owns the device memory and the streams here, so its runtime
        # is loaded first and this library binds to it.
        import torch  # noqa: F401

        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


NUM_KERNELS = 10


def profile_start(kinds=None) -> None:
    """Starts per-kernel event timing; kinds = iterable of kernel names restricts it to those kernels."""
    lib = load()
    if kinds is None:
        lib.mi355_moe_profile_start()
        return
    names = [lib.mi355_moe_kernel_name(k).decode() for k in range(NUM_KERNELS)]
    mask = 0
    for k in kinds:
        mask |= 1 << names.index(k)
    lib.mi355_moe_profile_start_kinds(C.c_uint32(mask))


def profile_stop() -> dict:
    """{kernel name: (total ms, launches)} for the kernels launched since profile_start()."""
    lib = load()
    ms = (C.c_double * NUM_KERNELS)()
    n = (C.c_int32 * NUM_KERNELS)()
    rc = lib.mi355_moe_profile_stop(ms, n)
    if rc != OK:
        raise RuntimeError(f"profile_stop failed ({rc}): {last_error()}")
    return {lib.mi355_moe_kernel_name(k).decode(): (ms[k], n[k]) for k in range(NUM_KERNELS) if n[k] > 0}


def mfma_sustained(prec: str, milliseconds: int = 1500, zero_operands: bool = False, stream=None) -> float:
    """TFLOP/s (TOP/s for int8) a loop of independent MFMAs on register operands sustains on this device."""
    out = C.c_double(0.0)
    rc = load().mi355_moe_mfma_sustained(DTYPES[prec], int(milliseconds), int(bool(zero_operands)), C.byref(out), stream)
    if rc != OK:
        raise RuntimeError(f"mfma_sustained failed ({rc}): {last_error()}")
    return out.value


def last_error() -> str:
    return load().mi355_moe_last_error().decode()
