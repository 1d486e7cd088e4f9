"""ctypes binding of ``libtorchtune_amd.so`` (the C ABI declared in ``include/torchtune_amd.h``).

The library is the only compute path of this package: if it cannot be loaded, every op raises.  There is no
eager-PyTorch or CPU substitute behind it.
"""
from __future__ import annotations

import ctypes
import os
import threading
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libtorchtune_amd.so"
ABI_VERSION = 1

TTAMD_BF16 = 0
TTAMD_F32 = 1

_c_void_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float
_size = ctypes.c_size_t

# name -> (restype, argtypes); one entry per symbol declared in include/torchtune_amd.h
SIGNATURES = {
    "ttamd_version": (_int, []),
    "ttamd_last_error": (ctypes.c_char_p, []),
    "ttamd_nf4_quantize_workspace_bytes": (_size, [_i64, _int]),
    "ttamd_nf4_quantize": (
        _int,
        [_c_void_p, _int, _i64, _int, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _size, _c_void_p],
    ),
    "ttamd_nf4_dequantize": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _i64, _int, _int, _c_void_p, _c_void_p],
    ),
    "ttamd_nf4_block_scalers": (_int, [_c_void_p, _c_void_p, _c_void_p, _int, _i64, _int, _c_void_p, _c_void_p]),
    "ttamd_nf4_dequantize_merge_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _f32, _c_void_p, _i64, _i64, _c_void_p]),
    "ttamd_lora_fwd_workspace_bytes": (_size, [_i64, _i64, _int]),
    "ttamd_lora_hidden_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _int, _c_void_p, _size, _c_void_p]),
    "ttamd_lora_hidden_static_max_bytes": (_size, []),
    "ttamd_lora_hidden_static_init": (_int, []),
    "ttamd_lora_hidden_static_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _int, _c_void_p]),
    "ttamd_nf4_lora_linear_fwd_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _f32, _c_void_p, _c_void_p, _i64, _i64, _i64,
         _c_void_p],
    ),
    "ttamd_dora_weight_norm_workspace_bytes": (_size, [_i64, _i64]),
    "ttamd_nf4_dora_weight_norm_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _f32, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _size,
         _c_void_p],
    ),
    "ttamd_nf4_dora_linear_fwd_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _f32, _c_void_p, _c_void_p, _c_void_p, _i64, _i64,
         _i64, _c_void_p],
    ),
    "ttamd_dora_bwd_workspace_bytes": (_size, [_i64]),
    "ttamd_dora_bwd_prologue_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _size, _c_void_p],
    ),
    "ttamd_nf4_transpose_for_backward": (_int, [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_nf4_linear_bwd_dx_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _c_void_p, _i64, _i64, _i64,
         _c_void_p],
    ),
    "ttamd_nf4_gemm_workspace_bytes": (_size, [_i64, _i64, _i64]),
    "ttamd_nf4_gemm_expands_weight": (_int, [_i64, _i64, _i64]),
    "ttamd_nf4_lora_linear_fwd_ws_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _f32, _c_void_p, _c_void_p, _c_void_p, _i64, _i64,
         _i64, _c_void_p, _size, _c_void_p],
    ),
    "ttamd_nf4_linear_bwd_dx_ws_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _c_void_p, _i64, _i64, _i64,
         _c_void_p, _size, _c_void_p],
    ),
    "ttamd_nf4_linear_bwd_dx_swiglu_ws_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _c_void_p, _c_void_p, _c_void_p,
         _c_void_p, _i64, _i64, _i64, _c_void_p, _size, _c_void_p],
    ),
    "ttamd_lora_bwd_workspace_bytes": (_size, [_i64, _i64, _i64, _int]),
    "ttamd_lora_bwd_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _f32, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _int,
         _c_void_p, _size, _c_void_p],
    ),
    "ttamd_qlora_linear_fwd_workspace_bytes": (_size, [_i64, _i64, _i64, _int]),
    "ttamd_qlora_linear_fwd_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _f32, _c_void_p, _c_void_p, _c_void_p, _i64, _i64,
         _i64, _c_void_p, _size, _c_void_p],
    ),
    "ttamd_qlora_linear_bwd_workspace_bytes": (_size, [_i64, _i64, _i64, _int]),
    "ttamd_qlora_linear_bwd_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _f32,
         _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _c_void_p, _size, _c_void_p],
    ),
    "ttamd_lora_group_hidden_workspace_bytes": (_size, [_c_void_p, _int, _i64, _i64]),
    "ttamd_lora_group_hidden_bf16": (_int, [_c_void_p, _c_void_p, _int, _c_void_p, _i64, _i64, _c_void_p, _size, _c_void_p]),
    "ttamd_lora_group_fwd_workspace_bytes": (_size, [_c_void_p, _int, _i64, _i64]),
    "ttamd_nf4_lora_group_fwd_bf16": (_int, [_c_void_p, _c_void_p, _int, _c_void_p, _i64, _i64, _c_void_p, _size, _c_void_p]),
    "ttamd_nf4_lora_group_swiglu_fwd_bf16": (_int, [_c_void_p, _c_void_p, _int, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _size,
                                                    _c_void_p]),
    "ttamd_lora_group_bwd_workspace_bytes": (_size, [_c_void_p, _int, _i64, _i64]),
    "ttamd_lora_group_bwd_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _int, _c_void_p, _i64, _i64, _c_void_p, _size, _c_void_p]),
    "ttamd_lora_group_swiglu_bwd_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _size, _c_void_p]),
    "ttamd_nf4_group_bwd_dx_bf16": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _i64, _i64, _c_void_p]),
    "ttamd_nf4_group_bwd_dx_workspace_bytes": (_size, [_c_void_p, _int, _i64, _i64]),
    "ttamd_nf4_group_bwd_dx_ws_bf16": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _size, _c_void_p]),
    "ttamd_nf4_group_fwd_leaves_tiles": (_int, [_c_void_p, _int, _i64, _i64, _int]),
    "ttamd_nf4_group_bwd_dx_tiles_bf16": (_int, [_c_void_p, _int, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _int, _c_void_p]),
    "ttamd_nf4_lora_group_fwd_tiles_bf16": (_int, [_c_void_p, _c_void_p, _int, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _int, _c_void_p]),
    "ttamd_tiled_weight_bytes": (_size, [_i64, _i64]),
    "ttamd_gemm_tn_applies": (_int, [_i64, _i64, _i64]),
    "ttamd_gemm_tn_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _c_void_p]),
    "ttamd_gemm_tn_group_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _int, _i64, _c_void_p, _i64, _c_void_p]),
    "ttamd_gemm_tn_workspace_bytes": (_size, [_i64, _i64, _i64]),
    "ttamd_gemm_tn_ws_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _c_void_p, _size, _c_void_p]),
    "ttamd_gemm_tn_group_ws_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _int, _i64, _c_void_p, _i64, _c_void_p, _size, _c_void_p]),
    "ttamd_fq_per_group_int4_sym_tiled_bf16": (_int, [_c_void_p, _i64, _i64, _int, _int, _f32, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_tiled_linear_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _c_void_p]),
    "ttamd_tiled_lora_linear_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _int, _f32, _c_void_p, _c_void_p, _i64, _i64,
                                            _i64, _c_void_p]),
    "ttamd_fq_per_group_int4_sym_tiled_at_bf16": (_int, [_c_void_p, _i64, _i64, _int, _int, _f32, _c_void_p, _int, _c_void_p, _i64, _i64,
                                                         _c_void_p, _c_void_p]),
    "ttamd_tiled_linear_group_fwd_bf16": (_int, [_c_void_p, _c_void_p, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64,
                                                 _c_void_p]),
    "ttamd_tiled_linear_group_dx_bf16": (_int, [_c_void_p, _c_void_p, _int, _c_void_p, _c_void_p, _i64, _i64, _c_void_p]),
    "ttamd_tiled_linear_dx_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _int, _c_void_p, _i64, _i64, _i64, _c_void_p]),
    "ttamd_fq_per_token_int8_asym": (_int, [_c_void_p, _int, _i64, _i64, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_fq_per_group_int4_sym": (_int, [_c_void_p, _int, _i64, _i64, _int, _int, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_quantize_per_group_int4": (
        _int,
        [_c_void_p, _int, _i64, _i64, _int, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p],
    ),
    "ttamd_dequantize_per_group_int4": (_int, [_c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _int, _c_void_p, _c_void_p]),
    "ttamd_fq_per_group_uint4_asym": (
        _int, [_c_void_p, _int, _i64, _i64, _int, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_quantize_per_group_uint4": (
        _int, [_c_void_p, _int, _i64, _i64, _int, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_dequantize_per_group_uint4": (_int, [_c_void_p, _c_void_p, _c_void_p, _int, _i64, _i64, _int, _c_void_p, _c_void_p]),
    "ttamd_fq_per_token_int8_asym_conv": (
        _int, [_c_void_p, _int, _i64, _i64, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_fq_per_group_int4_sym_conv": (
        _int, [_c_void_p, _int, _i64, _i64, _int, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_quantize_per_group_int4_conv": (
        _int, [_c_void_p, _int, _i64, _i64, _int, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_fq_per_group_uint4_asym_conv": (
        _int, [_c_void_p, _int, _i64, _i64, _int, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_quantize_per_group_uint4_conv": (
        _int, [_c_void_p, _int, _i64, _i64, _int, _int, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p]),
    "ttamd_rms_norm_fwd_bf16": (_int, [_c_void_p, _c_void_p, _f32, _c_void_p, _c_void_p, _i64, _i64, _c_void_p]),
    "ttamd_rms_norm_bwd_workspace_bytes": (_size, [_i64]),
    "ttamd_rms_norm_bwd_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _size, _c_void_p],
    ),
    "ttamd_add_rms_norm_fwd_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _f32, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _c_void_p]),
    "ttamd_rms_norm_bwd_add_bf16": (
        _int,
        [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _size, _c_void_p],
    ),
    "ttamd_rope_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _i64, _int, _c_void_p]),
    "ttamd_repeat_kv_bf16": (_int, [_c_void_p, _c_void_p, _i64, _i64, _i64, _i64, _c_void_p]),
    "ttamd_repeat_kv_bwd_bf16": (_int, [_c_void_p, _c_void_p, _i64, _i64, _i64, _i64, _c_void_p]),
    "ttamd_qkv_rope_repeat_bf16": (_int, [_c_void_p] * 7 + [_i64] * 5 + [_c_void_p]),
    "ttamd_qkv_rope_repeat_bwd_bf16": (_int, [_c_void_p] * 7 + [_i64] * 5 + [_c_void_p]),
    "ttamd_swiglu_fwd_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _i64, _c_void_p]),
    "ttamd_cross_entropy_fwd_bwd_bf16": (_int, [_c_void_p, _c_void_p, _i64, _f32, _c_void_p, _c_void_p, _i64, _i64, _c_void_p]),
    "ttamd_swiglu_bwd_bf16": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _c_void_p]),
}

class FqConventions(ctypes.Structure):
    """``ttamd_fq_conventions`` of the header: the version-dependent constants of the fake-quant schemes."""

    _fields_ = [("eps_per_token", ctypes.c_float), ("eps_per_group_sym", ctypes.c_float), ("min_scale_uint4", ctypes.c_float),
                ("uint4_clamp_range_first", ctypes.c_int)]


GROUP_MAX = 4


class LoraGroupMember(ctypes.Structure):
    """``ttamd_lora_group_member`` of the header: one linear of a group that shares its input."""

    _fields_ = [("quantized_data", _c_void_p), ("block_scalers", _c_void_p), ("block_scalers_t", _c_void_p),
                ("quantized_data_t", _c_void_p), ("lora_a", _c_void_p), ("lora_b", _c_void_p), ("bias", _c_void_p),
                ("y", _c_void_p), ("grad_lora_a", _c_void_p), ("grad_lora_b", _c_void_p), ("N", _i64), ("rank", _int),
                ("scale", _f32)]


_lock = threading.Lock()
_lib = None


class LibraryNotBuiltError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the shared library (once) and attach the prototypes.  Raises if it is missing or stale."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise LibraryNotBuiltError(
                f"{LIB_PATH} is missing: torchtune_amd has no compute path without its HIP library. "
                "Build it with `python -m torchtune_amd.build` (needs hipcc)."
            )
        lib = ctypes.CDLL(os.fspath(LIB_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as err:
                raise LibraryNotBuiltError(f"{LIB_PATH} does not export {name}; rebuild it") from err
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.ttamd_version() != ABI_VERSION:
            raise LibraryNotBuiltError(
                f"{LIB_PATH} has ABI version {lib.ttamd_version()}, this package needs {ABI_VERSION}; rebuild it"
            )
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    """Turn a negative C-ABI return code into the matching Python exception."""
    if rc == 0:
        return
    msg = load().ttamd_last_error().decode("utf-8", "replace")
    if rc == -1:
        raise ValueError(f"{what}: {msg}")
    raise RuntimeError(f"{what} failed (code {rc}): {msg}")
