"""Loads the compiled kernel library and declares its C interface for ctypes.

The library must be there on a GPU machine: nothing in this package falls back
to a CPU or to a library model when it is missing.  ``import torch`` happens
first so that the HIP runtime the kernels link against is the one PyTorch has
already loaded.
"""

from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_long, c_void_p
from typing import Optional

import torch  # noqa: F401  (loads libamdhip64 before our library asks for it)

from . import build as _build

ABI_VERSION = 10

_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()

P, I, L, F = c_void_p, c_int, c_long, c_float

_SIGNATURES = {
    "fmsamd_embed": [P, P, I, P, I, I, I, F, P],
    "fmsamd_add_norm": [P, P, I, P, P, I, P, P, I, I, F, I, P],
    "fmsamd_gated_act": [P, P, I, P, I, I, I, I, P],
    "fmsamd_cast": [P, I, P, I, L, P],
    "fmsamd_advance_positions": [P, P, I, P],
    "fmsamd_bias_add": [P, I, P, I, I, I, P],
    "fmsamd_rope_table": [P, P, P, I, I, P],
    "fmsamd_rope_kv_write": [P, I, L, P, P, P, I, P, P, I, I, P, P, I, I, I, I, I, P],
    "fmsamd_attn_generic": [P, L, P, L, I, P, P, P, I, P, P, I, I, I, I, F, I, P, F, I, I, I, P, P, I, P],
    "fmsamd_attn_prefill_bf16": [P, L, P, L, P, P, P, P, I, I, P, I, P, P, I, I, I, I, F, I, F, I, P, I, P, I, P],
    "fmsamd_attn_decode_bf16": [P, L, P, L, P, L, P, P, P, I, P, P, I, I, I, I, F, I, I, I, I, I, P, F, I, P, I, P, I, P],
    "fmsamd_qkv_rope_skinny_bf16": [P, L, P, P, I, P, L, I, I, P, P, P, I, P, P, I, I, P, P, I, I, I, P, P, L, P],
    "fmsamd_gemm_f32": [P, L, P, P, P, L, I, I, I, P],
    "fmsamd_gemm_bf16": [P, L, P, P, I, P, I, L, I, I, I, P],
    "fmsamd_gemm_bf16_any": [P, L, P, P, I, P, I, L, I, I, I, P],
    "fmsamd_gemm_skinny_workspace": [I, I, I],
    "fmsamd_gemm_skinny_bf16": [P, L, P, P, I, P, I, L, I, I, I, P, P, L, P],
    "fmsamd_gemm_skinny_gated_bf16": [P, L, P, P, I, P, I, L, I, I, I, I, P, P, L, P],
    "fmsamd_gemm_skinny_residual_partials": [I, I, I],
    "fmsamd_gemm_skinny_residual_bf16": [P, L, P, P, I, P, L, P, I, P, L, P, I, I, I, I, P, P, L, P],
    "fmsamd_sample": [P, L, I, I, I, F, I, P, P, P],
    "fmsamd_argmax": [P, L, I, I, P, L, P, P],
    "fmsamd_norm_add_norm": [P, P, I, P, F, P, I, F, P, P, I, I, P],
    "fmsamd_norm_add_norm_affine": [P, P, I, P, P, F, I, P, P, I, F, I, P, P, I, I, P],
    "fmsamd_rms_norm_cols": [P, L, I, I, P, I, F, P, I, L, I, P],
    "fmsamd_activate": [P, P, I, L, I, P],
    "fmsamd_clamped_gated_act": [P, P, I, I, I, F, F, F, P],
    "fmsamd_latent_kv_write": [P, L, I, I, I, P, I, F, P, P, P, I, P, P, I, P, P, I, I, P],
    "fmsamd_latent_attn_mfma": [P, L, P, L, P, L, P, P, P, I, P, P, P, I, I, I, I, F, I, I, P],
    "fmsamd_latent_q_rotate": [P, L, I, I, I, I, P, L, I, P, P, P, I, I, P],
    "fmsamd_headwise_linear": [P, L, L, P, P, L, L, P, L, I, I, I, I, I, P],
    "fmsamd_latent_attn_generic": [P, L, P, L, I, P, P, P, I, P, P, I, I, I, I, F, I, P],
    "fmsamd_moe_route": [P, L, I, I, I, I, P, P, P],
    "fmsamd_moe_group": [P, I, I, P, P, I, I, P],
    "fmsamd_moe_experts": [I, P, L, P, P, P, I, P, P, I, I, I, I, I, F, F, F, P, I, P],
    "fmsamd_moe_route_grouped": [P, L, I, I, I, P, I, I, F, P, P, P],
    "fmsamd_poly_norm": [P, L, I, F, F, F, F, F, P, I, L, I, P],
    "fmsamd_group_norm_chain": [P, P, I, P, I, I, F, P, I, I, F, P, I, P, I, I, P],
    "fmsamd_short_conv": [P, L, I, P, P, I, I, P, P, P, I, P, I, L, I, I, P],
    "fmsamd_rglru_gates": [P, L, P, P, P, P, I, P, F, P, P, P, I, I, I, P],
    "fmsamd_rglru_scan": [P, P, P, L, I, P, P, P, P, P, I, L, I, I, P],
    "fmsamd_rglru_scan_chunk": [I, I],
    "fmsamd_rglru_scan_chunked": [P, P, P, L, I, P, P, P, P, P, I, L, I, I, I, I, P, P],
    "fmsamd_qk_projection_norm": [P, L, I, I, I, P, P, I, F, P, I, L, P, I, I, P, L, P, P],
    "fmsamd_gate_mul": [P, L, P, L, I, F, P, L, I, I, I, I, P],
    "fmsamd_scale_f32": [P, L, F, P],
    "fmsamd_cast_cols": [P, L, P, I, L, I, I, P],
    "fmsamd_delta_prepare": [P, L, I, P, L, I, P, I, I, P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, F, P],
    "fmsamd_delta_rule": [P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, P],
    "fmsamd_gated_head_norm": [P, P, L, P, I, F, I, F, P, I, L, P, I, I, I, P],
    "fmsamd_moe_combine": [P, P, I, P, P, L, P, I, I, I, P, I, P, L, P],
    "fmsamd_probe_read": [P, L, I, I, P, P],
    "fmsamd_probe_mfma": [I, I, I, P, P, P],
}


class KernelLibraryMissing(RuntimeError):
    pass


def load(verbose: bool = True) -> ctypes.CDLL:
    """The kernel library, compiled first if no built copy is found."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        try:
            path = _build.ensure_built(verbose=verbose)
            lib = ctypes.CDLL(path)
        except Exception as err:  # no compiler, no writable folder, broken library
            raise KernelLibraryMissing(
                f"the HIP kernel library of fms_amd could not be built or loaded ({err}); "
                "there is no fallback path: build it with `python -m fms_amd.kernels.build` (needs hipcc)"
            ) from err
        lib.fmsamd_last_error.restype = c_char_p
        lib.fmsamd_last_error.argtypes = []
        lib.fmsamd_abi_version.restype = c_int
        lib.fmsamd_abi_version.argtypes = []
        if lib.fmsamd_abi_version() != ABI_VERSION:
            raise KernelLibraryMissing(
                f"{path} has interface version {lib.fmsamd_abi_version()}, this package needs {ABI_VERSION}: rebuild it"
            )
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = c_int
        lib.fmsamd_attn_prefill_qblock.restype = c_int
        lib.fmsamd_attn_prefill_qblock.argtypes = [I, I, I, I]
        lib.fmsamd_latent_attn_workspace.restype = c_long
        lib.fmsamd_latent_attn_workspace.argtypes = [I, I, I, I]
        lib.fmsamd_latent_attn_mfma_fits.restype = c_int
        lib.fmsamd_latent_attn_mfma_fits.argtypes = [I, I]
        lib.fmsamd_moe_max_tiles.restype = c_int
        lib.fmsamd_moe_max_tiles.argtypes = [I, I, I]
        lib.fmsamd_moe_tile_rows.restype = c_int
        lib.fmsamd_moe_tile_rows.argtypes = [I, I, I]
        lib.fmsamd_argmax_workspace.restype = c_long
        lib.fmsamd_argmax_workspace.argtypes = [I, I]
        lib.fmsamd_attn_decode_workspace.restype = c_long
        lib.fmsamd_gemm_skinny_workspace.restype = c_long
        lib.fmsamd_attn_decode_workspace.argtypes = [I, I, I, I]
        lib.path = path
        _lib = lib
    return _lib


class KernelError(RuntimeError):
    pass


def check(code: int) -> None:
    if code != 0:
        raise KernelError(load().fmsamd_last_error().decode())
