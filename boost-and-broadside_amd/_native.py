"""Loads ``_lib/libbnb_amd.so`` and declares its C ABI (see ``include/bnb_amd.h``).

There is no fallback: if the library is missing or an entry point is absent the
import-time caller gets an exception naming the build command.
"""

from __future__ import annotations

import ctypes
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "_lib", "libbnb_amd.so")

ABI_VERSION = 28
F32, BF16 = 0, 1
PATH_AUTO, PATH_VALU, PATH_MFMA, PATH_ENV, PATH_HEAD = 0, 1, 2, 3, 4
WGRAD_PATH_AUTO, WGRAD_PATH_STAGED, WGRAD_PATH_DMA = 0, 1, 2

_vp, _i, _i64, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float

# name -> (restype, argtypes); mirrors include/bnb_amd.h line for line
SIGNATURES = {
    "bnb_abi_version": (_i, []),
    "bnb_build_arch": (ctypes.c_char_p, []),
    "bnb_error_string": (ctypes.c_char_p, [_i]),
    "bnb_sdpa_masked_fwd": (_i, [_vp, _i64, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "bnb_sdpa_masked_fwd_path": (_i, [_vp, _i64, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp]),
    "bnb_sdpa_cross_fwd": (_i, [_vp, _i64, _i, _vp, _vp, _i64, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "bnb_sdpa_cross_ranges_fwd": (_i, [_vp, _i64, _i, _vp, _i64, _vp, _i64, _vp, _vp, _i, _i, _i, _i, _vp]),
    "bnb_sdpa_cross_ranges_fwd_lse": (_i, [_vp, _i64, _i, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "bnb_rglru_step_fwd": (_i, [_vp, _i, _vp, _i, _vp, _f, _vp, _i64, _vp, _i64, _vp, _i, _i64, _i, _vp]),
    "bnb_rglru_step_reset_fwd": (
        _i, [_vp, _i, _vp, _i, _vp, _f, _vp, _i64, _vp, _i64, _vp, _i, _vp, _i, _i64, _i, _vp]
    ),
    "bnb_rglru_step_rows_fwd": (
        _i, [_vp, _i, _vp, _i, _vp, _f, _vp, _i64, _vp, _i64, _vp, _i, _i64, _vp, _i, _i64, _i, _vp]
    ),
    "bnb_conv_step_rows_fwd": (_i, [_vp, _i, _i64, _i64, _vp, _i64, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i64, _i64, _i, _vp]),
    "bnb_linear_wgrad_slices": (_i, [_i64, _i, _i]),
    "bnb_linear_wgrad_path": (_i, [_i]),
    "bnb_linear_wgrad_fwd": (_i, [_vp, _i64, _vp, _i64, _vp, _i, _vp, _i, _i64, _i, _i, _vp]),
    "bnb_linear_wgrad_tiled_fwd": (_i, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _i, _vp, _i, _i64, _i, _i, _vp]),
    "bnb_conv_seq_bwd_blocks": (_i, [_i64, _i, _i]),
    "bnb_conv_seq_bwd": (_i, [_vp, _i, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "bnb_column_sums_slices": (_i, [_i64, _i]),
    "bnb_column_sums": (_i, [_vp, _i, _i64, _vp, _i, _vp, _i, _i64, _i, _vp]),
    "bnb_gelu_mul_bwd": (_i, [_vp, _i, _i64, _vp, _i, _i64, _vp, _i, _vp, _i64, _vp, _i64, _i64, _i, _vp]),
    "bnb_sdpa_masked_bwd": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _vp]),
    "bnb_sdpa_cross_bwd": (_i, [_vp, _i64, _i, _vp, _i64, _i, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "bnb_sdpa_cross_ranges_bwd": (_i, [_vp, _i64, _i, _vp, _i64, _vp, _i64, _i, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "bnb_sdpa_cross_stream_bwd": (_i, [_vp, _i64, _i, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "bnb_sdpa_cross_stream_bwd_lse": (_i, [_vp, _i64, _i, _vp, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _vp]),
    "bnb_sdpa_masked_bwd_path": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _i, _vp]),
    "bnb_rmsnorm_bwd_blocks": (_i, [_i64, _i]),
    "bnb_rmsnorm_bwd": (_i, [_vp, _i64, _vp, _i, _i64, _vp, _f, _vp, _vp, _vp, _vp, _i, _vp, _i64, _i, _vp]),
    "bnb_rmsnorm_bwd_static_limit": (_i64, []),
    "bnb_rmsnorm_bwd_static": (_i, [_vp, _i64, _vp, _i, _i64, _vp, _f, _vp, _vp, _vp, _vp, _i64, _i, _vp]),
    "bnb_team_attend_fwd": (_i, [_vp, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i, _i, _i, _i, _vp]),
    "bnb_team_attend_bwd": (_i, [_vp, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "bnb_team_attend_bwd_partial_rows": (_i, []),
    "bnb_team_gather_bwd": (_i, [_vp, _vp, _i64, _vp, _i64, _vp, _i, _i, _i, _vp]),
    "bnb_team_norm_broadcast_fwd": (_i, [_vp, _vp, _f, _vp, _i64, _vp, _vp, _i64, _i64, _i, _i, _i, _vp]),
    "bnb_temporal_step_fwd": (
        _i, [_vp, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _f, _vp, _i64, _i64,
             _vp, _i, _i64, _i, _vp]
    ),
    "bnb_conv_step_fwd": (_i, [_vp, _i, _vp, _i64, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i64, _i64, _i, _vp]),
    "bnb_conv_seq_fwd": (_i, [_vp, _i, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i, _i, _i, _i, _i, _vp]),
    "bnb_rglru_scan_fwd": (_i, [_vp, _i, _vp, _i, _vp, _f, _vp, _i64, _vp, _vp, _i, _vp, _i64, _i64, _i, _i, _i, _i, _i, _vp]),
    "bnb_rglru_scan_bwd": (
        _i, [_vp, _i, _vp, _i, _vp, _f, _vp, _i64, _vp, _vp, _i, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i, _i, _i, _i, _i, _vp]
    ),
    "bnb_add_rmsnorm_fwd": (_i, [_vp, _i64, _vp, _i, _vp, _f, _vp, _vp, _i, _i64, _i, _vp]),
    "bnb_norm_linear_fwd": (_i, [_vp, _i64, _vp, _vp, _vp, _f, _vp, _vp, _vp, _i64, _i, _i, _vp]),
    "bnb_norm_linear_train_fwd": (_i, [_vp, _i64, _vp, _f, _vp, _vp, _vp, _i64, _i, _i, _vp]),
    "bnb_linear_f32_fwd": (_i, [_vp, _i64, _vp, _i64, _vp, _f, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _i, _i, _i, _vp]),
    "bnb_mask_count": (_i, [_vp, _vp, _i, _i, _vp]),
    "bnb_mask_fill": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "bnb_ffn_fused_fwd": (_i, [_vp, _i64, _vp, _i, _vp, _f, _vp, _vp, _i64, _i, _i, _vp]),
    "bnb_ffn_fused_proj_next_fwd": (_i, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _f, _vp, _vp, _vp, _f, _vp, _vp, _i, _i64,
                                         _i64, _i, _i, _vp]),
    "bnb_ffn_fused_train_fwd": (_i, [_vp, _i64, _vp, _i, _vp, _f, _vp, _vp, _vp, _vp, _i64, _i, _i, _vp]),
    "bnb_ffn_fused_proj_train_fwd": (_i, [_vp, _i64, _vp, _i64, _vp, _vp, _f, _vp, _vp, _vp, _vp, _i64, _i, _i, _vp]),
    "bnb_ffn_bwd": (_i, [_vp, _vp, _i, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i, _i, _vp]),
    "bnb_ffn_fused_proj_fwd": (_i, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _f, _vp, _vp, _i64, _i, _i, _vp]),
    "bnb_gelu_mul_fwd": (_i, [_vp, _i, _i64, _vp, _i, _i64, _vp, _i, _i64, _i, _vp]),
    "bnb_copy_bytes": (_i, [_vp, _vp, _i64, _vp]),
    "bnb_issue_probe": (_i, [_i, _i, _i, _i, _i, _vp, _vp]),
}

_lib = None


class NativeLibraryError(RuntimeError):
    """The HIP library is missing, stale or returned an error code (``code``, 0 when none)."""

    def __init__(self, message: str, code: int = 0) -> None:
        super().__init__(message)
        self.code = code


ERR_UNSUPPORTED = 10004  # BNB_ERR_UNSUPPORTED: a shape outside what the kernels cover
ERR_SCRATCH_LIMIT = 10006  # BNB_ERR_SCRATCH_LIMIT: more workspace needed than the built-in buffer holds


def load() -> ctypes.CDLL:
    """Return the loaded library, loading and checking it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeLibraryError(
            f"{LIB_PATH} not found: build it with `python boost-and-broadside_amd/build.py` "
            "(hipcc, --offload-arch=gfx950). There is no non-HIP fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise NativeLibraryError(f"{LIB_PATH} does not export {name}; rebuild it") from exc
        fn.restype, fn.argtypes = restype, argtypes
    got = lib.bnb_abi_version()
    if got != ABI_VERSION:
        raise NativeLibraryError(f"{LIB_PATH} has ABI version {got}, this package expects {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    """Raise if an entry point returned a non-zero code."""
    if code != 0:
        msg = load().bnb_error_string(code).decode()
        raise NativeLibraryError(f"{what} failed with code {code}: {msg}", code)
