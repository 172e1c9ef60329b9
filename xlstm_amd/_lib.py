"""ctypes binding of the C ABI declared in ``include/xlstm_amd.h``.

The engine has no CPU fallback: if the shared library is missing, loading
fails loudly with the command that builds it.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("XLSTM_AMD_LIB", os.path.join(PKG, "lib", "libxlstm_amd.so"))

XS_F32, XS_BF16 = 0, 1
XS_ERR_UNSUPPORTED = -5
STATIC_SCRATCH_BYTES = (4 << 20) + (64 << 10)
ABI_VERSION = 16

EXPORTS = (
    "xs_abi_version",
    "xs_last_error",
    "xs_slstm_workspace_bytes",
    "xs_slstm_forward",
    "xs_slstm_step",
    "xs_slstm_forward_static",
    "xs_slstm_tile_r_for_steps",
    "xs_slstm_backward_prepare",
    "xs_slstm_backward",
    "xs_slstm_backward_params",
    "xs_slstm_backward_tile_r",
    "xs_causal_conv_silu",
    "xs_headwise_gates",
    "xs_headwise_group_norm",
    "xs_measure_stage",
)


class SlstmArgs(ctypes.Structure):
    """Mirror of ``xs_slstm_args``."""

    _fields_ = [
        ("B", ctypes.c_int32), ("T", ctypes.c_int32), ("NH", ctypes.c_int32), ("dh", ctypes.c_int32),
        ("wx_dtype", ctypes.c_int32), ("r_dtype", ctypes.c_int32),
        ("wx", ctypes.c_void_p),
        ("wx_stride_b", ctypes.c_int64), ("wx_stride_t", ctypes.c_int64),
        ("r", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("s0", ctypes.c_void_p),
        ("reset", ctypes.c_void_p),
        ("reset_stride_b", ctypes.c_int64),
        ("h_out", ctypes.c_void_p),
        ("s_out", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
        ("stream", ctypes.c_void_p),
        ("spin_limit", ctypes.c_int64),
        ("h_prev", ctypes.c_void_p),
        ("coef_out", ctypes.c_void_p),
        ("r_tiled", ctypes.c_void_p),
    ]


class SlstmBwdArgs(ctypes.Structure):
    """Mirror of ``xs_slstm_bwd_args``."""

    _fields_ = [
        ("B", ctypes.c_int32), ("T", ctypes.c_int32), ("NH", ctypes.c_int32), ("dh", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("wx", ctypes.c_void_p),
        ("wx_stride_b", ctypes.c_int64), ("wx_stride_t", ctypes.c_int64),
        ("ry", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("s0", ctypes.c_void_p),
        ("reset", ctypes.c_void_p),
        ("reset_stride_b", ctypes.c_int64),
        ("coef", ctypes.c_void_p),
        ("d_h", ctypes.c_void_p),
        ("d_s_final", ctypes.c_void_p),
        ("r_t", ctypes.c_void_p),
        ("d_wx", ctypes.c_void_p),
        ("d_wx_stride_b", ctypes.c_int64), ("d_wx_stride_t", ctypes.c_int64),
        ("d_s0", ctypes.c_void_p),
        ("stream", ctypes.c_void_p),
        ("split", ctypes.c_int32),
        ("exchange", ctypes.c_void_p),
        ("counters", ctypes.c_void_p),
        ("spin_limit", ctypes.c_int64),
        ("recurrent_cut", ctypes.c_int32),
        ("recurrent_clipval", ctypes.c_float),
        ("h_out", ctypes.c_void_p),
        ("r", ctypes.c_void_p),
        ("d_r", ctypes.c_void_p),
        ("d_bias", ctypes.c_void_p),
        ("d_wx_dtype", ctypes.c_int32),
    ]


class ConvArgs(ctypes.Structure):
    """Mirror of ``xs_conv_args``."""

    _fields_ = [
        ("B", ctypes.c_int32), ("T", ctypes.c_int32), ("D", ctypes.c_int32), ("K", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("x", ctypes.c_void_p),
        ("x_stride_b", ctypes.c_int64), ("x_stride_t", ctypes.c_int64),
        ("conv_state", ctypes.c_void_p),
        ("conv_state_stride_b", ctypes.c_int64),
        ("weight", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("reset", ctypes.c_void_p),
        ("reset_stride_b", ctypes.c_int64),
        ("out", ctypes.c_void_p),
        ("stream", ctypes.c_void_p),
        ("ring_out", ctypes.c_void_p),
    ]


class GatesArgs(ctypes.Structure):
    """Mirror of ``xs_gates_args``."""

    _fields_ = [
        ("M", ctypes.c_int32), ("NH", ctypes.c_int32), ("dh", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("x", ctypes.c_void_p),
        ("x_stride_row", ctypes.c_int64),
        ("x_conv", ctypes.c_void_p),
        ("x_conv_stride_row", ctypes.c_int64),
        ("w", ctypes.c_void_p * 4),
        ("out", ctypes.c_void_p),
        ("out_stride_row", ctypes.c_int64),
        ("stream", ctypes.c_void_p),
    ]


class NormArgs(ctypes.Structure):
    """Mirror of ``xs_norm_args``."""

    _fields_ = [
        ("B", ctypes.c_int32), ("T", ctypes.c_int32), ("NH", ctypes.c_int32), ("dh", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("eps", ctypes.c_float),
        ("x", ctypes.c_void_p),
        ("x_stride_b", ctypes.c_int64), ("x_stride_t", ctypes.c_int64), ("x_stride_h", ctypes.c_int64),
        ("weight", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("stream", ctypes.c_void_p),
    ]


STAGE_EXCHANGE, STAGE_CONTRACTION, STAGE_GATING, STAGE_LAUNCH, STAGE_CHAIN = 0, 1, 2, 3, 4


class MeasureArgs(ctypes.Structure):
    """Mirror of ``xs_measure_args``."""

    _fields_ = [
        ("stage", ctypes.c_int32), ("members", ctypes.c_int32), ("two_xcds", ctypes.c_int32), ("rows", ctypes.c_int32),
        ("steps", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
        ("stream", ctypes.c_void_p),
    ]


class SlstmStatus(ctypes.Structure):
    """Mirror of ``xs_slstm_status`` (first bytes of the workspace)."""

    _fields_ = [
        ("aborted", ctypes.c_uint32), ("abort_wg", ctypes.c_uint32), ("abort_step", ctypes.c_uint32),
        ("max_spins", ctypes.c_uint32), ("xcd_mixed", ctypes.c_uint32), ("launches", ctypes.c_uint32),
        ("step_kernel", ctypes.c_uint32), ("rows_per_workgroup", ctypes.c_uint32),
        ("pipelined_step", ctypes.c_uint32),
        ("reserved", ctypes.c_uint32 * 7),
    ]


_LIB: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """Loads the engine; raises if it has not been built."""
    global _LIB
    if _LIB is not None:
        return _LIB
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"xlstm_amd: HIP engine not built ({LIB_PATH} missing). "
            "Build it with `python -m xlstm_amd.build`; there is no CPU fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    lib.xs_abi_version.restype = ctypes.c_int
    lib.xs_abi_version.argtypes = []
    lib.xs_last_error.restype = ctypes.c_char_p
    lib.xs_last_error.argtypes = []
    lib.xs_slstm_workspace_bytes.restype = ctypes.c_size_t
    lib.xs_slstm_workspace_bytes.argtypes = [ctypes.c_int32] * 4
    for name in ("xs_slstm_forward", "xs_slstm_step", "xs_slstm_forward_static"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.POINTER(SlstmArgs)]
    for fn in (lib.xs_slstm_backward_prepare, lib.xs_slstm_backward, lib.xs_slstm_backward_params, lib.xs_slstm_backward_tile_r):
        fn.restype = ctypes.c_int
        fn.argtypes = [ctypes.POINTER(SlstmBwdArgs)]
    lib.xs_slstm_tile_r_for_steps.restype = ctypes.c_int
    lib.xs_slstm_tile_r_for_steps.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
    lib.xs_causal_conv_silu.restype = ctypes.c_int
    lib.xs_causal_conv_silu.argtypes = [ctypes.POINTER(ConvArgs)]
    lib.xs_headwise_gates.restype = ctypes.c_int
    lib.xs_headwise_gates.argtypes = [ctypes.POINTER(GatesArgs)]
    lib.xs_headwise_group_norm.restype = ctypes.c_int
    lib.xs_headwise_group_norm.argtypes = [ctypes.POINTER(NormArgs)]
    lib.xs_measure_stage.restype = ctypes.c_int
    lib.xs_measure_stage.argtypes = [ctypes.POINTER(MeasureArgs)]
    if lib.xs_abi_version() != ABI_VERSION:
        raise RuntimeError(f"xlstm_amd: ABI version {lib.xs_abi_version()} != expected {ABI_VERSION}; rebuild")
    _LIB = lib
    return lib


def last_error() -> str:
    return load().xs_last_error().decode()
