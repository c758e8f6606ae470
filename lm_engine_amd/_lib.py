"""ctypes binding of libgdn_hip.so (the C ABI declared in include/gdn_hip.h).

The library is loaded lazily and the load fails loudly: there is no CPU or PyTorch fallback
behind the HIP path.  Build it with ``python -m lm_engine_amd.build``.
"""

from __future__ import annotations

import ctypes
import os


GDN_ABI_VERSION = 2

GDN_BF16 = 0
GDN_F32 = 1

GDN_FLAG_L2NORM = 1
GDN_FLAG_STATE_INPLACE = 2
GDN_FLAG_LEFT_PADDED = 4
GDN_FLAG_FUSED_LAUNCH = 8
GDN_FLAG_READY_FLAGS_CLEAR = 16
GDN_FLAG_RECORDS_16X16 = 32
GDN_FLAG_DEBUG_NO_PRODUCERS = 64
GDN_FLAG_SKIP_EMPTY_CHUNKS = 128

GDN_ERR_TIMEOUT = -7

GDN_NOALLOC_SCRATCH_BYTES = 64 << 20  # built-in workspace of gdn_chunk_fwd_noalloc

GDN_ACT_NONE = 0
GDN_ACT_SILU = 1

LIBRARY_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libgdn_hip.so")

EXPORTED_SYMBOLS = (
    "gdn_abi_version",
    "gdn_strerror",
    "gdn_workspace_bytes",
    "gdn_workspace_header_bytes",
    "gdn_chunk_fwd",
    "gdn_chunk_fwd_status",
    "gdn_chunk_fwd_is_one_launch",
    "gdn_chunk_fwd_noalloc",
    "gdn_recurrent_fwd",
    "gdn_chunk_fwd_profile",
    "gdn_chunk_fwd_saving",
    "gdn_chunk_fwd_saving_is_staged",
    "gdn_chunk_bwd_local",
    "gdn_chunk_bwd_prepare",
    "gdn_causal_conv1d_fwd",
    "gdn_causal_conv1d_bwd",
    "gdn_gates_fwd",
    "gdn_gates_bwd",
    "gdn_gated_rmsnorm_fwd",
    "gdn_gated_rmsnorm_bwd",
)

GDN_CHUNK_KERNELS = 3
CHUNK_KERNEL_NAMES = ("chunk_offsets", "chunk_prepare", "chunk_scan")


class GdnChunkSaves(ctypes.Structure):
    _fields_ = [
        ("states", ctypes.c_void_p),
        ("v_new", ctypes.c_void_p),
        ("chunks_per_chain", ctypes.c_int32),
        ("records_given", ctypes.c_int32),
        ("save_every", ctypes.c_int32),
        ("save_reverse", ctypes.c_int32),
        ("states_dtype", ctypes.c_int32),
        ("v_new_dtype", ctypes.c_int32),
        ("no_output", ctypes.c_int32),
        ("mirror_reads", ctypes.c_int32),
        ("sliced", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("k_odd", ctypes.c_void_p),
        ("v_odd", ctypes.c_void_p),
        ("k_odd_stride_b", ctypes.c_int64),
        ("k_odd_stride_t", ctypes.c_int64),
        ("k_odd_stride_h", ctypes.c_int64),
        ("v_odd_stride_b", ctypes.c_int64),
        ("v_odd_stride_t", ctypes.c_int64),
        ("v_odd_stride_h", ctypes.c_int64),
        ("row_order", ctypes.c_void_p),
    ]


class GdnChunkLocalArgs(ctypes.Structure):
    _fields_ = (
        [(name, ctypes.c_void_p) for name in ("v_new", "states", "dstates", "gamma", "beta", "rq", "rk")]
        + [("saves_dtype", ctypes.c_int32), ("scale", ctypes.c_float), ("chunks", ctypes.c_int64), ("K", ctypes.c_int32),
           ("V", ctypes.c_int32)]
        + [(name, ctypes.c_void_p) for name in ("y_mirror", "y_chunks", "dq_out", "dk_out", "dv_out", "dg_out", "dbeta_out")]
        + [("H", ctypes.c_int32), ("NC", ctypes.c_int32)]
        + [(name, ctypes.c_void_p) for name in ("q_raw", "k_raw", "v_raw", "dout_raw")]
        + [(f"{x}_stride_{d}", ctypes.c_int64) for x in ("q", "k", "v", "dout") for d in ("b", "t", "h")]
        + [("seq_start", ctypes.c_void_p), ("seq_len", ctypes.c_void_p), ("T_rows", ctypes.c_int32), ("dstates_dtype", ctypes.c_int32),
           ("saves_sliced", ctypes.c_int32), ("reserved", ctypes.c_int32)]
    )  # fmt: skip


class GdnChunkBwdPrepareArgs(ctypes.Structure):
    _fields_ = (
        [(name, ctypes.c_void_p) for name in ("q", "k", "dout", "g", "beta")]
        + [(f"{x}_stride_{d}", ctypes.c_int64) for x in ("q", "k", "dout") for d in ("b", "t", "h")]
        + [(name, ctypes.c_int32) for name in ("N", "T", "H", "K", "V", "beta_dtype", "flags")]
        + [("scale", ctypes.c_float)]
        + [(name, ctypes.c_void_p) for name in ("gamma", "beta_packed", "rq", "rk", "k_mirror", "v_mirror", "records")]
        + [("records_bytes", ctypes.c_uint64), ("seq_start", ctypes.c_void_p), ("seq_len", ctypes.c_void_p),
           ("NC", ctypes.c_int32), ("reserved", ctypes.c_int32), ("records_fwd", ctypes.c_void_p),
           ("records_fwd_bytes", ctypes.c_uint64)]
    )  # fmt: skip


class GdnConvBwdArgs(ctypes.Structure):
    _fields_ = (
        [(name, ctypes.c_void_p) for name in ("x", "dy", "weight", "bias", "input_state", "mask", "dx", "dstate",
                                              "dweight_partial", "dbias_partial")]
        + [(name, ctypes.c_int64) for name in ("x_stride_b", "x_stride_s", "dy_stride_b", "dy_stride_s")]
        + [(name, ctypes.c_int32) for name in ("B", "S", "C", "kernel_size", "w_dtype", "activation", "tokens_per_block",
                                               "dtype")]
    )  # fmt: skip


class GdnNormBwdArgs(ctypes.Structure):
    _fields_ = (
        [(name, ctypes.c_void_p) for name in ("o", "gate", "weight", "dy", "d_o", "d_gate", "dweight_partial")]
        + [(name, ctypes.c_int64) for name in ("o_stride_t", "gate_stride_t", "tokens")]
        + [(name, ctypes.c_int32) for name in ("H", "V", "dtype", "w_dtype")]
        + [("eps", ctypes.c_float), ("partial_blocks", ctypes.c_int32)]
    )  # fmt: skip


class GdnArgs(ctypes.Structure):
    """Mirror of ``struct gdn_args``; field order and types must match include/gdn_hip.h."""

    _fields_ = (
        [(name, ctypes.c_void_p) for name in ("q", "k", "v", "beta", "g", "h0", "ht", "o", "cu_seqlens", "workspace")]
        + [("workspace_bytes", ctypes.c_uint64)]
        + [
            (f"{t}_stride_{d}", ctypes.c_int64)
            for t in ("q", "k", "v", "o")
            for d in ("b", "t", "h")
        ]
        + [(name, ctypes.c_int32) for name in ("B", "T", "H", "K", "V", "N", "chunk", "dtype", "beta_dtype", "flags")]
        + [("scale", ctypes.c_float), ("spin_limit", ctypes.c_int32), ("qk_heads", ctypes.c_int32), ("reserved", ctypes.c_int32), ("error_word", ctypes.c_void_p)]
    )


class GdnConvArgs(ctypes.Structure):
    """Mirror of ``struct gdn_conv_args``."""

    _fields_ = (
        [(name, ctypes.c_void_p) for name in ("x", "weight", "bias", "input_state", "mask", "y", "final_state")]
        + [(name, ctypes.c_int64) for name in ("x_stride_b", "x_stride_s", "y_stride_b", "y_stride_s")]
        + [(name, ctypes.c_int32) for name in ("B", "S", "C", "kernel_size", "dtype", "w_dtype", "activation", "reserved")]
    )


class GdnGateArgs(ctypes.Structure):
    """Mirror of ``struct gdn_gate_args``."""

    _fields_ = (
        [(name, ctypes.c_void_p) for name in ("a", "b", "A_log", "dt_bias", "g", "beta")]
        + [(name, ctypes.c_int64) for name in ("a_stride", "b_stride", "tokens")]
        + [("H", ctypes.c_int32), ("dtype", ctypes.c_int32), ("beta_scale", ctypes.c_float), ("reserved", ctypes.c_int32)]
    )


class GdnGateBwdArgs(ctypes.Structure):
    """Mirror of ``struct gdn_gate_bwd_args``."""

    _fields_ = (
        [(name, ctypes.c_void_p) for name in ("a", "b", "A_log", "dt_bias", "dg", "dbeta", "da", "db", "dA_log_partial",
                                              "ddt_bias_partial")]
        + [(name, ctypes.c_int64) for name in ("a_stride", "b_stride", "tokens")]
        + [("H", ctypes.c_int32), ("dtype", ctypes.c_int32), ("beta_scale", ctypes.c_float), ("partial_blocks", ctypes.c_int32)]
    )  # fmt: skip


class GdnNormArgs(ctypes.Structure):
    """Mirror of ``struct gdn_norm_args``."""

    _fields_ = (
        [(name, ctypes.c_void_p) for name in ("o", "gate", "weight", "y")]
        + [(name, ctypes.c_int64) for name in ("o_stride_t", "gate_stride_t", "y_stride_t", "tokens")]
        + [(name, ctypes.c_int32) for name in ("H", "V", "dtype", "w_dtype")]
        + [("eps", ctypes.c_float), ("reserved", ctypes.c_int32)]
    )


class GdnLibraryError(RuntimeError):
    pass


_lib = None


def load_library() -> ctypes.CDLL:
    """Loads libgdn_hip.so once, checks its ABI version and declares the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBRARY_PATH):
        raise GdnLibraryError(
            f"{LIBRARY_PATH} is missing: the gated delta-rule HIP library has not been built "
            "(run `python -m lm_engine_amd.build`); there is no fallback path."
        )
    lib = ctypes.CDLL(LIBRARY_PATH)
    for symbol in EXPORTED_SYMBOLS:
        if not hasattr(lib, symbol):
            raise GdnLibraryError(f"{LIBRARY_PATH} does not export {symbol}")

    lib.gdn_abi_version.argtypes = []
    lib.gdn_abi_version.restype = ctypes.c_int
    lib.gdn_strerror.argtypes = [ctypes.c_int]
    lib.gdn_strerror.restype = ctypes.c_char_p
    lib.gdn_workspace_bytes.argtypes = [ctypes.POINTER(GdnArgs)]
    lib.gdn_workspace_bytes.restype = ctypes.c_uint64
    lib.gdn_workspace_header_bytes.argtypes = [ctypes.POINTER(GdnArgs)]
    lib.gdn_workspace_header_bytes.restype = ctypes.c_uint64
    lib.gdn_chunk_fwd.argtypes = [ctypes.POINTER(GdnArgs), ctypes.c_void_p]
    lib.gdn_chunk_fwd.restype = ctypes.c_int
    lib.gdn_chunk_fwd_is_one_launch.argtypes = [ctypes.POINTER(GdnArgs)]
    lib.gdn_chunk_fwd_is_one_launch.restype = ctypes.c_int
    lib.gdn_chunk_fwd_status.argtypes = [ctypes.POINTER(GdnArgs), ctypes.c_void_p]
    lib.gdn_chunk_fwd_status.restype = ctypes.c_int
    lib.gdn_chunk_fwd_noalloc.argtypes = [ctypes.POINTER(GdnArgs), ctypes.c_void_p]
    lib.gdn_chunk_fwd_noalloc.restype = ctypes.c_int
    lib.gdn_recurrent_fwd.argtypes = [ctypes.POINTER(GdnArgs), ctypes.c_void_p]
    lib.gdn_recurrent_fwd.restype = ctypes.c_int
    lib.gdn_chunk_fwd_profile.argtypes = [ctypes.POINTER(GdnArgs), ctypes.c_void_p, ctypes.POINTER(ctypes.c_float)]
    lib.gdn_chunk_fwd_profile.restype = ctypes.c_int
    lib.gdn_chunk_fwd_saving.argtypes = [ctypes.POINTER(GdnArgs), ctypes.POINTER(GdnChunkSaves), ctypes.c_void_p]
    lib.gdn_chunk_fwd_saving.restype = ctypes.c_int
    lib.gdn_chunk_fwd_saving_is_staged.argtypes = [ctypes.POINTER(GdnArgs), ctypes.POINTER(GdnChunkSaves)]
    lib.gdn_chunk_fwd_saving_is_staged.restype = ctypes.c_int
    lib.gdn_chunk_bwd_local.argtypes = [ctypes.POINTER(GdnChunkLocalArgs), ctypes.c_void_p]
    lib.gdn_chunk_bwd_local.restype = ctypes.c_int
    lib.gdn_chunk_bwd_prepare.argtypes = [ctypes.POINTER(GdnChunkBwdPrepareArgs), ctypes.c_void_p]
    lib.gdn_chunk_bwd_prepare.restype = ctypes.c_int
    lib.gdn_causal_conv1d_fwd.argtypes = [ctypes.POINTER(GdnConvArgs), ctypes.c_void_p]
    lib.gdn_causal_conv1d_fwd.restype = ctypes.c_int
    lib.gdn_gated_rmsnorm_bwd.argtypes = [ctypes.POINTER(GdnNormBwdArgs), ctypes.c_void_p]
    lib.gdn_gated_rmsnorm_bwd.restype = ctypes.c_int
    lib.gdn_causal_conv1d_bwd.argtypes = [ctypes.POINTER(GdnConvBwdArgs), ctypes.c_void_p]
    lib.gdn_causal_conv1d_bwd.restype = ctypes.c_int
    lib.gdn_gates_fwd.argtypes = [ctypes.POINTER(GdnGateArgs), ctypes.c_void_p]
    lib.gdn_gates_fwd.restype = ctypes.c_int
    lib.gdn_gates_bwd.argtypes = [ctypes.POINTER(GdnGateBwdArgs), ctypes.c_void_p]
    lib.gdn_gates_bwd.restype = ctypes.c_int
    lib.gdn_gated_rmsnorm_fwd.argtypes = [ctypes.POINTER(GdnNormArgs), ctypes.c_void_p]
    lib.gdn_gated_rmsnorm_fwd.restype = ctypes.c_int

    version = lib.gdn_abi_version()
    if version != GDN_ABI_VERSION:
        raise GdnLibraryError(f"libgdn_hip.so has ABI version {version}, this binding expects {GDN_ABI_VERSION}")
    _lib = lib
    return lib


def strerror(status: int) -> str:
    return load_library().gdn_strerror(status).decode()


def check_status(status: int, what: str) -> None:
    """Negative codes are rejected arguments (ValueError), positive ones HIP errors (RuntimeError)."""
    if status == 0:
        return
    message = f"{what}: {strerror(status)} (status {status})"
    if status < 0:
        raise ValueError(message)
    raise RuntimeError(message)
