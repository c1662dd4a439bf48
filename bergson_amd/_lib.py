"""ctypes binding of libbergson_amd.so (the C ABI declared in include/bergson_amd.h).

The library is built in-tree by ``python -m bergson_amd.build_ext``; loading
fails loudly when it is missing -- there is no fallback implementation.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libbergson_amd.so"

BGX_F32, BGX_F16, BGX_BF16 = 0, 1, 2
ABI_VERSION = 12
STATIC_SCRATCH_BYTES = 16 << 20


class ModuleDesc(C.Structure):
    """Mirror of ``bgx_module_desc``."""

    _fields_ = [
        ("a", C.c_void_p),
        ("g", C.c_void_p),
        ("r_in", C.c_void_p),
        ("r_out", C.c_void_p),
        ("col_scale", C.c_void_p),
        ("row_scale", C.c_void_p),
        ("bias_col", C.c_void_p),
        ("bias_scale", C.c_void_p),
        ("a_seq_stride", C.c_int64),
        ("a_tok_stride", C.c_int64),
        ("g_seq_stride", C.c_int64),
        ("g_tok_stride", C.c_int64),
        ("out_col", C.c_int64),
        ("I", C.c_int32),
        ("O", C.c_int32),
    ]


class BlockDesc(C.Structure):
    """bgx_block_desc: one module's fp32 matrix and its columns in a gradient row."""

    _fields_ = [
        ("h_dev", C.c_void_p),
        ("col0", C.c_int64),
        ("dim", C.c_int32),
        ("reserved", C.c_int32),
    ]


# name -> (restype, argtypes); the one list every exported symbol is checked against
SIGNATURES: dict[str, tuple] = {
    "bgx_abi_version": (C.c_int, []),
    "bgx_last_error": (C.c_char_p, []),
    "bgx_reload_switches": (C.c_int, []),
    "bgx_last_kernel": (C.c_char_p, [C.c_int32]),
    "bgx_adafactor_scales": (
        C.c_int,
        [C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p],
    ),
    "bgx_collect_workspace_bytes": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "bgx_collect_workspace_bytes_for": (C.c_size_t, [C.POINTER(ModuleDesc), C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                                     C.c_int32]),
    "bgx_collect_seq": (
        C.c_int,
        [C.POINTER(ModuleDesc), C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_int64, C.c_int32, C.c_float, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "bgx_collect_tok": (
        C.c_int,
        [C.POINTER(ModuleDesc), C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_int64, C.c_int32, C.c_float, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "bgx_collect_seq_static": (
        C.c_int,
        [C.POINTER(ModuleDesc), C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_int64, C.c_int32, C.c_float, C.c_float, C.c_void_p],
    ),
    "bgx_adam_table_bytes": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "bgx_adam_prepare": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                                   C.c_int32, C.c_void_p, C.c_void_p]),
    "bgx_collect_adam_workspace_bytes": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                                      C.c_int32, C.c_int64]),
    "bgx_collect_adam": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32,
         C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p,
         C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int32, C.c_float, C.c_float, C.c_void_p, C.c_size_t,
         C.c_int64, C.c_void_p],
    ),
    "bgx_token_sum": (C.c_int, [C.c_void_p, C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                C.c_void_p, C.c_void_p]),
    "bgx_fullgrad_seq": (
        C.c_int,
        [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int32, C.c_float, C.c_float, C.c_void_p],
    ),
    "bgx_fullgrad_seq_gemm": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32,
         C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_int64, C.c_int64, C.c_int32, C.c_float, C.c_float, C.c_void_p],
    ),
    "bgx_collect_seq_weight_workspace_bytes": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "bgx_collect_seq_weight": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32,
         C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
         C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int32, C.c_float,
         C.c_float, C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "bgx_project_rows_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int64, C.c_int32, C.c_int32]),
    "bgx_project_rows": (
        C.c_int,
        [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p, C.c_int64,
         C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "bgx_fullgrad_tok": (
        C.c_int,
        [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32,
         C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_void_p, C.c_int64, C.c_int64, C.c_int32, C.c_float, C.c_float, C.c_void_p],
    ),
    "bgx_collect_timing_enable": (C.c_int, [C.c_int32]),
    "bgx_collect_timing_read": (C.c_int, [C.POINTER(C.c_float), C.c_int32, C.POINTER(C.c_int32)]),
    "bgx_unit_normalize_rows": (C.c_int, [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p]),
    "bgx_precond_workspace_bytes": (C.c_size_t, [C.c_int32]),
    "bgx_block_gemm": (
        C.c_int,
        [C.c_void_p, C.c_int32, C.c_int64, C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.POINTER(BlockDesc), C.c_int32,
         C.c_void_p, C.c_size_t, C.c_void_p],
    ),
    "bgx_gram_accumulate": (
        C.c_int,
        [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.POINTER(BlockDesc), C.c_int32, C.c_void_p, C.c_size_t,
         C.c_void_p],
    ),
    "bgx_scan_workspace_bytes": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int64]),
    "bgx_scan_workspace_bytes_for": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int64, C.c_int64, C.c_int32]),
    "bgx_scan": (
        C.c_int,
        [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_int32, C.c_float, C.c_int32,
         C.c_int32, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_size_t, C.c_int64, C.c_void_p],
    ),
    "bgx_row_sumsq": (C.c_int, [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]),
    "bgx_scan_known_norms": (
        C.c_int,
        [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_int32, C.c_float, C.c_int32,
         C.c_int32, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
         C.c_size_t, C.c_int64, C.c_void_p],
    ),
}

_lib = None


class BergsonAmdError(RuntimeError):
    """A C-ABI call returned non-zero."""


def load() -> C.CDLL:
    """Load the library once and bind every declared symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build the HIP extension first with "
            "`python -m bergson_amd.build_ext` (there is no CPU fallback)"
        )
    lib = C.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.bgx_abi_version()
    if got != ABI_VERSION:
        raise ImportError(f"{LIB_PATH}: ABI version {got}, expected {ABI_VERSION}")
    _lib = lib
    return lib


def reload_switches() -> None:
    """Make the library read its BGX_* environment switches again (they are read once otherwise)."""
    load().bgx_reload_switches()


FAMILY_COLLECT, FAMILY_ADAM, FAMILY_SCAN, FAMILY_FULLGRAD = 0, 1, 2, 3


def last_kernel(family: int) -> str:
    """Name of the main kernel this thread's last launch of a family enqueued ("" before the first)."""
    return load().bgx_last_kernel(family).decode()


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().bgx_last_error().decode("utf-8", "replace")
        raise BergsonAmdError(f"{what} failed with code {rc}: {msg}")
