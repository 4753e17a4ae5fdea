"""ctypes binding of libmxplace.so (the C ABI declared in include/mxp.h, plus the measurement entry points of
include/mxp_bench.h).

The library is the product: there is no Python or CPU fallback for anything it does.
If it is missing, or was built without a symbol the header declares, importing this
module's ``lib()`` raises immediately.
"""

from __future__ import annotations

import ctypes as C
from pathlib import Path

import os

PKG_DIR = Path(__file__).resolve().parent
# MXP_LIBRARY_PATH selects another build of the same library (same ABI), e.g. a tuning variant.
LIB_PATH = Path(os.environ["MXP_LIBRARY_PATH"]) if os.environ.get("MXP_LIBRARY_PATH") else PKG_DIR / "libmxplace.so"

MXP_MAX_DIMS = 8

ERR_NAMES = {
    -1: "MXP_ERR_IO", -2: "MXP_ERR_FORMAT", -3: "MXP_ERR_UNSUPPORTED", -4: "MXP_ERR_COVERAGE",
    -5: "MXP_ERR_ARG", -6: "MXP_ERR_DEVICE", -7: "MXP_ERR_STATE", -8: "MXP_ERR_VERIFY",
}
ERR_IO, ERR_FORMAT, ERR_UNSUPPORTED, ERR_COVERAGE, ERR_ARG, ERR_DEVICE, ERR_STATE, ERR_VERIFY = range(-1, -9, -1)

DTYPES = ("F64", "F32", "F16", "BF16", "F8_E4M3", "F8_E5M2", "I64", "I32", "I16", "I8", "U8", "BOOL")
DTYPE_CODE = {n: i for i, n in enumerate(DTYPES)}
DTYPE_SIZE = {"F64": 8, "F32": 4, "F16": 2, "BF16": 2, "F8_E4M3": 1, "F8_E5M2": 1,
              "I64": 8, "I32": 4, "I16": 2, "I8": 1, "U8": 1, "BOOL": 1}

PLAN_ALLOW_CAST_F32_BF16 = 0x1
PLAN_ALLOW_UNMAPPED = 0x2
PLAN_ALLOW_UNCOVERED = 0x4
PLAN_NO_FP8_BLOCK_CHECK = 0x8
PLAN_NONLOCAL_EXPERTS_UNMAPPED = 0x10

WRITE_KINDS = ("direct", "fused", "expert", "premerged")


class MxpLibraryMissing(ImportError):
    """libmxplace.so has not been built (run ``python -m modelexpress_amd.build``)."""


class MxpError(RuntimeError):
    """A negative status from the C ABI, with the library's message."""

    def __init__(self, code: int, message: str):
        super().__init__(f"{ERR_NAMES.get(code, code)}: {message}")
        self.code = code
        self.message = message


class TensorInfo(C.Structure):
    _fields_ = [("name", C.c_char_p), ("dtype", C.c_int32), ("ndim", C.c_int32),
                ("shape", C.c_int64 * MXP_MAX_DIMS), ("file_index", C.c_int32), ("reserved", C.c_int32),
                ("file_offset", C.c_uint64), ("nbytes", C.c_uint64)]


class FileInfo(C.Structure):
    _fields_ = [("path", C.c_char_p), ("file_size", C.c_uint64), ("data_start", C.c_uint64),
                ("n_tensors", C.c_int64)]


class WriteInfo(C.Structure):
    _fields_ = [("tensor_index", C.c_int64), ("param_index", C.c_int64), ("kind", C.c_int32), ("cast", C.c_int32),
                ("src_offset", C.c_uint64), ("src_pitch", C.c_uint64), ("dst_offset", C.c_uint64),
                ("dst_pitch", C.c_uint64), ("rows", C.c_uint64), ("row_bytes", C.c_uint64),
                ("paired_runs", C.c_uint64)]


class ParamInfo(C.Structure):
    _fields_ = [("name", C.c_char_p), ("dtype", C.c_int32), ("ndim", C.c_int32),
                ("shape", C.c_int64 * MXP_MAX_DIMS), ("nbytes", C.c_uint64), ("bytes_written", C.c_uint64),
                ("n_writes", C.c_int32), ("reserved", C.c_int32)]


class Box(C.Structure):
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("src_pitch", C.c_uint64), ("dst_pitch", C.c_uint64),
                ("rows", C.c_uint64), ("row_bytes", C.c_uint64), ("csum_index", C.c_uint64),
                ("csum_group", C.c_uint32), ("cast", C.c_uint32)]


class ViewCopy(C.Structure):
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("ndim", C.c_int32), ("elem_size", C.c_int32),
                ("cast", C.c_int32), ("contiguous_src", C.c_uint8), ("contiguous_dst", C.c_uint8),
                ("reserved", C.c_uint16), ("shape", C.c_int64 * 8), ("src_strides", C.c_int64 * 8),
                ("dst_strides", C.c_int64 * 8)]


class EngineOptions(C.Structure):
    _fields_ = [("device", C.c_int32), ("ring_slots", C.c_int32), ("slot_bytes", C.c_uint64),
                ("reader_threads", C.c_int32), ("streams", C.c_int32), ("tile_bytes", C.c_uint32),
                ("nan_bits", C.c_uint16), ("pack_strided_on_host", C.c_uint16), ("use_o_direct", C.c_int32)]


class ExecStats(C.Structure):
    _fields_ = [("wall_seconds", C.c_double), ("read_seconds", C.c_double), ("kernel_ms", C.c_double),
                ("file_bytes", C.c_uint64), ("h2d_bytes", C.c_uint64), ("placed_bytes", C.c_uint64),
                ("n_chunks", C.c_uint64), ("n_segments", C.c_uint64), ("n_workgroups", C.c_uint64),
                ("n_launches", C.c_uint64), ("mutated", C.c_int32), ("reserved", C.c_int32)]

    def as_dict(self) -> dict:
        return {k: getattr(self, k) for k, _ in self._fields_ if k != "reserved"}


_P = C.c_void_p
_PP = C.POINTER(C.c_void_p)
_U64P = C.POINTER(C.c_uint64)
_U32P = C.POINTER(C.c_uint32)

# name -> (restype, argtypes); every symbol include/mxp.h declares (the product ABI).
SIGNATURES = {
    "mxp_last_error": (C.c_char_p, []),
    "mxp_abi_version": (C.c_int, []),
    "mxp_dtype_size": (C.c_int, [C.c_int]),
    "mxp_dtype_from_name": (C.c_int, [C.c_char_p]),
    "mxp_dtype_name": (C.c_char_p, [C.c_int]),
    "mxp_ckpt_open": (C.c_int, [C.c_char_p, _PP]),
    "mxp_ckpt_close": (None, [_P]),
    "mxp_ckpt_tensor_count": (C.c_int64, [_P]),
    "mxp_ckpt_file_count": (C.c_int64, [_P]),
    "mxp_ckpt_tensor_info": (C.c_int, [_P, C.c_int64, C.POINTER(TensorInfo)]),
    "mxp_ckpt_file_info": (C.c_int, [_P, C.c_int64, C.POINTER(FileInfo)]),
    "mxp_ckpt_find": (C.c_int64, [_P, C.c_char_p]),
    "mxp_plan_create": (C.c_int, [_P, C.c_int32, C.c_int32, C.c_uint32, _PP]),
    "mxp_plan_destroy": (None, [_P]),
    "mxp_plan_add_param": (C.c_int64, [_P, C.c_char_p, C.c_int32, C.c_int32, C.POINTER(C.c_int64)]),
    "mxp_plan_add_stacked": (C.c_int, [_P, C.c_char_p, C.c_char_p]),
    "mxp_plan_add_expert": (C.c_int, [_P, C.c_char_p, C.c_char_p, C.c_int32, C.c_char_p, C.c_int32]),
    "mxp_plan_add_skip_prefix": (C.c_int, [_P, C.c_char_p]),
    "mxp_plan_add_virtual": (C.c_int64, [_P, C.c_char_p, C.c_int32, C.POINTER(C.c_int64)]),
    "mxp_plan_add_virtual_shard": (C.c_int, [_P, C.c_int64, C.c_char_p, C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                                             C.POINTER(C.c_int64)]),
    "mxp_plan_build": (C.c_int, [_P]),
    "mxp_plan_param_count": (C.c_int64, [_P]),
    "mxp_plan_write_count": (C.c_int64, [_P]),
    "mxp_plan_param_info": (C.c_int, [_P, C.c_int64, C.POINTER(ParamInfo)]),
    "mxp_plan_write_info": (C.c_int, [_P, C.c_int64, C.POINTER(WriteInfo)]),
    "mxp_plan_totals": (C.c_int, [_P, _U64P, _U64P, _U64P, _U64P]),
    "mxp_engine_set_fused_digests": (C.c_int, [_P, C.c_int32]),
    "mxp_plan_digests": (C.c_int, [_P, _P, C.POINTER(C.c_uint8), C.c_int64]),
    "mxp_engine_create": (C.c_int, [C.POINTER(EngineOptions), _PP]),
    "mxp_engine_destroy": (None, [_P]),
    "mxp_prepare": (C.c_int, [_P, _P]),
    "mxp_execute": (C.c_int, [_P, _P, _PP, C.POINTER(ExecStats)]),
    "mxp_execute_after": (C.c_int, [_P, _P, _PP, _P, C.POINTER(ExecStats)]),
    "mxp_execute_resident": (C.c_int, [_P, _P, _PP, _PP, _P, C.POINTER(ExecStats)]),
    "mxp_engine_set_direct_placement": (C.c_int, [_P, C.c_int64]),
    "mxp_plan_checksums": (C.c_int, [_P, _P, _U32P, C.c_int64]),
    "mxp_checksum32": (C.c_int, [_P, _PP, _U64P, C.c_int64, _U32P, _P]),
    "mxp_checksum32_static": (C.c_int, [_P, _PP, _U64P, C.c_int64, _U32P, _P]),
    "mxp_verify_plan_create": (C.c_int, [_P, _PP, _U64P, C.c_int64, C.POINTER(C.c_void_p)]),
    "mxp_verify_plan_checksums": (C.c_int, [_P, _P, _U32P, _P]),
    "mxp_verify_plan_digests": (C.c_int, [_P, _P, C.POINTER(C.c_uint8), _U64P, _P]),
    "mxp_verify_plan_destroy": (None, [_P]),
    "mxp_digest": (C.c_int, [_P, _PP, _U64P, C.c_int64, C.POINTER(C.c_uint8), _U64P, _P]),
    "mxp_cast_f32_bf16": (C.c_int, [_P, _P, _P, C.c_uint64, _U32P, _P]),
    "mxp_cast": (C.c_int, [_P, _P, _P, C.c_uint64, C.c_int32, _U32P, _P]),
    "mxp_gather2d": (C.c_int, [_P, _P, C.c_uint64, _P, C.c_uint64, C.c_uint64, C.c_uint64, _U32P, _P]),
    "mxp_place_boxes": (C.c_int, [_P, C.POINTER(Box), C.c_int64, C.c_uint32, _U32P, _P]),
    "mxp_permute_copy": (C.c_int, [_P, _P, _P, C.c_int32, C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                                   C.POINTER(C.c_int32), C.c_int32, _U32P, _P]),
    "mxp_copy_view": (C.c_int, [_P, _P, _P, C.c_int32, C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                                C.POINTER(C.c_int64), C.c_int32, C.c_int32, _U32P, _P]),
    "mxp_copy_views": (C.c_int, [_P, C.POINTER(ViewCopy), C.c_int64, _P]),
    "mxp_view_plan_create": (C.c_int, [_P, C.POINTER(ViewCopy), C.c_int64, C.POINTER(C.c_void_p)]),
    "mxp_view_plan_run": (C.c_int, [_P, _P, _P]),
    "mxp_view_plan_bytes": (C.c_int, [_P, _U64P]),
    "mxp_view_plan_destroy": (None, [_P]),
    "mxp_copy_batch": (C.c_int, [_P, _PP, _PP, _U64P, C.c_int64, _U32P, _P]),
    "mxp_digest_from_scalars": (C.c_int, [_U64P, C.POINTER(C.c_uint8)]),
    "mxp_crc32c": (C.c_uint32, [C.c_uint32, _P, C.c_uint64]),
    "mxp_file_crc32c": (C.c_int, [C.c_char_p, C.c_uint64, _U32P, _U32P, C.c_uint64, _U64P]),
}

# The measurement and test-input entry points of include/mxp_bench.h (same library, no part of the drop-in boundary).
BENCH_SIGNATURES = {
    "mxp_measure_gather": (C.c_int, [_P, C.c_uint64, C.c_uint32, C.c_uint64, C.c_uint32, C.c_int32, C.c_int32, C.POINTER(C.c_double)]),
    "mxp_engine_set_launch_timing": (C.c_int, [_P, C.c_int32]),
    "mxp_engine_launch_times": (C.c_int, [_P, C.POINTER(C.c_float), C.c_int32, C.POINTER(C.c_int32)]),
    "mxp_measure_h2d": (C.c_int, [_P, C.c_uint64, C.c_int32, C.POINTER(C.c_double)]),
    "mxp_describe_views": (C.c_int, [_P, C.POINTER(ViewCopy), C.c_int64, C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "mxp_set_transpose_form": (C.c_int, [C.c_int32]),
    "mxp_measure_read": (C.c_int, [C.POINTER(C.c_char_p), C.c_int64, C.c_int32, C.c_uint64, C.c_int32, _U64P, C.POINTER(C.c_double)]),
    "mxp_synth_host": (C.c_int, [_P, C.c_uint64, C.c_int32, C.c_uint32, C.c_uint64, C.c_int32]),
    "mxp_synth_device": (C.c_int, [_P, C.c_uint64, C.c_int32, C.c_uint32, C.c_uint64, _P]),
}

_lib = None


def lib() -> C.CDLL:
    """The loaded library, with every signature set. Raises if it is absent or incomplete."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise MxpLibraryMissing(
            f"{LIB_PATH} not found: the HIP placement library is not built. "
            "Run `python -m modelexpress_amd.build`; there is no fallback path."
        )
    handle = C.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in {**SIGNATURES, **BENCH_SIGNATURES}.items():
        try:
            fn = getattr(handle, name)
        except AttributeError as exc:
            raise MxpLibraryMissing(f"{LIB_PATH} does not export {name}; rebuild it") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    if handle.mxp_abi_version() != 1:
        raise MxpLibraryMissing(f"{LIB_PATH} has ABI version {handle.mxp_abi_version()}, expected 1")
    _lib = handle
    return handle


def check(rc: int) -> int:
    """Raise MxpError for a negative status; pass non-negative values through."""
    if rc < 0:
        raise MxpError(int(rc), lib().mxp_last_error().decode("utf-8", "replace"))
    return rc
