"""ctypes loader for the C part of the CPU oracle (test infrastructure only)."""

from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "libmxp_oracle.so"


class OrcWrite(C.Structure):
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("src_pitch", C.c_uint64), ("dst_pitch", C.c_uint64),
                ("rows", C.c_uint64), ("row_bytes", C.c_uint64), ("dst_index", C.c_uint64), ("param", C.c_uint32),
                ("cast", C.c_uint32)]


def build() -> Path:
    subprocess.run(["make", "-C", str(HERE), "-B", "libmxp_oracle.so"], check=True, capture_output=True)
    return LIB


class OracleC:
    def __init__(self, handle):
        self.h = handle
        h = handle
        h.orc_checksum32.restype = C.c_uint32
        h.orc_checksum32.argtypes = [C.c_void_p, C.c_uint64]
        h.orc_checksum32_at.restype = C.c_uint32
        h.orc_checksum32_at.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64]
        h.orc_digest_scalars.restype = None
        h.orc_digest_scalars.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(C.c_uint64)]
        h.orc_cast.restype = None
        h.orc_cast.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint16]
        h.orc_cast_f32_bf16.restype = None
        h.orc_cast_f32_bf16.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint16]
        h.orc_copy2d.restype = None
        h.orc_copy2d.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64]
        h.orc_run_writes.restype = C.c_int
        h.orc_run_writes.argtypes = [C.POINTER(OrcWrite), C.c_uint64, C.c_uint64, C.POINTER(C.c_uint32), C.c_int,
                                     C.c_uint16]

    def checksum32(self, arr: np.ndarray, first_index: int = 0) -> str:
        a = np.ascontiguousarray(arr).reshape(-1).view(np.uint8)
        return format(self.h.orc_checksum32_at(a.ctypes.data, a.shape[0], first_index), "08x")

    def digest_scalars(self, arr: np.ndarray) -> list:
        a = np.ascontiguousarray(arr).reshape(-1).view(np.uint8)
        out = (C.c_uint64 * 7)()
        self.h.orc_digest_scalars(a.ctypes.data, a.shape[0], out)
        return [int(v) for v in out]

    def cast_f32_bf16(self, u32: np.ndarray, nan_bits: int = 0x7FC0) -> np.ndarray:
        src = np.ascontiguousarray(u32, dtype=np.uint32)
        dst = np.empty(src.shape, dtype=np.uint16)
        self.h.orc_cast_f32_bf16(src.ctypes.data, dst.ctypes.data, src.size, nan_bits)
        return dst

    def cast(self, code: int, bits: np.ndarray, nan_bits: int = 0x7FC0) -> np.ndarray:
        """Conversion ``code`` (1 fp32->bf16, 2 bf16->fp32, 3 fp16->fp32, 4 fp32->fp16, 5 fp8-e4m3->bf16) on bit patterns."""
        src_t, dst_t = {1: (np.uint32, np.uint16), 2: (np.uint16, np.uint32), 3: (np.uint16, np.uint32),
                        4: (np.uint32, np.uint16), 5: (np.uint8, np.uint16), 6: (np.uint16, np.uint16),
                        7: (np.uint16, np.uint16)}[code]
        src = np.ascontiguousarray(bits, dtype=src_t)
        dst = np.empty(src.shape, dtype=dst_t)
        self.h.orc_cast(code, src.ctypes.data, dst.ctypes.data, src.size, nan_bits)
        return dst

    def run_writes(self, writes: list, n_params: int, threads: int, nan_bits: int = 0x7FC0) -> list:
        arr = (OrcWrite * max(1, len(writes)))(*writes)
        sums = (C.c_uint32 * max(1, n_params))()
        rc = self.h.orc_run_writes(arr, len(writes), n_params, sums, threads, nan_bits)
        if rc != 0:
            raise RuntimeError("orc_run_writes failed")
        return [format(sums[i], "08x") for i in range(n_params)]


def load() -> OracleC:
    if not LIB.exists():
        build()
    return OracleC(C.CDLL(str(LIB)))
