"""ctypes mirror of include/smelt_hip_import.h: the GPU weight-import producers.

`Importer` stands where SmeltCompiler's CPU routines stand in the reference
(SmeltAffineQuantizer.quantizeTensorAffine, SmeltAffineQuantizer.swift:399-513;
SmeltSignedQuantCodec.validateCodes / normalizeMLXScales, SmeltSignedQuantCodec.swift:128-215):
numpy arrays in, numpy arrays out, errors raised as exceptions that carry the offending index."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import runtime as rt

SRC_F32, SRC_F16, SRC_BF16 = 0, 1, 2
CLIP_MIN_MAX, CLIP_MSE_OPTIMAL = 0, 1
FORMAT_BINARY1, FORMAT_TERNARY2, FORMAT_TRIT5 = 0, 1, 2
ERR_INVALID_CODE, ERR_MLX_SCALE, ERR_MLX_BIAS, ERR_BUFFER_TOO_SMALL = -20, -21, -22, -23


class ImportError_(RuntimeError):
    """A failed import call: `code` is the C status, `index` the offending code / group if any."""

    def __init__(self, code: int, message: str, index: int | None = None):
        super().__init__(f"{message} (status {code})")
        self.code = code
        self.index = index


_declared = False


def _lib() -> C.CDLL:
    global _declared
    lib = rt.load_library()
    if not _declared:
        vp, i32, sz = C.c_void_p, C.c_int, C.c_size_t
        lib.smelt_hip_importer_create.restype = i32
        lib.smelt_hip_importer_create.argtypes = [i32, C.c_char_p, C.POINTER(vp)]
        lib.smelt_hip_importer_destroy.restype = None
        lib.smelt_hip_importer_destroy.argtypes = [vp]
        lib.smelt_hip_importer_last_error.restype = C.c_char_p
        lib.smelt_hip_importer_last_error.argtypes = [vp]
        lib.smelt_hip_import_quantize_affine_u4.restype = i32
        lib.smelt_hip_import_quantize_affine_u4.argtypes = [vp, vp, i32, i32, i32, i32, i32, vp, i32, vp, vp, vp]
        lib.smelt_hip_import_validate_signed_codes.restype = i32
        lib.smelt_hip_import_validate_signed_codes.argtypes = [vp, vp, sz, C.c_uint64, i32, C.POINTER(C.c_int64)]
        lib.smelt_hip_import_normalize_mlx_scales.restype = i32
        lib.smelt_hip_import_normalize_mlx_scales.argtypes = [vp, i32, vp, vp, sz, vp, C.POINTER(C.c_int64)]
        _declared = True
    return lib


def _ptr(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


class Importer:
    def __init__(self, device: int = 0):
        self.lib = _lib()
        self.h = C.c_void_p()
        rc = self.lib.smelt_hip_importer_create(device, rt.LIB_DIR.encode(), C.byref(self.h))
        if rc != 0:
            raise ImportError_(rc, self.lib.smelt_hip_importer_last_error(None).decode())

    def close(self) -> None:
        if self.h:
            self.lib.smelt_hip_importer_destroy(self.h)
            self.h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _raise(self, rc: int, index: int | None = None):
        raise ImportError_(rc, self.lib.smelt_hip_importer_last_error(self.h).decode(), index)

    def quantize_affine_u4(self, src: np.ndarray, src_dtype: int, rows: int, cols: int, group: int,
                           clip: int = CLIP_MIN_MAX, importance: np.ndarray | None = None,
                           scale_dtype: int = rt.ACT_F16):
        """src: fp32 values (SRC_F32) or raw 16-bit patterns (SRC_F16 / SRC_BF16), row-major.
        Returns (packed [rows, ceil(cols/2)] u8, scales [rows, groups] u16, biases [rows, groups] u16)."""
        src = np.ascontiguousarray(src)
        want = np.float32 if src_dtype == SRC_F32 else np.uint16
        if src.dtype != want or src.size != rows * cols:
            raise ValueError("source array does not match dtype / shape")
        gpr = (cols + group - 1) // group
        packed = np.empty((rows, (cols + 1) // 2), np.uint8)
        scales = np.empty((rows, gpr), np.uint16)
        biases = np.empty((rows, gpr), np.uint16)
        imp = None
        if importance is not None:
            imp = np.ascontiguousarray(importance, np.float32)
            if imp.size != cols:
                raise ValueError("importance needs one weight per column")
        rc = self.lib.smelt_hip_import_quantize_affine_u4(
            self.h, _ptr(src), src_dtype, rows, cols, group, clip, _ptr(imp) if imp is not None else None,
            scale_dtype, _ptr(packed), _ptr(scales), _ptr(biases))
        if rc != 0:
            self._raise(rc)
        return packed, scales, biases

    def validate_signed_codes(self, codes: np.ndarray, logical_count: int, fmt: int) -> None:
        codes = np.ascontiguousarray(codes, np.uint8)
        bad = C.c_int64(-1)
        rc = self.lib.smelt_hip_import_validate_signed_codes(self.h, _ptr(codes), codes.size, logical_count, fmt, C.byref(bad))
        if rc != 0:
            self._raise(rc, bad.value if bad.value >= 0 else None)

    def normalize_mlx_scales(self, fmt: int, scales: np.ndarray, biases: np.ndarray) -> np.ndarray:
        scales = np.ascontiguousarray(scales, np.uint16)
        biases = np.ascontiguousarray(biases, np.uint16)
        if scales.size != biases.size:
            raise ValueError("scales and biases differ in length")
        out = np.empty(scales.shape, np.uint16)
        bad = C.c_int64(-1)
        rc = self.lib.smelt_hip_import_normalize_mlx_scales(self.h, fmt, _ptr(scales), _ptr(biases), scales.size, _ptr(out), C.byref(bad))
        if rc != 0:
            self._raise(rc, bad.value if bad.value >= 0 else None)
        return out
