"""ctypes loader for the CPU oracle (test infrastructure; never imported by the product).

Only tests/, the smoke check and the benchmark's cpu_baseline leg may import this
module.  Array arguments are numpy arrays; every wrapper checks dtypes and
contiguity before handing pointers to C.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F16, BF16, F32 = 0, 1, 2
BINARY1, TERNARY2, TRIT5 = 0, 1, 2

OK = 0
ERR_GEOMETRY = -1
ERR_BUFFER_TOO_SMALL = -2
ERR_INVALID_CODE = -3
ERR_MLX_SCALE = -4
ERR_MLX_BIAS = -5


def build(force: bool = False) -> str:
    """Compile liboracle.so with the Makefile beside this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


def _p(a: np.ndarray, dtype) -> C.c_void_p:
    assert a.dtype == np.dtype(dtype), (a.dtype, dtype)
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def _declare(l: C.CDLL) -> None:
    vp, i32, i64, f32, u16, u32 = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_uint16, C.c_uint32
    sig = {
        "so_f16_to_f32": (f32, [u16]),
        "so_f32_to_f16": (u16, [f32]),
        "so_f32_to_bf16": (u16, [f32]),
        "so_bf16_to_f32": (f32, [u16]),
        "so_round_through": (f32, [f32, i32]),
        "so_affine_num_groups": (i32, [i32, i32]),
        "so_affine_packed_row_stride": (i32, [i32]),
        "so_affine_params": (None, [f32, f32, i32, vp, vp, vp, vp]),
        "so_affine_quantize_row": (None, [vp, i32, i32, i32, vp, i32, vp, vp, vp]),
        "so_affine_dequantize_row": (None, [vp, vp, vp, i32, i32, i32, vp]),
        "so_affine_dequantize_row_narrow": (None, [vp, vp, vp, i32, i32, i32, i32, vp]),
        "so_affine_matvec": (None, [vp, vp, vp, vp, i32, i32, i32, i32, vp]),
        "so_affine_matvec_mt": (None, [vp, vp, vp, vp, i32, i32, i32, i32, vp]),
        "so_affine_matvec_dequant_f64": (None, [vp, vp, vp, vp, i32, i32, i32, i32, vp]),
        "so_signed_packed_byte_count": (i64, [i64, i32]),
        "so_signed_groups_per_row": (i32, [i32, i32]),
        "so_signed_code_at": (i32, [i64, vp, i64, i32]),
        "so_signed_semantic": (i32, [i32, i32, vp]),
        "so_signed_validate_codes": (i32, [vp, i64, i64, i32, vp]),
        "so_signed_canonical_mlx_scale_bits": (i32, [i32, u16, u16, vp]),
        "so_signed_normalize_mlx_scales": (i32, [i32, vp, vp, i32, vp, vp]),
        "so_signed_dequantize_row": (i32, [i32, vp, i64, vp, i64, i32, i32, i32, vp]),
        "so_signed_dequantize_row_f16": (i32, [i32, vp, i64, vp, i64, i32, i32, i32, vp]),
        "so_signed_pack_row": (None, [i32, vp, i32, vp, i64]),
        "so_trit5_build_lut": (None, [vp]),
        "so_signed_matvec": (i32, [i32, vp, i64, vp, vp, i32, i32, i32, i32, i32, vp]),
        "so_signed_matvec_mt": (i32, [i32, vp, i64, vp, vp, i32, i32, i32, i32, vp]),
        "so_signed_matvec_f64": (i32, [i32, vp, i64, vp, vp, i32, i32, i32, i32, i32, vp]),
        "so_ternary_affine_qmv": (None, [vp, vp, vp, vp, i32, i32, i32, vp]),
        "so_ternary_affine_qmm_weights": (None, [vp, vp, vp, i32, i32, vp]),
        "so_ternary_affine_qmm": (None, [vp, vp, vp, vp, i32, i32, i32, vp]),
        "so_epilogue_residual_add": (u16, [f32, u16, i32]),
        "so_epilogue_affine_swiglu": (u16, [f32, f32, i32]),
        "so_epilogue_geglu": (u16, [f32, f32, i32]),
        "so_unary": (u16, [i32, u16, f32, i32]),
        "so_rms_norm_1pw_add_scalar": (None, [vp, vp, vp, u16, i32, f32, i32, vp]),
        "so_rms_norm_1pw_from_fp32": (None, [vp, vp, i32, f32, i32, vp]),
        "so_rms_norm_gated": (None, [vp, vp, vp, i32, i32, f32, i32, i32, vp]),
        "so_rms_norm_gated_signed_activation_bitplanes": (None, [vp, vp, vp, i32, f32, i32, i32, vp, vp]),
        "so_norm_scale_input": (None, [vp, f32, vp, i32, i32, vp]),
        "so_epilogue_signed_swiglu": (u16, [u16, u16, i32]),
        "so_rms_scale": (f32, [vp, i32, f32, i32]),
        "so_rms_norm_1pw": (None, [vp, vp, vp, i32, f32, i32, i32, vp]),
        "so_swiglu_fused": (None, [vp, vp, i32, i32, vp]),
        "so_elementwise": (None, [vp, vp, i32, i32, i32, vp]),
        "so_bitplane_max_q": (i32, [i32]),
        "so_signed_activation_bitplanes": (None, [vp, i32, i32, i32, vp, vp, vp]),
        "so_swiglu_signed_activation_bitplanes": (None, [vp, vp, i32, i32, i32, vp, vp]),
        "so_sigmoid_mul_signed_activation_bitplanes": (None, [vp, vp, i32, i32, i32, vp, vp]),
        "so_sigmoid_mul": (u16, [u16, u16, i32]),
        "so_norm_scale_signed_activation_bitplanes": (None, [f32, vp, vp, i32, i32, i32, vp, vp]),
        "so_signed_bitplane_matvec": (None, [i32, vp, vp, vp, vp, i32, i32, i32, i32, vp]),
        "so_lut_matvec": (None, [vp, vp, vp, i32, i32, i32, vp]),
        "so_epilogue_lut_add": (u16, [f32, u16, i32]),
        "so_lut_gather": (None, [vp, vp, i32, i32, i32, vp]),
        "so_tqh_prepare": (None, [vp, i32, i32, vp]),
        "so_tqh_matvec": (None, [vp, vp, vp, i32, i32, vp]),
        "so_tqh_dequantize_row": (None, [vp, vp, i32, vp]),
        "so_argmax_ordered_key16": (u32, [u16]),
        "so_argmax_pack_key": (C.c_uint64, [u16, u32]),
        "so_argmax16": (i32, [vp, i32]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(l, name)
        fn.restype = res
        fn.argtypes = args


# ---------------------------------------------------------------------------
# conversions (vectorised helpers built on the scalar C entry points)
# ---------------------------------------------------------------------------

def f16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    l = lib()
    flat = np.ascontiguousarray(bits, dtype=np.uint16).ravel()
    return np.array([l.so_f16_to_f32(int(b)) for b in flat], dtype=np.float32).reshape(bits.shape)


def f32_to_f16_bits(vals: np.ndarray) -> np.ndarray:
    l = lib()
    flat = np.ascontiguousarray(vals, dtype=np.float32).ravel()
    return np.array([l.so_f32_to_f16(float(v)) for v in flat], dtype=np.uint16).reshape(vals.shape)


def widen(bits: np.ndarray, dtype: int) -> np.ndarray:
    """Exact widening of fp16/bf16 bit patterns to float32 (numpy; pinned against C in tests)."""
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    if dtype == BF16:
        return (bits.astype(np.uint32) << 16).view(np.float32)
    return bits.view(np.float16).astype(np.float32)


def narrow(vals: np.ndarray, dtype: int) -> np.ndarray:
    """RNE narrowing float32 -> fp16/bf16 bit patterns."""
    vals = np.ascontiguousarray(vals, dtype=np.float32)
    if dtype == BF16:
        b = vals.view(np.uint32)
        return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)
    return vals.astype(np.float16).view(np.uint16)


# ---------------------------------------------------------------------------
# affine u4
# ---------------------------------------------------------------------------

def affine_quantize(w: np.ndarray, group: int, clip: int = 0, importance=None, dtype: int = F16):
    rows, cols = w.shape
    w = np.ascontiguousarray(w, dtype=np.float32)
    groups = (cols + group - 1) // group
    stride = (cols + 1) // 2
    packed = np.zeros((rows, stride), np.uint8)
    scales = np.zeros((rows, groups), np.uint16)
    biases = np.zeros((rows, groups), np.uint16)
    imp = None if importance is None else np.ascontiguousarray(importance, dtype=np.float32)
    l = lib()
    for r in range(rows):
        l.so_affine_quantize_row(_p(w[r], np.float32), cols, group, clip,
                                 None if imp is None else _p(imp, np.float32), dtype,
                                 _p(packed[r], np.uint8), _p(scales[r], np.uint16),
                                 _p(biases[r], np.uint16))
    return packed, scales, biases


def affine_dequantize(packed, scales, biases, cols: int, group: int, dtype: int = F16) -> np.ndarray:
    rows = packed.shape[0]
    out = np.zeros((rows, cols), np.float32)
    l = lib()
    for r in range(rows):
        l.so_affine_dequantize_row(_p(packed[r], np.uint8), _p(scales[r], np.uint16),
                                   _p(biases[r], np.uint16), cols, group, dtype,
                                   _p(out[r], np.float32))
    return out


def affine_dequantize_narrow(packed, scales, biases, cols, group, dtype=F16, out_dtype=F16):
    rows = packed.shape[0]
    out = np.zeros((rows, cols), np.uint16)
    l = lib()
    for r in range(rows):
        l.so_affine_dequantize_row_narrow(_p(packed[r], np.uint8), _p(scales[r], np.uint16),
                                          _p(biases[r], np.uint16), cols, group, dtype, out_dtype,
                                          _p(out[r], np.uint16))
    return out


def affine_matvec(packed, scales, biases, x_f32, rows, cols, group, dtype=F16, threads=False):
    """x_f32: [batch, cols] float32 (already widened).  Returns unrounded fp32 [batch, rows]."""
    x = np.ascontiguousarray(np.atleast_2d(x_f32), dtype=np.float32)
    out = np.zeros((x.shape[0], rows), np.float32)
    fn = lib().so_affine_matvec_mt if threads else lib().so_affine_matvec
    packed = np.ascontiguousarray(packed)
    scales = np.ascontiguousarray(scales)
    biases = np.ascontiguousarray(biases)
    for b in range(x.shape[0]):
        fn(_p(packed, np.uint8), _p(scales, np.uint16), _p(biases, np.uint16),
           _p(x[b], np.float32), rows, cols, group, dtype, _p(out[b], np.float32))
    return out


def affine_matvec_f64(packed, scales, biases, x_f32, rows, cols, group, dtype=F16):
    x = np.ascontiguousarray(np.atleast_2d(x_f32), dtype=np.float32)
    out = np.zeros((x.shape[0], rows), np.float64)
    for b in range(x.shape[0]):
        lib().so_affine_matvec_dequant_f64(_p(np.ascontiguousarray(packed), np.uint8),
                                           _p(np.ascontiguousarray(scales), np.uint16),
                                           _p(np.ascontiguousarray(biases), np.uint16),
                                           _p(x[b], np.float32), rows, cols, group, dtype,
                                           _p(out[b], np.float64))
    return out


# ---------------------------------------------------------------------------
# signed codec
# ---------------------------------------------------------------------------


def signed_validate(codes: np.ndarray, logical_count: int, fmt: int):
    """(status, index of the first invalid code or -1) — SmeltSignedQuantCodec.swift:128-145"""
    codes = np.ascontiguousarray(codes, np.uint8)
    bad = C.c_int64(-1)
    rc = lib().so_signed_validate_codes(_p(codes, np.uint8), codes.size, logical_count, fmt, C.byref(bad))
    return rc, bad.value


def signed_normalize_mlx(fmt: int, scales: np.ndarray, biases: np.ndarray):
    """(status, canonical scale bits, failing group or -1) — SmeltSignedQuantCodec.swift:154-215"""
    scales = np.ascontiguousarray(scales, np.uint16)
    biases = np.ascontiguousarray(biases, np.uint16)
    out = np.zeros(scales.shape, np.uint16)
    bad = C.c_int(-1)
    rc = lib().so_signed_normalize_mlx_scales(fmt, _p(scales, np.uint16), _p(biases, np.uint16), scales.size,
                                              _p(out, np.uint16), C.byref(bad))
    return rc, out, bad.value


def signed_row_stride(padded_cols: int, fmt: int, align: int = 1) -> int:
    n = int(lib().so_signed_packed_byte_count(padded_cols, fmt))
    return (n + align - 1) // align * align


def signed_pack(codes: np.ndarray, fmt: int, row_stride: int | None = None) -> np.ndarray:
    """codes: [rows, cols] uint8 of packed-domain codes (binary 0/1, ternary 0/1/2)."""
    rows, cols = codes.shape
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    stride = row_stride or signed_row_stride(cols, fmt)
    out = np.zeros((rows, stride), np.uint8)
    for r in range(rows):
        lib().so_signed_pack_row(fmt, _p(codes[r], np.uint8), cols, _p(out[r], np.uint8), stride)
    return out


def signed_dequantize(fmt, packed, scales, cols, padded_cols, group):
    rows = packed.shape[0]
    out = np.zeros((rows, cols), np.float32)
    for r in range(rows):
        rc = lib().so_signed_dequantize_row(fmt, _p(packed[r], np.uint8), packed.shape[1],
                                            _p(scales[r], np.uint16), scales.shape[1] * 2, cols,
                                            padded_cols, group, _p(out[r], np.float32))
        if rc != OK:
            raise ValueError(f"so_signed_dequantize_row rc={rc}")
    return out


def signed_matvec(fmt, packed, scales, x_f32, rows, cols, padded_cols, group, threads=False):
    x = np.ascontiguousarray(np.atleast_2d(x_f32), dtype=np.float32)
    batch = x.shape[0]
    out = np.zeros((batch, rows), np.float32)
    packed = np.ascontiguousarray(packed)
    scales = np.ascontiguousarray(scales)
    if threads:
        for b in range(batch):
            rc = lib().so_signed_matvec_mt(fmt, _p(packed, np.uint8), packed.shape[1],
                                           _p(scales, np.uint16), _p(x[b], np.float32), rows, cols,
                                           padded_cols, group, _p(out[b], np.float32))
            if rc != OK:
                raise ValueError(f"so_signed_matvec_mt rc={rc}")
        return out
    rc = lib().so_signed_matvec(fmt, _p(packed, np.uint8), packed.shape[1], _p(scales, np.uint16),
                                _p(x, np.float32), rows, cols, padded_cols, group, batch,
                                _p(out, np.float32))
    if rc != OK:
        raise ValueError(f"so_signed_matvec rc={rc}")
    return out


def signed_matvec_f64(fmt, packed, scales, x_f32, rows, cols, padded_cols, group):
    x = np.ascontiguousarray(np.atleast_2d(x_f32), dtype=np.float32)
    batch = x.shape[0]
    out = np.zeros((batch, rows), np.float64)
    rc = lib().so_signed_matvec_f64(fmt, _p(np.ascontiguousarray(packed), np.uint8),
                                    packed.shape[1], _p(np.ascontiguousarray(scales), np.uint16),
                                    _p(x, np.float32), rows, cols, padded_cols, group, batch,
                                    _p(out, np.float64))
    if rc != OK:
        raise ValueError(f"so_signed_matvec_f64 rc={rc}")
    return out


def ternary_affine_qmv(packed, scales, x_bits, rows, cols):
    x = np.ascontiguousarray(np.atleast_2d(x_bits), dtype=np.uint16)
    out = np.zeros((x.shape[0], rows), np.uint16)
    packed = np.ascontiguousarray(packed)
    scales = np.ascontiguousarray(scales)
    lib().so_ternary_affine_qmv(_p(packed, np.uint8), _p(scales, np.uint16), _p(scales, np.uint16),
                                _p(x, np.uint16), rows, cols, x.shape[0], _p(out, np.uint16))
    return out


def ternary_affine_qmm_weights(packed, scales, rows, cols, bias_scales=None):
    """fp16 bits [rows, cols] of the QMM weight tile with per-byte-lane rounded subscales."""
    packed = np.ascontiguousarray(packed)
    scales = np.ascontiguousarray(scales)
    bias_scales = scales if bias_scales is None else np.ascontiguousarray(bias_scales)
    out = np.zeros((rows, cols), np.uint16)
    lib().so_ternary_affine_qmm_weights(_p(packed, np.uint8), _p(scales, np.uint16),
                                        _p(bias_scales, np.uint16), rows, cols, _p(out, np.uint16))
    return out


def ternary_affine_qmm(packed, scales, x_bits, rows, cols, bias_scales=None):
    x = np.ascontiguousarray(np.atleast_2d(x_bits), dtype=np.uint16)
    packed = np.ascontiguousarray(packed)
    scales = np.ascontiguousarray(scales)
    bias_scales = scales if bias_scales is None else np.ascontiguousarray(bias_scales)
    out = np.zeros((x.shape[0], rows), np.float32)
    lib().so_ternary_affine_qmm(_p(packed, np.uint8), _p(scales, np.uint16), _p(bias_scales, np.uint16),
                                _p(x, np.uint16), rows, cols, x.shape[0], _p(out, np.float32))
    return out


def trit5_lut() -> np.ndarray:
    out = np.zeros(256, np.uint16)
    lib().so_trit5_build_lut(_p(out, np.uint16))
    return out


def argmax16(bits: np.ndarray) -> int:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    return int(lib().so_argmax16(_p(bits, np.uint16), bits.size))


def epilogue_residual_add(acc: np.ndarray, residual_bits: np.ndarray, dtype: int) -> np.ndarray:
    l = lib()
    return np.array([l.so_epilogue_residual_add(float(a), int(r), dtype)
                     for a, r in zip(np.ravel(acc), np.ravel(residual_bits))],
                    dtype=np.uint16).reshape(np.shape(acc))


def epilogue_affine_swiglu(gate: np.ndarray, up: np.ndarray, dtype: int) -> np.ndarray:
    l = lib()
    return np.array([l.so_epilogue_affine_swiglu(float(g), float(u), dtype)
                     for g, u in zip(np.ravel(gate), np.ravel(up))],
                    dtype=np.uint16).reshape(np.shape(gate))


def epilogue_geglu(gate: np.ndarray, up: np.ndarray, dtype: int) -> np.ndarray:
    l = lib()
    return np.array([l.so_epilogue_geglu(float(g), float(u), dtype)
                     for g, u in zip(np.ravel(gate), np.ravel(up))],
                    dtype=np.uint16).reshape(np.shape(gate))


def norm_scale_input(x_bits: np.ndarray, rs: float, w_bits: np.ndarray, dtype: int) -> np.ndarray:
    """The activation row a norm-scale matvec consumes (and stores): narrow((x * rs) * (1 + w))."""
    x = np.ascontiguousarray(x_bits, np.uint16).ravel()
    out = np.zeros(x.size, np.uint16)
    lib().so_norm_scale_input(_p(x, np.uint16), float(rs), _p(np.ascontiguousarray(w_bits, np.uint16).ravel(), np.uint16),
                              dtype, x.size, _p(out, np.uint16))
    return out.reshape(np.shape(x_bits))


def epilogue_signed_swiglu(gate_bits: np.ndarray, up_bits: np.ndarray, dtype: int) -> np.ndarray:
    l = lib()
    return np.array([l.so_epilogue_signed_swiglu(int(g), int(u), dtype)
                     for g, u in zip(np.ravel(gate_bits), np.ravel(up_bits))],
                    dtype=np.uint16).reshape(np.shape(gate_bits))


# ---------------------------------------------------------------------------
# layer ops between the matvecs (norms.metal, activations_precise.metal, activations.metal)
# ---------------------------------------------------------------------------

def rms_scale(x_bits: np.ndarray, eps: float, dtype: int) -> float:
    x = np.ascontiguousarray(x_bits, np.uint16)
    return float(lib().so_rms_scale(_p(x, np.uint16), x.size, eps, dtype))


def rms_norm_1pw(x_bits, w_bits, eps: float, dtype: int, two_step, residual_bits=None) -> np.ndarray:
    """two_step: False/0 = x * (rs * (1 + w)), True/1 = half(1 + w) * half(x * rs), 2 = (x * rs) * (1 + w)."""
    x = np.ascontiguousarray(x_bits, np.uint16)
    w = np.ascontiguousarray(w_bits, np.uint16)
    out = np.zeros(x.size, np.uint16)
    res = None if residual_bits is None else np.ascontiguousarray(residual_bits, np.uint16)
    lib().so_rms_norm_1pw(_p(x, np.uint16), _p(w, np.uint16), None if res is None else _p(res, np.uint16),
                          x.size, eps, dtype, int(two_step), _p(out, np.uint16))
    return out


def rms_norm_1pw_add_scalar(x_bits, w_bits, residual_bits, scalar_bits: int, eps: float, dtype: int) -> np.ndarray:
    x = np.ascontiguousarray(x_bits, np.uint16)
    out = np.zeros(x.size, np.uint16)
    lib().so_rms_norm_1pw_add_scalar(_p(x, np.uint16), _p(np.ascontiguousarray(w_bits, np.uint16), np.uint16),
                                     _p(np.ascontiguousarray(residual_bits, np.uint16), np.uint16), int(scalar_bits),
                                     x.size, eps, dtype, _p(out, np.uint16))
    return out


def rms_norm_1pw_from_fp32(x_f32, w_bits, eps: float, dtype: int) -> np.ndarray:
    x = np.ascontiguousarray(x_f32, np.float32)
    out = np.zeros(x.size, np.uint16)
    lib().so_rms_norm_1pw_from_fp32(_p(x, np.float32), _p(np.ascontiguousarray(w_bits, np.uint16), np.uint16), x.size,
                                    eps, dtype, _p(out, np.uint16))
    return out


def rms_norm_gated(x_bits, gate_bits, w_bits, heads: int, head_dim: int, eps: float, dtype: int, precise: bool = False) -> np.ndarray:
    x = np.ascontiguousarray(x_bits, np.uint16)
    out = np.zeros(x.size, np.uint16)
    lib().so_rms_norm_gated(_p(x, np.uint16), _p(np.ascontiguousarray(gate_bits, np.uint16), np.uint16),
                            _p(np.ascontiguousarray(w_bits, np.uint16), np.uint16), heads, head_dim, eps, dtype,
                            int(precise), _p(out, np.uint16))
    return out


def rms_norm_gated_activation_bitplanes(x_bits, gate_bits, w_bits, heads: int, eps: float, dtype: int, precise: bool):
    """(planes [heads, 6, 4] u32, scales [heads] u16) of the gated norm of `heads` heads of 128 values."""
    x = np.ascontiguousarray(x_bits, np.uint16)
    out = np.zeros((heads, 6, 4), np.uint32)
    scales = np.zeros(heads, np.uint16)
    lib().so_rms_norm_gated_signed_activation_bitplanes(
        _p(x, np.uint16), _p(np.ascontiguousarray(gate_bits, np.uint16), np.uint16),
        _p(np.ascontiguousarray(w_bits, np.uint16), np.uint16), heads, eps, dtype, int(precise), _p(out, np.uint32),
        _p(scales, np.uint16))
    return out, scales


UNARY_OPS = {"silu": 0, "sigmoid_kernel": 1, "softplus": 2, "scalar_mul": 3, "logit_cap": 4}


def unary(name: str, x_bits, dtype: int, param: float = 0.0) -> np.ndarray:
    l, op = lib(), UNARY_OPS[name]
    return np.array([l.so_unary(op, int(b), float(param), dtype) for b in np.ravel(x_bits)], np.uint16).reshape(np.shape(x_bits))


def swiglu_fused(gate_bits, up_bits, dtype: int) -> np.ndarray:
    g = np.ascontiguousarray(gate_bits, np.uint16)
    u = np.ascontiguousarray(up_bits, np.uint16)
    out = np.zeros(g.size, np.uint16)
    lib().so_swiglu_fused(_p(g, np.uint16), _p(u, np.uint16), g.size, dtype, _p(out, np.uint16))
    return out


def elementwise(a_bits, b_bits, dtype: int, multiply: bool = False) -> np.ndarray:
    a = np.ascontiguousarray(a_bits, np.uint16)
    b = np.ascontiguousarray(b_bits, np.uint16)
    out = np.zeros(a.size, np.uint16)
    lib().so_elementwise(_p(a, np.uint16), _p(b, np.uint16), a.size, dtype, int(multiply), _p(out, np.uint16))
    return out


# ---------------------------------------------------------------------------
# signed activation views (bit planes) — signed_quant.metal:746-2260
# ---------------------------------------------------------------------------

def activation_bitplanes(x_bits, planes: int, dtype: int):
    """(planes [groups, planes, 4] u32, scales [groups] u16, q [cols] int32)"""
    x = np.ascontiguousarray(x_bits, np.uint16)
    groups = x.size // 128
    out = np.zeros((groups, planes, 4), np.uint32)
    scales = np.zeros(groups, np.uint16)
    q = np.zeros(x.size, np.int32)
    lib().so_signed_activation_bitplanes(_p(x, np.uint16), x.size, planes, dtype, _p(out, np.uint32),
                                         _p(scales, np.uint16), _p(q, np.int32))
    return out, scales, q


def sigmoid_mul(a_bits, b_bits, dtype: int) -> np.ndarray:
    l = lib()
    return np.array([l.so_sigmoid_mul(int(a), int(b), dtype) for a, b in zip(np.ravel(a_bits), np.ravel(b_bits))],
                    dtype=np.uint16).reshape(np.shape(a_bits))


def sigmoid_mul_activation_bitplanes(a_bits, b_bits, planes: int, dtype: int):
    a = np.ascontiguousarray(a_bits, np.uint16)
    b = np.ascontiguousarray(b_bits, np.uint16)
    out = np.zeros((a.size // 128, planes, 4), np.uint32)
    scales = np.zeros(a.size // 128, np.uint16)
    lib().so_sigmoid_mul_signed_activation_bitplanes(_p(a, np.uint16), _p(b, np.uint16), a.size, planes, dtype,
                                                     _p(out, np.uint32), _p(scales, np.uint16))
    return out, scales


def swiglu_activation_bitplanes(gate_bits, up_bits, planes: int, dtype: int):
    g = np.ascontiguousarray(gate_bits, np.uint16)
    u = np.ascontiguousarray(up_bits, np.uint16)
    out = np.zeros((g.size // 128, planes, 4), np.uint32)
    scales = np.zeros(g.size // 128, np.uint16)
    lib().so_swiglu_signed_activation_bitplanes(_p(g, np.uint16), _p(u, np.uint16), g.size, planes, dtype,
                                                _p(out, np.uint32), _p(scales, np.uint16))
    return out, scales


def norm_scale_activation_bitplanes(rs: float, x_bits, w_bits, planes: int, dtype: int):
    x = np.ascontiguousarray(x_bits, np.uint16)
    w = np.ascontiguousarray(w_bits, np.uint16)
    out = np.zeros((x.size // 128, planes, 4), np.uint32)
    scales = np.zeros(x.size // 128, np.uint16)
    lib().so_norm_scale_signed_activation_bitplanes(rs, _p(x, np.uint16), _p(w, np.uint16), x.size, planes, dtype,
                                                    _p(out, np.uint32), _p(scales, np.uint16))
    return out, scales


def signed_bitplane_matvec(fmt, packed, weight_scales, planes_arr, act_scales, rows, cols, dtype):
    packed = np.ascontiguousarray(packed, np.uint8)
    ws = np.ascontiguousarray(weight_scales, np.uint16)
    pl = np.ascontiguousarray(planes_arr, np.uint32)
    sc = np.ascontiguousarray(act_scales, np.uint16)
    out = np.zeros(rows, np.float32)
    lib().so_signed_bitplane_matvec(fmt, _p(packed, np.uint8), _p(ws, np.uint16), _p(pl, np.uint32), _p(sc, np.uint16),
                                    rows, cols, pl.shape[1], dtype, _p(out, np.float32))
    return out


# ---------------------------------------------------------------------------
# u4_lut — lut_matvec.metal:28-790, 967-992
# ---------------------------------------------------------------------------

def lut_matvec(indices, lut_bits, x_f32, rows, cols, group) -> np.ndarray:
    idx = np.ascontiguousarray(indices, np.uint8)
    lut = np.ascontiguousarray(lut_bits, np.uint16)
    x = np.ascontiguousarray(x_f32, np.float32)
    out = np.zeros(rows, np.float32)
    lib().so_lut_matvec(_p(idx, np.uint8), _p(lut, np.uint16), _p(x, np.float32), rows, cols, group, _p(out, np.float32))
    return out


def epilogue_lut_add(acc: np.ndarray, residual_bits: np.ndarray, dtype: int) -> np.ndarray:
    l = lib()
    return np.array([l.so_epilogue_lut_add(float(a), int(r), dtype) for a, r in zip(np.ravel(acc), np.ravel(residual_bits))],
                    dtype=np.uint16)


def lut_gather(indices, lut_bits, row, cols, group) -> np.ndarray:
    idx = np.ascontiguousarray(indices, np.uint8)
    lut = np.ascontiguousarray(lut_bits, np.uint16)
    out = np.zeros(cols, np.uint16)
    lib().so_lut_gather(_p(idx, np.uint8), _p(lut, np.uint16), row, cols, group, _p(out, np.uint16))
    return out


# ---------------------------------------------------------------------------
# turbo_quant_h — lut_matvec.metal:1045-1079, 9207-9355
# ---------------------------------------------------------------------------

def tqh_prepare(x_bits, dtype: int) -> np.ndarray:
    x = np.ascontiguousarray(x_bits, np.uint16)
    out = np.zeros((x.size + 127) // 128 * 128, np.float32)
    lib().so_tqh_prepare(_p(x, np.uint16), x.size, dtype, _p(out, np.float32))
    return out


def tqh_matvec(codes, codebook_bits, xhat, rows, cols) -> np.ndarray:
    c = np.ascontiguousarray(codes, np.uint8)
    cb = np.ascontiguousarray(codebook_bits, np.uint16)
    xh = np.ascontiguousarray(xhat, np.float32)
    out = np.zeros(rows, np.float32)
    lib().so_tqh_matvec(_p(c, np.uint8), _p(cb, np.uint16), _p(xh, np.float32), rows, cols, _p(out, np.float32))
    return out


def tqh_dequantize_row(row_codes, codebook_bits, cols) -> np.ndarray:
    c = np.ascontiguousarray(row_codes, np.uint8)
    cb = np.ascontiguousarray(codebook_bits, np.uint16)
    out = np.zeros(cols, np.float32)
    lib().so_tqh_dequantize_row(_p(c, np.uint8), _p(cb, np.uint16), cols, _p(out, np.float32))
    return out
