"""ctypes binding of include/smelt_hip_compiler.h: dtype gateway, weights.bin layout, shape
routes and dispatch-record emitters (host-only entry points of libsmelt_hip.so)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import runtime as rt

DTYPES = ["fp16", "fp32", "bf16", "int32", "u4_lut", "affine_u4", "binary1", "ternary2",
          "turbo_quant_h", "raw", "trit5"]
(FP16, FP32, BF16, INT32, U4_LUT, AFFINE_U4, BINARY1, TERNARY2, TURBO_QUANT_H, RAW, TRIT5) = range(11)
ACT_FP16, ACT_BF16, ACT_FP32 = 0, 1, 2
GEMV, GEMM, GEMM_TN = 0, 1, 2
FUSION_NONE, FUSION_DUAL, FUSION_GATE_UP_SWIGLU, FUSION_GATE_UP_GEGLU = 0, 1, 2, 3
OUT_FP16, OUT_BF16, OUT_FP32 = 0, 1, 2
SLOT_FIXED, SLOT_VARIABLE = 0, 1
FAMILY_DENSE, FAMILY_AFFINE_U4, FAMILY_BINARY1, FAMILY_TERNARY2, FAMILY_LUT_U4, FAMILY_TQH, FAMILY_TRIT5 = 0, 100, 101, 102, 103, 104, 105
SELECT_OK, SELECT_MISSING, SELECT_NOT_MEANINGFUL = 0, -20, -21


class MatvecCell(C.Structure):
    _fields_ = [("activation", C.c_int), ("weight", C.c_int), ("shape", C.c_int),
                ("fusion", C.c_int), ("output", C.c_int), ("slot", C.c_int)]


class WeightEntry(C.Structure):
    _fields_ = [("offset", C.c_uint64), ("size_bytes", C.c_uint64), ("rows", C.c_int32),
                ("cols", C.c_int32), ("dtype", C.c_int32), ("group_size", C.c_int32),
                ("packed_row_stride", C.c_int32), ("padded_cols", C.c_int32),
                ("scales_offset", C.c_uint64), ("scales_size_bytes", C.c_uint64),
                ("biases_offset", C.c_uint64), ("biases_size_bytes", C.c_uint64)]


class Route(C.Structure):
    _fields_ = [("pipeline", C.c_char * 128), ("specialized", C.c_int32),
                ("rows_per_group", C.c_int32), ("batch_tile", C.c_int32), ("threads", C.c_int32),
                ("grid_w", C.c_int32)]


class Binding(C.Structure):
    _fields_ = [("slot", C.c_int32), ("offset", C.c_uint64), ("offset_kind", C.c_uint8)]


def bind(slot: int, offset: int = 0, kind: int = 0) -> Binding:
    return Binding(slot, offset, kind)


_declared = False


def lib() -> C.CDLL:
    global _declared
    l = rt.load_library()
    if _declared:
        return l
    vp, i32, u32, sz = C.c_void_p, C.c_int, C.c_uint32, C.c_size_t
    we, u64p = C.POINTER(WeightEntry), C.POINTER(C.c_uint64)
    sig = {
        "smelt_dtype_name": (C.c_char_p, [i32]),
        "smelt_dtype_from_name": (i32, [C.c_char_p]),
        "smelt_kernel_table_select": (i32, [C.POINTER(MatvecCell), i32, C.POINTER(i32)]),
        "smelt_kernel_table_meaningful_cells": (i32, [C.POINTER(MatvecCell), i32]),
        "smelt_layout_make_affine_entry": (i32, [i32, i32, i32, u64p, we]),
        "smelt_layout_make_signed_entry": (i32, [i32, i32, i32, i32, u64p, we]),
        "smelt_layout_make_dense_entry": (i32, [i32, i32, i32, u64p, we]),
        "smelt_layout_make_affine_bank": (i32, [C.POINTER(i32), i32, i32, i32, u64p, we]),
        "smelt_layout_make_signed_bank": (i32, [C.POINTER(i32), i32, i32, i32, i32, u64p, we]),
        "smelt_emit_bank_matvec": (i32, [vp, i32, we, i32, Binding, C.POINTER(Binding)]),
        "smelt_route_decode_affine": (i32, [i32, i32, i32, i32, i32, C.POINTER(Route)]),
        "smelt_route_prefill_affine": (i32, [i32, i32, i32, i32, i32, i32, C.POINTER(Route)]),
        "smelt_emitter_create": (i32, [i32, i32, C.POINTER(vp)]),
        "smelt_emitter_destroy": (None, [vp]),
        "smelt_emitter_last_error": (C.c_char_p, [vp]),
        "smelt_emit_matvec": (i32, [vp, i32, we, Binding, Binding, i32, i32]),
        "smelt_emit_matvec_add": (i32, [vp, i32, we, Binding, Binding, Binding]),
        "smelt_emit_gate_up_swiglu": (i32, [vp, i32, we, we, Binding, Binding, i32, i32]),
        "smelt_emit_rms_norm_scale_only": (i32, [vp, Binding, Binding, i32, C.c_float, i32]),
        "smelt_emit_fused_norm_matvec": (i32, [vp, i32, we, we, Binding, Binding, C.POINTER(Binding), Binding, Binding, C.c_float]),
        "smelt_emit_norm_scale_matvec": (i32, [vp, i32, we, Binding, Binding, Binding, Binding, Binding]),
        "smelt_emit_norm_scale_gate_up": (i32, [vp, i32, we, we, i32, Binding, Binding, Binding, Binding]),
        "smelt_emit_dual_matvec": (i32, [vp, i32, we, we, Binding, Binding, Binding]),
        "smelt_emit_lm_head_argmax": (i32, [vp, i32, we, Binding, Binding, Binding, i32, C.c_float]),
        "smelt_emit_swap": (i32, [vp]),
        "smelt_emit_activation_view": (i32, [vp, i32, Binding, Binding, Binding, i32, i32]),
        "smelt_emit_view_matvec": (i32, [vp, i32, we, i32, Binding, Binding, Binding, C.POINTER(Binding), i32]),
        "smelt_emit_view_gate_up_swiglu": (i32, [vp, i32, we, we, i32, Binding, Binding, Binding, i32]),
        "smelt_emit_rms_norm_1pw": (i32, [vp, Binding, Binding, Binding, C.POINTER(Binding), i32, C.c_float, i32]),
        "smelt_emit_elementwise": (i32, [vp, i32, Binding, Binding, Binding, i32]),
        "smelt_emit_swiglu_fused": (i32, [vp, Binding, Binding, Binding, i32]),
        "smelt_emitter_record_count": (sz, [vp]),
        "smelt_emitter_records": (C.POINTER(rt.DispatchRecord), [vp]),
        "smelt_emitter_pipeline_count": (sz, [vp]),
        "smelt_emitter_pipeline_name": (C.c_char_p, [vp, sz]),
        "smelt_emitter_argmax_partial_bytes": (sz, [vp]),
        "smelt_hip_resolve_pipeline_name": (i32, [C.c_char_p, i32, C.c_char_p, sz, C.c_char_p, sz]),
        "smelt_hip_plan_qmm": (i32, [u32, u32, u32, u32, u32, u32, sz, sz, C.POINTER(u32)]),
        "smelt_hip_plan_matvec": (i32, [i32, u32, u32, u32, u32, sz, i32, C.POINTER(u32)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(l, name)
        fn.restype = res
        fn.argtypes = args
    _declared = True
    return l


def select(activation, weight, shape=GEMV, fusion=FUSION_NONE, output=OUT_FP16, slot=SLOT_FIXED,
           hip_backend=False):
    cell = MatvecCell(activation, weight, shape, fusion, output, slot)
    fam = C.c_int(-1)
    rc = lib().smelt_kernel_table_select(C.byref(cell), int(hip_backend), C.byref(fam))
    return rc, fam.value


def meaningful_cells() -> list[MatvecCell]:
    n = lib().smelt_kernel_table_meaningful_cells(None, 0)
    arr = (MatvecCell * n)()
    lib().smelt_kernel_table_meaningful_cells(arr, n)
    return list(arr)


class Layout:
    """Running weights.bin layout (SmeltWeightLayout.computeLayout): entries advance one offset."""

    def __init__(self):
        self.offset = C.c_uint64(0)
        self.entries: list[WeightEntry] = []

    def _check(self, rc):
        if rc != 0:
            raise ValueError(f"layout call failed with {rc}")

    def affine(self, rows, cols, group) -> WeightEntry:
        e = WeightEntry()
        self._check(lib().smelt_layout_make_affine_entry(rows, cols, group, C.byref(self.offset), C.byref(e)))
        self.entries.append(e)
        return e

    def signed(self, rows, cols, dtype, group=128) -> WeightEntry:
        e = WeightEntry()
        self._check(lib().smelt_layout_make_signed_entry(rows, cols, dtype, group, C.byref(self.offset), C.byref(e)))
        self.entries.append(e)
        return e

    def affine_bank(self, member_rows, cols, group) -> list[WeightEntry]:
        n = len(member_rows)
        rows = (C.c_int * n)(*member_rows)
        out = (WeightEntry * n)()
        self._check(lib().smelt_layout_make_affine_bank(rows, n, cols, group, C.byref(self.offset), out))
        members = [WeightEntry.from_buffer_copy(bytes(out[i])) for i in range(n)]
        self.entries.extend(members)
        return members

    def signed_bank(self, member_rows, cols, dtype, group=128) -> list[WeightEntry]:
        n = len(member_rows)
        rows = (C.c_int * n)(*member_rows)
        out = (WeightEntry * n)()
        self._check(lib().smelt_layout_make_signed_bank(rows, n, cols, dtype, group, C.byref(self.offset), out))
        members = [WeightEntry.from_buffer_copy(bytes(out[i])) for i in range(n)]
        self.entries.extend(members)
        return members

    def dense(self, rows, cols, dtype) -> WeightEntry:
        e = WeightEntry()
        self._check(lib().smelt_layout_make_dense_entry(rows, cols, dtype, C.byref(self.offset), C.byref(e)))
        self.entries.append(e)
        return e

    @property
    def total_bytes(self) -> int:
        return int(self.offset.value)


def write_affine(image: np.ndarray, e: WeightEntry, packed, scales, biases) -> None:
    for off, arr, size in ((e.offset, packed, e.size_bytes), (e.scales_offset, scales, e.scales_size_bytes),
                           (e.biases_offset, biases, e.biases_size_bytes)):
        a = np.ascontiguousarray(arr).view(np.uint8).ravel()
        assert a.size == size, (a.size, size)
        image[off:off + a.size] = a


def write_signed(image: np.ndarray, e: WeightEntry, packed, scales) -> None:
    for off, arr, size in ((e.offset, packed, e.size_bytes), (e.scales_offset, scales, e.scales_size_bytes)):
        a = np.ascontiguousarray(arr).view(np.uint8).ravel()
        assert a.size == size, (a.size, size)
        image[off:off + a.size] = a


def route_decode_affine(rows, cols, group, fusion=FUSION_NONE, compute_units=256) -> Route:
    r = Route()
    rc = lib().smelt_route_decode_affine(rows, cols, group, fusion, compute_units, C.byref(r))
    if rc != 0:
        raise ValueError(f"no decode route ({rc})")
    return r


def route_prefill_affine(rows, cols, group, max_batch, fusion=FUSION_NONE, compute_units=256) -> Route:
    r = Route()
    rc = lib().smelt_route_prefill_affine(rows, cols, group, fusion, max_batch, compute_units, C.byref(r))
    if rc != 0:
        raise ValueError(f"no prefill route ({rc})")
    return r


def resolve_pipeline_name(entry: str, act=rt.ACT_F16):
    sym = C.create_string_buffer(128)
    kinds = C.create_string_buffer(64)
    rc = lib().smelt_hip_resolve_pipeline_name(entry.encode(), act, sym, 128, kinds, 64)
    return rc, sym.value.decode(), kinds.value.decode()


QMM_PLAN_FIELDS = ("kernel", "row_tiles", "k_waves", "per_wave", "ksplit", "grid_x", "grid_y", "grid_z",
                   "threads", "lds", "workspace")
MATVEC_PLAN_FIELDS = ("segments", "waves", "workgroups", "threads", "lds")
LAYOUT_U4, LAYOUT_BINARY1, LAYOUT_TERNARY2, LAYOUT_TRIT5 = range(4)


def plan_qmm(rows, cols, group, nmat, batch, compute_units=256, lds_limit=160 * 1024, workspace_bytes=1 << 30):
    """Launch plan of an affine qmm record, or None when it keeps the kernel its pipeline names."""
    out = (C.c_uint32 * 11)()
    rc = lib().smelt_hip_plan_qmm(rows, cols, group, nmat, batch, compute_units, lds_limit, workspace_bytes, out)
    if rc < 0:
        raise ValueError(f"smelt_hip_plan_qmm: {rc}")
    return dict(zip(QMM_PLAN_FIELDS, out)) if rc else None


def plan_matvec(layout, rows, cols, group, nmat=1, lds_limit=160 * 1024, force=False):
    """Launch plan of the single-pass matrix-core matvec, or None when the shape stays on its own kernel."""
    out = (C.c_uint32 * 5)()
    rc = lib().smelt_hip_plan_matvec(layout, rows, cols, group, nmat, lds_limit, int(force), out)
    if rc < 0:
        raise ValueError(f"smelt_hip_plan_matvec: {rc}")
    return dict(zip(MATVEC_PLAN_FIELDS, out)) if rc else None


class EmitError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"emit error {code}: {message}")
        self.code = code
        self.message = message


class Emitter:
    """Collects dispatch records and the pipeline-name list they index (SmeltCodeEmitter)."""

    def __init__(self, act_dtype=rt.ACT_F16, compute_units=256):
        self.l = lib()
        h = C.c_void_p()
        rc = self.l.smelt_emitter_create(act_dtype, compute_units, C.byref(h))
        if rc != 0:
            raise EmitError(rc, "cannot create emitter")
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            self.l.smelt_emitter_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc):
        if rc != 0:
            raise EmitError(rc, (self.l.smelt_emitter_last_error(self.h) or b"").decode())

    def matvec(self, weights_slot, w, x: Binding, y: Binding, batch=1, dynamic=False):
        self._check(self.l.smelt_emit_matvec(self.h, weights_slot, C.byref(w), x, y, batch, int(dynamic)))

    def matvec_add(self, weights_slot, w, x, y, residual):
        self._check(self.l.smelt_emit_matvec_add(self.h, weights_slot, C.byref(w), x, y, residual))

    def gate_up_swiglu(self, weights_slot, gate, up, x, y, batch=1, dynamic=False):
        self._check(self.l.smelt_emit_gate_up_swiglu(self.h, weights_slot, C.byref(gate), C.byref(up), x, y,
                                                     batch, int(dynamic)))

    def rms_norm_scale_only(self, x, scale, dim, eps=1e-6, batch=1):
        self._check(self.l.smelt_emit_rms_norm_scale_only(self.h, x, scale, dim, eps, batch))

    def norm_scale_matvec(self, weights_slot, w, scale, x, norm_weight, norm_output, y):
        """The affine matvec that normalises its input inline from a precomputed RMS scale."""
        self._check(self.l.smelt_emit_norm_scale_matvec(self.h, weights_slot, C.byref(w), scale, x, norm_weight,
                                                        norm_output, y))

    def norm_scale_gate_up(self, weights_slot, gate, up, scale, x, norm_weight, y, geglu=False):
        self._check(self.l.smelt_emit_norm_scale_gate_up(self.h, weights_slot, C.byref(gate), C.byref(up), int(geglu),
                                                         scale, x, norm_weight, y))

    def fused_norm_matvec(self, weights_slot, w, x, norm_weight, y, scratch, norm_output=None, up=None, eps=1e-6):
        """rms_norm_1pw + affine matvec (or gate+up+SwiGLU when `up` is given) in one dispatch."""
        self._check(self.l.smelt_emit_fused_norm_matvec(self.h, weights_slot, C.byref(w), C.byref(up) if up is not None else None,
                                                        x, norm_weight, C.byref(norm_output) if norm_output is not None else None,
                                                        y, scratch, eps))

    def dual_matvec(self, weights_slot, w1, w2, x, y1, y2):
        self._check(self.l.smelt_emit_dual_matvec(self.h, weights_slot, C.byref(w1), C.byref(w2), x, y1, y2))

    def bank_matvec(self, weights_slot, members, x, outputs) -> bool:
        """One dispatch for 2-4 contiguous same-input members; False if they do not form a bank."""
        n = len(members)
        arr = (WeightEntry * n)(*members)
        outs = (Binding * n)(*outputs)
        rc = self.l.smelt_emit_bank_matvec(self.h, weights_slot, arr, n, x, outs)
        if rc == 1:
            return False
        self._check(rc)
        return True

    def lm_head_argmax(self, weights_slot, w, x, keys, out, batch=1, logit_cap=0.0):
        self._check(self.l.smelt_emit_lm_head_argmax(self.h, weights_slot, C.byref(w), x, keys, out, batch,
                                                     C.c_float(logit_cap)))

    def rms_norm_1pw(self, x, weight, y, dim, eps=1e-6, batch=1, residual=None):
        res = None if residual is None else C.byref(residual)
        self._check(self.l.smelt_emit_rms_norm_1pw(self.h, x, weight, y, res, dim, C.c_float(eps), batch))

    def elementwise_add(self, a, b, y, count):
        self._check(self.l.smelt_emit_elementwise(self.h, 0, a, b, y, count))

    def elementwise_mul(self, a, b, y, count):
        self._check(self.l.smelt_emit_elementwise(self.h, 1, a, b, y, count))

    def swiglu_fused(self, gate, up, y, count):
        self._check(self.l.smelt_emit_swiglu_fused(self.h, gate, up, y, count))

    def activation_view(self, planes, x, view_planes, view_scales, cols, batch=1):
        self._check(self.l.smelt_emit_activation_view(self.h, planes, x, view_planes, view_scales, cols, batch))

    def view_matvec(self, weights_slot, w, planes, view_planes, view_scales, y, residual=None, batch=1):
        res = None if residual is None else C.byref(residual)
        self._check(self.l.smelt_emit_view_matvec(self.h, weights_slot, C.byref(w), planes, view_planes, view_scales, y, res, batch))

    def view_gate_up_swiglu(self, weights_slot, gate, up, planes, view_planes, view_scales, y, batch=1):
        self._check(self.l.smelt_emit_view_gate_up_swiglu(self.h, weights_slot, C.byref(gate), C.byref(up), planes,
                                                          view_planes, view_scales, y, batch))

    def swap(self):
        self._check(self.l.smelt_emit_swap(self.h))

    @property
    def pipelines(self) -> list[str]:
        n = self.l.smelt_emitter_pipeline_count(self.h)
        return [self.l.smelt_emitter_pipeline_name(self.h, i).decode() for i in range(n)]

    @property
    def argmax_partial_bytes(self) -> int:
        return int(self.l.smelt_emitter_argmax_partial_bytes(self.h))

    def records(self):
        """A copy of the record table (the bytes of dispatches.bin)."""
        n = self.l.smelt_emitter_record_count(self.h)
        arr = (rt.DispatchRecord * n)()
        if n:
            C.memmove(arr, self.l.smelt_emitter_records(self.h), n * C.sizeof(rt.DispatchRecord))
        return arr

    def install(self, ctx: rt.Context) -> None:
        """Create the context's pipeline table in manifest order (index == record.pipeline)."""
        for i, name in enumerate(self.pipelines):
            idx = ctx.pipeline(name)
            assert idx == i, (idx, i, name)
