"""MLX safetensors triplets -> one semantic signed tensor, and the writer that streams such tensors
and dense ones into a planned weights.bin.

Mirrors SmeltPrequantizedSafetensors / SmeltPrequantizedTensorView
(Sources/SmeltCompiler/SmeltPrequantizedTensor.swift:52-300) and SmeltNativeWeightWriter.write
(Sources/SmeltCompiler/SmeltNativeWeightWriter.swift:70-389): the same discovery rules, geometry
checks and error kinds.  Code validation and the (scale, bias) -> canonical scale normalisation
run on the GPU through `Importer`; there is no CPU path for them here.
"""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass

import numpy as np

from . import importer as im
from .package import WeightRecord, total_bytes

# element sizes of the safetensors dtypes this adapter meets
_ST_ITEMSIZE = {"U32": 4, "I32": 4, "F32": 4, "F16": 2, "BF16": 2, "U8": 1, "I8": 1, "I64": 8, "F64": 8,
                "U16": 2, "I16": 2, "BOOL": 1, "U64": 8}
FORMAT_NAMES = {im.FORMAT_BINARY1: "binary1", im.FORMAT_TERNARY2: "ternary2"}
_BITS = {im.FORMAT_BINARY1: 1, im.FORMAT_TERNARY2: 2}


class PrequantizedError(ValueError):
    """SmeltPrequantizedTensorError; `kind` is the case name."""

    def __init__(self, kind: str, message: str):
        super().__init__(message)
        self.kind = kind


class NativeWriterError(ValueError):
    """SmeltNativeWeightWriterError; `kind` is the case name."""

    def __init__(self, kind: str, message: str):
        super().__init__(message)
        self.kind = kind


@dataclass
class TensorInfo:
    name: str
    dtype: str          # safetensors spelling: "U32", "F16", ...
    shape: list
    data: np.ndarray    # uint8 view of the payload (a memory map for files)

    @property
    def byte_count(self) -> int:
        return int(self.data.size)


def read_safetensors(paths) -> list[TensorInfo]:
    """Header parse + zero-copy payload views of one or more .safetensors files, in file order.
    Nothing in the file is executed: the header is JSON, payloads are raw little-endian arrays."""
    out = []
    for path in ([paths] if isinstance(paths, (str, os.PathLike)) else paths):
        with open(path, "rb") as f:
            head = f.read(8)
            if len(head) != 8:
                raise PrequantizedError("invalidPayload", f"{path}: truncated safetensors header")
            (hlen,) = struct.unpack("<Q", head)
            header = json.loads(f.read(hlen).decode("utf-8"), object_pairs_hook=list)
        base = 8 + hlen
        size = os.path.getsize(path)
        mm = np.memmap(path, dtype=np.uint8, mode="r") if size > base else np.zeros(0, np.uint8)
        for name, meta in header:
            if name == "__metadata__":
                continue
            meta = dict(meta)
            lo, hi = meta["data_offsets"]
            if not (0 <= lo <= hi <= size - base):
                raise PrequantizedError("invalidPayload", f"tensor '{name}': data_offsets outside the file")
            out.append(TensorInfo(name, meta["dtype"], [int(s) for s in meta["shape"]], mm[base + lo:base + hi]))
    return out


def packed_byte_count(logical_count: int, fmt: int) -> int:
    """SmeltSignedQuantCodec.packedByteCount (SmeltSignedQuantCodec.swift:83-100)."""
    return (logical_count * _BITS[fmt] + 7) // 8


@dataclass
class PrequantizedDescriptor:
    source_name: str
    format: int
    logical_shape: list
    group_size: int
    packed_row_stride: int
    padded_cols: int
    code_byte_count: int
    scale_count: int


@dataclass
class PrequantizedView:
    descriptor: PrequantizedDescriptor
    codes: np.ndarray             # uint8, code_byte_count
    mlx_scales: np.ndarray        # uint16 bit patterns, scale_count
    mlx_biases: np.ndarray
    canonical_scales: np.ndarray  # uint16, proven for every group when the view is made

    def canonical_scale_bits(self, group: int) -> int:
        if not 0 <= group < self.descriptor.scale_count:
            raise PrequantizedError("invalidGeometry",
                                    f"prequantized tensor '{self.descriptor.source_name}' has invalid geometry: "
                                    f"scale group {group} outside 0..<{self.descriptor.scale_count}")
        return int(self.canonical_scales[group])


class MlxTriplets:
    """The MLX spelling of one logical tensor is `<base>.weight` (U32 words of packed codes) with
    `<base>.scales` and `<base>.biases` (F16).  Everything else stays a dense checkpoint tensor."""

    norm_weight_semantics = "directWeight"   # MLX conversion stores direct multiplicative norm weights

    def __init__(self, tensors: list[TensorInfo], fmt: int, group_size: int, importer: im.Importer):
        if group_size <= 0:
            raise PrequantizedError("invalidGeometry", "prequantized tensor 'checkpoint' has invalid geometry: "
                                                       "group size must be positive")
        by_name = {}
        for t in tensors:
            if t.name in by_name:
                raise PrequantizedError("duplicateTensor", f"prequantized checkpoint contains duplicate tensor '{t.name}'")
            by_name[t.name] = t
        packed = [t for t in tensors if t.dtype == "U32" and t.name.endswith(".weight")]
        packed_names = {t.name for t in packed}
        for t in tensors:
            for suffix in (".scales", ".biases"):
                if t.name.endswith(suffix) and t.name[:-len(suffix)] + ".weight" not in packed_names:
                    raise PrequantizedError("orphanCompanion", f"prequantized companion '{t.name}' has no packed weight")

        self.prequantized: list[PrequantizedView] = []
        self.consumed_names: set[str] = set()
        for w in sorted(packed, key=lambda t: t.name):
            base = w.name[:-len(".weight")]
            companions = []
            for suffix in (".scales", ".biases"):
                c = by_name.get(base + suffix)
                if c is None:
                    raise PrequantizedError("missingCompanion",
                                            f"prequantized tensor '{w.name}' is missing companion '{base + suffix}'")
                companions.append(c)
            scales, biases = companions
            for c in companions:
                if c.dtype != "F16":
                    raise PrequantizedError("invalidDType", f"prequantized tensor '{c.name}' needs dtype F16, got {c.dtype}")

            def bad_geometry(detail, name=w.name):
                return PrequantizedError("invalidGeometry", f"prequantized tensor '{name}' has invalid geometry: {detail}")

            if not (len(w.shape) == 2 and len(scales.shape) == 2 and biases.shape == scales.shape
                    and w.shape[0] == scales.shape[0]):
                raise bad_geometry("expected weight [rows,packed_u32] and matching scales/biases [rows,groups]")
            rows, groups_per_row = w.shape[0], scales.shape[1]
            logical_cols = groups_per_row * group_size
            if rows <= 0 or groups_per_row <= 0 or logical_cols >= 1 << 63:
                raise bad_geometry("row/column count is empty or overflows")
            row_bytes = packed_byte_count(logical_cols, fmt)
            # U32 storage may only add whole words; bit padding inside a row is rejected
            if row_bytes % 4 != 0 or w.shape[1] != row_bytes // 4:
                raise bad_geometry(f"U32 row width {w.shape[1]} does not encode {logical_cols} "
                                   f"{FORMAT_NAMES[fmt]} values exactly")
            code_bytes, scale_count = rows * row_bytes, rows * groups_per_row
            if w.byte_count != code_bytes or scales.byte_count != scale_count * 2 or biases.byte_count != scale_count * 2:
                raise bad_geometry("payload byte counts do not match resolved geometry")

            codes = np.ascontiguousarray(w.data)
            mlx_scales = np.ascontiguousarray(scales.data).view(np.uint16)
            mlx_biases = np.ascontiguousarray(biases.data).view(np.uint16)
            try:
                importer.validate_signed_codes(codes, rows * logical_cols, fmt)
                # every group is proven to be a signed group before the bias plane is dropped
                canonical = importer.normalize_mlx_scales(fmt, mlx_scales, mlx_biases)
            except im.ImportError_ as e:
                raise PrequantizedError("invalidPayload", f"prequantized tensor '{w.name}' has invalid payload: {e}") from e
            desc = PrequantizedDescriptor(w.name, fmt, [rows, logical_cols], group_size, row_bytes, logical_cols,
                                          code_bytes, scale_count)
            self.prequantized.append(PrequantizedView(desc, codes, mlx_scales, mlx_biases, canonical))
            self.consumed_names.update((w.name, scales.name, biases.name))
        self.checkpoint_tensors = [t for t in tensors if t.name not in self.consumed_names]


# ---- SmeltNativeWeightWriter ------------------------------------------------------------------

def _element_count(shape, name: str) -> int:
    if not shape:
        raise NativeWriterError("shapeMismatch", f"tensor '{name}': expected shape [1], got []")
    n = 1
    for d in shape:
        if d <= 0:
            raise NativeWriterError("shapeMismatch", f"tensor '{name}': expected {[max(1, s) for s in shape]}, got {list(shape)}")
        n *= int(d)
    return n


_DENSE_SOURCES = {"fp16": ("F16", "BF16", "F32"), "bf16": ("BF16",), "fp32": ("F16", "BF16", "F32"), "int32": ("I32",)}
_DENSE_BYTES = {"fp16": 2, "bf16": 2, "fp32": 4, "int32": 4}


def _validate_packed(view: PrequantizedView, e: WeightRecord) -> None:
    expected = im.FORMAT_BINARY1 if e.dtype == "binary1" else im.FORMAT_TERNARY2
    d = view.descriptor
    if d.format != expected:
        raise NativeWriterError("signedFormatMismatch",
                                f"tensor '{e.name}': expected {FORMAT_NAMES[expected]}, got {FORMAT_NAMES[d.format]}")
    meta = [e.get(k) for k in ("group_size", "packed_row_stride", "padded_cols", "scales_offset", "scales_size_bytes")]
    if len(e.shape) != 2 or any(m is None for m in meta):
        raise NativeWriterError("invalidSignedEntry", f"tensor '{e.name}': missing rank-2/group/stride/scale metadata")
    group, stride, padded, scales_offset, scales_size = meta
    if d.logical_shape != [e.shape[0], padded]:
        raise NativeWriterError("shapeMismatch", f"tensor '{e.name}': expected {[e.shape[0], padded]}, got {d.logical_shape}")
    if (d.group_size, d.packed_row_stride, d.padded_cols, d.code_byte_count, d.scale_count * 2) != \
            (group, stride, padded, e.size_bytes, scales_size):
        raise NativeWriterError("invalidSignedEntry", f"tensor '{e.name}': source geometry does not match planned packed regions")
    if scales_offset < e.offset + e.size_bytes:
        raise NativeWriterError("invalidSignedEntry", f"tensor '{e.name}': scale region overlaps packed codes")


def _validate_dense(t: TensorInfo, e: WeightRecord) -> None:
    if list(t.shape) != list(e.shape):
        raise NativeWriterError("shapeMismatch", f"tensor '{e.name}': expected {list(e.shape)}, got {list(t.shape)}")
    n = _element_count(e.shape, e.name)
    if t.dtype not in ("F16", "BF16", "F32", "I32"):
        raise NativeWriterError("unsupportedSourceDtype", f"tensor '{e.name}': entry {e.dtype} cannot take source {t.dtype}")
    if t.byte_count != n * _ST_ITEMSIZE[t.dtype]:
        raise NativeWriterError("sourceByteMismatch",
                                f"tensor '{e.name}': expected {n * _ST_ITEMSIZE[t.dtype]} source bytes, got {t.byte_count}")
    if t.dtype not in _DENSE_SOURCES[e.dtype]:
        raise NativeWriterError("unsupportedSourceDtype", f"tensor '{e.name}': entry {e.dtype} cannot take source {t.dtype}")
    if e.size_bytes != n * _DENSE_BYTES[e.dtype]:
        raise NativeWriterError("invalidSignedEntry", f"tensor '{e.name}': dense byte count does not match shape/dtype")


def _dense_bytes(t: TensorInfo, e: WeightRecord) -> np.ndarray:
    """Element type conversion of a dense tensor; IEEE round-to-nearest-even narrowing, exact widening."""
    raw = np.ascontiguousarray(t.data)
    if e.dtype in ("bf16", "int32") or (e.dtype == "fp16" and t.dtype == "F16") or (e.dtype == "fp32" and t.dtype == "F32"):
        return raw
    if t.dtype == "BF16":
        f32 = (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
    elif t.dtype == "F16":
        f32 = raw.view(np.float16).astype(np.float32)
    else:
        f32 = raw.view(np.float32)
    if e.dtype == "fp32":
        return np.ascontiguousarray(f32).view(np.uint8)
    with np.errstate(over="ignore"):
        return f32.astype(np.float16).view(np.uint8)


def write_native(packed: list, dense: list, expected_layout: list[WeightRecord], output_path: str) -> list[WeightRecord]:
    """packed: [(runtime_name, PrequantizedView)], dense: [(runtime_name, TensorInfo)].  The whole
    plan is validated before the file is created; a failed write leaves no file behind."""
    def unique(pairs):
        out = {}
        for name, item in pairs:
            if name in out:
                raise NativeWriterError("duplicateSource", f"tensor '{name}' has more than one source")
            out[name] = item
        return out

    packed_by, dense_by = unique(packed), unique(dense)
    for name in packed_by:
        if name in dense_by:
            raise NativeWriterError("sourceKindCollision", f"tensor '{name}' is both a packed and a dense source")
    live = [e for e in expected_layout if e.size_bytes > 0]
    expected_names = {e.name for e in live}
    for name in list(packed_by) + list(dense_by):
        if name not in expected_names:
            raise NativeWriterError("unexpectedSource", f"tensor '{name}' is not in the planned layout")
    for e in live:
        if e.dtype in ("binary1", "ternary2"):
            if e.name not in packed_by:
                raise NativeWriterError("missingSource", f"tensor '{e.name}' has no source")
            _validate_packed(packed_by[e.name], e)
        elif e.dtype in _DENSE_SOURCES:
            if e.name not in dense_by:
                raise NativeWriterError("missingSource", f"tensor '{e.name}' has no source")
            _validate_dense(dense_by[e.name], e)
        else:
            raise NativeWriterError("unsupportedEntryDtype", f"tensor '{e.name}': dtype {e.dtype} is not written by this writer")
    total = total_bytes(expected_layout)
    if total <= 0:
        raise NativeWriterError("fileResizeFailed", output_path)

    done = False
    try:
        out = np.memmap(output_path, dtype=np.uint8, mode="w+", shape=(total,))
        for e in live:
            if e.dtype in ("binary1", "ternary2"):
                v = packed_by[e.name]
                out[e.offset:e.offset + e.size_bytes] = v.codes
                so = e.get("scales_offset")
                out[so:so + v.descriptor.scale_count * 2] = v.canonical_scales.view(np.uint8)
            else:
                b = _dense_bytes(dense_by[e.name], e)
                out[e.offset:e.offset + b.size] = b
        out.flush()
        del out
        done = True
    finally:
        if not done and os.path.exists(output_path):
            os.remove(output_path)
    return expected_layout
