"""Reader / writer of a Smelt package's weight table: `weights.bin` plus the `weights` object of
manifest.json (SmeltWeightManifest / SmeltWeightEntry, Sources/SmeltSchema/SmeltManifest.swift:
1597-1725) and the older name-keyed weights.json (SmeltWeightManifestLoader.load,
Sources/SmeltCompiler/SmeltWeightManifestLoader.swift:17-133).

The byte layout of every tensor is the reference's, so an existing package's weights.bin is
uploaded unchanged (`PackageWeights.upload`); `PackageBuilder` goes the other way and lays out,
quantises on the GPU and writes a package this backend and the reference both read."""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field

import numpy as np

from . import compiler as cc

# SmeltDType raw values (SmeltManifest.swift:1614-1630); trit5 exists only in this backend
DTYPE_NAMES = {"fp16": cc.FP16, "fp32": cc.FP32, "bf16": cc.BF16, "int32": cc.INT32, "u4_lut": cc.U4_LUT,
               "affine_u4": cc.AFFINE_U4, "binary1": cc.BINARY1, "ternary2": cc.TERNARY2,
               "turbo_quant_h": cc.TURBO_QUANT_H, "raw": cc.RAW, "trit5": cc.TRIT5}
DTYPE_OF = {v: k for k, v in DTYPE_NAMES.items()}
BYTES_PER_ELEMENT = {cc.FP16: 2, cc.BF16: 2, cc.FP32: 4, cc.INT32: 4}

# optional SmeltWeightEntry fields in CodingKeys order: (snake_case key, camelCase key)
_OPTIONAL = [("group_size", "groupSize"), ("lut_offset", "lutOffset"), ("lut_size_bytes", "lutSizeBytes"),
             ("packed_row_stride", "packedRowStride"), ("padded_cols", "paddedCols"),
             ("scales_offset", "scalesOffset"), ("scales_size_bytes", "scalesSizeBytes"),
             ("biases_offset", "biasesOffset"), ("biases_size_bytes", "biasesSizeBytes"),
             ("codebook_offset", "codebookOffset"), ("codebook_size_bytes", "codebookSizeBytes")]


class PackageError(ValueError):
    pass


@dataclass
class WeightRecord:
    """One SmeltWeightEntry: required fields plus whichever optional ones the manifest carries."""
    name: str
    offset: int
    size_bytes: int
    shape: list
    dtype: str
    optional: dict = field(default_factory=dict)

    def get(self, key: str):
        return self.optional.get(key)

    @property
    def rows(self) -> int:
        return int(self.shape[0]) if self.shape else 0

    @property
    def cols(self) -> int:
        return int(self.shape[1]) if len(self.shape) > 1 else 1

    def regions(self):
        """(what, offset, size) of every byte range the entry owns."""
        out = [("data", self.offset, self.size_bytes)]
        for what in ("lut", "scales", "biases", "codebook"):
            off, size = self.get(f"{what}_offset"), self.get(f"{what}_size_bytes")
            if off is not None and size is not None:
                out.append((what, off, size))
        return out

    def to_json(self) -> dict:
        d = {"name": self.name, "offset": self.offset, "size_bytes": self.size_bytes,
             "shape": list(self.shape), "dtype": self.dtype}
        for snake, _ in _OPTIONAL:     # absent optionals are omitted, as Codable's encodeIfPresent does
            if self.optional.get(snake) is not None:
                d[snake] = self.optional[snake]
        return d

    def to_entry(self) -> cc.WeightEntry:
        """The C-ABI view the record emitters take; validates what the kernels rely on."""
        if self.dtype not in DTYPE_NAMES:
            raise PackageError(f"tensor '{self.name}': unknown dtype '{self.dtype}'")
        e = cc.WeightEntry()
        e.offset, e.size_bytes = self.offset, self.size_bytes
        e.rows, e.cols = self.rows, self.cols
        e.dtype = DTYPE_NAMES[self.dtype]
        e.group_size = self.get("group_size") or 0
        e.packed_row_stride = self.get("packed_row_stride") or 0
        e.padded_cols = self.get("padded_cols") or 0
        e.scales_offset = self.get("scales_offset") or 0
        e.scales_size_bytes = self.get("scales_size_bytes") or 0
        e.biases_offset = self.get("biases_offset") or 0
        e.biases_size_bytes = self.get("biases_size_bytes") or 0
        if e.dtype in (cc.AFFINE_U4, cc.BINARY1, cc.TERNARY2, cc.TRIT5):
            if len(self.shape) != 2 or e.rows <= 0 or e.cols <= 0:
                raise PackageError(f"tensor '{self.name}': packed formats are 2-D")
            if e.group_size <= 0 or e.packed_row_stride <= 0 or not e.scales_size_bytes:
                raise PackageError(f"tensor '{self.name}': {self.dtype} needs group_size, packed_row_stride and scales")
            padded = e.padded_cols or e.cols
            groups = (padded + e.group_size - 1) // e.group_size
            if e.size_bytes != e.rows * e.packed_row_stride:
                raise PackageError(f"tensor '{self.name}': size_bytes {e.size_bytes} is not rows x packed_row_stride")
            if e.scales_size_bytes != e.rows * groups * 2:
                raise PackageError(f"tensor '{self.name}': scales region holds {e.scales_size_bytes} bytes, "
                                   f"{e.rows} x {groups} groups need {e.rows * groups * 2}")
            if e.dtype == cc.AFFINE_U4 and e.biases_size_bytes != e.scales_size_bytes:
                raise PackageError(f"tensor '{self.name}': affine_u4 needs a bias per scale")
        elif e.dtype in BYTES_PER_ELEMENT:
            n = int(np.prod(self.shape)) if self.shape else 0
            if e.size_bytes != n * BYTES_PER_ELEMENT[e.dtype]:
                raise PackageError(f"tensor '{self.name}': size_bytes does not match shape x element size")
        return e


def record_from_entry(name: str, e: cc.WeightEntry) -> WeightRecord:
    opt = {}
    if e.dtype in (cc.AFFINE_U4, cc.BINARY1, cc.TERNARY2, cc.TRIT5):
        opt = {"group_size": e.group_size, "packed_row_stride": e.packed_row_stride, "padded_cols": e.padded_cols,
               "scales_offset": e.scales_offset, "scales_size_bytes": e.scales_size_bytes}
        if e.dtype == cc.AFFINE_U4:
            opt.update({"biases_offset": e.biases_offset, "biases_size_bytes": e.biases_size_bytes})
    return WeightRecord(name, int(e.offset), int(e.size_bytes), [int(e.rows), int(e.cols)], DTYPE_OF[e.dtype], opt)


def _int(meta: dict, snake: str, camel: str):
    for k in (camel, snake):       # the loader looks the camelCase spelling up first
        v = meta.get(k)
        if isinstance(v, bool):
            continue
        if isinstance(v, (int, float)) and float(v).is_integer():
            return int(v)
    return None


def parse_weight_manifest(obj: dict) -> tuple[int, list[WeightRecord]]:
    """manifest.json (its "weights" object or that object itself) -> (total_bytes, entries in file order)."""
    w = obj.get("weights", obj)
    if not isinstance(w, dict) or "entries" not in w or "total_bytes" not in w:
        raise PackageError("no weights.total_bytes / weights.entries in the manifest")
    out = []
    for m in w["entries"]:
        for key in ("name", "offset", "size_bytes", "shape", "dtype"):
            if key not in m:
                raise PackageError(f"weight entry lacks '{key}'")
        if m["dtype"] not in DTYPE_NAMES:
            raise PackageError(f"tensor '{m['name']}': unknown dtype '{m['dtype']}'")
        opt = {snake: int(m[snake]) for snake, _ in _OPTIONAL if m.get(snake) is not None}
        out.append(WeightRecord(m["name"], int(m["offset"]), int(m["size_bytes"]), [int(s) for s in m["shape"]],
                                m["dtype"], opt))
    total = int(w["total_bytes"])
    check_regions(out, total)
    return total, out


def parse_legacy_weights_json(obj: dict) -> list[WeightRecord]:
    """Name-keyed weights.json of the Python quantiser (SmeltWeightManifestLoader.swift:17-133):
    camelCase or snake_case keys, dtype defaulting to u4_lut for `quantized: true` and fp16
    otherwise, packed_row_stride / padded_cols derived from shape[1] when absent, sorted by offset."""
    out = []
    for name, meta in obj.items():
        if not isinstance(meta, dict):
            continue
        shape = [int(s) for s in meta.get("shape", [])] if isinstance(meta.get("shape"), list) else []
        quantized = meta.get("quantized") is True
        dtype = meta.get("dtype") if meta.get("dtype") in DTYPE_NAMES and meta.get("dtype") != "trit5" else None
        if dtype is None:
            dtype = "u4_lut" if quantized else "fp16"
        opt = {}
        for snake, camel in _OPTIONAL:
            v = _int(meta, snake, camel)
            if v is not None:
                opt[snake] = v
        explicit = "packed_row_stride" in opt and "padded_cols" in opt
        packed_kind = quantized or dtype in ("u4_lut", "affine_u4", "binary1", "ternary2", "turbo_quant_h")
        if not explicit:
            opt.pop("packed_row_stride", None)
            opt.pop("padded_cols", None)
            if packed_kind and len(shape) >= 2:
                opt["padded_cols"] = shape[1]
                opt["packed_row_stride"] = {"affine_u4": (shape[1] + 1) // 2, "binary1": (shape[1] + 7) // 8,
                                            "ternary2": (shape[1] + 3) // 4}.get(dtype, shape[1] // 2)
        out.append(WeightRecord(name, _int(meta, "offset", "offset") or 0, _int(meta, "size_bytes", "sizeBytes") or 0,
                                shape, dtype, opt))
    out.sort(key=lambda r: r.offset)
    return out


def total_bytes(entries: list[WeightRecord]) -> int:
    """File size the entries imply: the furthest end of any data / lut / scales / biases / codebook
    region (SmeltWeightManifestLoader.totalBytes, :136-155)."""
    return max((off + size for r in entries for _, off, size in r.regions()), default=0)


def check_regions(entries: list[WeightRecord], total: int) -> None:
    spans = []
    for r in entries:
        for what, off, size in r.regions():
            if off < 0 or size < 0 or off + size > total:
                raise PackageError(f"tensor '{r.name}': {what} region [{off}, {off + size}) is outside the {total}-byte file")
            if size:
                spans.append((off, off + size, r.name, what))
    spans.sort()
    for (s0, e0, n0, w0), (s1, e1, n1, w1) in zip(spans, spans[1:]):
        if s1 < e0 and (n0, w0) != (n1, w1):
            raise PackageError(f"'{n0}' {w0} and '{n1}' {w1} overlap in weights.bin")


def weight_manifest_json(entries: list[WeightRecord], total: int) -> dict:
    return {"total_bytes": int(total), "entries": [r.to_json() for r in entries]}


class PackageWeights:
    """weights.bin of a package directory, memory-mapped, with its entry table."""

    def __init__(self, directory: str):
        self.directory = directory
        mpath = os.path.join(directory, "manifest.json")
        lpath = os.path.join(directory, "weights.json")
        if os.path.exists(mpath):
            self.total, self.entries = parse_weight_manifest(json.load(open(mpath)))
        elif os.path.exists(lpath):
            self.entries = parse_legacy_weights_json(json.load(open(lpath)))
            self.total = total_bytes(self.entries)
            check_regions(self.entries, self.total)
        else:
            raise PackageError(f"{directory}: neither manifest.json nor weights.json")
        path = os.path.join(directory, "weights.bin")   # the file name is fixed (SmeltPackageSpec.swift:83)
        size = os.path.getsize(path)
        if size < self.total:
            raise PackageError(f"{path} holds {size} bytes, the manifest describes {self.total}")
        self.image = np.memmap(path, dtype=np.uint8, mode="r")
        self.by_name = {r.name: r for r in self.entries}

    def entry(self, name: str) -> cc.WeightEntry:
        return self.by_name[name].to_entry()

    def region(self, name: str, what: str = "data") -> np.ndarray:
        for w, off, size in self.by_name[name].regions():
            if w == what:
                return self.image[off:off + size]
        raise KeyError(what)

    def upload(self, ctx, slot: int) -> None:
        """One device allocation for the whole file; logical offsets are device offsets."""
        ctx.upload_weights(slot, self.image[:self.total])


class PackageBuilder:
    """Lays tensors out as SmeltWeightLayout does, fills weights.bin and writes the weight table."""

    def __init__(self):
        self.layout = cc.Layout()
        self.records: list[WeightRecord] = []
        self._pending = []   # (entry, arrays) written when the image is materialised

    def add_affine_u4(self, name: str, importer, src: np.ndarray, src_dtype: int, rows: int, cols: int,
                      group: int = 64, clip: int = 0, importance=None, scale_dtype: int = 0) -> cc.WeightEntry:
        """Quantises on the GPU (bit-identical to SmeltAffineQuantizer) and records the entry."""
        e = self.layout.affine(rows, cols, group)
        packed, scales, biases = importer.quantize_affine_u4(src, src_dtype, rows, cols, group, clip, importance, scale_dtype)
        self._pending.append((e, (packed, scales, biases)))
        self.records.append(record_from_entry(name, e))
        return e

    def add_signed(self, name: str, importer, codes: np.ndarray, mlx_scales: np.ndarray, mlx_biases: np.ndarray,
                   rows: int, cols: int, dtype: int, group: int = 128) -> cc.WeightEntry:
        """An MLX-packed signed tensor: codes are validated and copied, (scale, bias) pairs become
        canonical signed scales (SmeltPrequantizedTensor.swift:147-300)."""
        from . import importer as im
        fmt = {cc.BINARY1: im.FORMAT_BINARY1, cc.TERNARY2: im.FORMAT_TERNARY2}[dtype]
        e = self.layout.signed(rows, cols, dtype, group)
        codes = np.ascontiguousarray(codes).view(np.uint8).reshape(rows, -1)
        if codes.shape[1] != e.packed_row_stride:
            raise PackageError(f"tensor '{name}': {codes.shape[1]} code bytes per row, layout needs {e.packed_row_stride}")
        importer.validate_signed_codes(codes, rows * cols, fmt)
        scales = importer.normalize_mlx_scales(fmt, mlx_scales, mlx_biases)
        self._pending.append((e, (codes, scales)))
        self.records.append(record_from_entry(name, e))
        return e

    def add_dense(self, name: str, array: np.ndarray, dtype: int) -> cc.WeightEntry:
        rows = array.shape[0]
        cols = int(np.prod(array.shape[1:])) if array.ndim > 1 else 1
        e = self.layout.dense(rows, cols, dtype)
        self._pending.append((e, (array,)))
        rec = record_from_entry(name, e)
        rec.shape = [int(s) for s in array.shape]
        self.records.append(rec)
        return e

    def image(self) -> np.ndarray:
        img = np.zeros(self.layout.total_bytes, np.uint8)
        for e, arrays in self._pending:
            if len(arrays) == 3:
                cc.write_affine(img, e, *arrays)
            elif len(arrays) == 2:
                cc.write_signed(img, e, *arrays)
            else:
                a = np.ascontiguousarray(arrays[0]).view(np.uint8).ravel()
                img[e.offset:e.offset + a.size] = a
        return img

    def write(self, directory: str, extra_manifest: dict | None = None) -> None:
        os.makedirs(directory, exist_ok=True)
        self.image().tofile(os.path.join(directory, "weights.bin"))
        manifest = dict(extra_manifest or {})
        manifest["weights"] = weight_manifest_json(self.records, self.layout.total_bytes)
        with open(os.path.join(directory, "manifest.json"), "w") as f:
            json.dump(manifest, f, indent=1)
