"""Weight-table reader / writer against the schema of SmeltManifest.swift:1597-1725 and the legacy
loader rules of SmeltWeightManifestLoader.swift:17-155 (no GPU needed)."""
import json

import numpy as np
import pytest

from smelt_amd import compiler as cc
from smelt_amd import package as pk


def sample_layout():
    lay = cc.Layout()
    a = lay.affine(48, 200, 64)
    b = lay.signed(16, 256, cc.BINARY1)
    t = lay.signed(16, 300, cc.TERNARY2)
    d = lay.dense(8, 32, cc.FP16)
    recs = [pk.record_from_entry(n, e) for n, e in (("l0.q", a), ("l0.bin", b), ("l0.ter", t), ("norm", d))]
    return lay, recs


def test_manifest_round_trip_keeps_every_field_and_omits_absent_ones():
    lay, recs = sample_layout()
    doc = {"weights": pk.weight_manifest_json(recs, lay.total_bytes)}
    text = json.dumps(doc)
    total, back = pk.parse_weight_manifest(json.loads(text))
    assert total == lay.total_bytes and [r.to_json() for r in back] == [r.to_json() for r in recs]
    aff = doc["weights"]["entries"][0]
    # SmeltWeightEntry.CodingKeys spellings; affine_u4 carries scales and biases, no lut / codebook
    assert set(aff) == {"name", "offset", "size_bytes", "shape", "dtype", "group_size", "packed_row_stride",
                        "padded_cols", "scales_offset", "scales_size_bytes", "biases_offset", "biases_size_bytes"}
    assert aff["dtype"] == "affine_u4" and aff["packed_row_stride"] == 100 and aff["shape"] == [48, 200]
    assert "biases_offset" not in doc["weights"]["entries"][1]          # signed formats have no bias plane
    assert set(doc["weights"]["entries"][3]) == {"name", "offset", "size_bytes", "shape", "dtype"}
    for r, src in zip(back, lay.entries):
        e = r.to_entry()
        for f, _ in cc.WeightEntry._fields_:
            assert getattr(e, f) == getattr(src, f), (r.name, f)


def test_total_bytes_counts_trailing_scale_and_bias_regions():
    lay, recs = sample_layout()
    assert pk.total_bytes(recs[:1]) == recs[0].get("biases_offset") + recs[0].get("biases_size_bytes")
    assert pk.total_bytes(recs) == lay.total_bytes
    lut = pk.WeightRecord("w", 0, 64, [8, 16], "u4_lut", {"lut_offset": 4096, "lut_size_bytes": 512})
    assert pk.total_bytes([lut]) == 4608


def test_regions_outside_the_file_or_overlapping_are_rejected():
    lay, recs = sample_layout()
    with pytest.raises(pk.PackageError):
        pk.parse_weight_manifest({"weights": pk.weight_manifest_json(recs, lay.total_bytes - 1)})
    clash = pk.WeightRecord("dup", recs[0].offset + 4, 16, [8], "fp16")
    with pytest.raises(pk.PackageError):
        pk.check_regions(recs + [clash], lay.total_bytes)
    bad = pk.WeightRecord("q", 0, 10, [4, 64], "affine_u4",
                          {"group_size": 64, "packed_row_stride": 32, "padded_cols": 64, "scales_offset": 128,
                           "scales_size_bytes": 8, "biases_offset": 256, "biases_size_bytes": 8})
    with pytest.raises(pk.PackageError):
        bad.to_entry()                                  # size_bytes != rows x stride
    with pytest.raises(pk.PackageError):
        pk.parse_weight_manifest({"weights": {"total_bytes": 64, "entries": [
            {"name": "x", "offset": 0, "size_bytes": 8, "shape": [4], "dtype": "fp8"}]}})


def test_legacy_weights_json_rules():
    legacy = {
        "b.weight": {"offset": 4096, "sizeBytes": 1024, "shape": [32, 64], "quantized": True,
                     "lutOffset": 8192, "lutSizeBytes": 512, "groupSize": 32},
        "a.weight": {"offset": 0, "size_bytes": 3200, "shape": [32, 200], "dtype": "affine_u4", "group_size": 64,
                     "scales_offset": 3200, "scales_size_bytes": 256, "biases_offset": 3456, "biases_size_bytes": 256},
        "n.weight": {"offset": 16384, "size_bytes": 128, "shape": [64]},
        "t.weight": {"offset": 20000, "size_bytes": 32 * 75, "shape": [32, 300], "dtype": "ternary2"},
        "c.weight": {"offset": 30000, "size_bytes": 32 * 38, "shape": [32, 300], "dtype": "binary1"},
        "s.weight": {"offset": 40000, "size_bytes": 10, "shape": [4, 20], "dtype": "affine_u4",
                     "packedRowStride": 16, "paddedCols": 32},
        "comment": "not a tensor",
    }
    recs = pk.parse_legacy_weights_json(legacy)
    assert [r.name for r in recs] == ["a.weight", "b.weight", "n.weight", "t.weight", "c.weight", "s.weight"]
    a, b, n, t, c, s = recs
    assert (a.dtype, a.get("packed_row_stride"), a.get("padded_cols")) == ("affine_u4", 100, 200)
    assert (b.dtype, b.get("packed_row_stride"), b.get("lut_offset"), b.get("group_size")) == ("u4_lut", 32, 8192, 32)
    assert (n.dtype, n.get("packed_row_stride"), n.size_bytes) == ("fp16", None, 128)
    assert t.get("packed_row_stride") == 75 and c.get("packed_row_stride") == 38
    assert (s.get("packed_row_stride"), s.get("padded_cols")) == (16, 32)   # explicit pair wins
    assert pk.total_bytes(recs) == 40010


def test_package_directory_round_trip(tmp_path):
    """A written package reads back byte for byte (dense tensors only: no GPU in this test)."""
    b = pk.PackageBuilder()
    rng = np.random.default_rng(0)
    norm = rng.normal(0, 1, 64).astype(np.float16)
    table = rng.normal(0, 1, (8, 16)).astype(np.float32)
    b.add_dense("norm.weight", norm, cc.FP16)
    b.add_dense("table", table, cc.FP32)
    b.write(str(tmp_path), {"format_version": 1})
    pw = pk.PackageWeights(str(tmp_path))
    assert [r.name for r in pw.entries] == ["norm.weight", "table"]
    assert np.array_equal(pw.region("norm.weight").view(np.float16), norm)
    assert np.array_equal(pw.region("table").view(np.float32).reshape(8, 16), table)
    assert pw.by_name["table"].shape == [8, 16] and pw.entry("table").dtype == cc.FP32
    with open(tmp_path / "weights.bin", "r+b") as f:
        f.truncate(pw.total - 1)
    with pytest.raises(pk.PackageError):
        pk.PackageWeights(str(tmp_path))
