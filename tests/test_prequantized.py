"""MLX safetensors triplet adapter and the native weights.bin writer.

Cases follow Tests/SmeltCompilerTests/SmeltPrequantizedTensorTests.swift: the same synthetic
safetensors files (`writeSyntheticSafetensors`, :14-39), the same expected descriptors, bytes and
errors.  Discovery errors are raised before any payload is touched and run without a GPU; the
cases that validate codes and scales go through the GPU importer.
"""
import json
import os
import struct

import numpy as np
import pytest

import oracle.oracle as orc
from smelt_amd import importer as im
from smelt_amd import prequantized as pq
from smelt_amd.package import WeightRecord


def f16(values):
    return np.asarray(values, np.float16).tobytes()


def write_synthetic(path, tensors):
    """[(name, dtype, shape, bytes)] -> a safetensors file with an MLX metadata block."""
    header, payload, offset = {"__metadata__": {"format": "mlx"}}, b"", 0
    for name, dtype, shape, data in tensors:
        header[name] = {"dtype": dtype, "shape": shape, "data_offsets": [offset, offset + len(data)]}
        payload += data
        offset += len(data)
    h = json.dumps(header, sort_keys=True).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + payload)
    return path


BINARY_TRIPLET = [
    ("model.proj.weight", "U32", [2, 1], bytes([0x55] * 4 + [0xAA] * 4)),
    ("model.proj.scales", "F16", [2, 1], f16([0.5, 0.25])),
    ("model.proj.biases", "F16", [2, 1], f16([-0.25, -0.125])),
    ("model.norm.weight", "F16", [2], f16([1, 1])),
]


def test_safetensors_reader(tmp_path):
    p = write_synthetic(tmp_path / "a.safetensors", BINARY_TRIPLET)
    ts = pq.read_safetensors(str(p))
    assert sorted(t.name for t in ts) == sorted(t[0] for t in BINARY_TRIPLET)
    by = {t.name: t for t in ts}
    assert by["model.proj.weight"].dtype == "U32" and by["model.proj.weight"].shape == [2, 1]
    assert bytes(by["model.proj.weight"].data) == BINARY_TRIPLET[0][3]
    assert bytes(by["model.norm.weight"].data) == f16([1, 1])
    # two files concatenate in order
    p2 = write_synthetic(tmp_path / "b.safetensors", [("x", "F32", [1], np.float32([2.5]).tobytes())])
    assert [t.name for t in pq.read_safetensors([str(p), str(p2)])][-1] == "x"


def test_reader_rejects_offsets_outside_the_file(tmp_path):
    h = json.dumps({"w": {"dtype": "F16", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p = tmp_path / "bad.safetensors"
    p.write_bytes(struct.pack("<Q", len(h)) + h + b"\0\0")
    with pytest.raises(pq.PrequantizedError) as e:
        pq.read_safetensors(str(p))
    assert e.value.kind == "invalidPayload"


def test_missing_and_orphan_companions(tmp_path):
    """SmeltPrequantizedTensorTests.swift:129-156."""
    missing = pq.read_safetensors(str(write_synthetic(tmp_path / "m.safetensors", [
        ("proj.weight", "U32", [1, 1], bytes(4)), ("proj.scales", "F16", [1, 1], f16([0.5]))])))
    with pytest.raises(pq.PrequantizedError) as e:
        pq.MlxTriplets(missing, im.FORMAT_BINARY1, 32, importer=None)
    assert e.value.kind == "missingCompanion" and "proj.biases" in str(e.value)
    orphan = pq.read_safetensors(str(write_synthetic(tmp_path / "o.safetensors", [
        ("orphan.scales", "F16", [1, 1], f16([0.5]))])))
    with pytest.raises(pq.PrequantizedError) as e:
        pq.MlxTriplets(orphan, im.FORMAT_BINARY1, 32, importer=None)
    assert e.value.kind == "orphanCompanion"


def test_discovery_errors_before_any_payload_is_read():
    def t(name, dtype, shape, n):
        return pq.TensorInfo(name, dtype, shape, np.zeros(n, np.uint8))
    ok = [t("p.weight", "U32", [2, 1], 8), t("p.scales", "F16", [2, 1], 4), t("p.biases", "F16", [2, 1], 4)]
    with pytest.raises(pq.PrequantizedError) as e:
        pq.MlxTriplets(ok, im.FORMAT_BINARY1, 0, importer=None)
    assert e.value.kind == "invalidGeometry"
    with pytest.raises(pq.PrequantizedError) as e:
        pq.MlxTriplets(ok + [ok[0]], im.FORMAT_BINARY1, 32, importer=None)
    assert e.value.kind == "duplicateTensor"
    bad_dtype = [ok[0], t("p.scales", "F32", [2, 1], 8), ok[2]]
    with pytest.raises(pq.PrequantizedError) as e:
        pq.MlxTriplets(bad_dtype, im.FORMAT_BINARY1, 32, importer=None)
    assert e.value.kind == "invalidDType"
    # scales of another row count, a U32 width that does not encode the columns exactly, short payloads
    for bad in ([ok[0], t("p.scales", "F16", [3, 1], 6), t("p.biases", "F16", [3, 1], 6)],
                [t("p.weight", "U32", [2, 2], 16), ok[1], ok[2]],
                [t("p.weight", "U32", [2, 1], 4), ok[1], ok[2]],
                [ok[0], ok[1], t("p.biases", "F16", [2, 1], 2)]):
        with pytest.raises(pq.PrequantizedError) as e:
            pq.MlxTriplets(bad, im.FORMAT_BINARY1, 32, importer=None)
        assert e.value.kind == "invalidGeometry"
    # ternary group of 16 = one word; a binary group of 16 would be half a word: bit padding is rejected
    with pytest.raises(pq.PrequantizedError) as e:
        pq.MlxTriplets(ok, im.FORMAT_BINARY1, 16, importer=None)
    assert e.value.kind == "invalidGeometry" and "exactly" in str(e.value)
    # a U32 tensor that is not a `.weight`, and dense tensors, are left alone
    src = pq.MlxTriplets([t("ids", "U32", [4], 16), t("norm.weight", "F16", [2], 4)], im.FORMAT_BINARY1, 32, importer=None)
    assert src.prequantized == [] and [x.name for x in src.checkpoint_tensors] == ["ids", "norm.weight"]


def test_native_writer_plan_errors(tmp_path):
    d = pq.PrequantizedDescriptor("p.weight", im.FORMAT_BINARY1, [1, 32], 32, 4, 32, 4, 1)
    view = pq.PrequantizedView(d, np.full(4, 0x55, np.uint8), np.zeros(1, np.uint16), np.zeros(1, np.uint16),
                               np.array([0x3400], np.uint16))
    signed = WeightRecord("proj", 128, 4, [1, 32], "binary1", {"group_size": 32, "packed_row_stride": 4, "padded_cols": 32,
                                                                "scales_offset": 256, "scales_size_bytes": 2})
    norm = WeightRecord("norm", 0, 4, [2], "fp16")
    dense = pq.TensorInfo("n", "F32", [2], np.float32([1.5, -2.0]).view(np.uint8))
    out = str(tmp_path / "w.bin")

    def expect(kind, packed, dense_list, layout):
        with pytest.raises(pq.NativeWriterError) as e:
            pq.write_native(packed, dense_list, layout, out)
        assert e.value.kind == kind
        assert not os.path.exists(out)

    expect("duplicateSource", [("proj", view), ("proj", view)], [], [signed])
    expect("sourceKindCollision", [("proj", view)], [("proj", dense)], [signed])
    expect("unexpectedSource", [("other", view)], [], [signed])
    expect("missingSource", [], [("norm", dense)], [norm, signed])
    expect("missingSource", [("proj", view)], [], [norm, signed])
    expect("signedFormatMismatch", [("proj", view)], [],
           [WeightRecord("proj", 128, 4, [1, 32], "ternary2", dict(signed.optional))])
    expect("invalidSignedEntry", [("proj", view)], [], [WeightRecord("proj", 128, 4, [1, 32], "binary1", {"group_size": 32})])
    expect("shapeMismatch", [("proj", view)], [],
           [WeightRecord("proj", 128, 4, [2, 32], "binary1", dict(signed.optional))])
    expect("invalidSignedEntry", [("proj", view)], [],
           [WeightRecord("proj", 128, 4, [1, 32], "binary1", {**signed.optional, "scales_offset": 130})])
    expect("shapeMismatch", [], [("norm", dense)], [WeightRecord("norm", 0, 6, [3], "fp16")])
    expect("unsupportedSourceDtype", [], [("norm", dense)], [WeightRecord("norm", 0, 4, [2], "bf16")])
    expect("unsupportedSourceDtype", [], [("norm", pq.TensorInfo("n", "U8", [2], np.zeros(2, np.uint8)))], [norm])
    expect("sourceByteMismatch", [], [("norm", pq.TensorInfo("n", "F32", [2], np.zeros(4, np.uint8)))], [norm])
    expect("unsupportedEntryDtype", [], [], [WeightRecord("q", 0, 16, [1, 32], "affine_u4")])


def test_native_writer_dense_conversions(tmp_path):
    """SmeltNativeWeightWriter.swift:318-371: F32/BF16 -> fp16 by IEEE narrowing, F16/BF16 -> fp32 exact,
    bf16 and int32 copied."""
    vals = np.float32([1.5, -2.0, 65504.0, 1e-8, 0.1])
    bf = (vals.view(np.uint32) >> 16).astype(np.uint16)
    layout = [WeightRecord("a", 0, 10, [5], "fp16"), WeightRecord("b", 16, 10, [5], "fp16"),
              WeightRecord("c", 32, 20, [5], "fp32"), WeightRecord("d", 64, 20, [5], "fp32"),
              WeightRecord("e", 96, 10, [5], "bf16"), WeightRecord("f", 112, 8, [2], "int32")]
    dense = [("a", pq.TensorInfo("a", "F32", [5], vals.view(np.uint8))),
             ("b", pq.TensorInfo("b", "BF16", [5], bf.view(np.uint8))),
             ("c", pq.TensorInfo("c", "BF16", [5], bf.view(np.uint8))),
             ("d", pq.TensorInfo("d", "F16", [5], vals.astype(np.float16).view(np.uint8))),
             ("e", pq.TensorInfo("e", "BF16", [5], bf.view(np.uint8))),
             ("f", pq.TensorInfo("f", "I32", [2], np.int32([-7, 9]).view(np.uint8)))]
    out = str(tmp_path / "dense.bin")
    pq.write_native([], dense, layout, out)
    img = np.fromfile(out, np.uint8)
    assert img.size == 120
    bf_f32 = (bf.astype(np.uint32) << 16).view(np.float32)
    assert (img[0:10].view(np.uint16) == orc.f32_to_f16_bits(vals)).all()
    assert (img[16:26].view(np.uint16) == orc.f32_to_f16_bits(bf_f32)).all()
    assert (img[32:52].view(np.float32) == bf_f32).all()
    assert (img[64:84].view(np.float32) == vals.astype(np.float16).astype(np.float32)).all()
    assert (img[96:106].view(np.uint16) == bf).all()
    assert (img[112:120].view(np.int32) == [-7, 9]).all()


# ---- through the GPU importer -----------------------------------------------------------------

@pytest.fixture(scope="module")
def importer():
    with im.Importer() as imp:
        yield imp


@pytest.mark.gpu
def test_mlx_triplets_become_one_binary_tensor(tmp_path, importer):
    """SmeltPrequantizedTensorTests.swift:51-88."""
    ts = pq.read_safetensors(str(write_synthetic(tmp_path / "b.safetensors", BINARY_TRIPLET)))
    src = pq.MlxTriplets(ts, im.FORMAT_BINARY1, 32, importer)
    assert len(src.prequantized) == 1
    v = src.prequantized[0]
    d = v.descriptor
    assert d.source_name == "model.proj.weight" and d.logical_shape == [2, 32]
    assert d.packed_row_stride == 4 and d.scale_count == 2 and d.code_byte_count == 8
    assert v.canonical_scale_bits(0) == 0x3400          # fp16 0.25 = 0.5 * 0.5
    assert v.canonical_scale_bits(1) == 0x3000          # 0.125
    with pytest.raises(pq.PrequantizedError):
        v.canonical_scale_bits(2)
    assert [t.name for t in src.checkpoint_tensors] == ["model.norm.weight"]
    assert src.consumed_names == {"model.proj.weight", "model.proj.scales", "model.proj.biases"}
    assert src.norm_weight_semantics == "directWeight"


@pytest.mark.gpu
def test_mlx_triplets_validate_ternary_codes_and_affine_relationship(tmp_path, importer):
    """SmeltPrequantizedTensorTests.swift:90-127."""
    def source(first_byte, bias):
        return pq.read_safetensors(str(write_synthetic(tmp_path / f"t{first_byte}_{bias}.safetensors", [
            ("proj.weight", "U32", [1, 1], bytes([first_byte, 0x55, 0x55, 0x55])),
            ("proj.scales", "F16", [1, 1], f16([0.25])), ("proj.biases", "F16", [1, 1], f16([bias]))])))
    ok = pq.MlxTriplets(source(0b10_01_00_10, -0.25), im.FORMAT_TERNARY2, 16, importer)
    assert ok.prequantized[0].descriptor.logical_shape == [1, 16]
    assert ok.prequantized[0].canonical_scale_bits(0) == 0x3400
    for first_byte, bias in ((0b11, -0.25), (0x55, -0.5)):
        with pytest.raises(pq.PrequantizedError) as e:
            pq.MlxTriplets(source(first_byte, bias), im.FORMAT_TERNARY2, 16, importer)
        assert e.value.kind == "invalidPayload"


@pytest.mark.gpu
def test_native_writer_streams_signed_and_dense_regions(tmp_path, importer):
    """SmeltPrequantizedTensorTests.swift:158-235: 258-byte file, fp16 norm at 0, codes at 128,
    canonical scale at 256, dequantised row +-0.25."""
    ts = pq.read_safetensors(str(write_synthetic(tmp_path / "s.safetensors", [
        ("model.proj.weight", "U32", [1, 1], bytes([0x55] * 4)),
        ("model.proj.scales", "F16", [1, 1], f16([0.5])), ("model.proj.biases", "F16", [1, 1], f16([-0.25])),
        ("model.norm.weight", "F32", [2], np.float32([1.5, -2.0]).tobytes())])))
    src = pq.MlxTriplets(ts, im.FORMAT_BINARY1, 32, importer)
    layout = [WeightRecord("norm_weight", 0, 4, [2], "fp16"),
              WeightRecord("proj_weight", 128, 4, [1, 32], "binary1",
                           {"group_size": 32, "packed_row_stride": 4, "padded_cols": 32,
                            "scales_offset": 256, "scales_size_bytes": 2})]
    out = str(tmp_path / "native.bin")
    pq.write_native([("proj_weight", src.prequantized[0])], [("norm_weight", src.checkpoint_tensors[0])], layout, out)
    img = np.fromfile(out, np.uint8)
    assert img.size == 258
    assert (img[0:4].view(np.float16) == [1.5, -2.0]).all()
    assert list(img[128:132]) == [0x55] * 4
    assert img[256:258].view(np.float16)[0] == 0.25
    row = orc.signed_dequantize(orc.BINARY1, img[128:132].reshape(1, 4), img[256:258].view(np.uint16).reshape(1, 1), 32, 32, 32)[0]
    assert row[0] == 0.25 and row[1] == -0.25


@pytest.mark.gpu
def test_native_writer_preserves_interleaved_ternary_codes(tmp_path, importer):
    """SmeltPrequantizedTensorTests.swift:237-293."""
    inter = np.zeros(8, np.uint8)
    for col in range(32):
        inter[col // 4] |= (col % 3) << ((col & 3) * 2)
    ts = pq.read_safetensors(str(write_synthetic(tmp_path / "t.safetensors", [
        ("model.proj.weight", "U32", [1, 2], inter.tobytes()),
        ("model.proj.scales", "F16", [1, 1], f16([0.5])), ("model.proj.biases", "F16", [1, 1], f16([-0.5]))])))
    src = pq.MlxTriplets(ts, im.FORMAT_TERNARY2, 32, importer)
    layout = [WeightRecord("proj_weight", 0, 8, [1, 32], "ternary2",
                           {"group_size": 32, "packed_row_stride": 8, "padded_cols": 32,
                            "scales_offset": 128, "scales_size_bytes": 2})]
    out = str(tmp_path / "tern.bin")
    pq.write_native([("proj_weight", src.prequantized[0])], [], layout, out)
    img = np.fromfile(out, np.uint8)
    assert (img[:8] == inter).all() and img[128:130].view(np.float16)[0] == 0.5
    row = orc.signed_dequantize(orc.TERNARY2, img[0:8].reshape(1, 8), img[128:130].view(np.uint16).reshape(1, 1), 32, 32, 32)[0]
    assert (row == [(c % 3 - 1) * 0.5 for c in range(32)]).all()
