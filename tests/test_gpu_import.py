"""GPU parity of the weight-import producers (affine 4-bit quantiser, signed code validation, MLX
scale normalisation) against the CPU oracle, bit for bit, through include/smelt_hip_import.h and
through the device-resident pipelines."""
import json
import os

import numpy as np
import pytest

import fixtures as fx
from oracle import oracle as so
from smelt_amd import importer as im
from smelt_amd import runtime as rt

pytestmark = pytest.mark.gpu

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


@pytest.fixture(scope="module")
def imp():
    i = im.Importer()
    yield i
    i.close()


def weights(seed, rows, cols, outliers=True):
    rng = fx.rng_for(77, seed)
    w = rng.normal(0, 0.05, (rows, cols)).astype(np.float32)
    if outliers:
        idx = rng.integers(0, w.size, max(1, w.size // 97))
        w.ravel()[idx] *= 6.0
    return w


def as_source(w, src_dtype):
    """(array handed to the importer, fp32 values the oracle sees)"""
    if src_dtype == im.SRC_F32:
        return w, w
    bits = so.narrow(w, so.F16 if src_dtype == im.SRC_F16 else so.BF16)
    return bits, so.widen(bits, so.F16 if src_dtype == im.SRC_F16 else so.BF16)


@pytest.mark.parametrize("rows,cols,group", [
    (5, 64, 64), (33, 1024, 64), (7, 200, 64), (3, 129, 32), (9, 96, 32), (64, 4096, 128),
    (2, 130, 128), (1, 1, 32), (300, 2560, 64)])
@pytest.mark.parametrize("src_dtype", [im.SRC_F32, im.SRC_F16, im.SRC_BF16])
def test_affine_quantiser_min_max_is_bit_exact(imp, rows, cols, group, src_dtype):
    src, vals = as_source(weights(rows * 131 + cols, rows, cols), src_dtype)
    for scale_dtype, odt in ((rt.ACT_F16, so.F16), (rt.ACT_BF16, so.BF16)):
        got = imp.quantize_affine_u4(src, src_dtype, rows, cols, group, im.CLIP_MIN_MAX, None, scale_dtype)
        ref = so.affine_quantize(vals, group, 0, None, odt)
        for g, r, name in zip(got, ref, ("packed", "scales", "biases")):
            assert np.array_equal(g, r), (name, scale_dtype)


@pytest.mark.parametrize("rows,cols,group", [(17, 512, 64), (4, 200, 32), (6, 1024, 128), (1, 70, 64)])
@pytest.mark.parametrize("weighted", [False, True])
def test_affine_quantiser_least_error_endpoints_are_bit_exact(imp, rows, cols, group, weighted):
    w = weights(rows + 7 * cols, rows, cols)
    importance = None
    if weighted:
        importance = np.abs(fx.rng_for(78, cols).normal(1.0, 0.7, cols)).astype(np.float32)
    for scale_dtype, odt in ((rt.ACT_F16, so.F16), (rt.ACT_BF16, so.BF16)):
        got = imp.quantize_affine_u4(w, im.SRC_F32, rows, cols, group, im.CLIP_MSE_OPTIMAL, importance, scale_dtype)
        ref = so.affine_quantize(w, group, 1, importance, odt)
        for g, r, name in zip(got, ref, ("packed", "scales", "biases")):
            assert np.array_equal(g, r), (name, scale_dtype)
    # the search must actually move some endpoints on data with outliers
    mm = so.affine_quantize(w, group, 0, None, so.F16)
    assert not np.array_equal(mm[1], so.affine_quantize(w, group, 1, importance, so.F16)[1])


def test_affine_quantiser_reference_fixtures(imp):
    """SmeltAffineU4Tests.swift:67-80 (ramp 0..15, group 16 is below this kernel's group sizes, so the
    same ramp is laid over a group of 32) and :120-128 (constant group -> scale 1, bias = the value)."""
    ramp = np.tile(np.arange(16, dtype=np.float32), 2)[None, :]
    packed, scales, biases = imp.quantize_affine_u4(ramp, im.SRC_F32, 1, 32, 32)
    assert scales[0, 0] == 0x3C00 and biases[0, 0] == 0      # scale 1.0, bias 0
    assert packed[0].tolist() == [((2 * i + 1) << 4) | (2 * i) for i in range(8)] * 2
    const = np.full((1, 64), 0.123, np.float32)
    packed, scales, biases = imp.quantize_affine_u4(const, im.SRC_F32, 1, 64, 64)
    assert scales[0, 0] == 0x3C00 and biases[0, 0] == so.narrow(np.float32([0.123]), so.F16)[0]
    assert not packed.any()


def test_affine_quantised_output_feeds_the_matvec_kernel(imp):
    """producer -> consumer: what the GPU quantiser writes is what the decode kernel reads."""
    import gpu_harness as gh
    rows, cols, group = 256, 1024, 64
    w = weights(5, rows, cols)
    packed, scales, biases = imp.quantize_affine_u4(w, im.SRC_F32, rows, cols, group)
    x = fx.rng_for(79, 1).normal(0, 1, (1, cols)).astype(np.float32)
    x_bits = so.narrow(x, so.F16)
    ctx = rt.Context()
    try:
        wf = gh.WeightFile()
        a, b, c = wf.add(packed), wf.add(scales), wf.add(biases)
        ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
        ctx.put(gh.X_SLOT, x_bits)
        ctx.alloc(gh.Y_SLOT, rows * 2)
        pipe = ctx.pipeline(f"affine_matvec:{cols}:{group}")
        rec = rt.make_record(pipe, [(0, 0, a), (0, 1, b), (0, 2, c), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)],
                             [(5, rows)], (64, 1, 1), (256, 1, 1))
        ctx.interpret_decode(ctx.table([rec]))
        ctx.wait()
        got = ctx.read(gh.Y_SLOT, np.uint16, rows)
    finally:
        ctx.close()
    ref = so.affine_matvec(packed, scales, biases, so.widen(x_bits, so.F16)[0], rows, cols, group, so.F16)
    gh.check_outputs(got, ref, so.F16, "matvec over GPU-quantised weights")
    # and the quantised matrix is a faithful image of w: within half a step per element
    deq = so.affine_dequantize(packed, scales, biases, cols, group, so.F16)
    step = so.widen(scales, so.F16).repeat(group, axis=1)
    assert np.all(np.abs(deq - w) <= 0.51 * step + 1e-3)


def ternary_stream(seed, count):
    rng = fx.rng_for(80, seed)
    codes = rng.integers(0, 3, count).astype(np.uint8)
    pad = (-count) % 4
    c = np.concatenate([codes, np.zeros(pad, np.uint8)]).reshape(-1, 4)
    return (c[:, 0] | (c[:, 1] << 2) | (c[:, 2] << 4) | (c[:, 3] << 6)).astype(np.uint8)


@pytest.mark.parametrize("count", [1, 5, 64, 1023, 4096 * 33 + 3])
def test_signed_code_validation_matches_the_oracle(imp, count):
    stream = ternary_stream(count, count)
    imp.validate_signed_codes(stream, count, im.FORMAT_TERNARY2)
    imp.validate_signed_codes(stream, count, im.FORMAT_BINARY1)     # any bits are binary codes
    rng = fx.rng_for(81, count)
    for _ in range(4):
        bad = stream.copy()
        where = sorted(int(i) for i in rng.integers(0, count, 3))
        for i in where:
            bad[i // 4] |= 3 << (2 * (i % 4))
        rc, ref_idx = so.signed_validate(bad, count, so.TERNARY2)
        assert rc == so.ERR_INVALID_CODE and ref_idx == where[0]
        with pytest.raises(im.ImportError_) as e:
            imp.validate_signed_codes(bad, count, im.FORMAT_TERNARY2)
        assert e.value.code == im.ERR_INVALID_CODE and e.value.index == ref_idx
    # a code 3 in the padding bits after the last logical code is not an error
    if count % 4:
        tail = stream.copy()
        tail[-1] |= 3 << (2 * (count % 4))
        assert so.signed_validate(tail, count, so.TERNARY2)[0] == 0
        imp.validate_signed_codes(tail, count, im.FORMAT_TERNARY2)
    with pytest.raises(im.ImportError_) as e:
        imp.validate_signed_codes(stream[:-1] if stream.size > 1 else stream[:0], count, im.FORMAT_TERNARY2)
    assert e.value.code == im.ERR_BUFFER_TOO_SMALL


def test_trit5_byte_validation(imp):
    rng = fx.rng_for(82, 0)
    count = 5 * 1000 + 2
    stream = rng.integers(0, 243, (count + 4) // 5).astype(np.uint8)
    imp.validate_signed_codes(stream, count, im.FORMAT_TRIT5)
    bad = stream.copy()
    bad[777] = 250
    bad[900] = 243
    rc, ref_idx = so.signed_validate(bad, count, so.TRIT5)
    assert rc == so.ERR_INVALID_CODE and ref_idx == 777 * 5
    with pytest.raises(im.ImportError_) as e:
        imp.validate_signed_codes(bad, count, im.FORMAT_TRIT5)
    assert e.value.index == 777 * 5


def test_mlx_scale_normalisation_reference_cases(imp):
    """SmeltSignedQuantCodecTests.swift:109-204."""
    g = GOLDEN["mlx_scale_normalisation"]
    fmt = {"binary1": im.FORMAT_BINARY1, "ternary2": im.FORMAT_TERNARY2}
    f16 = lambda v: so.narrow(np.float32([v]), so.F16)
    for name, s, b, want in g["ok_f32"]:
        assert imp.normalize_mlx_scales(fmt[name], f16(s), f16(b))[0] == f16(want)[0]
    for name, s, b in g["reject_f32"]:
        with pytest.raises(im.ImportError_) as e:
            imp.normalize_mlx_scales(fmt[name], f16(s), f16(b))
        assert e.value.code == im.ERR_MLX_BIAS and e.value.index == 0
    for name, s, b, want in g["ok_bits"]:
        assert imp.normalize_mlx_scales(fmt[name], np.uint16([s]), np.uint16([b]))[0] == want
    for name, s, b in g["reject_bits"]:
        with pytest.raises(im.ImportError_):
            imp.normalize_mlx_scales(fmt[name], np.uint16([s]), np.uint16([b]))


@pytest.mark.parametrize("fmt", [im.FORMAT_BINARY1, im.FORMAT_TERNARY2])
def test_mlx_scale_normalisation_matches_the_oracle(imp, fmt):
    rng = fx.rng_for(83, fmt)
    n = 70001
    scale = np.abs(rng.normal(0, 0.05, n)).astype(np.float32)
    scale[::97] = rng.uniform(1e-7, 1e-5, scale[::97].size)       # fp16 subnormal range
    s_bits = so.narrow(scale, so.F16)
    canon = so.widen(s_bits, so.F16) * (0.5 if fmt == im.FORMAT_BINARY1 else 1.0)
    b_bits = so.narrow(-so.widen(so.narrow(canon.astype(np.float32), so.F16), so.F16), so.F16)
    # one-ulp drift of the bias is accepted
    drift = rng.integers(0, 3, n) == 0
    b_bits = np.where(drift & (b_bits > 0x8001), b_bits - 1, b_bits).astype(np.uint16)
    rc, ref, _ = so.signed_normalize_mlx(fmt, s_bits, b_bits)
    assert rc == 0
    assert np.array_equal(imp.normalize_mlx_scales(fmt, s_bits, b_bits), ref)
    # failures: the lowest failing group and its reason are reported
    for bad_at, s_val, b_val, code in ((60000, 0x7C00, None, im.ERR_MLX_SCALE), (123, None, 0x3C00, im.ERR_MLX_BIAS),
                                       (5, 0x8400, None, im.ERR_MLX_SCALE)):
        s2, b2 = s_bits.copy(), b_bits.copy()
        if s_val is not None:
            s2[bad_at] = s_val
        if b_val is not None:
            b2[bad_at] = b_val
        b2[65000] = 0x3C00   # a later failure must not win
        rc, _, bad = so.signed_normalize_mlx(fmt, s2, b2)
        assert bad == bad_at
        with pytest.raises(im.ImportError_) as e:
            imp.normalize_mlx_scales(fmt, s2, b2)
        assert e.value.index == bad_at and e.value.code == code
        assert {so.ERR_MLX_SCALE: im.ERR_MLX_SCALE, so.ERR_MLX_BIAS: im.ERR_MLX_BIAS}[rc] == code


def test_device_resident_quantiser_pipeline_and_bad_launches():
    """The same kernel through a dispatch record, sources and outputs resident in slots."""
    rows, cols, group = 128, 2048, 64
    w = weights(11, rows, cols)
    ctx = rt.Context(act_dtype=rt.ACT_BF16)
    try:
        gpr = cols // group
        ctx.put(1, w)
        ctx.alloc(2, rows * cols // 2)
        ctx.alloc(3, rows * gpr * 2)
        ctx.alloc(4, rows * gpr * 2)
        pipe = ctx.pipeline(f"affine_quantize_u4:{cols}:{group}")
        bufs = [(1, 0, 0), (2, 1, 0), (3, 2, 0), (4, 3, 0)]
        rec = rt.make_record(pipe, bufs, [(5, rows), (6, im.SRC_F32), (7, 0)], (32, 1, 1), (128, 1, 1))
        ctx.interpret_decode(ctx.table([rec]))
        ctx.wait()
        ref = so.affine_quantize(w, group, 0, None, so.BF16)
        assert np.array_equal(ctx.read(2, np.uint8, rows * cols // 2).reshape(rows, -1), ref[0])
        assert np.array_equal(ctx.read(3, np.uint16, rows * gpr).reshape(rows, -1), ref[1])
        assert np.array_equal(ctx.read(4, np.uint16, rows * gpr).reshape(rows, -1), ref[2])
        # wrong workgroup size, source too small, unknown group: refused before any launch
        with pytest.raises(rt.SmeltHipError):
            ctx.interpret_decode(ctx.table([rt.make_record(pipe, bufs, [(5, rows), (6, 0), (7, 0)], (32, 1, 1), (256, 1, 1))]))
        with pytest.raises(rt.SmeltHipError):
            ctx.interpret_decode(ctx.table([rt.make_record(pipe, bufs, [(5, rows + 1), (6, 0), (7, 0)], (32, 1, 1), (128, 1, 1))]))
        with pytest.raises(rt.SmeltHipError):
            ctx.pipeline(f"affine_quantize_u4:{cols}:48")
    finally:
        ctx.close()


def test_package_built_on_the_gpu_reads_back_and_decodes(imp, tmp_path):
    """checkpoint tensors -> GPU producers -> weights.bin + manifest.json -> reader -> upload ->
    matvec records: every stage against the oracle."""
    import gpu_harness as gh
    from smelt_amd import compiler as cc
    from smelt_amd import package as pk
    rows, cols = 96, 512
    w = weights(21, rows, cols)
    rng = fx.rng_for(84, 0)
    codes = rng.integers(0, 3, (rows, cols)).astype(np.uint8)
    ter_packed = so.signed_pack(codes, so.TERNARY2)
    mlx_scale = so.narrow(np.abs(rng.normal(0, 0.03, (rows, cols // 128))).astype(np.float32) + 1e-3, so.F16)
    mlx_bias = so.narrow(-so.widen(mlx_scale, so.F16), so.F16)
    b = pk.PackageBuilder()
    b.add_affine_u4("layers.0.q_proj.weight", imp, w, im.SRC_F32, rows, cols, 64)
    b.add_signed("layers.0.o_proj.weight", imp, ter_packed, mlx_scale, mlx_bias, rows, cols, cc.TERNARY2)
    b.add_dense("norm.weight", np.ones(cols, np.float16), cc.FP16)
    b.write(str(tmp_path))
    pw = pk.PackageWeights(str(tmp_path))
    ref_q = so.affine_quantize(w, 64, 0, None, so.F16)
    assert np.array_equal(pw.region("layers.0.q_proj.weight").reshape(rows, -1), ref_q[0])
    assert np.array_equal(pw.region("layers.0.q_proj.weight", "scales").view(np.uint16).reshape(rows, -1), ref_q[1])
    assert np.array_equal(pw.region("layers.0.q_proj.weight", "biases").view(np.uint16).reshape(rows, -1), ref_q[2])
    assert np.array_equal(pw.region("layers.0.o_proj.weight", "scales").view(np.uint16).reshape(rows, -1), mlx_scale)
    # a ternary tensor with a forbidden code never reaches the file
    bad = ter_packed.copy()
    bad[5, 7] |= 0xC0
    with pytest.raises(im.ImportError_) as e:
        pk.PackageBuilder().add_signed("x", imp, bad, mlx_scale, mlx_bias, rows, cols, cc.TERNARY2)
    assert e.value.index == 5 * cols + 7 * 4 + 3
    ctx = rt.Context()
    try:
        pw.upload(ctx, gh.WEIGHTS_SLOT)
        x = so.narrow(rng.normal(0, 1, (1, cols)).astype(np.float32), so.F16)
        ctx.put(gh.X_SLOT, x)
        ctx.alloc(gh.Y_SLOT, rows * 2)
        em = cc.Emitter(rt.ACT_F16, ctx.device_info()["compute_units"])
        eq, eo = pw.entry("layers.0.q_proj.weight"), pw.entry("layers.0.o_proj.weight")
        em.matvec(gh.WEIGHTS_SLOT, eq, cc.bind(gh.X_SLOT), cc.bind(gh.Y_SLOT))
        em.install(ctx)
        ctx.interpret_decode(em.records())
        ctx.wait()
        got = ctx.read(gh.Y_SLOT, np.uint16, rows)
        gh.check_outputs(got, so.affine_matvec(*ref_q, so.widen(x, so.F16)[0], rows, cols, 64, so.F16), so.F16, "q_proj from package")
    finally:
        ctx.close()
    ctx = rt.Context()
    try:
        pw.upload(ctx, gh.WEIGHTS_SLOT)
        ctx.put(gh.X_SLOT, x)
        ctx.alloc(gh.Y_SLOT, rows * 2)
        em = cc.Emitter(rt.ACT_F16, ctx.device_info()["compute_units"])
        em.matvec(gh.WEIGHTS_SLOT, eo, cc.bind(gh.X_SLOT), cc.bind(gh.Y_SLOT))
        em.install(ctx)
        ctx.interpret_decode(em.records())
        ctx.wait()
        got = ctx.read(gh.Y_SLOT, np.uint16, rows)
        ref = so.signed_matvec(so.TERNARY2, ter_packed, mlx_scale, so.widen(x, so.F16)[0], rows, cols, cols, 128)
        gh.check_outputs(got, ref, so.F16, "o_proj from package")
    finally:
        ctx.close()
