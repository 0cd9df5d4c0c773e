"""GPU parity of the single-pass matrix-core matvec (the kernel large single-token records take):
every format and both activation types against the oracle, through the C-ABI, with the engine
forced to the matrix cores so that small, ragged and odd-width shapes exercise it too."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import runtime as rt
from test_gpu_matvec import run_affine, run_signed

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = rt.Context()
    c.set_matvec_engine(rt.MATVEC_MATRIX_CORE)
    yield c
    c.close()


@pytest.fixture(scope="module")
def vec():
    c = rt.Context()
    c.set_matvec_engine(rt.MATVEC_VECTOR)
    yield c
    c.close()


# rows: multiples of 8, ragged tails, fewer than one tile; cols: one 16-byte piece per row, a partial
# 128-byte segment, several segments per wave, several waves per row
# (28672 columns: 112 segments, seven per wave on sixteen waves; 8192: four per wave on eight; 30720: eight on fifteen)
AFFINE_SHAPES = [(8, 32, 32), (5, 64, 64), (50, 1152, 64), (130, 3584, 64), (24, 2560, 128), (264, 5120, 64),
                 (72, 17408, 64), (33, 9216, 32), (40, 28672, 64), (8200, 8192, 64), (19, 30720, 128)]


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("shape", AFFINE_SHAPES)
def test_affine_matrix_core_matvec(ctx, dtype, shape):
    rows, cols, group = shape
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=rows)
    x = fx.synth_activation(1, cols, dtype, config=1, tensor=cols)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, dtype), rows, cols, group, dtype)
    y = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    w = gh.check_outputs(y, ref, dtype, f"matrix-core affine {shape}")
    print(f"\n  matrix-core affine {shape} dtype={dtype} max rel err {w:.2e}")


@pytest.mark.parametrize("cols", [2560, 3584])
def test_affine_tall_matrix_two_waves_per_tile(ctx, cols):
    """A vocabulary-sized matrix of rows of ten and fourteen segments: two waves per tile, five and seven segments each.
    Against the oracle on the first and last rows (ragged last tile), and against the vector kernel everywhere: at most
    one step of the output type apart."""
    rows, group, dtype = 131075, 64, fx.BF16
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=cols)
    x = fx.synth_activation(1, cols, dtype, config=1, tensor=cols + 1)
    y = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    for sl in (slice(0, 96), slice(rows - 99, rows)):
        n = sl.stop - sl.start
        ref = so.affine_matvec(packed[sl], scales[sl], biases[sl], fx.from_bits(x, dtype), n, cols, group, dtype)
        gh.check_outputs(y[:, sl], ref, dtype, f"tall affine {rows}x{cols} rows {sl.start}..{sl.stop}")
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)
    try:
        y_vec = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    finally:
        ctx.set_matvec_engine(rt.MATVEC_AUTO)
    gh.check_steps(y, y_vec, dtype, f"tall affine {rows}x{cols}, single-pass against vector kernel", max_steps=1, min_exact=0.9)


def test_affine_matrix_core_exact_on_dyadic_fixture(ctx):
    """KernelLab.swift:2829-2855 buffers: every partial sum is an exact dyadic rational, so the
    matrix cores must give the oracle's bits too."""
    rows, cols, group = 64, 1024, 64
    packed, scales, biases, x = fx.kernel_lab_qmm_fixture(rows, cols, group, 1)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, fx.F16), rows, cols, group)
    y = run_affine(ctx, packed, scales, biases, x, fx.F16, f"affine_matvec:{cols}:{group}", generic=True)
    assert np.array_equal(y, ref.astype(np.float16).view(np.uint16))


# (28672 columns: a ternary row of 56 segments takes four per wave)
SIGNED_SHAPES = [(5, 128), (8, 256), (50, 1152), (1024, 5120), (264, 17408), (77, 9216), (40, 28672)]


def pack_signed(codes, fmt, garbage_padding=False):
    """Packed rows at the stride the kernels expect (trit5: five digits per byte, rows padded to 16 bytes).
    With garbage_padding the trit5 bytes past the last column's byte hold arbitrary valid digit bytes."""
    if fmt != fx.TRIT5:
        return fx.pack_signed_np(codes, fmt)
    cols = codes.shape[1]
    stride = (((cols + 4) // 5) + 15) // 16 * 16
    packed = fx.pack_signed_np(codes, fmt, stride)
    used = (cols + 4) // 5
    if garbage_padding and used < stride:
        packed[:, used:] = fx.rng_for(3, cols).integers(0, 243, (codes.shape[0], stride - used), dtype=np.uint8)
    return packed


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("fmt,name", [(fx.BINARY1, "binary"), (fx.TERNARY2, "ternary"), (fx.TRIT5, "trit5")])
@pytest.mark.parametrize("shape", SIGNED_SHAPES)
def test_signed_matrix_core_matvec(ctx, fmt, name, dtype, shape):
    rows, cols = shape
    codes = fx.synth_signed_codes(fmt, rows, cols, config=2 + fmt, tensor=rows % 7)
    scales = fx.synth_signed_scales(rows, cols, config=2 + fmt, tensor=rows % 7)
    packed = pack_signed(codes, fmt, garbage_padding=True)
    x = fx.synth_activation(1, cols, dtype, config=2 + fmt)
    ref = so.signed_matvec(fmt, packed, scales, fx.from_bits(x, dtype), rows, cols, cols, 128)
    y = run_signed(ctx, name, packed, scales, x, dtype, rows, cols)
    w = gh.check_outputs(y, ref, dtype, f"matrix-core signed {name} {shape}")
    print(f"\n  matrix-core {name} {shape} dtype={dtype} max rel err {w:.2e}")


def test_ternary_matrix_core_reproduces_mlx_golden_bits(ctx):
    """MLX v0.31.1 bit patterns held by SignedQuantKernelTests.swift:87-199: all partial sums of
    these fixtures are exact in fp32, so the matrix-core kernel must reproduce them as well."""
    g = fx.golden_vectors()
    for key in ("ternary_qmv_mlx_k512", "ternary_qmv_mlx_k5120_m3"):
        case = g[key]
        codes, scales, x = fx.mlx_ternary_fixture(case["rows"], case["cols"], case["batch"], case["scale_unit"])
        packed = fx.pack_signed_np(codes, fx.TERNARY2)
        want = np.array([int(b, 16) for b in case["expected_bits"]], np.uint16).reshape(case["batch"], case["rows"])
        for b in range(case["batch"]):   # the matrix-core kernel is the single-token one
            y = run_signed(ctx, "ternary", packed, scales, x[b:b + 1], fx.F16, case["rows"], case["cols"])
            assert np.array_equal(y[0], want[b]), (key, b)


@pytest.mark.parametrize("fmt,name", [(fx.BINARY1, "binary"), (fx.TERNARY2, "ternary"), (fx.TRIT5, "trit5")])
def test_signed_matrix_core_fused_forms_equal_staged(ctx, fmt, name):
    rows, cols = 100, 2560
    dtype = fx.BF16
    gc = fx.synth_signed_codes(fmt, rows, cols, tensor=1)
    uc = fx.synth_signed_codes(fmt, rows, cols, tensor=2)
    gs = fx.synth_signed_scales(rows, cols, tensor=1)
    us = fx.synth_signed_scales(rows, cols, tensor=2)
    gp, up = pack_signed(gc, fmt), pack_signed(uc, fmt)
    x = fx.synth_activation(1, cols, dtype, config=2)
    g = run_signed(ctx, name, gp, gs, x, dtype, rows, cols)
    u = run_signed(ctx, name, up, us, x, dtype, rows, cols)
    res = fx.to_bits(fx.rng_for(2, 78).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    fused_add = run_signed(ctx, name, gp, gs, x, dtype, rows, cols, kind="add", residual=res)
    assert np.array_equal(fused_add, so.narrow(fx.from_bits(g, dtype) + fx.from_bits(res, dtype), dtype))
    fused = run_signed(ctx, name, gp, gs, x, dtype, rows, cols, kind="gate_up", second=(up, us))
    staged = so.epilogue_signed_swiglu(g, u, so.BF16)
    diff = np.abs(fused.astype(np.int32) - staged.astype(np.int32))
    assert diff.max() <= 1, diff.max()   # the low-precision exp() is not pinned bit-exactly


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_affine_matrix_core_fused_forms_equal_staged(ctx, dtype):
    rows, cols, group = 200, 5120, 64
    gw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=4)
    uw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=5)
    x = fx.synth_activation(1, cols, dtype, config=1)
    y = run_affine(ctx, *gw, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    res = fx.to_bits(fx.rng_for(1, 77).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    fused = run_affine(ctx, *gw, x, dtype, f"fused_affine_matvec_add:{cols}:{group}", residual=res, generic=True)
    assert np.array_equal(fused, so.narrow(fx.from_bits(y, dtype) + fx.from_bits(res, dtype), dtype))
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, group, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, group, dtype)
    ref = fx.from_bits(so.epilogue_affine_swiglu(g, u, so.BF16 if dtype == fx.BF16 else so.F16), dtype)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.alloc(gh.Y_SLOT, rows * 2)
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
    pipe = ctx.pipeline(f"fused_affine_gate_up_swiglu_c{cols}_r{rows}_g{group}_rows4" + gh.t_suffix(dtype))
    ctx.encode_decode(rt.make_record(pipe, bufs, [], (512, 1, 1), (256, 1, 1)))
    ctx.wait()
    got = ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows)
    gh.check_outputs(got, gh.swiglu_unrounded(g, u), dtype, "matrix-core affine gate_up_swiglu")


def test_engines_agree_within_tolerance_and_auto_switches_by_size(ctx, vec):
    """The two engines differ in summation order only; AUTO keeps a small matrix on the vector
    kernel (bit-identical to VECTOR) and moves a large one to the matrix cores (bit-identical to
    MATRIX_CORE)."""
    dtype = fx.BF16
    auto = rt.Context()
    try:
        for rows, cols, large in ((256, 1024, False), (2048, 5120, True)):
            w = fx.synth_affine(rows, cols, 64, dtype, config=1, tensor=3)
            x = fx.synth_activation(1, cols, dtype, config=1, tensor=4)
            name = f"affine_matvec:{cols}:64"
            ym = run_affine(ctx, *w, x, dtype, name, generic=True)
            yv = run_affine(vec, *w, x, dtype, name, generic=True)
            ya = run_affine(auto, *w, x, dtype, name, generic=True)
            ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
            gh.check_outputs(ym, ref, dtype, "matrix-core")
            gh.check_outputs(yv, ref, dtype, "vector")
            assert np.array_equal(ya, ym if large else yv)
    finally:
        auto.close()


def test_bf16_activations_beyond_the_fp16_range(ctx):
    """bf16 activations enter the bf16 MFMA unconverted: magnitudes past 65504 are not clamped."""
    rows, cols, group = 64, 1024, 64
    dtype = fx.BF16
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=8)
    xf = fx.rng_for(1, 555).normal(0, 1, (1, cols)).astype(np.float32)
    xf[0, ::37] *= 3.0e5
    x = fx.to_bits(xf, dtype)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, dtype), rows, cols, group, dtype)
    y = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    gh.check_outputs(y, ref, dtype, "matrix-core affine with |x| > 65504")


def test_vector_engine_converts_bf16_activations_to_fp16(vec):
    """The vector-ALU kernels feed v_dot2_f32_f16: bf16 activations are converted to fp16 on staging,
    exact for |x| in [2^-14, 65504] and saturating beyond.  Pinned here: with |x| > 65504 the kernel
    matches the oracle run on the clamped activations, not on the raw ones."""
    rows, cols, group = 64, 1024, 64
    dtype = fx.BF16
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=8)
    xf = fx.rng_for(1, 555).normal(0, 1, (1, cols)).astype(np.float32)
    xf[0, ::37] *= 3.0e5
    x = fx.to_bits(xf, dtype)
    raw = fx.from_bits(x, dtype)
    clamped = np.clip(raw, -65504.0, 65504.0)
    y = run_affine(vec, packed, scales, biases, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    gh.check_outputs(y, so.affine_matvec(packed, scales, biases, clamped, rows, cols, group, dtype), dtype, "vector engine, clamped reference")
    ref_raw = so.affine_matvec(packed, scales, biases, raw, rows, cols, group, dtype)
    assert np.abs(fx.from_bits(y, dtype) - ref_raw).max() > 0.1 * np.abs(ref_raw).max()


def test_ternary_affine_names_on_both_engines(ctx, vec):
    """signed_ternary_affine_{matvec, matvec_add, gate_up_swiglu}_g128_rows8 (the production ternary
    names: codes, scales, scales again, x, y): the matrix-core kernels against the oracle and the
    vector kernels, ragged row count."""
    dtype = fx.BF16
    rows, cols = 203, 2560
    gc = fx.synth_signed_codes(fx.TERNARY2, rows, cols, config=3, tensor=5)
    uc = fx.synth_signed_codes(fx.TERNARY2, rows, cols, config=3, tensor=6)
    gs = fx.synth_signed_scales(rows, cols, config=3, tensor=5)
    us = fx.synth_signed_scales(rows, cols, config=3, tensor=6)
    gp, up = fx.pack_signed_np(gc, fx.TERNARY2), fx.pack_signed_np(uc, fx.TERNARY2)
    x = fx.synth_activation(1, cols, dtype, config=3, tensor=7)
    res = fx.to_bits(fx.rng_for(3, 80).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    xf = fx.from_bits(x, dtype)
    g_ref = so.signed_matvec(so.TERNARY2, gp, gs, xf, rows, cols, cols, 128)
    u_ref = so.signed_matvec(so.TERNARY2, up, us, xf, rows, cols, cols, 128)
    got = {}
    for name, c in (("matrix", ctx), ("vector", vec)):
        wf = gh.WeightFile()
        ogp, ogs, oup, ous = wf.add(gp), wf.add(gs), wf.add(up), wf.add(us)
        c.upload_weights(0, wf.image())
        c.put(gh.X_SLOT, x)
        c.put(gh.RES_SLOT, res)
        for s in (gh.Y_SLOT, gh.AUX_SLOT, gh.AUX2_SLOT):
            c.alloc(s, rows * 2)
        grid = ((rows + 7) // 8, 1, 1)

        def run(pipe, bufs, consts):
            c.encode_decode(rt.make_record(c.pipeline(pipe + gh.t_suffix(dtype)), bufs, consts, grid, (256, 1, 1)))
            c.wait()

        run("signed_ternary_affine_matvec_g128_rows8",
            [(0, 0, ogp), (0, 1, ogs), (0, 2, ogs), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)], [(5, rows), (6, cols)])
        run("signed_ternary_affine_matvec_add_g128_rows8",
            [(0, 0, ogp), (0, 1, ogs), (0, 2, ogs), (gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0), (gh.RES_SLOT, 5, 0)], [(6, rows), (7, cols)])
        run("signed_ternary_affine_gate_up_swiglu_g128_rows8",
            [(0, 0, ogp), (0, 1, ogs), (0, 2, ogs), (0, 3, oup), (0, 4, ous), (0, 5, ous), (gh.X_SLOT, 6, 0), (gh.AUX2_SLOT, 7, 0)],
            [(8, rows), (9, cols)])
        y = c.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows)
        ya = c.read(gh.AUX_SLOT, np.uint16, rows).reshape(1, rows)
        yg = c.read(gh.AUX2_SLOT, np.uint16, rows).reshape(1, rows)
        gh.check_outputs(y, g_ref, dtype, f"ternary-affine matvec ({name})")
        assert np.array_equal(ya, so.narrow(fx.from_bits(y, dtype) + fx.from_bits(res, dtype), dtype))
        staged = so.epilogue_signed_swiglu(so.narrow(g_ref, dtype), so.narrow(u_ref, dtype), so.BF16)
        assert np.abs(yg.astype(np.int32) - staged.astype(np.int32)).max() <= 2, name
        got[name] = y
    assert np.abs(got["matrix"].astype(np.int32) - got["vector"].astype(np.int32)).max() <= 1


def test_affine_bank4_on_the_matrix_cores(ctx, vec):
    """affine_bank4_matvec:K:G over q|k|v: the matrix-core bank kernel gives each member the bits of
    its own matrix-core matvec, and the oracle's values."""
    dtype = fx.BF16
    cols, group = 2560, 64
    member_rows = [264, 72, 61]
    rows = sum(member_rows)
    w = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=9)
    x = fx.synth_activation(1, cols, dtype, config=1, tensor=10)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype)
    whole = run_affine(ctx, *w, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    gh.check_outputs(whole, ref, dtype, "matrix-core matvec over the whole slab")
    for c in (ctx, vec):
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in w]
        c.upload_weights(gh.WEIGHTS_SLOT, wf.image())
        c.put(gh.X_SLOT, x)
        outs = [gh.Y_SLOT, gh.AUX_SLOT, gh.AUX2_SLOT]
        for s, r in zip(outs, member_rows):
            c.alloc(s, r * 2)
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0)] + [(outs[min(i, 2)], 4 + i, 0) for i in range(4)]
        consts = [(8 + i, member_rows[i] if i < 3 else 0) for i in range(4)]
        pipe = c.pipeline(f"affine_bank4_matvec:{cols}:{group}" + gh.t_suffix(dtype))
        c.encode_decode(rt.make_record(pipe, bufs, consts, ((rows + 7) // 8, 1, 1), (256, 1, 1)))
        c.wait()
        start = 0
        for s, r in zip(outs, member_rows):
            y = c.read(s, np.uint16, r).reshape(1, r)
            gh.check_outputs(y, ref[:, start:start + r], dtype, "bank member")
            if c is ctx:
                assert np.array_equal(y, whole[:, start:start + r])
            start += r


def test_operands_off_a_16_byte_boundary_keep_the_vector_kernel(ctx, vec):
    """The matrix-core kernels fetch scales and biases 16 bytes at a time; a record that binds a
    scale plane 2 bytes past a boundary is served by the kernel its pipeline names (bit-identical to
    the vector engine), not faulted on."""
    dtype = fx.BF16
    rows, cols, group = 96, 2560, 64
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=12)
    x = fx.synth_activation(1, cols, dtype, config=1, tensor=13)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, dtype), rows, cols, group, dtype)
    image = np.zeros(1 << 20, np.uint8)
    o_w, o_s, o_b = 0, 256 * 1024 + 2, 512 * 1024
    for off, a in ((o_w, packed), (o_s, scales), (o_b, biases)):
        b = np.ascontiguousarray(a).view(np.uint8).ravel()
        image[off:off + b.size] = b
    out = []
    for c in (ctx, vec):
        c.upload_weights(gh.WEIGHTS_SLOT, image)
        c.put(gh.X_SLOT, x)
        c.alloc(gh.Y_SLOT, rows * 2)
        pipe = c.pipeline(f"affine_matvec:{cols}:{group}" + gh.t_suffix(dtype))
        bufs = [(0, 0, o_w), (0, 1, o_s), (0, 2, o_b), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
        c.encode_decode(rt.make_record(pipe, bufs, [(5, rows)], ((rows + 7) // 8, 1, 1), (256, 1, 1)))
        c.wait()
        out.append(c.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows))
    gh.check_outputs(out[0], ref, dtype, "misaligned scale plane")
    assert np.array_equal(out[0], out[1])


@pytest.mark.parametrize("fmt,name", [(fx.BINARY1, "binary"), (fx.TERNARY2, "ternary"), (fx.TRIT5, "trit5")])
@pytest.mark.parametrize("kind", ["matvec", "gate_up"])
@pytest.mark.parametrize("batch", [6, 5, 2])
def test_signed_four_token_forms_run_one_grid_row_per_token(fmt, name, kind, batch):
    """`*_batched_b4` records (four tokens per grid row) and per-token records with several grid rows take the
    single-pass kernel under the default engine: two tokens per pass for binary and ternary codes (the second token
    in the MFMA's free token slots), one grid row per token for five-digit bytes.  Each token's row is the
    single-token kernel's bits and, for the plain matvec, the oracle's values to the usual bar.  Ragged batches
    (6 = 4 + 2; 5: the last pass holds one token) and ragged rows."""
    rows, cols, dtype = 1003, 5120, fx.BF16
    c = rt.Context()
    try:
        mats = []
        for t in range(2 if kind == "gate_up" else 1):
            codes = fx.synth_signed_codes(fmt, rows, cols, config=2 + fmt, tensor=t)
            mats.append((pack_signed(codes, fmt), fx.synth_signed_scales(rows, cols, config=2 + fmt, tensor=t)))
        x = fx.synth_activation(batch, cols, dtype, config=2 + fmt, tensor=77)
        second = mats[1] if kind == "gate_up" else None
        y4 = run_signed(c, name, *mats[0], x, dtype, rows, cols, kind=kind, second=second, b4=True)
        yr = run_signed(c, name, *mats[0], x, dtype, rows, cols, kind=kind, second=second)
        assert np.array_equal(y4, yr)
        for b in range(batch):
            y1 = run_signed(c, name, *mats[0], x[b:b + 1], dtype, rows, cols, kind=kind, second=second)
            assert np.array_equal(y4[b], y1[0]), b
        if kind == "matvec":
            ref = so.signed_matvec(fmt, *mats[0], fx.from_bits(x, dtype), rows, cols, cols, 128)
            gh.check_outputs(y4, ref, dtype, f"four-token {name}")
    finally:
        c.close()


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_ternary_affine_rows_over_several_tokens(dtype):
    """`signed_ternary_affine_matvec_g128_rows8` with one grid row per token (what the reference launches below six
    tokens): two tokens per pass on the single-pass kernel; every row is the one-token launch's bits."""
    rows, cols, batch = 777, 2560, 5
    c = rt.Context()
    try:
        codes = fx.synth_signed_codes(fx.TERNARY2, rows, cols, config=3, tensor=5)
        scales = fx.synth_signed_scales(rows, cols, config=3, tensor=5)
        packed = fx.pack_signed_np(codes, fx.TERNARY2)
        x = fx.synth_activation(batch, cols, dtype, config=3, tensor=15)
        wf = gh.WeightFile()
        oc, os_ = wf.add(packed), wf.add(scales)
        c.upload_weights(0, wf.image())
        pipe = c.pipeline("signed_ternary_affine_matvec_g128_rows8" + gh.t_suffix(dtype))

        def run(xb):
            n = xb.shape[0]
            c.put(gh.X_SLOT, xb)
            c.alloc(gh.Y_SLOT, n * rows * 2)
            bufs = [(0, 0, oc), (0, 1, os_), (0, 2, os_), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
            assert c.encode_decode(rt.make_record(pipe, bufs, [(5, rows), (6, cols)], ((rows + 7) // 8, n, 1), (256, 1, 1))) == 1
            c.wait()
            return c.read(gh.Y_SLOT, np.uint16, n * rows).reshape(n, rows)

        y = run(x)
        for b in range(batch):
            assert np.array_equal(y[b], run(x[b:b + 1])[0]), b
        ref = so.signed_matvec(so.TERNARY2, packed, scales, fx.from_bits(x, dtype), rows, cols, cols, 128)
        gh.check_outputs(y, ref, dtype, "ternary affine rows, five tokens")
    finally:
        c.close()


@pytest.mark.parametrize("fmt,name", [(fx.BINARY1, "binary"), (fx.TERNARY2, "ternary")])
@pytest.mark.parametrize("kind", ["matvec", "add", "gate_up"])
@pytest.mark.parametrize("shape", [(1003, 5120, 13), (40, 768, 8), (264, 2560, 33)])
@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_signed_rows_over_many_tokens_stream(fmt, name, kind, shape, dtype):
    """Per-token binary and ternary records (one grid row per token) from eight tokens on (bf16 rows converted to fp16): the
    streaming kernel of the format (the weights pass once per sixteen tokens).  Against the single-token kernel's
    rows (the same exact operands and fp32 scales in another summation order: one output step at most for the
    plain and +residual forms, the SwiGLU step bound for gate+up) and, for the plain matvec, the oracle."""
    rows, cols, batch = shape
    c = rt.Context()
    try:
        mats = []
        for t in range(2 if kind == "gate_up" else 1):
            codes = fx.synth_signed_codes(fmt, rows, cols, config=2 + fmt, tensor=10 + t)
            mats.append((pack_signed(codes, fmt), fx.synth_signed_scales(rows, cols, config=2 + fmt, tensor=10 + t)))
        x = fx.synth_activation(batch, cols, dtype, config=2 + fmt, tensor=78)
        res = fx.to_bits(fx.rng_for(2, 79).normal(0, 1, (batch, rows)).astype(np.float32), dtype) if kind == "add" else None
        second = mats[1] if kind == "gate_up" else None
        y = run_signed(c, name, *mats[0], x, dtype, rows, cols, kind=kind, second=second, residual=res)
        assert np.array_equal(y, run_signed(c, name, *mats[0], x, dtype, rows, cols, kind=kind, second=second, residual=res))
        if kind != "add":
            # the four-token form of the same record takes the same kernel
            assert np.array_equal(y, run_signed(c, name, *mats[0], x, dtype, rows, cols, kind=kind, second=second, b4=True))
        if kind == "add":
            # the residual form is the plain form's rounded sums plus the residual, bit for bit (a comparison with the
            # single-token rows would measure the projection's last place against a sum that may cancel)
            plain = run_signed(c, name, *mats[0], x, dtype, rows, cols, kind="matvec")
            assert np.array_equal(y, so.narrow(fx.from_bits(plain, dtype) + fx.from_bits(res, dtype), dtype))
        else:
            rows1 = np.concatenate([run_signed(c, name, *mats[0], x[b:b + 1], dtype, rows, cols, kind=kind, second=second)
                                    for b in range(batch)])
            gh.check_steps(y, rows1, dtype, f"{name} {kind} over {batch} tokens against single-token rows",
                           max_steps=4 if kind == "gate_up" else 1, min_exact=0.8 if kind == "gate_up" else 0.9)
        if kind == "matvec":
            ref = so.signed_matvec(fmt, *mats[0], fx.from_bits(x, dtype), rows, cols, cols, 128)
            gh.check_outputs(y, ref, dtype, f"{name} over {batch} tokens")
    finally:
        c.close()


def test_ternary_affine_rows_over_many_tokens_stream():
    """`signed_ternary_affine_matvec_g128_rows8` with one grid row per token at thirteen tokens (fp16): the streaming
    kernel, the second binding of the scale plane ignored as in the single-token kernel."""
    rows, cols, batch, dtype = 777, 2560, 13, fx.F16
    c = rt.Context()
    try:
        codes = fx.synth_signed_codes(fx.TERNARY2, rows, cols, config=3, tensor=6)
        scales = fx.synth_signed_scales(rows, cols, config=3, tensor=6)
        other = np.roll(scales, 2, axis=0)
        packed = fx.pack_signed_np(codes, fx.TERNARY2)
        x = fx.synth_activation(batch, cols, dtype, config=3, tensor=16)
        wf = gh.WeightFile()
        oc, os_, oo = wf.add(packed), wf.add(scales), wf.add(other)
        c.upload_weights(0, wf.image())
        c.put(gh.X_SLOT, x)
        c.alloc(gh.Y_SLOT, batch * rows * 2)
        pipe = c.pipeline("signed_ternary_affine_matvec_g128_rows8")
        bufs = [(0, 0, oc), (0, 1, os_), (0, 2, oo), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
        assert c.encode_decode(rt.make_record(pipe, bufs, [(5, rows), (6, cols)], ((rows + 7) // 8, batch, 1), (256, 1, 1))) == 1
        c.wait()
        y = c.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
        ref = so.signed_matvec(so.TERNARY2, packed, scales, fx.from_bits(x, dtype), rows, cols, cols, 128)
        gh.check_outputs(y, ref, dtype, "ternary affine rows, thirteen tokens")
    finally:
        c.close()
