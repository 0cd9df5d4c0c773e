"""GPU parity: quantized matvec kernels vs the CPU oracle, driven through the C-ABI with
hand-built dispatch records (the same bindings the reference emitter produces)."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import runtime as rt

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = rt.Context()
    yield c
    c.close()


@pytest.fixture
def vector_ctx(ctx):
    """The module's context on the vector-ALU kernels: comparisons that are bit for bit between a fused kernel and
    its staged pair, or a small-batch kernel and the single-token one, hold there; under AUTO a single-token affine
    matvec takes the single-pass matrix-core kernel, whose order of accumulation differs (same tolerance against
    the oracle)."""
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)
    yield ctx
    ctx.set_matvec_engine(rt.MATVEC_AUTO)


def run_affine(ctx, packed, scales, biases, x_bits, dtype, entry, *, residual=None, grid=None,
               tg=256, generic=False, batched=False, batch_tile=8):
    rows, cols = packed.shape[0], packed.shape[1] * 2
    batch = x_bits.shape[0]
    wf = gh.WeightFile()
    ow, os_, ob = wf.add(packed), wf.add(scales), wf.add(biases)
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, x_bits)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    bufs = [(0, 0, ow), (0, 1, os_), (0, 2, ob), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
    consts = []
    nxt = 5
    if residual is not None:
        ctx.put(gh.RES_SLOT, residual)
        bufs.append((gh.RES_SLOT, 5, 0))
        nxt = 6
    if generic:
        consts.append((nxt, rows))
    if batched:
        consts.append((nxt, batch))
    pipe = ctx.pipeline(entry + gh.t_suffix(dtype))
    gw = grid or min(1024, (rows + 7) // 8)
    gy = (batch + batch_tile - 1) // batch_tile if batched else batch
    rec = rt.make_record(pipe, bufs, consts, (gw, gy, 1), (tg, 1, 1))
    assert ctx.encode_decode(rec) == 1
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_affine_matvec_config0(ctx, dtype):
    """K=1024, N=3584, g64: seeded synthetic tensors; generic and fixed-shape pipeline names."""
    rows, cols, group = 3584, 1024, 64
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=0, tensor=0)
    x = fx.synth_activation(1, cols, dtype, config=0)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, dtype), rows, cols, group, dtype)
    y = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    w1 = gh.check_outputs(y, ref, dtype, "affine_matvec generic")
    y2 = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec_c{cols}_r{rows}_g{group}_rows4")
    assert np.array_equal(y, y2)
    # launch geometry is a tuning knob only: a Metal-shaped grid (N/8 x 64 threads) gives the same bits
    y3 = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec_c{cols}_r{rows}_g{group}",
                    grid=rows // 8, tg=64)
    assert np.array_equal(y, y3)
    print(f"\n  affine c0 dtype={dtype} max rel err {w1:.2e}")


@pytest.mark.parametrize("shape", [(8, 64, 32), (5, 256, 64), (33, 512, 128), (130, 3584, 64), (24, 2560, 64), (17, 9216, 64)])
def test_affine_matvec_closed_form_fixture_shapes(ctx, shape):
    """Closed-form fixture (PrefillKernelTests.swift:220-264) at ragged row counts and every
    lanes-per-row regime; reference tolerance there is 0.02 absolute."""
    rows, cols, group = shape
    packed, scales, biases, x, _ = fx.affine_synthetic_fixture(rows, cols, group, seed=rows)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, fx.F16), rows, cols, group)
    y = run_affine(ctx, packed, scales, biases, x, fx.F16, f"affine_matvec:{cols}:{group}", generic=True)
    gh.check_outputs(y, ref, fx.F16, f"affine fixture {shape}")
    assert np.abs(fx.from_bits(y, fx.F16) - ref).max() < 0.02


def test_affine_exact_on_dyadic_fixture(ctx):
    """KernelLab.swift:2829-2855 buffers: every partial sum is an exact dyadic rational, so any
    summation order must give the oracle's bits."""
    rows, cols, group = 64, 1024, 64
    packed, scales, biases, x = fx.kernel_lab_qmm_fixture(rows, cols, group, 1)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, fx.F16), rows, cols, group)
    y = run_affine(ctx, packed, scales, biases, x, fx.F16, f"affine_matvec:{cols}:{group}", generic=True)
    assert np.array_equal(y, ref.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_affine_fused_add_equals_staged(ctx, dtype):
    rows, cols, group = 1024, 3584, 64
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=6)
    x = fx.synth_activation(1, cols, dtype, config=1)
    res = fx.to_bits(fx.rng_for(1, 77).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    y = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    fused = run_affine(ctx, packed, scales, biases, x, dtype, f"fused_affine_matvec_add:{cols}:{group}",
                       residual=res, generic=True)
    staged = so.narrow(fx.from_bits(y, dtype) + fx.from_bits(res, dtype), dtype)
    assert np.array_equal(fused, staged)


def run_signed(ctx, fmt_name, packed, scales, x_bits, dtype, rows, cols, *, kind="matvec",
               residual=None, second=None, b4=False, grid=None, tg=256):
    batch = x_bits.shape[0]
    wf = gh.WeightFile()
    oc, os_ = wf.add(packed), wf.add(scales)
    bufs = [(0, 0, oc), (0, 1, os_)]
    nxt = 2
    if second is not None:
        oc2, os2 = wf.add(second[0]), wf.add(second[1])
        bufs += [(0, 2, oc2), (0, 3, os2)]
        nxt = 4
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, x_bits)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    bufs += [(gh.X_SLOT, nxt, 0), (gh.Y_SLOT, nxt + 1, 0)]
    nxt += 2
    if residual is not None:
        ctx.put(gh.RES_SLOT, residual)
        bufs.append((gh.RES_SLOT, nxt, 0))
        nxt += 1
    consts = [(nxt, rows), (nxt + 1, cols)]
    name = {"matvec": f"signed_{fmt_name}_matvec_g128_rows8",
            "add": f"signed_{fmt_name}_matvec_add_g128_rows8",
            "gate_up": f"signed_{fmt_name}_gate_up_swiglu_g128_rows8"}[kind]
    if b4:
        name += "_batched_b4"
        consts.append((nxt + 2, batch))
    pipe = ctx.pipeline(name + gh.t_suffix(dtype))
    gy = (batch + 3) // 4 if b4 else batch
    rec = rt.make_record(pipe, bufs, consts, (grid or min(1024, (rows + 7) // 8), gy, 1), (tg, 1, 1))
    assert ctx.encode_decode(rec) == 1
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)


@pytest.mark.parametrize("fmt,name", [(fx.BINARY1, "binary"), (fx.TERNARY2, "ternary")])
def test_signed_matvec_reference_fixture_batch_and_row_tail(ctx, fmt, name):
    """SignedQuantKernelTests.swift:989-1047: rows 5, cols 256, 5 batch rows,
    tolerance max(0.02, 1%) there; the 2e-3 bar here."""
    codes, scales, x = fx.signed_synthetic_fixture(fmt)
    rows, cols = codes.shape
    packed = fx.pack_signed_np(codes, fmt)
    ref = so.signed_matvec(fmt, packed, scales, fx.from_bits(x, fx.F16), rows, cols, cols, 128)
    y = run_signed(ctx, name, packed, scales, x, fx.F16, rows, cols)
    gh.check_outputs(y, ref, fx.F16, f"signed {name} fixture")
    y4 = run_signed(ctx, name, packed, scales, x, fx.F16, rows, cols, b4=True)
    assert np.array_equal(y, y4), "batched_b4 must equal the per-row kernel bit for bit"


def test_ternary_matvec_reproduces_mlx_golden_bits(ctx):
    """MLX v0.31.1 bit patterns held by SignedQuantKernelTests.swift:87-199. All partial sums of
    these fixtures are exact in fp32, so the result is independent of reduction order."""
    g = fx.golden_vectors()
    for key in ("ternary_qmv_mlx_k512", "ternary_qmv_mlx_k5120_m3"):
        case = g[key]
        codes, scales, x = fx.mlx_ternary_fixture(case["rows"], case["cols"], case["batch"], case["scale_unit"])
        packed = fx.pack_signed_np(codes, fx.TERNARY2)
        y = run_signed(ctx, "ternary", packed, scales, x, fx.F16, case["rows"], case["cols"])
        want = np.array([int(b, 16) for b in case["expected_bits"]], np.uint16)
        assert np.array_equal(y.ravel(), want), key


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("fmt,name", [(fx.BINARY1, "binary"), (fx.TERNARY2, "ternary")])
@pytest.mark.parametrize("shape", [(1024, 5120), (640, 17408)])
def test_signed_matvec_27b_shapes(ctx, fmt, name, dtype, shape):
    rows, cols = shape
    codes = fx.synth_signed_codes(fmt, rows, cols, config=2 + fmt, tensor=rows % 7)
    scales = fx.synth_signed_scales(rows, cols, config=2 + fmt, tensor=rows % 7)
    packed = fx.pack_signed_np(codes, fmt)
    x = fx.synth_activation(1, cols, dtype, config=2 + fmt)
    ref = so.signed_matvec(fmt, packed, scales, fx.from_bits(x, dtype), rows, cols, cols, 128)
    y = run_signed(ctx, name, packed, scales, x, dtype, rows, cols)
    w = gh.check_outputs(y, ref, dtype, f"signed {name} {shape}")
    print(f"\n  {name} {shape} dtype={dtype} max rel err {w:.2e}")


@pytest.mark.parametrize("fmt,name", [(fx.BINARY1, "binary"), (fx.TERNARY2, "ternary")])
def test_signed_fused_add_and_gate_up_equal_staged(ctx, fmt, name):
    rows, cols = 96, 1024
    dtype = fx.F16
    gc = fx.synth_signed_codes(fmt, rows, cols, tensor=1)
    uc = fx.synth_signed_codes(fmt, rows, cols, tensor=2)
    gs = fx.synth_signed_scales(rows, cols, tensor=1)
    us = fx.synth_signed_scales(rows, cols, tensor=2)
    gp, up = fx.pack_signed_np(gc, fmt), fx.pack_signed_np(uc, fmt)
    x = fx.synth_activation(2, cols, dtype, config=2)
    g = run_signed(ctx, name, gp, gs, x, dtype, rows, cols)
    u = run_signed(ctx, name, up, us, x, dtype, rows, cols)
    res = fx.to_bits(fx.rng_for(2, 78).normal(0, 1, (2, rows)).astype(np.float32), dtype)
    fused_add = run_signed(ctx, name, gp, gs, x, dtype, rows, cols, kind="add", residual=res)
    staged_add = so.narrow(fx.from_bits(g, dtype) + fx.from_bits(res, dtype), dtype)
    assert np.array_equal(fused_add, staged_add)
    fused = run_signed(ctx, name, gp, gs, x, dtype, rows, cols, kind="gate_up", second=(up, us))
    staged = so.epilogue_signed_swiglu(g, u, so.F16)
    diff = np.abs(fused.astype(np.int32) - staged.astype(np.int32))
    # the half-precision exp() is not pinned bit-exactly; one output ulp of slack
    assert diff.max() <= 1, diff.max()


def test_affine_gate_up_swiglu_and_dual(vector_ctx):
    ctx = vector_ctx
    rows, cols, group = 3584, 1024, 64
    dtype = fx.F16
    gw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=4)
    uw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=5)
    x = fx.synth_activation(1, cols, dtype, config=1)
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, group, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, group, dtype)
    ref = fx.from_bits(so.epilogue_affine_swiglu(g, u, so.F16), fx.F16)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.alloc(gh.Y_SLOT, rows * 2)
    ctx.alloc(gh.AUX_SLOT, rows * 2)
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
    pipe = ctx.pipeline(f"fused_affine_gate_up_swiglu_c{cols}_r{rows}_g{group}_rows4")
    ctx.encode_decode(rt.make_record(pipe, bufs, [], (512, 1, 1), (256, 1, 1)))
    ctx.wait()
    y = ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows)
    gh.check_outputs(y, gh.swiglu_unrounded(g, u), fx.F16, "affine gate_up_swiglu")
    # dual: two outputs equal two single matvecs bit for bit
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0), (gh.AUX_SLOT, 8, 0)]
    pipe = ctx.pipeline(f"fused_dual_affine_matvec:{cols}:{group}")
    ctx.encode_decode(rt.make_record(pipe, bufs, [(9, rows)], (512, 1, 1), (256, 1, 1)))
    ctx.wait()
    y1 = ctx.read(gh.Y_SLOT, np.uint16, rows)
    y2 = ctx.read(gh.AUX_SLOT, np.uint16, rows)
    s1 = run_affine(ctx, *gw, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    s2 = run_affine(ctx, *uw, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    assert np.array_equal(y1, s1.ravel()) and np.array_equal(y2, s2.ravel())


@pytest.mark.parametrize("batch,tile", [(3, 3), (4, 4), (7, 8), (9, 4)])
def test_affine_small_batch_equals_per_row_matvec(vector_ctx, batch, tile):
    """Per-token results of the small-batch kernel are the batch-1 kernel's bits
    (the reference asserts the same of its batched variants).  On the vector-ALU kernels: under AUTO the
    single-token record runs the matrix-core kernel, which adds up a row in another order."""
    ctx = vector_ctx
    rows, cols, group = 512, 1024, 64
    dtype = fx.F16
    w = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=2)
    x = fx.synth_activation(batch, cols, dtype, config=1, tensor=50 + batch)
    suffix = {3: "_batched_tile3", 4: "_batched_tile4", 8: "_batched"}[tile]
    yb = run_affine(ctx, *w, x, dtype, f"affine_matvec_c{cols}_r{rows}_g{group}{suffix}",
                    batched=True, batch_tile=tile)
    for b in range(batch):
        y1 = run_affine(ctx, *w, x[b:b + 1], dtype, f"affine_matvec:{cols}:{group}", generic=True)
        assert np.array_equal(yb[b], y1[0]), b


def test_dequant_is_bit_exact_through_embedding_gather(ctx):
    """Per-element dequant contract: gather every row and compare with the oracle's rows."""
    rows, cols, group = 96, 512, 64
    for dtype in (fx.F16, fx.BF16):
        packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=0, tensor=9)
        want = so.affine_dequantize_narrow(packed, scales, biases, cols, group, dtype, dtype)
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in (packed, scales, biases)]
        ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
        ids = np.arange(rows, dtype=np.int32)[::-1].copy()
        ctx.put(gh.X_SLOT, ids)
        ctx.alloc(gh.Y_SLOT, rows * cols * 2)
        pipe = ctx.pipeline("affine_embedding_gather_batched" + gh.t_suffix(dtype))
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
        rec = rt.make_record(pipe, bufs, [(5, cols), (6, rows), (7, group)], (cols // 2, rows, 1),
                             (64, 1, 1), style=rt.STYLE_THREADS)
        assert ctx.encode_prefill(rec, seq_len=rows) == 1
        ctx.wait()
        got = ctx.read(gh.Y_SLOT, np.uint16, rows * cols).reshape(rows, cols)
        assert np.array_equal(got, want[ids])
    for fmt, name in ((fx.BINARY1, "binary"), (fx.TERNARY2, "ternary"), (fx.TRIT5, "trit5")):
        cols = 640
        base = fx.TERNARY2 if fmt == fx.TRIT5 else fmt
        codes = fx.synth_signed_codes(base, rows, cols, tensor=3)
        scales = fx.synth_signed_scales(rows, cols, tensor=3)
        stride = (((cols + 4) // 5) + 15) // 16 * 16 if fmt == fx.TRIT5 else None
        packed = fx.pack_signed_np(codes, fmt, stride)
        wide = so.signed_dequantize(fmt, packed, scales, cols, cols, 128)
        want = wide.astype(np.float16).view(np.uint16)
        wf = gh.WeightFile()
        oc, os_ = wf.add(packed), wf.add(scales)
        ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
        ids = np.arange(rows, dtype=np.int32)
        ctx.put(gh.X_SLOT, ids)
        ctx.alloc(gh.Y_SLOT, rows * cols * 2)
        pipe = ctx.pipeline(f"signed_{name}_embedding_gather_g128")
        rec = rt.make_record(pipe, [(0, 0, oc), (0, 1, os_), (gh.X_SLOT, 2, 0), (gh.Y_SLOT, 3, 0)],
                             [(4, cols)], (cols, rows, 1), (128, 1, 1), style=rt.STYLE_THREADS)
        assert ctx.encode_decode(rec) == 1
        ctx.wait()
        got = ctx.read(gh.Y_SLOT, np.uint16, rows * cols).reshape(rows, cols)
        assert np.array_equal(got, want), name
