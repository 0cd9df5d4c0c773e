"""The fused affine forms of the single-pass matrix-core matvec: two projections of one input (with and without a
residual each), GeGLU, and the norm-scale prologue in front of a projection, a pair or a gate+up
(lut_matvec.metal:1294-1460, 2030-2150, 2235-2243, 2333-2401, 2896-2990).  On the matrix-core engine a fused kernel
equals its staged pair bit for bit, as on the vector engine; across the two engines the results agree to one
step of the output type (different summation orders), and they do differ somewhere, which is how these
tests know the matrix-core kernel ran."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
import oracle.oracle as so
from smelt_amd import runtime as rt
from test_gpu_matvec import run_affine
from test_gpu_norm_scale import RS_SLOT, NW_SLOT, XN_SLOT, norm_inputs, run_norm_scale_matvec, run_gate_up

pytestmark = pytest.mark.gpu

SHAPES = [(2048, 1536, 128), (777, 1056, 32), (5120, 1024, 64)]


@pytest.fixture(scope="module")
def ctx():
    c = rt.Context()
    c.set_matvec_engine(rt.MATVEC_MATRIX_CORE)
    yield c
    c.close()


def on_vector(ctx, fn):
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)
    try:
        return fn()
    finally:
        ctx.set_matvec_engine(rt.MATVEC_MATRIX_CORE)


def other_engine_agrees(got, vec, dtype, what):
    assert not np.array_equal(got, vec), f"{what}: identical to the vector kernel's bits - was the record re-routed?"
    gh.check_steps(got, vec, dtype, what, max_steps=1, min_exact=0.9)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("rows,cols,group", SHAPES)
def test_norm_scale_matvec_on_the_matrix_cores(ctx, dtype, rows, cols, group):
    weights = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=3)
    x, w, rs = norm_inputs(1, cols, dtype, seed=rows)
    xn_ref = so.norm_scale_input(x[0], rs[0], w, dtype)
    entry = f"norm_scale_affine_matvec:{cols}:{group}"
    y, xn = run_norm_scale_matvec(ctx, weights, x, w, rs, dtype, entry, [(8, rows)])
    assert np.array_equal(xn[0], xn_ref)                     # the stored normalised row, bit for bit
    staged = run_affine(ctx, *weights, xn, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    assert np.array_equal(y, staged)                          # fused == staged on this engine
    ref = so.affine_matvec(*weights, fx.from_bits(xn_ref, dtype).reshape(1, cols), rows, cols, group, dtype)
    gh.check_outputs(y, ref, dtype, "norm_scale_affine_matvec (matrix cores)")
    vec, _ = on_vector(ctx, lambda: run_norm_scale_matvec(ctx, weights, x, w, rs, dtype, entry, [(8, rows)]))
    other_engine_agrees(y, vec, dtype, "norm_scale_affine_matvec")


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_norm_add_scale_matvec_on_the_matrix_cores(ctx, dtype):
    rows, cols, group = 2048, 2560, 128
    weights = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=5)
    x, w, rs = norm_inputs(1, cols, dtype, seed=41)
    res = fx.to_bits(np.random.default_rng(42).normal(0, 1, (1, cols)).astype(np.float32), dtype)
    row_ref = so.elementwise(so.norm_scale_input(x[0], rs[0], w, dtype), res[0], dtype)
    wf = gh.WeightFile()
    ow, os_, ob = (wf.add(a) for a in weights)

    def fused():
        ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
        ctx.put(RS_SLOT, rs); ctx.put(gh.X_SLOT, x); ctx.put(NW_SLOT, w); ctx.put(gh.RES_SLOT, res)
        ctx.alloc(XN_SLOT, cols * 2); ctx.alloc(gh.Y_SLOT, rows * 2)
        bufs = [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0), (gh.RES_SLOT, 3, 0), (XN_SLOT, 4, 0), (0, 5, ow),
                (0, 6, os_), (0, 7, ob), (gh.Y_SLOT, 8, 0)]
        pipe = ctx.pipeline(f"norm_add_scale_affine_matvec_c{cols}_r{rows}_g{group}_rows4" + gh.t_suffix(dtype))
        assert ctx.encode_decode(rt.make_record(pipe, bufs, [], (rows // 4, 1, 1), (64, 1, 1))) == 1
        ctx.wait()
        return ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows), ctx.read(XN_SLOT, np.uint16, cols)

    y, row = fused()
    assert np.array_equal(row, row_ref)
    staged = run_affine(ctx, *weights, row.reshape(1, cols), dtype, f"affine_matvec:{cols}:{group}", generic=True)
    assert np.array_equal(y, staged)
    ref = so.affine_matvec(*weights, fx.from_bits(row_ref, dtype).reshape(1, cols), rows, cols, group, dtype)
    gh.check_outputs(y, ref, dtype, "norm_add_scale_affine_matvec (matrix cores)")
    other_engine_agrees(y, on_vector(ctx, fused)[0], dtype, "norm_add_scale_affine_matvec")


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("act", ["swiglu", "geglu"])
@pytest.mark.parametrize("rows,cols,group", [(3584, 1024, 64), (1000, 1056, 32)])
def test_gate_up_forms_on_the_matrix_cores(ctx, dtype, act, rows, cols, group):
    gw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=4)
    uw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=5)
    x, w, rs = norm_inputs(1, cols, dtype, seed=17)
    xn = so.norm_scale_input(x[0], rs[0], w, dtype).reshape(1, cols)
    fused = run_gate_up(ctx, gw, uw, dtype, f"norm_scale_affine_gate_up_{act}:{cols}:{group}", [(10, rows)], x, norm=(w, rs))
    staged = run_gate_up(ctx, gw, uw, dtype, f"fused_affine_gate_up_{act}:{cols}:{group}", [(8, rows)], xn)
    assert np.array_equal(fused, staged)
    # the plain gate+up equals the two projections, rounded, through the oracle's epilogue on those bits (GeGLU
    # rounds gate and up first, so this is exact up to the tanh; SwiGLU is checked against the unrounded sums)
    xf = fx.from_bits(xn, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, group, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, group, dtype)
    if act == "swiglu":
        gh.check_outputs(fused, gh.swiglu_unrounded(g, u), dtype, "norm_scale gate_up swiglu (matrix cores)")
    else:
        gh.check_steps(fused, so.epilogue_geglu(g, u, dtype).reshape(np.shape(fused)), dtype, "gate_up geglu (matrix cores)",
                       max_steps=gh.GEGLU_STEPS)
    vec = on_vector(ctx, lambda: run_gate_up(ctx, gw, uw, dtype, f"fused_affine_gate_up_{act}:{cols}:{group}", [(8, rows)], xn))
    assert not np.array_equal(staged, vec)
    gh.check_steps(staged, vec, dtype, f"gate_up {act} across engines", max_steps=2 if act == "geglu" else 1, min_exact=0.85)


def run_dual(ctx, w1, w2, dtype, entry, x, consts, grid, residuals=None, norm=None):
    rows, cols = w1[0].shape[0], w1[0].shape[1] * 2
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*w1, *w2)]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, x); ctx.alloc(gh.Y_SLOT, rows * 2); ctx.alloc(gh.AUX_SLOT, rows * 2)
    if norm is not None:
        w, rs = norm
        ctx.put(RS_SLOT, rs); ctx.put(NW_SLOT, w)
        bufs = [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0)] + [(0, 3 + i, o) for i, o in enumerate(offs)] + \
               [(gh.Y_SLOT, 9, 0), (gh.AUX_SLOT, 10, 0)]
    else:
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0), (gh.AUX_SLOT, 8, 0)]
        if residuals is not None:
            ctx.put(gh.RES_SLOT, residuals[0]); ctx.put(gh.AUX2_SLOT, residuals[1])
            bufs += [(gh.RES_SLOT, 9, 0), (gh.AUX2_SLOT, 10, 0)]
    pipe = ctx.pipeline(entry + gh.t_suffix(dtype))
    assert ctx.encode_decode(rt.make_record(pipe, bufs, consts, grid, (64, 1, 1))) == 1
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows), ctx.read(gh.AUX_SLOT, np.uint16, rows).reshape(1, rows)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_dual_matvec_forms_on_the_matrix_cores(ctx, dtype):
    rows, cols, group = 1024, 2560, 128
    shape = f"c{cols}_r{rows}_g{group}"
    w1 = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=6)
    w2 = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=7)
    x = fx.synth_activation(1, cols, dtype, config=4, tensor=74)
    s1 = run_affine(ctx, *w1, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    s2 = run_affine(ctx, *w2, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    y1, y2 = run_dual(ctx, w1, w2, dtype, f"fused_dual_affine_matvec_{shape}_batched", x, [], (rows // 8, 1, 1))
    assert np.array_equal(y1, s1) and np.array_equal(y2, s2)          # the pair == two projections on this engine
    v1, _ = on_vector(ctx, lambda: run_dual(ctx, w1, w2, dtype, f"fused_dual_affine_matvec_{shape}_batched", x, [], (rows // 8, 1, 1)))
    other_engine_agrees(y1, v1, dtype, "dual matvec")
    # a residual per output: round, then add in the 16-bit type
    r1 = fx.to_bits(fx.rng_for(5, 1).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    r2 = fx.to_bits(fx.rng_for(5, 2).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    a1, a2 = run_dual(ctx, w1, w2, dtype, f"fused_dual_affine_matvec_add_{shape}_rows4", x, [], (rows // 4, 1, 1), residuals=(r1, r2))
    assert np.array_equal(a1, so.elementwise(s1[0], r1[0], dtype).reshape(1, rows))
    assert np.array_equal(a2, so.elementwise(s2[0], r2[0], dtype).reshape(1, rows))
    # norm-scale prologue in front of the pair: equals two norm-scale projections
    xr, w, rs = norm_inputs(1, cols, dtype, seed=rows)
    n1, n2 = run_dual(ctx, w1, w2, dtype, f"norm_scale_fused_dual_affine_matvec_{shape}_batched", xr, [], (rows // 8, 1, 1), norm=(w, rs))
    t1, _ = run_norm_scale_matvec(ctx, w1, xr, w, rs, dtype, f"norm_scale_affine_matvec:{cols}:{group}", [(8, rows)])
    t2, _ = run_norm_scale_matvec(ctx, w2, xr, w, rs, dtype, f"norm_scale_affine_matvec:{cols}:{group}", [(8, rows)])
    assert np.array_equal(n1, t1) and np.array_equal(n2, t2)
