"""Norm-scale affine kernels and the GeGLU epilogue on the GPU.

The norm-scale kernels (lut_matvec.metal:1288-1575, fixed forms :2743-3170, batched :4268-4440) read
a precomputed RMS scale and normalise their input inline, x_norm = half((x * rs) * (1 + w)); the
invariant the reference leans on is that the fused kernel equals the staged pair (a norm that
stores x_norm, then the plain matvec) bit for bit.  GeGLU: lut_matvec.metal:2235-2243.
"""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
import oracle.oracle as so
from smelt_amd import runtime as rt
from test_gpu_matvec import run_affine

pytestmark = pytest.mark.gpu

RS_SLOT, NW_SLOT, XN_SLOT = 6, 7, 8


@pytest.fixture(scope="module")
def ctx():
    c = rt.Context()
    yield c
    c.close()


@pytest.fixture
def vector_ctx(ctx):
    """The module's context on the vector-ALU kernels: a fused kernel and its staged pair are bit for bit equal on
    one engine (tests/test_gpu_mm1_fused.py makes the same comparisons on the matrix cores); a per-token batched
    form runs the vector kernel whatever the engine, so comparing it with a single-token record needs this."""
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)
    yield ctx
    ctx.set_matvec_engine(rt.MATVEC_AUTO)


def norm_inputs(batch, cols, dtype, seed):
    rng = np.random.default_rng(seed)
    x = fx.to_bits(rng.normal(0, 2.0, (batch, cols)).astype(np.float32), dtype)
    w = fx.to_bits(rng.normal(0, 0.3, cols).astype(np.float32), dtype)
    rs = np.array([so.rms_scale(x[b], 1e-6, dtype) for b in range(batch)], np.float32)
    return x, w, rs


def run_norm_scale_matvec(ctx, weights, x, w, rs, dtype, entry, consts, batch_tile=None):
    packed, scales, biases = weights
    rows, cols = packed.shape[0], packed.shape[1] * 2
    batch = x.shape[0]
    wf = gh.WeightFile()
    ow, os_, ob = wf.add(packed), wf.add(scales), wf.add(biases)
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(RS_SLOT, rs)
    ctx.put(gh.X_SLOT, x)
    ctx.put(NW_SLOT, w)
    ctx.alloc(XN_SLOT, batch * cols * 2)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    bufs = [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0), (XN_SLOT, 3, 0), (0, 4, ow), (0, 5, os_), (0, 6, ob),
            (gh.Y_SLOT, 7, 0)]
    gy = batch if batch_tile is None else (batch + batch_tile - 1) // batch_tile
    pipe = ctx.pipeline(entry + gh.t_suffix(dtype))
    assert ctx.encode_decode(rt.make_record(pipe, bufs, consts, (min(1024, (rows + 7) // 8), gy, 1), (256, 1, 1))) == 1
    ctx.wait()
    return (ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows),
            ctx.read(XN_SLOT, np.uint16, batch * cols).reshape(batch, cols))


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("rows,cols,group", [(2048, 1536, 128), (777, 1056, 32), (6144, 1024, 64)])
def test_norm_scale_matvec_equals_staged_pair(vector_ctx, dtype, rows, cols, group):
    ctx = vector_ctx
    weights = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=3)
    x, w, rs = norm_inputs(1, cols, dtype, seed=rows)
    xn_ref = so.norm_scale_input(x[0], rs[0], w, dtype)
    y, xn = run_norm_scale_matvec(ctx, weights, x, w, rs, dtype, f"norm_scale_affine_matvec:{cols}:{group}", [(8, rows)])
    assert np.array_equal(xn[0], xn_ref)                     # the stored normalised row, bit for bit
    staged = run_affine(ctx, *weights, xn, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    assert np.array_equal(y, staged)                          # fused == staged
    ref = so.affine_matvec(*weights, fx.from_bits(xn_ref, dtype).reshape(1, cols), rows, cols, group, dtype)
    gh.check_outputs(y, ref, dtype, "norm_scale_affine_matvec")
    if cols % 32 == 0 and (group & (group - 1)) == 0:
        for suffix in ("_rows4", "_rows8", ""):
            y2, _ = run_norm_scale_matvec(ctx, weights, x, w, rs, dtype,
                                          f"norm_scale_affine_matvec_c{cols}_r{rows}_g{group}{suffix}", [])
            assert np.array_equal(y, y2)


@pytest.mark.parametrize("batch,tile", [(3, 8), (8, 8), (11, 8)])
def test_norm_scale_matvec_batched_rows_use_their_own_scale(vector_ctx, batch, tile):
    """Per-token scale scalePtr[token] (lut_matvec.metal:4318-4322); every row equals the batch-1 kernel (on one
    engine: under AUTO the batch-1 record of this 5M-weight matrix takes the matrix-core kernel and the token tiles
    the vector kernel, equal to one output step only)."""
    ctx = vector_ctx
    rows, cols, group, dtype = 2048, 2560, 128, fx.F16
    weights = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=1)
    x, w, rs = norm_inputs(batch, cols, dtype, seed=batch)
    y, xn = run_norm_scale_matvec(ctx, weights, x, w, rs, dtype,
                                  f"norm_scale_affine_matvec_c{cols}_r{rows}_g{group}_batched", [(8, batch)], batch_tile=tile)
    for b in range(batch):
        assert np.array_equal(xn[b], so.norm_scale_input(x[b], rs[b], w, dtype))
        y1, _ = run_norm_scale_matvec(ctx, weights, x[b:b + 1], w, rs[b:b + 1], dtype,
                                      f"norm_scale_affine_matvec:{cols}:{group}", [(8, rows)])
        assert np.array_equal(y[b], y1[0])
    # grid.y of the single-token kernel is the token index as well
    yg, xg = run_norm_scale_matvec(ctx, weights, x, w, rs, dtype, f"norm_scale_affine_matvec:{cols}:{group}", [(8, rows)])
    assert np.array_equal(yg, y) and np.array_equal(xg, xn)


def run_gate_up(ctx, gw, uw, dtype, entry, consts, x, norm=None):
    rows, cols = gw[0].shape[0], gw[0].shape[1] * 2
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.alloc(gh.Y_SLOT, rows * 2)
    if norm is None:
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
    else:
        w, rs = norm
        ctx.put(RS_SLOT, rs)
        ctx.put(NW_SLOT, w)
        bufs = [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0)] + [(0, 3 + i, o) for i, o in enumerate(offs)] + \
               [(gh.Y_SLOT, 9, 0)]
    pipe = ctx.pipeline(entry + gh.t_suffix(dtype))
    assert ctx.encode_decode(rt.make_record(pipe, bufs, consts, (512, 1, 1), (256, 1, 1))) == 1
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("act", ["swiglu", "geglu"])
def test_norm_scale_gate_up_equals_staged_pair(vector_ctx, dtype, act):
    ctx = vector_ctx
    rows, cols, group = 3584, 1024, 64
    gw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=4)
    uw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=5)
    x, w, rs = norm_inputs(1, cols, dtype, seed=17)
    xn = so.norm_scale_input(x[0], rs[0], w, dtype).reshape(1, cols)
    fused = run_gate_up(ctx, gw, uw, dtype, f"norm_scale_affine_gate_up_{act}:{cols}:{group}", [(10, rows)], x, norm=(w, rs))
    staged = run_gate_up(ctx, gw, uw, dtype, f"fused_affine_gate_up_{act}:{cols}:{group}", [(8, rows)], xn)
    assert np.array_equal(fused, staged)
    fixed = run_gate_up(ctx, gw, uw, dtype, f"norm_scale_affine_gate_up_{act}_c{cols}_r{rows}_g{group}_rows4", [], x, norm=(w, rs))
    assert np.array_equal(fused, fixed)
    xf = fx.from_bits(xn, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, group, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, group, dtype)
    epi = so.epilogue_affine_swiglu if act == "swiglu" else so.epilogue_geglu
    if act == "swiglu":
        gh.check_outputs(fused, gh.swiglu_unrounded(g, u), dtype, f"norm_scale gate_up {act}")
    else:   # GeGLU rounds gate and up to the 16-bit type before the activation: counted in output steps
        gh.check_steps(fused, epi(g, u, dtype).reshape(np.shape(fused)), dtype, f"norm_scale gate_up {act}", max_steps=gh.GEGLU_STEPS)


def test_geglu_fixed_name_and_clamps(ctx):
    """Large gates saturate tanh (argument clamped to +-20) and the product is clamped to +-65504."""
    rows, cols, group, dtype = 512, 1024, 64, fx.F16
    gw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=6)
    uw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=7)
    x = fx.to_bits(np.full((1, cols), 30.0, np.float32) * np.where(np.arange(cols) % 2, 1.0, 0.75), dtype)
    y = run_gate_up(ctx, gw, uw, dtype, f"fused_affine_gate_up_geglu_c{cols}_r{rows}_g{group}_rows4", [], x)
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, group, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, group, dtype)
    assert np.abs(g).max() > 30                                  # the clamp region is exercised
    ref_bits = so.epilogue_geglu(g, u, dtype)
    got = fx.from_bits(y, dtype).ravel().astype(np.float64)
    ref = fx.from_bits(ref_bits, dtype).ravel().astype(np.float64)
    assert np.isfinite(got).all() and np.abs(got).max() <= 65504
    tol = 4e-3 * np.maximum(np.abs(ref), np.abs(ref).max() * 2.0 ** -6) + gh.ulp_of(ref, dtype)
    assert (np.abs(got - ref) <= tol).all()


def test_norm_scale_launches_are_validated(ctx):
    rows, cols, group, dtype = 256, 1024, 64, fx.F16
    weights = fx.synth_affine(rows, cols, group, dtype, config=0, tensor=0)
    x, w, rs = norm_inputs(1, cols, dtype, seed=5)
    wf = gh.WeightFile()
    ow, os_, ob = wf.add(weights[0]), wf.add(weights[1]), wf.add(weights[2])
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(RS_SLOT, rs); ctx.put(gh.X_SLOT, x); ctx.put(NW_SLOT, w)
    ctx.alloc(XN_SLOT, cols * 2 - 64)                             # too small for the normalised row
    ctx.alloc(gh.Y_SLOT, rows * 2)
    bufs = [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0), (XN_SLOT, 3, 0), (0, 4, ow), (0, 5, os_), (0, 6, ob),
            (gh.Y_SLOT, 7, 0)]
    pipe = ctx.pipeline(f"norm_scale_affine_matvec:{cols}:{group}")
    with pytest.raises(rt.SmeltHipError):
        ctx.encode_decode(rt.make_record(pipe, bufs, [(8, rows)], (32, 1, 1), (256, 1, 1)))
    # forms that are not built fail to resolve instead of running something else
    for name in (f"norm_scale_affine_matvec_c{cols}_r{rows}_g{group}_batched_skinny",
                 f"norm_scale_affine_gate_up_swiglu_c{cols}_r{rows}_g{group}_batched",
                 f"fused_affine_gate_up_geglu_c{cols}_r{rows}_g{group}_batched_tile4"):
        with pytest.raises(rt.SmeltHipError):
            ctx.pipeline(name)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_emitted_scale_only_plus_norm_scale_pair_equals_norm_then_matvec(dtype):
    """The pair the reference emits (rms_norm_scale_only, then the norm-scale kernel;
    SmeltCodeEmitter.swift:2680-2754) against the unfused records: same projection bits, and the
    stored normalised row is the oracle's."""
    from smelt_amd import compiler as cc
    hidden, rows, ffn, group = 1536, 2048, 6144, 128
    lay = cc.Layout()
    wq, wg, wu = lay.affine(rows, hidden, group), lay.affine(ffn, hidden, group), lay.affine(ffn, hidden, group)
    image = np.zeros(lay.total_bytes, np.uint8)
    for i, e in enumerate((wq, wg, wu)):
        cc.write_affine(image, e, *fx.synth_affine(e.rows, e.cols, group, dtype, config=1, tensor=40 + i))
    X, NW, SCALE, XN, Q, F1, F2, Q2, F3 = range(1, 10)
    act = rt.ACT_BF16 if dtype == fx.BF16 else rt.ACT_F16
    em = cc.Emitter(act)
    em.rms_norm_scale_only(cc.bind(X), cc.bind(SCALE), hidden)
    em.norm_scale_matvec(0, wq, cc.bind(SCALE), cc.bind(X), cc.bind(NW), cc.bind(XN), cc.bind(Q))
    em.norm_scale_gate_up(0, wg, wu, cc.bind(SCALE), cc.bind(X), cc.bind(NW), cc.bind(F1))
    em.norm_scale_gate_up(0, wg, wu, cc.bind(SCALE), cc.bind(X), cc.bind(NW), cc.bind(F2), geglu=True)
    # unfused: plain matvec / gate+up on the stored normalised row
    em.matvec(0, wq, cc.bind(XN), cc.bind(Q2))
    em.gate_up_swiglu(0, wg, wu, cc.bind(XN), cc.bind(F3))
    # norm inside the consumer (one dispatch each)
    XN2, Q3, F4, SCR = 10, 11, 12, 13
    em.fused_norm_matvec(0, wq, cc.bind(X), cc.bind(NW), cc.bind(Q3), cc.bind(SCR), norm_output=cc.bind(XN2))
    em.fused_norm_matvec(0, wg, cc.bind(X), cc.bind(NW), cc.bind(F4), cc.bind(SCR), up=wu)
    ctx = rt.Context(act_dtype=act)
    try:
        # fused == unfused bit for bit holds between kernels of one engine: the norm-scale prologue
        # exists on the vector-ALU kernels only, so the unfused records are kept there as well
        ctx.set_matvec_engine(rt.MATVEC_VECTOR)
        em.install(ctx)
        ctx.upload_weights(0, image)
        x, w, _ = norm_inputs(1, hidden, dtype, seed=3)
        ctx.put(X, x); ctx.put(NW, w)
        ctx.alloc(SCALE, 4); ctx.alloc(XN, hidden * 2)
        for slot, n in ((Q, rows), (Q2, rows), (F1, ffn), (F2, ffn), (F3, ffn), (XN2, hidden), (Q3, rows), (F4, ffn)):
            ctx.alloc(slot, n * 2)
        ctx.alloc(SCR, 8)
        assert ctx.interpret_decode(em.records()) == 8
        ctx.wait()
        rs = float(ctx.read(SCALE, np.float32, 1)[0])
        assert abs(rs - so.rms_scale(x[0], 1e-6, dtype)) <= 5e-6 * rs
        assert np.array_equal(ctx.read(XN, np.uint16, hidden), so.norm_scale_input(x[0], rs, w, dtype))
        assert np.array_equal(ctx.read(Q, np.uint16, rows), ctx.read(Q2, np.uint16, rows))
        assert np.array_equal(ctx.read(F1, np.uint16, ffn), ctx.read(F3, np.uint16, ffn))
        assert np.abs(fx.from_bits(ctx.read(F2, np.uint16, ffn), dtype)).max() > 0
        # the in-kernel scale is summed in another order than rms_norm_scale_only's: last-place agreement
        rs2 = float(ctx.read(SCR, np.float32, 1)[0])
        assert abs(rs2 - rs) <= 2e-6 * rs and ctx.read(SCR, np.uint32, 2)[1] == 1
        assert np.array_equal(ctx.read(XN2, np.uint16, hidden), so.norm_scale_input(x[0], rs2, w, dtype))
        # the consumer forms the norm scale itself (another summation order): a staged activation can sit one
        # step of the 16-bit type away, which moves an output by whole steps too
        gh.check_steps(ctx.read(Q3, np.uint16, rows).reshape(1, rows), ctx.read(Q, np.uint16, rows).reshape(1, rows),
                       dtype, "fused norm matvec against the pair", max_steps=2, min_exact=0.9)
        gh.check_steps(ctx.read(F4, np.uint16, ffn).reshape(1, ffn), ctx.read(F1, np.uint16, ffn).reshape(1, ffn),
                       dtype, "fused norm gate+up against the pair", max_steps=2, min_exact=0.9)
    finally:
        ctx.close()


def run_qmm(ctx, entry, dtype, batch, bufs_fn, rows, grid_w, bt, batch_index, launches=1):
    pipe = ctx.pipeline(entry + gh.t_suffix(dtype))
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    rec = rt.make_record(pipe, bufs_fn(), [(batch_index, batch)], (grid_w, (batch + bt - 1) // bt, 1), (256, 1, 1))
    assert ctx.encode_decode(rec) == launches
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("batch,suffix,bt", [(14, "_batched_full", 16), (37, "_batched_full", 16), (70, "_batched_full_b64", 64)])
def test_norm_scale_qmm_equals_plain_qmm_on_the_stored_rows(ctx, dtype, batch, suffix, bt):
    """agent_norm_scale_affine_qmm_fixed_batched_full (lut_matvec.metal:8496-8530): per-token scales,
    normalised rows stored, and the product equal to the plain qmm run on those rows bit for bit
    (the plain record kept on the token-slab kernel the fused form shares its tile code with)."""
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)
    rows, cols, group = 1000, 1024, 64
    weights = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=2)
    x, w, rs = norm_inputs(batch, cols, dtype, seed=batch)
    wf = gh.WeightFile()
    ow, os_, ob = (wf.add(a) for a in weights)
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(RS_SLOT, rs); ctx.put(gh.X_SLOT, x); ctx.put(NW_SLOT, w)
    ctx.alloc(XN_SLOT, batch * cols * 2)
    shape = f"_c{cols}_r{rows}_g{group}"
    fused = run_qmm(ctx, "norm_scale_affine_matvec" + shape + suffix, dtype, batch,
                    lambda: [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0), (XN_SLOT, 3, 0), (0, 4, ow), (0, 5, os_),
                             (0, 6, ob), (gh.Y_SLOT, 7, 0)], rows, (rows + 63) // 64, bt, 8)
    xn = ctx.read(XN_SLOT, np.uint16, batch * cols).reshape(batch, cols)
    for b in range(batch):
        assert np.array_equal(xn[b], so.norm_scale_input(x[b], rs[b], w, dtype)), b
    ctx.put(gh.X_SLOT, xn)
    staged = run_qmm(ctx, "affine_matvec" + shape + suffix, dtype, batch,
                     lambda: [(0, 0, ow), (0, 1, os_), (0, 2, ob), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)],
                     rows, (rows + 63) // 64, bt, 5)
    ctx.set_matvec_engine(rt.MATVEC_AUTO)
    assert np.array_equal(fused, staged)
    ref = so.affine_matvec(*weights, fx.from_bits(xn, dtype), rows, cols, group, dtype)
    gh.check_outputs(fused, ref, dtype, "norm_scale qmm")


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("batch,suffix,bt,rows,cols", [(14, "_batched_full", 16, 1000, 1024), (140, "_batched_full_b64", 64, 2100, 2560),
                                                       (3, "_batched", 8, 1000, 1024), (37, "_batched_full", 16, 200, 11008)])
def test_norm_scale_qmm_under_the_default_engine_is_the_staged_pair(ctx, dtype, batch, suffix, bt, rows, cols):
    """Under AUTO the norm-scale qmm records (token-slab and per-token small-batch names) run as two launches: the
    normalised rows (stored to the record's output, the bits of a staged norm), then the streaming or token-tile
    kernel of the plain record (140 tokens of a 5.4M-weight matrix: token tiles).  Equal bit for bit to the plain
    record run on the stored rows, which takes the same kernel."""
    group = 64
    weights = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=2)
    x, w, rs = norm_inputs(batch, cols, dtype, seed=batch)
    wf = gh.WeightFile()
    ow, os_, ob = (wf.add(a) for a in weights)
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(RS_SLOT, rs); ctx.put(gh.X_SLOT, x); ctx.put(NW_SLOT, w)
    ctx.alloc(XN_SLOT, batch * cols * 2)
    shape = f"_c{cols}_r{rows}_g{group}"
    grid_w = (rows + 63) // 64 if "full" in suffix else min(1024, (rows + 7) // 8)
    fused = run_qmm(ctx, "norm_scale_affine_matvec" + shape + suffix, dtype, batch,
                    lambda: [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0), (XN_SLOT, 3, 0), (0, 4, ow), (0, 5, os_),
                             (0, 6, ob), (gh.Y_SLOT, 7, 0)], rows, grid_w, bt, 8, launches=2)
    xn = ctx.read(XN_SLOT, np.uint16, batch * cols).reshape(batch, cols)
    for b in range(batch):
        assert np.array_equal(xn[b], so.norm_scale_input(x[b], rs[b], w, dtype)), b
    ctx.put(gh.X_SLOT, xn)
    plain = "_batched_full" if suffix == "_batched" else suffix     # (three tokens of a 1M-weight matrix stream either way)
    staged = run_qmm(ctx, "affine_matvec" + shape + plain, dtype, batch,
                     lambda: [(0, 0, ow), (0, 1, os_), (0, 2, ob), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)],
                     rows, (rows + 63) // 64, 16 if plain == "_batched_full" else bt, 5)
    assert np.array_equal(fused, staged)
    ref = so.affine_matvec(*weights, fx.from_bits(xn, dtype), rows, cols, group, dtype, threads=True)
    gh.check_outputs(fused, ref, dtype, "norm_scale qmm, default engine")


@pytest.mark.parametrize("act", ["swiglu", "geglu"])
def test_norm_scale_gate_up_qmm_and_geglu_qmm(ctx, act):
    rows, cols, group, dtype, batch, bt = 640, 1024, 64, fx.F16, 21, 16
    gw = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=3)
    uw = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=4)
    x, w, rs = norm_inputs(batch, cols, dtype, seed=77)
    xn = np.stack([so.norm_scale_input(x[b], rs[b], w, dtype) for b in range(batch)])
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(RS_SLOT, rs); ctx.put(gh.X_SLOT, x); ctx.put(NW_SLOT, w)
    shape = f"_c{cols}_r{rows}_g{group}_batched_full"
    # on either engine the fused record equals the staged pair bit for bit: under AUTO two launches (the normalised rows
    # into the workspace, then the streaming kernel of the plain gate+up), under VECTOR the token-slab kernel both share
    for engine, launches in ((rt.MATVEC_AUTO, 2), (rt.MATVEC_VECTOR, 1)):
        ctx.set_matvec_engine(engine)
        try:
            ctx.put(gh.X_SLOT, x)
            fused = run_qmm(ctx, f"norm_scale_affine_gate_up_{act}" + shape, dtype, batch,
                            lambda: [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0)] + [(0, 3 + i, o) for i, o in enumerate(offs)] +
                                    [(gh.Y_SLOT, 9, 0)], rows, (rows + 63) // 64, bt, 10, launches=launches)
            ctx.put(gh.X_SLOT, xn)
            staged = run_qmm(ctx, f"fused_affine_gate_up_{act}" + shape, dtype, batch,
                             lambda: [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)],
                             rows, (rows + 63) // 64, bt, 8)
        finally:
            ctx.set_matvec_engine(rt.MATVEC_AUTO)
        assert np.array_equal(fused, staged), engine
    xf = fx.from_bits(xn, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, group, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, group, dtype)
    epi = so.epilogue_affine_swiglu if act == "swiglu" else so.epilogue_geglu
    if act == "swiglu":
        gh.check_outputs(fused, gh.swiglu_unrounded(g, u), dtype, f"gate_up {act} qmm")
    else:
        gh.check_steps(fused, epi(g, u, dtype).reshape(np.shape(fused)), dtype, f"gate_up {act} qmm", max_steps=gh.GEGLU_STEPS)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_norm_add_scale_matvec(ctx, dtype):
    """norm_add_scale_affine_matvec_c2560_r256_g128_rows4 (lut_matvec.metal:2896-3040): the row the
    matvec multiplies, and stores, is half(half(norm) + residual)."""
    rows, cols, group = 256, 2560, 128
    weights = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=5)
    x, w, rs = norm_inputs(1, cols, dtype, seed=41)
    res = fx.to_bits(np.random.default_rng(42).normal(0, 1, (1, cols)).astype(np.float32), dtype)
    normed = so.norm_scale_input(x[0], rs[0], w, dtype)
    row_ref = so.elementwise(normed, res[0], dtype)
    wf = gh.WeightFile()
    ow, os_, ob = (wf.add(a) for a in weights)
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(RS_SLOT, rs); ctx.put(gh.X_SLOT, x); ctx.put(NW_SLOT, w); ctx.put(gh.RES_SLOT, res)
    ctx.alloc(XN_SLOT, cols * 2); ctx.alloc(gh.Y_SLOT, rows * 2)
    bufs = [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0), (gh.RES_SLOT, 3, 0), (XN_SLOT, 4, 0), (0, 5, ow), (0, 6, os_),
            (0, 7, ob), (gh.Y_SLOT, 8, 0)]
    pipe = ctx.pipeline(f"norm_add_scale_affine_matvec_c{cols}_r{rows}_g{group}_rows4" + gh.t_suffix(dtype))
    assert ctx.encode_decode(rt.make_record(pipe, bufs, [], (rows // 4, 1, 1), (64, 1, 1))) == 1
    ctx.wait()
    row = ctx.read(XN_SLOT, np.uint16, cols)
    y = ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows)
    assert np.array_equal(row, row_ref)
    staged = run_affine(ctx, *weights, row.reshape(1, cols), dtype, f"affine_matvec:{cols}:{group}", generic=True)
    assert np.array_equal(y, staged)
    ref = so.affine_matvec(*weights, fx.from_bits(row_ref, dtype).reshape(1, cols), rows, cols, group, dtype)
    gh.check_outputs(y, ref, dtype, "norm_add_scale_affine_matvec")


@pytest.mark.parametrize("rows", [512, 1024])
def test_norm_scale_dual_matvec_per_token(ctx, rows):
    """norm_scale_fused_dual_affine_matvec_c2560_r{512,1024}_g128_batched (lut_matvec.metal:2030-2150):
    grid.y is the token, scalePtr[token] its scale; both outputs equal single norm-scale matvecs."""
    cols, group, dtype, batch = 2560, 128, fx.F16, 3
    w1 = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=6)
    w2 = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=7)
    x, w, rs = norm_inputs(batch, cols, dtype, seed=rows)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*w1, *w2)]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(RS_SLOT, rs); ctx.put(gh.X_SLOT, x); ctx.put(NW_SLOT, w)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2); ctx.alloc(gh.AUX_SLOT, batch * rows * 2)
    bufs = [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0)] + [(0, 3 + i, o) for i, o in enumerate(offs)] + \
           [(gh.Y_SLOT, 9, 0), (gh.AUX_SLOT, 10, 0)]
    pipe = ctx.pipeline(f"norm_scale_fused_dual_affine_matvec_c{cols}_r{rows}_g{group}_batched")
    assert ctx.encode_decode(rt.make_record(pipe, bufs, [], (rows // 8, batch, 1), (64, 1, 1))) == 1
    ctx.wait()
    y1 = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    y2 = ctx.read(gh.AUX_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    s1, _ = run_norm_scale_matvec(ctx, w1, x, w, rs, dtype, f"norm_scale_affine_matvec:{cols}:{group}", [(8, rows)])
    s2, _ = run_norm_scale_matvec(ctx, w2, x, w, rs, dtype, f"norm_scale_affine_matvec:{cols}:{group}", [(8, rows)])
    assert np.array_equal(y1, s1) and np.array_equal(y2, s2)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("threads", [64, 256])
def test_norm_fused_into_matvec_and_gate_up(vector_ctx, dtype, threads):
    """atomic_norm_affine_matvec / _gate_up_swiglu (fused_norm_matvec.metal:19-297): the norm's scale is
    computed inside the consumer.  The scale lands in scratch[0] with the ready flag in scratch[1]; the
    stored row and the products equal the scale-only + norm-scale pair run with that scale."""
    ctx = vector_ctx
    rows, cols, group = 1024, 2048, 64
    weights = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=8)
    uw = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=9)
    x, w, _ = norm_inputs(1, cols, dtype, seed=threads)
    SCR = 9
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*weights, *uw)]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, x); ctx.put(NW_SLOT, w)
    ctx.alloc(XN_SLOT, cols * 2); ctx.alloc(gh.Y_SLOT, rows * 2); ctx.alloc(SCR, 8)
    bufs = [(gh.X_SLOT, 0, 0), (NW_SLOT, 1, 0), (XN_SLOT, 2, 0), (0, 3, offs[0]), (0, 4, offs[1]), (0, 5, offs[2]),
            (gh.Y_SLOT, 6, 0), (SCR, 7, 0)]
    pipe = ctx.pipeline(f"atomic_norm_affine_matvec:{cols}:{group}" + gh.t_suffix(dtype))
    assert ctx.encode_decode(rt.make_record(pipe, bufs, [(8, rows), (9, 1e-6)], (rows // 8, 1, 1), (threads, 1, 1))) == 1
    ctx.wait()
    scratch = ctx.read(SCR, np.uint32, 2)
    rs = float(scratch[:1].view(np.float32)[0])
    assert scratch[1] == 1
    ref_rs = so.rms_scale(x[0], 1e-6, dtype)
    assert abs(rs - ref_rs) <= 5e-6 * ref_rs
    xn = ctx.read(XN_SLOT, np.uint16, cols)
    assert np.array_equal(xn, so.norm_scale_input(x[0], rs, w, dtype))
    y = ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows)
    staged = run_affine(ctx, *weights, xn.reshape(1, cols), dtype, f"affine_matvec:{cols}:{group}", generic=True)
    assert np.array_equal(y, staged)
    # gate + up + SwiGLU with the norm inside
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())      # run_affine replaced the image
    ctx.put(gh.X_SLOT, x); ctx.alloc(gh.Y_SLOT, rows * 2); ctx.alloc(SCR, 8)
    bufs = [(gh.X_SLOT, 0, 0), (NW_SLOT, 1, 0)] + [(0, 2 + i, o) for i, o in enumerate(offs)] + [(gh.Y_SLOT, 8, 0), (SCR, 9, 0)]
    pipe = ctx.pipeline(f"atomic_norm_affine_gate_up_swiglu:{cols}:{group}" + gh.t_suffix(dtype))
    assert ctx.encode_decode(rt.make_record(pipe, bufs, [(10, rows), (11, 1e-6)], (rows // 8, 1, 1), (threads, 1, 1))) == 1
    ctx.wait()
    fused = ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows)
    assert ctx.read(SCR, np.uint32, 2)[1] == 1
    staged = run_gate_up(ctx, weights, uw, dtype, f"fused_affine_gate_up_swiglu:{cols}:{group}", [(8, rows)], xn.reshape(1, cols))
    assert np.array_equal(fused, staged)


def test_dual_matvec_per_token_and_small_batch_geglu(vector_ctx):
    """fused_dual_affine_matvec_*_batched (lut_matvec.metal:7570-7591: grid.y = token) and the
    small-batch GeGLU kernels (:8342-8364, token tiles of 3 and 4): per-token results are the
    single-token kernels' bits."""
    ctx = vector_ctx
    rows, cols, group, dtype, batch = 512, 1024, 64, fx.F16, 5
    w1 = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=10)
    w2 = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=11)
    x = fx.synth_activation(batch, cols, dtype, config=1, tensor=72)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*w1, *w2)]
    image = wf.image()
    ctx.upload_weights(gh.WEIGHTS_SLOT, image)
    ctx.put(gh.X_SLOT, x); ctx.alloc(gh.Y_SLOT, batch * rows * 2); ctx.alloc(gh.AUX_SLOT, batch * rows * 2)
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0), (gh.AUX_SLOT, 8, 0)]
    pipe = ctx.pipeline(f"fused_dual_affine_matvec_c{cols}_r{rows}_g{group}_batched")
    assert ctx.encode_decode(rt.make_record(pipe, bufs, [], (rows // 8, batch, 1), (64, 1, 1))) == 1
    ctx.wait()
    y1 = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    y2 = ctx.read(gh.AUX_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    s1 = run_affine(ctx, *w1, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    s2 = run_affine(ctx, *w2, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    assert np.array_equal(y1, s1) and np.array_equal(y2, s2)
    single = np.stack([run_gate_up(ctx, w1, w2, dtype, f"fused_affine_gate_up_geglu:{cols}:{group}", [(8, rows)], x[b:b + 1])[0]
                       for b in range(batch)])
    for suffix, bt in (("_batched", 3), ("_batched_bt4_sg4", 4)):
        ctx.upload_weights(gh.WEIGHTS_SLOT, image)
        ctx.put(gh.X_SLOT, x); ctx.alloc(gh.Y_SLOT, batch * rows * 2)
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
        pipe = ctx.pipeline(f"fused_affine_gate_up_geglu_c{cols}_r{rows}_g{group}{suffix}")
        assert ctx.encode_decode(rt.make_record(pipe, bufs, [(8, batch)], (rows // 8, (batch + bt - 1) // bt, 1), (256, 1, 1))) == 1
        ctx.wait()
        assert np.array_equal(ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows), single), suffix


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_generated_small_batch_and_dual_add_names(vector_ctx, dtype):
    """The compiler's generated variants (SmeltGeneratedKernelVariants.swift:17-35, 66-68):
    `_batched_verify_b4` forms of the matvec, gate+up+SwiGLU and dual matvec (token tiles of 4, the token
    count at the binding after the outputs; lut_matvec.metal:3816-3922) and the decode dual matvec with two
    residuals (`fused_dual_affine_matvec_add_*_rows4`, :4660-4733).  Per token they are the single-token
    kernels' bits; the residual form is checked against the oracle's round-then-add."""
    ctx = vector_ctx
    rows, cols, group, batch = 264, 1024, 64, 6
    w1 = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=20)
    w2 = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=21)
    x = fx.synth_activation(batch, cols, dtype, config=1, tensor=73)
    s1 = run_affine(ctx, *w1, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    s2 = run_affine(ctx, *w2, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)
    shape = f"c{cols}_r{rows}_g{group}"
    tiles = (batch + 3) // 4

    got = run_affine(ctx, *w1, x, dtype, f"affine_matvec_{shape}_batched_verify_b4", batched=True, batch_tile=4)
    assert np.array_equal(got, s1)

    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*w1, *w2)]
    image = wf.image()
    weights = [(0, i, o) for i, o in enumerate(offs)]

    # gate+up+SwiGLU, tiles of 4 tokens against the single-token fused kernel
    single = np.stack([run_gate_up(ctx, w1, w2, dtype, f"fused_affine_gate_up_swiglu:{cols}:{group}", [(8, rows)], x[b:b + 1])[0]
                       for b in range(batch)])
    ctx.upload_weights(gh.WEIGHTS_SLOT, image)
    ctx.put(gh.X_SLOT, x); ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    pipe = ctx.pipeline(f"fused_affine_gate_up_swiglu_{shape}_batched_verify_b4" + gh.t_suffix(dtype))
    rec = rt.make_record(pipe, weights + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)], [(8, batch)], ((rows + 7) // 8, tiles, 1), (64, 1, 1))
    assert ctx.encode_decode(rec) == 1
    ctx.wait()
    assert np.array_equal(ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows), single)

    # dual matvec, tiles of 4 tokens; a grid one tile short is refused
    ctx.alloc(gh.Y_SLOT, batch * rows * 2); ctx.alloc(gh.AUX_SLOT, batch * rows * 2)
    pipe = ctx.pipeline(f"fused_dual_affine_matvec_{shape}_batched_verify_b4" + gh.t_suffix(dtype))
    bufs = weights + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0), (gh.AUX_SLOT, 8, 0)]
    assert ctx.encode_decode(rt.make_record(pipe, bufs, [(9, batch)], ((rows + 7) // 8, tiles, 1), (64, 1, 1))) == 1
    ctx.wait()
    assert np.array_equal(ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows), s1)
    assert np.array_equal(ctx.read(gh.AUX_SLOT, np.uint16, batch * rows).reshape(batch, rows), s2)
    with pytest.raises(rt.SmeltHipError):
        ctx.encode_decode(rt.make_record(pipe, bufs, [(9, batch)], ((rows + 7) // 8, tiles - 1, 1), (64, 1, 1)))

    # decode dual matvec with a residual per output (each output may alias its residual)
    r1 = fx.to_bits(fx.rng_for(5, 1).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    r2 = fx.to_bits(fx.rng_for(5, 2).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    ctx.put(gh.X_SLOT, x[:1]); ctx.put(gh.Y_SLOT, r1); ctx.alloc(gh.AUX_SLOT, rows * 2); ctx.put(gh.AUX2_SLOT, r2)
    pipe = ctx.pipeline(f"fused_dual_affine_matvec_add_{shape}_rows4" + gh.t_suffix(dtype))
    bufs = weights + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0), (gh.AUX_SLOT, 8, 0), (gh.Y_SLOT, 9, 0), (gh.AUX2_SLOT, 10, 0)]
    assert ctx.encode_decode(rt.make_record(pipe, bufs, [], (rows // 4, 1, 1), (64, 1, 1))) == 1
    ctx.wait()
    odt = so.F16 if dtype == fx.F16 else so.BF16
    xf = fx.from_bits(x[:1], dtype)
    a1 = so.affine_matvec(*w1, xf, rows, cols, group, dtype)
    a2 = so.affine_matvec(*w2, xf, rows, cols, group, dtype)
    y1 = ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows)
    y2 = ctx.read(gh.AUX_SLOT, np.uint16, rows).reshape(1, rows)
    # the projections agree with the oracle to tolerance; rounded to the activation type and added to the residual
    # in that type they are the fused kernel's bits (the oracle's epilogue on the GPU's own projections)
    gh.check_outputs(s1[:1], a1, dtype, "dual, first projection")
    gh.check_outputs(s2[:1], a2, dtype, "dual, second projection")
    assert np.array_equal(y1, so.epilogue_residual_add(fx.from_bits(s1[:1], dtype), r1, odt))
    assert np.array_equal(y2, so.epilogue_residual_add(fx.from_bits(s2[:1], dtype), r2, odt))


def test_two_launch_routes_replay_in_a_graph(ctx):
    """A captured table of records that the default engine runs as several launches (a norm-scale qmm: normalised rows
    plus the streaming kernel; a norm-scale gate+up, whose rows live in the context workspace) replayed three times
    with new inputs in between: every replay equals the eager result."""
    rows, cols, group, dtype, batch = 640, 1024, 64, fx.BF16, 11
    weights = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=2)
    gw = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=3)
    uw = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=4)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*weights, *gw, *uw)]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    F2 = 12
    ctx.alloc(XN_SLOT, batch * cols * 2); ctx.alloc(gh.Y_SLOT, batch * rows * 2); ctx.alloc(F2, batch * rows * 2)
    shape = f"_c{cols}_r{rows}_g{group}_batched_full"
    t = gh.t_suffix(dtype)
    r1 = rt.make_record(ctx.pipeline("norm_scale_affine_matvec" + shape + t),
                        [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0), (XN_SLOT, 3, 0)] + [(0, 4 + i, offs[i]) for i in range(3)] +
                        [(gh.Y_SLOT, 7, 0)], [(8, batch)], ((rows + 63) // 64, 1, 1), (256, 1, 1))
    r2 = rt.make_record(ctx.pipeline("norm_scale_affine_gate_up_swiglu" + shape + t),
                        [(RS_SLOT, 0, 0), (gh.X_SLOT, 1, 0), (NW_SLOT, 2, 0)] + [(0, 3 + i, offs[3 + i]) for i in range(6)] + [(F2, 9, 0)],
                        [(10, batch)], ((rows + 63) // 64, 1, 1), (256, 1, 1))
    table = ctx.table([r1, r2])
    x0, w0, rs0 = norm_inputs(batch, cols, dtype, seed=5)
    ctx.put(RS_SLOT, rs0); ctx.put(gh.X_SLOT, x0); ctx.put(NW_SLOT, w0)
    graph, n = ctx.capture_decode(table)
    assert n == 4
    try:
        for seed in (6, 7, 8):
            x, w, rs = norm_inputs(batch, cols, dtype, seed=seed)
            ctx.put(RS_SLOT, rs); ctx.put(gh.X_SLOT, x); ctx.put(NW_SLOT, w)
            assert ctx.interpret_decode(table) == 4
            ctx.wait()
            eager = (ctx.read(gh.Y_SLOT, np.uint16, batch * rows).copy(), ctx.read(F2, np.uint16, batch * rows).copy())
            ctx.put(gh.Y_SLOT, np.zeros(batch * rows, np.uint16)); ctx.put(F2, np.zeros(batch * rows, np.uint16))
            ctx.graph_launch(graph); ctx.wait()
            assert np.array_equal(ctx.read(gh.Y_SLOT, np.uint16, batch * rows), eager[0]), seed
            assert np.array_equal(ctx.read(F2, np.uint16, batch * rows), eager[1]), seed
            assert np.abs(fx.from_bits(eager[0], dtype)).max() > 0
    finally:
        ctx.graph_destroy(graph)
