"""u4_lut family (lut_matvec.metal:28-790, 967-992): oracle pins on the CPU, GPU parity against the
oracle through dispatch records."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import runtime as rt


def lut_case(seed, rows, cols, group):
    rng = fx.rng_for(130, seed)
    idx = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    ngroups = (rows + group - 1) // group
    lut = np.sort(rng.normal(0, 0.05, (ngroups, 16)).astype(np.float32), axis=1)   # k-means tables are sorted
    return idx, so.narrow(lut, so.F16)


def dense(idx, lut_bits, rows, cols, group):
    nib = np.stack([idx & 15, idx >> 4], axis=2).reshape(rows, cols)
    table = so.widen(lut_bits, so.F16)
    return table[np.arange(rows)[:, None] // group, nib]


def test_oracle_lut_matvec_against_closed_forms():
    rows, cols, group = 37, 256, 16
    idx, lut = lut_case(1, rows, cols, group)
    x = fx.rng_for(131, 0).normal(0, 1, cols).astype(np.float32)
    got = so.lut_matvec(idx, lut, x, rows, cols, group)
    exact = dense(idx, lut, rows, cols, group).astype(np.float64) @ x.astype(np.float64)
    assert np.all(np.abs(got - exact) <= 1e-5 * np.abs(exact).max())
    # an identity table turns the product into the plain sum of nibble * x: low nibble = even column
    ident = so.narrow(np.tile(np.arange(16, dtype=np.float32), ((rows + group - 1) // group, 1)), so.F16)
    e0 = np.zeros(cols, np.float32); e0[0] = 1.0
    e1 = np.zeros(cols, np.float32); e1[1] = 1.0
    assert np.array_equal(so.lut_matvec(idx, ident, e0, rows, cols, group), (idx[:, 0] & 15).astype(np.float32))
    assert np.array_equal(so.lut_matvec(idx, ident, e1, rows, cols, group), (idx[:, 0] >> 4).astype(np.float32))
    # tables belong to groups of ROWS: changing table 1 moves rows 16..31 only
    lut2 = lut.copy(); lut2[1] = so.narrow(so.widen(lut[1], so.F16) * 2, so.F16)
    got2 = so.lut_matvec(idx, lut2, x, rows, cols, group)
    assert np.array_equal(got2[:16], got[:16]) and np.array_equal(got2[32:], got[32:])
    assert np.all(np.abs(got2[16:32] - 2 * got[16:32]) <= 1e-5 * np.abs(got).max())
    assert np.array_equal(so.lut_gather(idx, lut, 20, cols, group), so.narrow(dense(idx, lut, rows, cols, group)[20], so.F16))
    assert so.epilogue_lut_add(np.float32([0.25]), so.narrow(np.float32([1.5]), so.F16), so.F16)[0] == so.narrow(np.float32([1.75]), so.F16)[0]


W, X, Y, RES, Y2, TOK = 0, 1, 2, 3, 4, 5


@pytest.fixture(scope="module", params=[fx.F16, fx.BF16], ids=["f16", "bf16"])
def env(request):
    act, odt = (rt.ACT_F16, so.F16) if request.param == fx.F16 else (rt.ACT_BF16, so.BF16)
    c = rt.Context(act_dtype=act)
    yield c, request.param, odt
    c.close()


def bits(values, dtype):
    return fx.f16_bits(values) if dtype == fx.F16 else fx.bf16_bits(values)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols,group,grid", [(9, 256, 16, None), (37, 1024, 16, None), (300, 2048, 32, None),
                                                  (1024, 4096, 64, 64), (151, 3584, 8, None), (4096, 1024, 16, 256)])
def test_lut_matvec_family(env, rows, cols, group, grid):
    ctx, dtype, odt = env
    idx, lut = lut_case(rows + cols, rows, cols, group)
    idx2, lut2 = lut_case(rows + cols + 1, rows, cols, group)
    x = bits(fx.rng_for(132, cols).normal(0, 1, cols).astype(np.float32), dtype)
    res = bits(fx.rng_for(133, rows).normal(0, 1, rows).astype(np.float32), dtype)
    xf = so.widen(x, odt)
    wf = gh.WeightFile()
    a, b, c, d = wf.add(idx), wf.add(lut), wf.add(idx2), wf.add(lut2)
    ctx.upload_weights(W, wf.image())
    ctx.put(X, x); ctx.put(RES, res); ctx.alloc(Y, rows * 2); ctx.alloc(Y2, rows * 2)
    g = (grid or (rows + 7) // 8, 1, 1)
    tg = (256, 1, 1)
    r1, r2 = so.lut_matvec(idx, lut, xf, rows, cols, group), so.lut_matvec(idx2, lut2, xf, rows, cols, group)

    def run(name, bufs, nconst):
        rec = rt.make_record(ctx.pipeline(f"{name}:{cols}:{group}"), bufs, [(nconst, rows)], g, tg)
        ctx.interpret_decode(ctx.table([rec])); ctx.wait()

    run("fused_lut_matvec", [(W, 0, a), (W, 1, b), (X, 2, 0), (Y, 3, 0)], 4)
    gh.check_outputs(ctx.read(Y, np.uint16, rows), r1, dtype, "fused_lut_matvec")
    run("fused_lut_matvec_add", [(W, 0, a), (W, 1, b), (X, 2, 0), (Y, 3, 0), (RES, 4, 0)], 5)
    # the projection is rounded before the residual is added: a sum on a rounding boundary moves the result one step
    gh.check_steps(ctx.read(Y, np.uint16, rows), so.epilogue_lut_add(r1, res, odt), dtype, "fused_lut_matvec_add", max_steps=1, min_exact=0.95)
    run("fused_dual_lut_matvec", [(W, 0, a), (W, 1, b), (W, 2, c), (W, 3, d), (X, 4, 0), (Y, 5, 0), (Y2, 6, 0)], 7)
    gh.check_outputs(ctx.read(Y, np.uint16, rows), r1, dtype, "dual output 1")
    gh.check_outputs(ctx.read(Y2, np.uint16, rows), r2, dtype, "dual output 2")
    run("fused_gate_up_swiglu", [(W, 0, a), (W, 1, b), (W, 2, c), (W, 3, d), (X, 4, 0), (Y, 5, 0)], 6)
    gh.check_outputs(ctx.read(Y, np.uint16, rows), gh.swiglu_unrounded(r1, r2), dtype, "lut gate+up+SwiGLU")


@pytest.mark.gpu
def test_lut_matmul_rows_equal_the_single_token_kernel(env):
    """fused_lut_matmul (prefill_matmul.metal:13-62): one token per grid row, constants cols, group, rows;
    every row of the output is the single-token kernel's."""
    ctx, dtype, odt = env
    rows, cols, group, tokens = 300, 1024, 16, 5
    idx, lut = lut_case(77, rows, cols, group)
    x = bits(fx.rng_for(134, 0).normal(0, 1, (tokens, cols)).astype(np.float32), dtype)
    wf = gh.WeightFile()
    a, b = wf.add(idx), wf.add(lut)
    ctx.upload_weights(W, wf.image())
    ctx.put(X, x); ctx.alloc(Y, tokens * rows * 2)
    rec = rt.make_record(ctx.pipeline("fused_lut_matmul"), [(W, 0, a), (W, 1, b), (X, 2, 0), (Y, 3, 0)],
                         [(4, cols), (5, group), (6, rows)], (rows, tokens, 1), (256, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    got = ctx.read(Y, np.uint16, tokens * rows).reshape(tokens, rows)
    for t in range(tokens):
        ctx.put(X, x[t]); ctx.alloc(Y2, rows * 2)
        one = rt.make_record(ctx.pipeline(f"fused_lut_matvec:{cols}:{group}"), [(W, 0, a), (W, 1, b), (X, 2, 0), (Y2, 3, 0)],
                             [(4, rows)], ((rows + 7) // 8, 1, 1), (256, 1, 1))
        ctx.interpret_decode(ctx.table([one])); ctx.wait()
        assert np.array_equal(got[t], ctx.read(Y2, np.uint16, rows))
        gh.check_outputs(got[t], so.lut_matvec(idx, lut, so.widen(x[t], odt), rows, cols, group), dtype, "fused_lut_matmul")


@pytest.mark.gpu
def test_lut_embedding_gather_and_bad_records(env):
    ctx, dtype, odt = env
    rows, cols, group = 100, 1024, 16
    idx, lut = lut_case(7, rows, cols, group)
    wf = gh.WeightFile()
    a, b = wf.add(idx), wf.add(lut)
    ctx.upload_weights(W, wf.image())
    ctx.alloc(Y, cols * 2)
    pipe = ctx.pipeline("lut_embedding_gather")
    for token in (0, 17, 99):
        ctx.put(TOK, np.int32([token]))
        rec = rt.make_record(pipe, [(W, 0, a), (W, 1, b), (TOK, 2, 0), (Y, 3, 0)], [(4, cols), (5, group)], (cols // 2, 1, 1), (256, 1, 1), style=rt.STYLE_THREADS)
        ctx.interpret_decode(ctx.table([rec])); ctx.wait()
        assert np.array_equal(ctx.read(Y, np.uint16, cols), so.lut_gather(idx, lut, token, cols, group))
    with pytest.raises(rt.SmeltHipError):
        ctx.pipeline("fused_lut_matvec:1000:16")           # cols not a multiple of 32
    ctx.put(X, np.zeros(cols, np.uint16))
    mv = ctx.pipeline(f"fused_lut_matvec:{cols}:{group}")
    with pytest.raises(rt.SmeltHipError):                  # more rows than the index plane holds
        ctx.interpret_decode(ctx.table([rt.make_record(mv, [(W, 0, a), (W, 1, b), (X, 2, 0), (Y, 3, 0)], [(4, rows * 40)], (8, 1, 1), (256, 1, 1))]))
