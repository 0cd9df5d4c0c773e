"""turbo_quant_h family (lut_matvec.metal:1045-1079, 9207-9486): oracle pins on the CPU (Hadamard
identities; the two-kernel matvec against the dequantised matrix, which is how the reference's own
TQHMatvecKernelTests check the kernels), and GPU parity through dispatch records on the shapes of
those tests (rows 64 x cols 256; partial final group, cols 130; FFN scale, cols 10240; batch 5)."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import runtime as rt


def tqh_case(seed, rows, cols):
    rng = fx.rng_for(140, seed)
    groups = (cols + 127) // 128
    codes = rng.integers(0, 256, (rows, groups * 32), dtype=np.uint8)
    codebook = so.narrow(np.sort(rng.normal(0, 0.1, (groups, 4)).astype(np.float32), axis=1), so.F16)
    return codes, codebook


def hadamard128():
    idx = np.arange(128)
    par = np.array([[bin(p & j).count("1") & 1 for j in idx] for p in idx])
    return np.where(par == 1, -1.0, 1.0)


def test_oracle_tqh_identities():
    h = hadamard128()
    assert np.array_equal(h @ h, 128 * np.eye(128))                       # Sylvester-Hadamard: H H = G I
    cols = 256
    x = so.narrow(fx.rng_for(141, 0).normal(0, 1, cols).astype(np.float32), so.F16)
    xhat = so.tqh_prepare(x, so.F16)
    xf = so.widen(x, so.F16).astype(np.float64)
    assert np.allclose(xhat.reshape(2, 128), (xf.reshape(2, 128) @ h), rtol=0, atol=2e-5)
    assert np.allclose((xhat.reshape(2, 128).astype(np.float64) @ h) / 128, xf.reshape(2, 128), atol=1e-5)   # rotating back
    # partial final group: columns beyond cols are zeros
    x130 = x[:130]
    xhat130 = so.tqh_prepare(x130, so.F16)
    padded = np.zeros(256); padded[:130] = xf[:130]
    assert np.allclose(xhat130.reshape(2, 128), padded.reshape(2, 128) @ h, atol=2e-5)


@pytest.mark.parametrize("rows,cols", [(64, 256), (32, 130), (16, 1280)])
def test_oracle_tqh_matvec_equals_the_dequantised_matrix(rows, cols):
    """y = W x with W[r, g*128 + p] = sum_j sign(p, j) cb[g][code_j] / sqrt(128): a missing 1/sqrt(128),
    a transposed sign index or a wrong code position breaks the equality."""
    codes, cb = tqh_case(rows + cols, rows, cols)
    x = so.narrow(fx.rng_for(142, cols).normal(0, 0.5, cols).astype(np.float32), so.F16)
    padded_cols = (cols + 127) // 128 * 128
    w = np.stack([so.tqh_dequantize_row(codes[r], cb, padded_cols) for r in range(rows)]).astype(np.float64)
    got = so.tqh_matvec(codes, cb, so.tqh_prepare(x, so.F16), rows, cols)
    xf = np.zeros(padded_cols); xf[:cols] = so.widen(x, so.F16)
    exact = w @ xf
    assert np.all(np.abs(got - exact) <= 2e-5 * np.abs(exact).max() + 1e-7)
    # independent dequant: numpy Hadamard on the looked-up entries
    g0 = so.widen(cb, so.F16)[0][((codes[0, :32, None] >> (2 * np.arange(4))) & 3).reshape(-1)]
    assert np.allclose(w[0, :128], (hadamard128() @ g0) * 0.0883883476483184405, atol=1e-6)


W, X, XH, Y, TOK = 0, 1, 2, 3, 4


@pytest.fixture(scope="module", params=[fx.F16, fx.BF16], ids=["f16", "bf16"])
def env(request):
    act, odt = (rt.ACT_F16, so.F16) if request.param == fx.F16 else (rt.ACT_BF16, so.BF16)
    c = rt.Context(act_dtype=act)
    yield c, request.param, odt
    c.close()


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols,batch", [(64, 256, 1), (32, 130, 1), (256, 10240, 1), (64, 256, 5), (256, 10240, 5), (1003, 2560, 2)])
def test_tqh_prepare_and_matvec(env, rows, cols, batch):
    ctx, dtype, odt = env
    codes, cb = tqh_case(rows * 3 + cols, rows, cols)
    groups = (cols + 127) // 128
    phase = np.arange(cols)[None, :] * 0.0731 + np.arange(batch)[:, None] * 0.137      # the reference tests' inputs
    x = (fx.f16_bits if dtype == fx.F16 else fx.bf16_bits)((np.sin(phase) * 0.5).astype(np.float32))
    wf = gh.WeightFile()
    a, b = wf.add(codes), wf.add(cb)
    ctx.upload_weights(W, wf.image())
    ctx.put(X, x); ctx.alloc(XH, batch * groups * 128 * 4); ctx.alloc(Y, batch * rows * 2)
    suffix = "_batched" if batch > 1 else ""
    prep = rt.make_record(ctx.pipeline("tqh_matvec_prepare_input" + suffix), [(X, 0, 0), (XH, 1, 0)], [(2, cols)],
                          (groups * 128, batch, 1), (128, 1, 1), style=rt.STYLE_THREADS)
    mv = rt.make_record(ctx.pipeline("tqh_matvec" + suffix), [(W, 0, a), (W, 1, b), (XH, 2, 0), (Y, 3, 0)],
                        [(4, rows), (5, cols), (6, groups * 32)], ((rows + 15) // 16, batch, 1), (256, 1, 1))
    ctx.interpret_decode(ctx.table([prep, mv])); ctx.wait()
    xhat = ctx.read(XH, np.float32, batch * groups * 128).reshape(batch, -1)
    got = ctx.read(Y, np.uint16, batch * rows).reshape(batch, rows)
    for t in range(batch):
        ref_hat = so.tqh_prepare(x[t], odt)
        assert np.array_equal(xhat[t], ref_hat)                       # same fp32 additions in the same order
        gh.check_outputs(got[t], so.tqh_matvec(codes, cb, ref_hat, rows, cols), dtype, f"tqh_matvec {rows}x{cols}")


@pytest.mark.gpu
def test_tqh_embedding_gather_and_bad_records(env):
    ctx, dtype, odt = env
    rows, cols = 50, 640
    codes, cb = tqh_case(9, rows, cols)
    wf = gh.WeightFile()
    a, b = wf.add(codes), wf.add(cb)
    ctx.upload_weights(W, wf.image())
    ctx.alloc(Y, cols * 2)
    pipe = ctx.pipeline("tqh_embedding_gather")
    for token in (0, 31, 49):
        ctx.put(TOK, np.int32([token]))
        rec = rt.make_record(pipe, [(W, 0, a), (W, 1, b), (TOK, 2, 0), (Y, 3, 0)], [(4, 5 * 32), (5, cols)], (cols, 1, 1), (128, 1, 1), style=rt.STYLE_THREADS)
        ctx.interpret_decode(ctx.table([rec])); ctx.wait()
        ref = so.narrow(so.tqh_dequantize_row(codes[token], cb, cols), odt)
        assert np.array_equal(ctx.read(Y, np.uint16, cols), ref)
    with pytest.raises(rt.SmeltHipError):       # codes_per_row that does not match the column groups
        ctx.interpret_decode(ctx.table([rt.make_record(pipe, [(W, 0, a), (W, 1, b), (TOK, 2, 0), (Y, 3, 0)], [(4, 100), (5, cols)], (cols, 1, 1), (128, 1, 1), style=rt.STYLE_THREADS)]))
