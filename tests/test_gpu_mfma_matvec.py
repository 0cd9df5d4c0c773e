"""GPU parity: the matrix-core matvec variants ("_mfma" pipeline names, affine u4 g64, matrices of 8M
weights and more): every K-split (1, 2, 4 waves per row tile), ragged row tiles, 1..8 and
more than 8 tokens, the fused epilogues, and agreement with the vector-ALU kernels."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import compiler as cc
from smelt_amd import runtime as rt
from test_gpu_matvec import run_affine

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = rt.Context()
    yield c
    c.close()


def mm_symbol(entry):
    rc, sym, kinds = cc.resolve_pipeline_name(entry)
    assert rc == 0, entry
    return sym


# rows chosen so that the row-tile count selects 4, 2 and 1 waves per tile; none is a multiple of 32
SHAPES = [(8200, 1024, 4), (33000, 512, 2), (70001, 256, 1), (5000, 2560, 4)]


@pytest.mark.parametrize("rows,cols,kw", SHAPES)
@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_mfma_matvec_matches_oracle(ctx, rows, cols, kw, dtype):
    entry = f"affine_matvec_c{cols}_r{rows}_g64_mfma"
    assert mm_symbol(entry) == f"smelt_affine_mm_matvec_{'stream' if kw == 1 else 'split'}_f16"
    w = fx.synth_affine(rows, cols, 64, dtype, config=1, tensor=60 + kw)
    x = fx.synth_activation(1, cols, dtype, config=1, tensor=61, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    y = run_affine(ctx, *w, x, dtype, entry, grid=1024)
    worst = gh.check_outputs(y, ref, dtype, f"mfma matvec {rows}x{cols}")
    print(f"\n  mfma matvec {rows}x{cols} kw={kw} dtype={dtype}: max rel err {worst:.2e}")
    # any grid covers every row; the generic entry runs the vector-ALU kernel on the same bytes
    y_small = run_affine(ctx, *w, x, dtype, entry, grid=7)
    assert np.array_equal(y, y_small)
    y_valu = run_affine(ctx, *w, x, dtype, f"affine_matvec:{cols}:64", generic=True)
    gh.check_outputs(y_valu, ref, dtype, "vector-ALU matvec")


@pytest.mark.parametrize("batch,tile,suffix", [(1, 8, "_batched"), (3, 3, "_batched_tile3"), (8, 8, "_batched"),
                                               (11, 8, "_batched"), (13, 4, "_batched_tile4")])
def test_mfma_small_batch(ctx, batch, tile, suffix):
    rows, cols = 8300, 1024
    dtype = fx.BF16
    entry = f"affine_matvec_c{cols}_r{rows}_g64{suffix}_mfma"
    assert mm_symbol(entry + "@bf16") == "smelt_affine_mm_matvec_batched_split_bf16"
    w = fx.synth_affine(rows, cols, 64, dtype, config=1, tensor=70)
    x = fx.synth_activation(batch, cols, dtype, config=1, tensor=71 + batch, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    y = run_affine(ctx, *w, x, dtype, entry, batched=True, batch_tile=tile)
    gh.check_outputs(y, ref, dtype, f"mfma batched M={batch}")
    # per-token results do not depend on the batch they ride in
    y1 = run_affine(ctx, *w, x[batch - 1:batch], dtype, f"affine_matvec_c{cols}_r{rows}_g64_mfma")
    assert np.array_equal(y[batch - 1], y1[0])


def test_mfma_fused_add_and_gate_up(ctx):
    rows, cols = 8192, 1024
    dtype = fx.F16
    gw = fx.synth_affine(rows, cols, 64, dtype, config=1, tensor=80)
    uw = fx.synth_affine(rows, cols, 64, dtype, config=1, tensor=81)
    x = fx.synth_activation(1, cols, dtype, config=1, tensor=82)
    res = fx.to_bits(fx.rng_for(1, 83).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    assert mm_symbol(f"fused_affine_matvec_add_c{cols}_r{rows}_g64_mfma") == "smelt_affine_mm_matvec_add_split_f16"
    y = run_affine(ctx, *gw, x, dtype, f"affine_matvec_c{cols}_r{rows}_g64_mfma")
    fused = run_affine(ctx, *gw, x, dtype, f"fused_affine_matvec_add_c{cols}_r{rows}_g64_mfma", residual=res)
    assert np.array_equal(fused, so.narrow(fx.from_bits(y, dtype) + fx.from_bits(res, dtype), dtype))
    entry = f"fused_affine_gate_up_swiglu_c{cols}_r{rows}_g64_mfma"
    assert mm_symbol(entry) == "smelt_affine_mm_gate_up_swiglu_split_f16"
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.alloc(gh.Y_SLOT, rows * 2)
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
    ctx.encode_decode(rt.make_record(ctx.pipeline(entry), bufs, [], (256, 1, 1), (256, 1, 1)))
    ctx.wait()
    got = ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows)
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, 64, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, 64, dtype)
    ref = fx.from_bits(so.epilogue_affine_swiglu(g, u, so.F16), fx.F16)
    gh.check_outputs(got, gh.swiglu_unrounded(g, u), dtype, "mfma gate_up_swiglu")


def test_mfma_argmax_and_selection_rules(ctx):
    """Fused lm_head argmax through the matrix-core kernel equals the oracle's argmax; the default
    names stay on the vector-ALU kernels and ineligible shapes are refused."""
    rows, cols, batch = 20000, 1024, 3
    dtype = fx.BF16
    w = fx.synth_affine(rows, cols, 64, dtype, config=1, tensor=7)
    x = fx.synth_activation(batch, cols, dtype, config=1, tensor=33)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    want = [so.argmax16(so.narrow(ref, dtype)[b]) for b in range(batch)]
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in w]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x)
    grid_w = 160
    ctx.alloc(gh.AUX_SLOT, batch * grid_w * 8)
    ctx.alloc(gh.Y_SLOT, batch * 4)
    entry = f"affine_matvec_argmax_c{cols}_r{rows}_g64_batched_mfma@bf16"
    assert mm_symbol(entry) == "smelt_affine_mm_matvec_argmax_split_bf16"
    p1, p2 = ctx.pipeline(entry), ctx.pipeline(f"lm_head_argmax_reduce_r{rows}")
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0)]
    r1 = rt.make_record(p1, bufs, [(5, batch), (6, 0.0)], (grid_w, 1, 1), (256, 1, 1))
    r2 = rt.make_record(p2, [(gh.AUX_SLOT, 0, 0), (gh.Y_SLOT, 1, 0)], [(2, batch), (3, grid_w)], (batch, 1, 1), (256, 1, 1))
    assert ctx.interpret_decode(ctx.table([r1, r2])) == 2
    ctx.wait()
    assert ctx.read(gh.Y_SLOT, np.int32, batch).tolist() == want
    assert mm_symbol("affine_matvec_c1024_r151936_g64@bf16") == "smelt_affine_matvec_bf16"
    assert mm_symbol("affine_matvec_c1024_r151936_g64_mfma@bf16") == "smelt_affine_mm_matvec_stream_bf16"
    for bad in ("affine_matvec_c1024_r3584_g64_mfma",        # under 8M weights
                "affine_matvec_c1024_r16384_g128_mfma",      # group != window
                "affine_matvec_c1088_r16384_g64_mfma"):      # cols % 256 != 0
        assert cc.resolve_pipeline_name(bad)[0] != 0


# ---- signed g128 formats: the runtime moves large matrices to the matrix cores per launch ---------
from test_gpu_matvec import run_signed  # noqa: E402


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("fmt,name", [(fx.BINARY1, "binary"), (fx.TERNARY2, "ternary")])
@pytest.mark.parametrize("shape", [(2050, 5120), (1030, 17408), (40010, 1024), (70001, 1024)])
def test_signed_large_matrices_match_oracle(ctx, fmt, name, dtype, shape):
    """27B-layer-like shapes of 8M weights and more (row counts off the 32-row tile, K split 4, 2 and 1
    ways): same pipeline names, same records, matrix-core kernels underneath."""
    rows, cols = shape
    codes = fx.synth_signed_codes(fmt, rows, cols, config=2 + fmt, tensor=rows % 7)
    scales = fx.synth_signed_scales(rows, cols, config=2 + fmt, tensor=rows % 7)
    packed = fx.pack_signed_np(codes, fmt)
    x = fx.synth_activation(2, cols, dtype, config=2 + fmt, outlier_frac=0.01)
    ref = so.signed_matvec(fmt, packed, scales, fx.from_bits(x, dtype), rows, cols, cols, 128)
    y = run_signed(ctx, name, packed, scales, x, dtype, rows, cols)
    w = gh.check_outputs(y, ref, dtype, f"signed {name} {shape}")
    print(f"\n  mfma {name} {shape} dtype={dtype} max rel err {w:.2e}")
    y_small = run_signed(ctx, name, packed, scales, x, dtype, rows, cols, grid=5)
    assert np.array_equal(y, y_small)


def test_signed_large_fused_add_and_ternary_affine_names(ctx):
    rows, cols = 2048, 5120
    dtype = fx.BF16
    for fmt, name in ((fx.BINARY1, "binary"), (fx.TERNARY2, "ternary")):
        codes = fx.synth_signed_codes(fmt, rows, cols, config=2 + fmt, tensor=3)
        scales = fx.synth_signed_scales(rows, cols, config=2 + fmt, tensor=3)
        packed = fx.pack_signed_np(codes, fmt)
        x = fx.synth_activation(1, cols, dtype, config=2 + fmt)
        res = fx.to_bits(fx.rng_for(2, 90).normal(0, 1, (1, rows)).astype(np.float32), dtype)
        y = run_signed(ctx, name, packed, scales, x, dtype, rows, cols)
        fused = run_signed(ctx, name, packed, scales, x, dtype, rows, cols, kind="add", residual=res)
        assert np.array_equal(fused, so.narrow(fx.from_bits(y, dtype) + fx.from_bits(res, dtype), dtype))
        if fmt == fx.TERNARY2:
            # production ternary pipeline name: scales bound twice, same arithmetic
            wf = gh.WeightFile()
            oc, os_ = wf.add(packed), wf.add(scales)
            ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
            ctx.put(gh.X_SLOT, x)
            ctx.alloc(gh.Y_SLOT, rows * 2)
            pipe = ctx.pipeline("signed_ternary_affine_matvec_g128_rows8@bf16")
            bufs = [(0, 0, oc), (0, 1, os_), (0, 2, os_), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
            ctx.encode_decode(rt.make_record(pipe, bufs, [(5, rows), (6, cols)], (256, 1, 1), (256, 1, 1)))
            ctx.wait()
            assert np.array_equal(ctx.read(gh.Y_SLOT, np.uint16, rows).reshape(1, rows), y)
