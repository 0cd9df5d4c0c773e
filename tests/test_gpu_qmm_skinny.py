"""GPU parity: the split-K skinny qmm kernels (M <= 32 per pass, affine u4 g64) against the oracle,
for every K split the launch can express, ragged row tiles, several token blocks, the fused
epilogues, and repeated launches that reuse the split-K workspace."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import compiler as cc
from smelt_amd import runtime as rt

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = rt.Context()
    c.set_matvec_engine(rt.MATVEC_VECTOR)   # keeps skinny records on the split-K kernels tested here
    yield c
    c.close()


def skinny(ctx, w, x_bits, dtype, rows, cols, ksplit, group=64, bt=32, threads=256):
    batch = x_bits.shape[0]
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in w]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x_bits)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    pipe = ctx.pipeline(f"affine_matvec_c{cols}_r{rows}_g{group}_batched_skinny" + gh.t_suffix(dtype))
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
    tiles = (rows + 31) // 32
    rec = rt.make_record(pipe, bufs, [(5, 0, rt.CONST_SEQ_LEN)], (tiles * ksplit, bt, 1), (threads, 1, 1),
                         grid_kinds=(0, rt.GRID_SEQ_LEN_CEIL_DIV, 0))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("batch", [1, 7, 8, 9, 32])
def test_skinny_qmm_4b_shapes(ctx, dtype, batch):
    """Qwen3.5-4B-shaped slab (K=2560, 384 of the 9216 rows), 1% outlier channels x10, K split 4 ways."""
    rows, cols = 384, 2560
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=0)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=batch, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    y = skinny(ctx, w, x, dtype, rows, cols, ksplit=4)
    worst = gh.check_outputs(y, ref, dtype, f"skinny qmm M={batch}")
    print(f"\n  skinny qmm M={batch} dtype={dtype} max rel err {worst:.2e}")


def test_skinny_qmm_every_split_is_the_same_sum_within_tolerance(ctx):
    """K = 1536 (24 windows) split 1, 2, 3, 5, 7 and 24 ways over workgroups of 4 to 8 waves (uneven
    chunks, one-window chunks, waves with no window): all within tolerance of the oracle, and a
    repeated launch is bit-identical (fixed summation order, counters back at zero)."""
    dtype = fx.BF16
    rows, cols, batch = 100, 1536, 13        # 100 rows: the last tile has 4 live rows
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=11)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=113, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    for ksplit, threads in ((1, 256), (1, 512), (2, 512), (3, 256), (5, 448), (7, 320), (24, 256)):
        y = skinny(ctx, w, x, dtype, rows, cols, ksplit, threads=threads)
        gh.check_outputs(y, ref, dtype, f"skinny qmm ksplit={ksplit} threads={threads}")
        again = skinny(ctx, w, x, dtype, rows, cols, ksplit, threads=threads)
        assert np.array_equal(y, again), (ksplit, threads)


def test_skinny_qmm_long_rows_and_token_blocks(ctx):
    """down-projection shape (K=9216) split 12 ways; 40 tokens = two 32-token passes, the second
    with 8 live tokens; also a 16-token tile (three passes)."""
    dtype = fx.F16
    rows, cols, batch = 96, 9216, 40
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=12)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=140, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    y = skinny(ctx, w, x, dtype, rows, cols, ksplit=12)
    gh.check_outputs(y, ref, dtype, "skinny qmm K=9216 M=40")
    y = skinny(ctx, w, x, dtype, rows, cols, ksplit=6, threads=512)
    gh.check_outputs(y, ref, dtype, "skinny qmm K=9216 M=40, 8 waves")
    y16 = skinny(ctx, w, x, dtype, rows, cols, ksplit=12, bt=16)
    gh.check_outputs(y16, ref, dtype, "skinny qmm K=9216 M=40 bt=16")


def test_skinny_qmm_closed_form_fixture(ctx):
    """Closed-form fixture of PrefillKernelTests.swift:220-264 (tolerance 0.07 absolute there)."""
    rows, cols, batch = 128, 1024, 9
    packed, scales, biases, x, _ = fx.affine_synthetic_fixture(rows, cols, 64, seed=3, batch=batch)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, fx.F16), rows, cols, 64)
    y = skinny(ctx, (packed, scales, biases), x, fx.F16, rows, cols, ksplit=2)
    assert np.abs(fx.from_bits(y, fx.F16) - ref).max() < 0.07
    gh.check_outputs(y, ref, fx.F16, "skinny qmm fixture")


def test_skinny_qmm_fused_add_and_gate_up(ctx):
    dtype = fx.BF16
    rows, cols, batch, ksplit = 192, 1024, 8, 4
    gw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=3)
    uw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=4)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=8)
    res = fx.to_bits(fx.rng_for(4, 79).normal(0, 1, (batch, rows)).astype(np.float32), dtype)
    plain = skinny(ctx, gw, x, dtype, rows, cols, ksplit)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.put(gh.RES_SLOT, res)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    ctx.alloc(gh.AUX_SLOT, batch * rows * 2)
    tiles = (rows + 31) // 32
    pipe = ctx.pipeline(f"fused_affine_matvec_add_c{cols}_r{rows}_g64_batched_skinny@bf16")
    bufs = [(0, i, offs[i]) for i in range(3)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0), (gh.RES_SLOT, 5, 0), (gh.Y_SLOT, 6, 0)]
    rec = rt.make_record(pipe, bufs, [(7, batch)], (tiles * ksplit, 1, 1), (256, 1, 1))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    mv = ctx.read(gh.AUX_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    out = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    assert np.array_equal(mv, plain)                       # fused == staged, bit for bit
    assert np.array_equal(out, so.narrow(fx.from_bits(plain, dtype) + fx.from_bits(res, dtype), dtype))
    pipe = ctx.pipeline(f"fused_affine_gate_up_swiglu_c{cols}_r{rows}_g64_batched_skinny@bf16")
    bufs = [(0, i, offs[i]) for i in range(6)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
    rec = rt.make_record(pipe, bufs, [(8, batch)], (tiles * ksplit, 1, 1), (512, 1, 1))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    y = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, 64, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, 64, dtype)
    ref = fx.from_bits(so.epilogue_affine_swiglu(g, u, so.BF16), fx.BF16)
    gh.check_outputs(y, gh.swiglu_unrounded(g, u), dtype, "skinny gate_up_swiglu")


def test_skinny_qmm_rejects_bad_launches(ctx):
    rows, cols = 64, 1024
    dtype = fx.F16
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=5)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in w]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, fx.synth_activation(4, cols, dtype, config=4, tensor=6))
    ctx.alloc(gh.Y_SLOT, 4 * rows * 2)
    pipe = ctx.pipeline(f"affine_matvec_c{cols}_r{rows}_g64_batched_skinny")
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
    bad = rt.make_record(pipe, bufs, [(5, 4)], (3, 1, 1), (256, 1, 1))       # 3 is not a multiple of 2 tiles
    with pytest.raises(rt.SmeltHipError):
        ctx.encode_prefill(bad, seq_len=4)
    bad = rt.make_record(pipe, bufs, [(5, 4)], (2, 1, 1), (128, 1, 1))       # fewer than four waves
    with pytest.raises(rt.SmeltHipError):
        ctx.encode_prefill(bad, seq_len=4)
    with pytest.raises(rt.SmeltHipError):                                    # group 128 has no skinny kernel
        ctx.pipeline("affine_matvec_c1024_r64_g128_batched_skinny")
    with pytest.raises(rt.SmeltHipError):                                    # cols % 512 != 0
        ctx.pipeline("affine_matvec_c1088_r64_g64_batched_skinny")


def test_emitter_routes_small_batches_to_skinny(ctx):
    """The emitter's M = 8 lowering of a 4B-shaped projection runs the skinny kernel and matches."""
    dtype = fx.BF16
    rows, cols, batch = 512, 2560, 8
    c = rt.Context(act_dtype=rt.ACT_BF16)
    try:
        lay = cc.Layout()
        e = lay.affine(rows, cols, 64)
        image = np.zeros(lay.total_bytes, np.uint8)
        w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=20)
        cc.write_affine(image, e, *w)
        em = cc.Emitter(rt.ACT_BF16, 256)
        em.matvec(0, e, cc.bind(1), cc.bind(2), batch=batch)
        assert any("_batched_skinny" in n for n in em.pipelines)
        em.install(c)
        c.upload_weights(0, image)
        x = fx.synth_activation(batch, cols, dtype, config=4, tensor=21, outlier_frac=0.01)
        c.put(1, x)
        c.alloc(2, batch * rows * 2)
        assert c.interpret_prefill(em.records(), seq_len=batch) == 1
        c.wait()
        y = c.read(2, np.uint16, batch * rows).reshape(batch, rows)
        ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
        gh.check_outputs(y, ref, dtype, "emitter skinny qmm")
    finally:
        c.close()
