"""GPU parity of the streaming small-batch qmm (the kernel a skinny qmm record takes by default):
affine u4 g64 against the oracle through the C-ABI, for every batch size around the 16-token pass,
ragged row tiles, one and two row tiles per wave, short and long rows, the fused epilogues, both
activation types, and against the split-K kernels the same records take under the vector engine."""
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


@pytest.fixture(scope="module")
def split_k():
    c = rt.Context()
    c.set_matvec_engine(rt.MATVEC_VECTOR)   # keeps skinny records on the split-K kernels
    yield c
    c.close()


def qmm(ctx, w, x_bits, dtype, rows, cols, ksplit=4):
    """A skinny qmm record as the emitter writes it (32-row tiles x ksplit, 32-token grid rows)."""
    batch = x_bits.shape[0]
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in w]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x_bits)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    pipe = ctx.pipeline(f"affine_matvec_c{cols}_r{rows}_g64_batched_skinny" + gh.t_suffix(dtype))
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
    tiles = (rows + 31) // 32
    rec = rt.make_record(pipe, bufs, [(5, 0, rt.CONST_SEQ_LEN)], (tiles * ksplit, 32, 1), (256, 1, 1),
                         grid_kinds=(0, rt.GRID_SEQ_LEN_CEIL_DIV, 0))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("batch", [1, 7, 8, 9, 15, 16, 17, 32, 40])
def test_stream_qmm_4b_shapes(ctx, dtype, batch):
    """Qwen3.5-4B-shaped slab (K=2560, 392 of the 9216 rows: the last tile has 8 live rows), 1% outlier
    channels x10; 17 and 40 tokens end in passes of 1 and 8 live tokens."""
    rows, cols = 392, 2560
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=0)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=batch, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    y = qmm(ctx, w, x, dtype, rows, cols)
    worst = gh.check_outputs(y, ref, dtype, f"stream qmm M={batch}")
    print(f"\n  stream qmm M={batch} dtype={dtype} max rel err {worst:.2e}")


# (rows, cols): one run of eight groups per row (512), 1536 = 12 pairs over three waves, long rows
# (9216 = 72 pairs, six steps for each of twelve waves), 40 pairs, and 8200 rows = 32-row workgroups
# (two row tiles per wave once a pass stages more than eight tokens) with a ragged last tile
SHAPES = [(40, 512), (100, 1536), (96, 9216), (130, 5120), (8200, 1024), (8200, 2560)]


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("shape", SHAPES)
def test_stream_qmm_shapes(ctx, dtype, shape):
    rows, cols = shape
    batch = 13
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=rows % 11)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=cols % 13, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype, threads=True)
    ksplit = max(1, cols // 1024)   # what the record asks of the split-K kernel; the streaming kernel has its own split
    y = qmm(ctx, w, x, dtype, rows, cols, ksplit=ksplit)
    gh.check_outputs(y, ref, dtype, f"stream qmm {shape}")
    again = qmm(ctx, w, x, dtype, rows, cols, ksplit=ksplit)
    assert np.array_equal(y, again)   # fixed summation order


# rows of a multiple of 256 but not of 512 columns (11008: a Llama-7B down projection, 86 pairs; 768 = six pairs; 256 =
# two): scale rows start on 8-byte boundaries only and are staged four groups at a time
@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("shape", [(100, 11008, 13), (40, 768, 5), (8200, 2816, 24), (24, 256, 2), (130, 11008, 100)])
def test_stream_qmm_rows_of_odd_multiples_of_256_columns(ctx, split_k, dtype, shape):
    rows, cols, batch = shape
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=rows % 7)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=cols % 17, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype, threads=True)
    y = qmm_full(ctx, w, x, dtype, rows, cols)
    gh.check_outputs(y, ref, dtype, f"stream qmm {shape}")
    assert np.array_equal(y, qmm_full(ctx, w, x, dtype, rows, cols))   # fixed summation order
    # the token-slab kernel the record names (vector engine) agrees to the output tolerance
    slab = qmm_full(split_k, w, x, dtype, rows, cols)
    gh.check_outputs(slab, ref, dtype, f"slab qmm {shape}")
    gh.check_steps(y, slab, dtype, f"stream against slab {shape}", max_steps=1)


# groups of 128 columns: one scale per step instead of two; 1536 columns = twelve groups, staged four at a time.
# groups of 32: four scales per step, every 64-column half multiplied once per group; 768 and 11008 columns = odd
# multiples of 256
@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("group,shape", [(128, (200, 4096, 13)), (128, (8200, 1024, 24)), (128, (100, 11264, 40)), (128, (40, 1536, 3)),
                                         (128, (130, 5120, 200)), (32, (200, 4096, 13)), (32, (8200, 1024, 24)), (32, (100, 11008, 40)),
                                         (32, (40, 768, 3)), (32, (130, 5120, 200))])
def test_stream_qmm_groups_of_128_and_32_columns(ctx, split_k, dtype, group, shape):
    rows, cols, batch = shape
    w = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=rows % 5)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=cols % 19, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype, threads=True)
    y = qmm_full(ctx, w, x, dtype, rows, cols, group=group)
    gh.check_outputs(y, ref, dtype, f"stream qmm g{group} {shape}")
    assert np.array_equal(y, qmm_full(ctx, w, x, dtype, rows, cols, group=group))
    slab = qmm_full(split_k, w, x, dtype, rows, cols, group=group)
    gh.check_steps(y, slab, dtype, f"stream against slab, g{group} {shape}", max_steps=1)
    if batch <= 4:
        # the per-token small-batch form of the same matrix: the streaming kernel, or (small matrices) the single-token
        # kernel with a grid row per token; either way within the tolerance
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in w]
        ctx.upload_weights(0, wf.image())
        ctx.put(gh.X_SLOT, x)
        ctx.alloc(gh.Y_SLOT, batch * rows * 2)
        pipe = ctx.pipeline(f"affine_matvec_c{cols}_r{rows}_g{group}_batched_tile4" + gh.t_suffix(dtype))
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
        assert ctx.encode_decode(rt.make_record(pipe, bufs, [(5, batch)], (min(1024, (rows + 7) // 8), 1, 1), (256, 1, 1))) == 1
        ctx.wait()
        gh.check_outputs(ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows), ref, dtype, f"tile4 g{group}")


def test_stream_qmm_is_exact_where_the_sums_are(ctx):
    """KernelLab.swift:2829-2855 buffers: every partial sum is an exact dyadic rational, so the
    streaming kernel gives the oracle's bits for every token."""
    rows, cols, group, batch = 64, 1024, 64, 9
    packed, scales, biases, x = fx.kernel_lab_qmm_fixture(rows, cols, group, batch)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, fx.F16), rows, cols, group)
    y = qmm(ctx, (packed, scales, biases), x, fx.F16, rows, cols, ksplit=2)
    assert np.array_equal(y, ref.astype(np.float16).view(np.uint16))


def test_stream_qmm_closed_form_fixture(ctx):
    """Closed-form fixture of PrefillKernelTests.swift:220-264 (tolerance 0.07 absolute there)."""
    rows, cols, batch = 128, 1024, 9
    packed, scales, biases, x, _ = fx.affine_synthetic_fixture(rows, cols, 64, seed=3, batch=batch)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, fx.F16), rows, cols, 64)
    y = qmm(ctx, (packed, scales, biases), x, fx.F16, rows, cols, ksplit=2)
    assert np.abs(fx.from_bits(y, fx.F16) - ref).max() < 0.07
    gh.check_outputs(y, ref, fx.F16, "stream qmm fixture")


def test_stream_and_split_k_kernels_agree(ctx, split_k):
    """The two kernels of a skinny record differ in summation order only."""
    dtype = fx.BF16
    rows, cols, batch = 416, 2560, 13
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=31)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=131, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    a = qmm(ctx, w, x, dtype, rows, cols)
    b = qmm(split_k, w, x, dtype, rows, cols)
    gh.check_outputs(a, ref, dtype, "stream")
    gh.check_outputs(b, ref, dtype, "split-K")
    ulp = np.abs(a.astype(np.int32) - b.astype(np.int32))
    assert ulp.max() <= 1 or np.mean(ulp > 1) < 1e-3


def test_stream_qmm_very_long_rows(ctx):
    """K = 17408 (136 pairs of groups): twelve waves, twelve steps each, the last one partly idle."""
    dtype = fx.F16
    rows, cols, batch = 64, 17408, 5
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=41)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=141)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    gh.check_outputs(qmm(ctx, w, x, dtype, rows, cols, ksplit=16), ref, dtype, "stream qmm K=17408")


def test_stream_qmm_bf16_activations_beyond_the_fp16_range(ctx):
    """bf16 activations enter the bf16 MFMA unconverted: magnitudes past 65504 are not clamped."""
    dtype = fx.BF16
    rows, cols, batch = 64, 1024, 6
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=8)
    xf = fx.rng_for(4, 555).normal(0, 1, (batch, cols)).astype(np.float32)
    xf[:, ::37] *= 3.0e5
    x = fx.to_bits(xf, dtype)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
    gh.check_outputs(qmm(ctx, w, x, dtype, rows, cols, ksplit=1), ref, dtype, "stream qmm with |x| > 65504")


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_stream_qmm_fused_add_and_gate_up(ctx, dtype):
    rows, cols, batch, ksplit = 200, 2560, 11, 4
    gw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=3)
    uw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=4)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=8)
    res = fx.to_bits(fx.rng_for(4, 79).normal(0, 1, (batch, rows)).astype(np.float32), dtype)
    plain = qmm(ctx, gw, x, dtype, rows, cols, ksplit)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.put(gh.RES_SLOT, res)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    ctx.alloc(gh.AUX_SLOT, batch * rows * 2)
    tiles = (rows + 31) // 32
    t = gh.t_suffix(dtype)
    pipe = ctx.pipeline(f"fused_affine_matvec_add_c{cols}_r{rows}_g64_batched_skinny" + t)
    bufs = [(0, i, offs[i]) for i in range(3)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0), (gh.RES_SLOT, 5, 0), (gh.Y_SLOT, 6, 0)]
    rec = rt.make_record(pipe, bufs, [(7, batch)], (tiles * ksplit, 1, 1), (256, 1, 1))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    mv = ctx.read(gh.AUX_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    out = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    assert np.array_equal(mv, plain)                       # fused == staged, bit for bit
    assert np.array_equal(out, so.narrow(fx.from_bits(plain, dtype) + fx.from_bits(res, dtype), dtype))
    pipe = ctx.pipeline(f"fused_affine_gate_up_swiglu_c{cols}_r{rows}_g64_batched_skinny" + t)
    bufs = [(0, i, offs[i]) for i in range(6)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
    rec = rt.make_record(pipe, bufs, [(8, batch)], (tiles * ksplit, 1, 1), (512, 1, 1))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    y = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, 64, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, 64, dtype)
    sd = so.BF16 if dtype == fx.BF16 else so.F16
    ref = fx.from_bits(so.epilogue_affine_swiglu(g, u, sd), dtype)
    gh.check_outputs(y, gh.swiglu_unrounded(g, u), dtype, "stream gate_up_swiglu")


# ---- token-tile form: 128 tokens and more; below, 16-token passes of the streaming kernel ------

def qmm_full(ctx, w, x_bits, dtype, rows, cols, bt=64, group=64):
    """A token-slab qmm record as the emitter writes it for prefill chunks (64-row slabs, bt-token grid rows)."""
    batch = x_bits.shape[0]
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in w]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x_bits)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    pipe = ctx.pipeline(f"affine_matvec_c{cols}_r{rows}_g{group}_batched_full_b{bt}" + gh.t_suffix(dtype))
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
    rec = rt.make_record(pipe, bufs, [(5, 0, rt.CONST_SEQ_LEN)], ((rows + 63) // 64, bt, 1), (256, 1, 1),
                         grid_kinds=(0, rt.GRID_SEQ_LEN_CEIL_DIV, 0))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("batch", [49, 64, 100, 127, 128, 129, 300])
def test_tile_qmm_4b_shapes(ctx, dtype, batch):
    """Qwen3.5-4B-shaped slab (K=2560, 2088 rows: ragged last row tile; a matrix of more than 5M weights, which the
    token-tile kernel takes from 128 tokens; the smaller batches run the streaming kernel), ragged last token tile."""
    rows, cols = 2088, 2560
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=0)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=batch, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype, threads=True)
    y = qmm_full(ctx, w, x, dtype, rows, cols)
    worst = gh.check_outputs(y, ref, dtype, f"tile qmm M={batch}")
    print(f"\n  tile qmm M={batch} dtype={dtype} max rel err {worst:.2e}")


@pytest.mark.parametrize("batch", [33, 64, 70, 127])
def test_tile_qmm_takes_large_matrices_from_33_tokens(ctx, split_k, batch):
    """From 40M weights (and 3584 rows) the token-tile kernel takes the record from 33 tokens on: one ragged 64-token
    block, one full, two; ragged last row tile.  Against the oracle and against the token-slab kernel."""
    rows, cols, dtype = 3600, 12288, fx.BF16
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=5)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=batch, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype, threads=True)
    y = qmm_full(ctx, w, x, dtype, rows, cols)
    gh.check_outputs(y, ref, dtype, f"tile qmm {rows}x{cols} M={batch}")
    assert np.array_equal(y, qmm_full(ctx, w, x, dtype, rows, cols))
    gh.check_steps(y, qmm_full(split_k, w, x, dtype, rows, cols), dtype, f"tile against slab M={batch}", max_steps=1)


@pytest.mark.parametrize("shape", [(600, 9216, 512), (8200, 1024, 96), (40, 512, 1100), (2600, 2560, 520), (2560, 9216, 256),
                                   (1000, 6144, 200)])
def test_tile_qmm_shapes(ctx, split_k, shape):
    """Long rows at a 512-token chunk (three workgroups share each tile along K), many rows in several
    16-token passes, a matrix smaller than one tile (which the token-tile kernel takes from 1024 tokens), ragged row and token tiles, the 4B down projection
    at 256 tokens (64-row tiles, three-way split), a two-way split with uneven halves; against the oracle
    and the token-slab kernel, and twice in a row (the split leaves its counters at zero)."""
    rows, cols, batch = shape
    dtype = fx.BF16
    w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=rows % 11)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=cols % 13, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype, threads=True)
    y = qmm_full(ctx, w, x, dtype, rows, cols)
    gh.check_outputs(y, ref, dtype, f"tile qmm {shape}")
    assert np.array_equal(y, qmm_full(ctx, w, x, dtype, rows, cols))
    gh.check_outputs(qmm_full(split_k, w, x, dtype, rows, cols), ref, dtype, f"slab qmm {shape}")


def test_tile_qmm_is_exact_where_the_sums_are(ctx):
    rows, cols, group, batch = 5120, 1024, 64, 150      # 5M weights: the token-tile kernel from 128 tokens
    packed, scales, biases, x = fx.kernel_lab_qmm_fixture(rows, cols, group, batch)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, fx.F16), rows, cols, group)
    y = qmm_full(ctx, (packed, scales, biases), x, fx.F16, rows, cols)
    assert np.array_equal(y, ref.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_tile_qmm_fused_add_and_gate_up(ctx, dtype):
    rows, cols, batch = 2100, 2560, 140                 # 5.4M weights: the token-tile kernel from 128 tokens
    gw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=3)
    uw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=4)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=8)
    res = fx.to_bits(fx.rng_for(4, 79).normal(0, 1, (batch, rows)).astype(np.float32), dtype)
    plain = qmm_full(ctx, gw, x, dtype, rows, cols)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.put(gh.RES_SLOT, res)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    ctx.alloc(gh.AUX_SLOT, batch * rows * 2)
    t = gh.t_suffix(dtype)
    grid = ((rows + 63) // 64, (batch + 63) // 64, 1)
    pipe = ctx.pipeline(f"fused_affine_matvec_add_c{cols}_r{rows}_g64_batched_full_b64" + t)
    bufs = [(0, i, offs[i]) for i in range(3)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0), (gh.RES_SLOT, 5, 0), (gh.Y_SLOT, 6, 0)]
    rec = rt.make_record(pipe, bufs, [(7, batch)], grid, (256, 1, 1))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    mv = ctx.read(gh.AUX_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    out = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    assert np.array_equal(mv, plain)                       # fused == staged, bit for bit
    assert np.array_equal(out, so.narrow(fx.from_bits(plain, dtype) + fx.from_bits(res, dtype), dtype))
    pipe = ctx.pipeline(f"fused_affine_gate_up_swiglu_c{cols}_r{rows}_g64_batched_full_b64" + t)
    bufs = [(0, i, offs[i]) for i in range(6)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
    rec = rt.make_record(pipe, bufs, [(8, batch)], grid, (256, 1, 1))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    y = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, 64, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, 64, dtype)
    sd = so.BF16 if dtype == fx.BF16 else so.F16
    ref = fx.from_bits(so.epilogue_affine_swiglu(g, u, sd), dtype)
    gh.check_outputs(y, gh.swiglu_unrounded(g, u), dtype, "tile gate_up_swiglu")


def test_tile_qmm_gate_up_on_a_grid_that_fills_the_machine(ctx):
    """6144 rows at 512 tokens: enough 64-row tiles for three workgroups per compute unit, which is where
    the gate+up record takes the four-wave kernel with both matrices in every wave (the smaller grids of
    the test above take the one-matrix-per-wave kernel)."""
    dtype = fx.BF16
    rows, cols, batch = 6144, 512, 512
    gw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=13)
    uw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=14)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=18)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    pipe = ctx.pipeline(f"fused_affine_gate_up_swiglu_c{cols}_r{rows}_g64_batched_full_b64@bf16")
    bufs = [(0, i, offs[i]) for i in range(6)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
    rec = rt.make_record(pipe, bufs, [(8, batch)], ((rows + 63) // 64, (batch + 63) // 64, 1), (256, 1, 1))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    y = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, 64, dtype, threads=True)
    u = so.affine_matvec(*uw, xf, rows, cols, 64, dtype, threads=True)
    ref = fx.from_bits(so.epilogue_affine_swiglu(g, u, so.BF16), dtype)
    gh.check_outputs(y, gh.swiglu_unrounded(g, u), dtype, "tile gate_up_swiglu, full grid")


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("shape", [(640, 1024, 21), (2100, 2560, 140), (200, 11008, 9), (512, 1024, 3)])
def test_geglu_qmm_streams_and_tiles(ctx, split_k, dtype, shape):
    """The GeGLU gate+up qmm (Gemma-shaped layers) on the streaming kernel (21 and 9 tokens; 11008 columns), on the
    token-tile kernel (140 tokens of a matrix pair of 10M weights) and, three tokens of a small pair through the per-token
    small-batch name, on the single-token kernel with a grid row per token: against the oracle's epilogue to the step
    bound of the GeGLU tests, and against the token-slab kernel the qmm record names."""
    rows, cols, batch = shape
    gw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=23)
    uw = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=24)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=28)
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, 64, dtype, threads=True)
    u = so.affine_matvec(*uw, xf, rows, cols, 64, dtype, threads=True)
    ref = so.epilogue_geglu(g, u, dtype)

    def run(c, name, consts, grid):
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in (*gw, *uw)]
        c.upload_weights(0, wf.image())
        c.put(gh.X_SLOT, x)
        c.alloc(gh.Y_SLOT, batch * rows * 2)
        pipe = c.pipeline(name + gh.t_suffix(dtype))
        bufs = [(0, i, offs[i]) for i in range(6)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
        assert c.encode_prefill(rt.make_record(pipe, bufs, consts, grid, (256, 1, 1)), seq_len=batch) == 1
        c.wait()
        return c.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)

    full = f"fused_affine_gate_up_geglu_c{cols}_r{rows}_g64_batched_full_b64"
    grid = ((rows + 63) // 64, (batch + 63) // 64, 1)
    y = run(ctx, full, [(8, batch)], grid)
    gh.check_steps(y, ref, dtype, f"geglu qmm {shape}", max_steps=gh.GEGLU_STEPS)
    assert np.array_equal(y, run(ctx, full, [(8, batch)], grid))
    gh.check_steps(y, run(split_k, full, [(8, batch)], grid), dtype, f"geglu qmm against slab {shape}", max_steps=gh.GEGLU_STEPS)
    if batch <= 3:
        small = run(ctx, f"fused_affine_gate_up_geglu_c{cols}_r{rows}_g64_batched", [(8, batch)], (min(1024, (rows + 7) // 8), 1, 1))
        gh.check_steps(small, ref, dtype, f"geglu small batch {shape}", max_steps=gh.GEGLU_STEPS)
