"""GPU parity: MFMA qmm kernels, lm_head argmax, ternary-affine pipeline names, projection
banks and the trit5 format, all through the C-ABI with hand-built records."""
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
    c.set_matvec_engine(rt.MATVEC_VECTOR)   # keeps qmm records on the token-slab kernels tested here
    yield c
    c.close()


def qmm_affine(ctx, w, x_bits, dtype, rows, cols, group, suffix="_batched_full", bt=16, grid_w=None):
    batch = x_bits.shape[0]
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in w]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x_bits)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    pipe = ctx.pipeline(f"affine_matvec_c{cols}_r{rows}_g{group}{suffix}" + gh.t_suffix(dtype))
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
    # prefill-style record: actualBatch = seqLen, grid height = ceil(seqLen / batch tile)
    rec = rt.make_record(pipe, bufs, [(5, 0, rt.CONST_SEQ_LEN)], (grid_w or (rows + 63) // 64, bt, 1),
                         (256, 1, 1), grid_kinds=(0, rt.GRID_SEQ_LEN_CEIL_DIV, 0))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("batch", [7, 8, 9, 32])
def test_affine_qmm_small_batch_4b_shapes(ctx, dtype, batch):
    """Qwen3.5-4B-shaped slab (K=2560, 384 of the 9216 rows), 1% outlier channels x10."""
    rows, cols, group = 384, 2560, 64
    w = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=0)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=batch, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype)
    y = qmm_affine(ctx, w, x, dtype, rows, cols, group)
    worst = gh.check_outputs(y, ref, dtype, f"affine qmm M={batch}")
    print(f"\n  qmm M={batch} dtype={dtype} max rel err {worst:.2e}")
    if batch == 8:
        y8 = qmm_affine(ctx, w, x, dtype, rows, cols, group, suffix="_batched_full_b8", bt=8)
        assert np.array_equal(y, y8)


def test_affine_qmm_prefill_chunk_and_ragged_edges(ctx):
    """512-token chunk through the 64-token tile variant; rows and K not multiples of the tile."""
    dtype = fx.F16
    rows, cols, group, batch = 200, 9216, 64, 512
    w = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=1)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=512, outlier_frac=0.01)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype)
    y = qmm_affine(ctx, w, x, dtype, rows, cols, group, suffix="_batched_full_b64", bt=64)
    gh.check_outputs(y, ref, dtype, "affine qmm M=512")
    # K = 96 (not a multiple of the 128-column step), M = 19, group 32
    rows, cols, group, batch = 70, 96, 32, 19
    w = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=2)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=19)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype)
    y = qmm_affine(ctx, w, x, dtype, rows, cols, group)
    gh.check_outputs(y, ref, dtype, "affine qmm ragged")


def test_affine_qmm_against_reference_tolerance_fixture(ctx):
    """Closed-form fixture of PrefillKernelTests.swift:220-264, qmm vs iterated matvec
    tolerance 0.07 absolute there (:9775-9883)."""
    rows, cols, group, batch = 128, 1024, 64, 9
    packed, scales, biases, x, _ = fx.affine_synthetic_fixture(rows, cols, group, seed=3, batch=batch)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, fx.F16), rows, cols, group)
    y = qmm_affine(ctx, (packed, scales, biases), x, fx.F16, rows, cols, group)
    assert np.abs(fx.from_bits(y, fx.F16) - ref).max() < 0.07
    gh.check_outputs(y, ref, fx.F16, "affine qmm fixture")


def test_affine_qmm_fused_add_and_gate_up(ctx):
    dtype = fx.F16
    rows, cols, group, batch = 192, 1024, 64, 8
    gw = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=3)
    uw = fx.synth_affine(rows, cols, group, dtype, config=4, tensor=4)
    x = fx.synth_activation(batch, cols, dtype, config=4, tensor=8)
    res = fx.to_bits(fx.rng_for(4, 79).normal(0, 1, (batch, rows)).astype(np.float32), dtype)
    plain = qmm_affine(ctx, gw, x, dtype, rows, cols, group)
    plain_u = qmm_affine(ctx, uw, x, dtype, rows, cols, group)
    # fused add: bindings 0 W,1 S,2 B,3 X,4 matvecOut,5 residual,6 out, const 7 actualBatch
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in (*gw, *uw)]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.put(gh.RES_SLOT, res)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    ctx.alloc(gh.AUX_SLOT, batch * rows * 2)
    pipe = ctx.pipeline(f"fused_affine_matvec_add_c{cols}_r{rows}_g{group}_batched_full_b8")
    bufs = [(0, i, offs[i]) for i in range(3)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0), (gh.RES_SLOT, 5, 0), (gh.Y_SLOT, 6, 0)]
    rec = rt.make_record(pipe, bufs, [(7, batch)], ((rows + 63) // 64, 1, 1), (256, 1, 1))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    mv = ctx.read(gh.AUX_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    out = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    assert np.array_equal(mv, plain)
    assert np.array_equal(out, so.narrow(fx.from_bits(plain, dtype) + fx.from_bits(res, dtype), dtype))
    # fused gate-up SwiGLU against the fp32 oracle epilogue
    pipe = ctx.pipeline(f"fused_affine_gate_up_swiglu_c{cols}_r{rows}_g{group}_batched_full")
    bufs = [(0, i, offs[i]) for i in range(6)] + [(gh.X_SLOT, 6, 0), (gh.Y_SLOT, 7, 0)]
    rec = rt.make_record(pipe, bufs, [(8, batch)], ((rows + 63) // 64, 1, 1), (256, 1, 1))
    assert ctx.encode_prefill(rec, seq_len=batch) == 1
    ctx.wait()
    y = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    xf = fx.from_bits(x, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, group, dtype)
    u = so.affine_matvec(*uw, xf, rows, cols, group, dtype)
    ref = fx.from_bits(so.epilogue_affine_swiglu(g, u, so.F16), fx.F16)
    gh.check_outputs(y, gh.swiglu_unrounded(g, u), dtype, "qmm gate_up_swiglu")
    assert plain_u.shape == plain.shape


def test_ternary_qmm_matches_per_row_matvec_and_oracle(ctx):
    """M >= 6 route (QMM) vs the M < 6 route (QMV): same logical result within tolerance; the
    dequantised ternary tile is exact in fp16, so the only difference is summation order."""
    rows, cols, batch = 96, 5120, 14
    codes = fx.synth_signed_codes(fx.TERNARY2, rows, cols, config=3, tensor=1)
    scales = fx.synth_signed_scales(rows, cols, config=3, tensor=1)
    packed = fx.pack_signed_np(codes, fx.TERNARY2)
    x = fx.synth_activation(batch, cols, fx.F16, config=3, tensor=14)
    ref = so.signed_matvec(so.TERNARY2, packed, scales, fx.from_bits(x, fx.F16), rows, cols, cols, 128)
    wf = gh.WeightFile()
    oc, os_ = wf.add(packed), wf.add(scales)
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    bufs = [(0, 0, oc), (0, 1, os_), (0, 2, os_), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
    qmv = ctx.pipeline("signed_ternary_affine_matvec_g128_rows8")
    qmm = ctx.pipeline("signed_ternary_affine_qmm_g128_bm32_bn32_bk32")
    # the reference emits both records, guarded by sequence length (SmeltCodeEmitter.swift:1120-1182)
    r1 = rt.make_record(qmv, bufs, [(5, rows), (6, cols), (0xFF, 6, 13)], ((rows + 7) // 8, 0, 1), (256, 1, 1),
                        grid_kinds=(0, rt.GRID_SEQ_LEN, 0))
    r2 = rt.make_record(qmm, bufs, [(5, rows), (6, cols), (7, 0, rt.CONST_SEQ_LEN)], ((rows + 63) // 64, 32, 1),
                        (256, 1, 1), grid_kinds=(0, rt.GRID_SEQ_LEN_CEIL_DIV, 0), min_seq_len=6)
    table = ctx.table([r1, r2])
    assert ctx.interpret_prefill(table, seq_len=batch) == 1      # only the QMM record runs at M=14
    ctx.wait()
    y_mm = ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
    gh.check_outputs(y_mm, ref, fx.F16, "ternary qmm")
    assert ctx.interpret_prefill(table, seq_len=5) == 1           # only the QMV record runs at M=5
    ctx.wait()
    y_mv = ctx.read(gh.Y_SLOT, np.uint16, 5 * rows).reshape(5, rows)
    gh.check_outputs(y_mv, ref[:5], fx.F16, "ternary qmv")


def test_ternary_qmm_reproduces_mlx_golden_bits_and_byte_lane_subscales(ctx):
    """SignedQuantKernelTests.swift:527-601: the 112 bit patterns MLX's affine_qmm_t gives for
    M=14, and the same shape with scales small enough that scale/16 and scale/64 round in the
    fp16 subnormal range (signed_quant_precise.metal:407-439). Every fp32 partial sum of both
    fixtures is exact, so summation order cannot matter and the bits must be equal; on the
    second fixture (code - 1) * scale would miss by up to 6 % on the small outputs."""
    case = fx.golden_vectors()["ternary_qmm_mlx_m14"]
    rows, cols, batch = case["rows"], case["cols"], case["batch"]
    golden = np.array([int(b, 16) for b in case["expected_bits"]], np.uint16)
    small = ["1b95", "1797", "1b93", "17ff", "1a01"]
    for scale_bits, want, separate_bias in ((case["scale_bits"], golden, False), (small, None, False),
                                            (small, None, True)):
        codes, scales, x = fx.mlx_ternary_qmm_fixture(rows, cols, batch, scale_bits)
        bias_scales = np.roll(scales, 1, axis=0) if separate_bias else scales
        packed = fx.pack_signed_np(codes, fx.TERNARY2)
        ref = so.ternary_affine_qmm(packed, scales, x, rows, cols, bias_scales=bias_scales)
        ref_bits = ref.astype(np.float16).view(np.uint16).ravel()
        if want is None:
            want = ref_bits
            naive = so.signed_matvec(so.TERNARY2, packed, scales, fx.from_bits(x, fx.F16), rows, cols, cols, 128)
            assert (naive.astype(np.float16).view(np.uint16).ravel() != want).sum() > 40
        else:
            assert np.array_equal(ref_bits, want)
        wf = gh.WeightFile()
        oc, os_, ob = wf.add(packed), wf.add(scales), wf.add(bias_scales)
        ctx.upload_weights(0, wf.image())
        ctx.put(gh.X_SLOT, x)
        ctx.alloc(gh.Y_SLOT, batch * rows * 2)
        ctx.encode_decode(rt.make_record(
            ctx.pipeline("signed_ternary_affine_qmm_g128_bm32_bn32_bk32"),
            [(0, 0, oc), (0, 1, os_), (0, 2, ob), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)],
            [(5, rows), (6, cols), (7, batch)], (1, 1, 1), (256, 1, 1)))
        ctx.wait()
        assert np.array_equal(ctx.read(gh.Y_SLOT, np.uint16, want.size), want), (scale_bits, separate_bias)


def test_lm_head_argmax_fused_and_staged(ctx):
    """Identical argmax over the lm_head row block: fused matvec+argmax, and argmax over the
    materialised logits, both equal the oracle's argmax of its rounded logits."""
    rows, cols, group = 20000, 1024, 64
    for dtype in (fx.F16, fx.BF16):
        w = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=7)
        batch = 3
        x = fx.synth_activation(batch, cols, dtype, config=1, tensor=33)
        ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype)
        ref_bits = so.narrow(ref, dtype)
        want = [so.argmax16(ref_bits[b]) for b in range(batch)]
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in w]
        ctx.upload_weights(0, wf.image())
        ctx.put(gh.X_SLOT, x)
        grid_w = 160
        ctx.alloc(gh.AUX_SLOT, batch * grid_w * 8)
        ctx.alloc(gh.Y_SLOT, batch * 4)
        p1 = ctx.pipeline(f"affine_matvec_argmax_c{cols}_r{rows}_g{group}_batched" + gh.t_suffix(dtype))
        p2 = ctx.pipeline(f"lm_head_argmax_reduce_r{rows}")
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0)]
        r1 = rt.make_record(p1, bufs, [(5, batch), (6, 0.0)], (grid_w, 1, 1), (256, 1, 1))
        r2 = rt.make_record(p2, [(gh.AUX_SLOT, 0, 0), (gh.Y_SLOT, 1, 0)], [(2, batch), (3, grid_w)], (batch, 1, 1), (256, 1, 1))
        assert ctx.interpret_decode(ctx.table([r1, r2])) == 2
        ctx.wait()
        got = ctx.read(gh.Y_SLOT, np.int32, batch).tolist()
        # top-2 margin of the oracle logits, to show the comparison is not a coin flip
        margins = [float(np.sort(ref[b])[-1] - np.sort(ref[b])[-2]) for b in range(batch)]
        assert got == want, (got, want, margins)
        # staged: matvec -> logits, argmax partials -> reduce
        ctx.alloc(gh.RES_SLOT, rows * 2)
        pm = ctx.pipeline(f"affine_matvec:{cols}:{group}" + gh.t_suffix(dtype))
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.RES_SLOT, 4, 0)]
        rm = rt.make_record(pm, bufs, [(5, rows)], (512, 1, 1), (256, 1, 1))
        chunk = 1024
        parts = (rows + chunk - 1) // chunk
        pa = ctx.pipeline("argmax_fp16_partials")
        pr = ctx.pipeline("argmax_key_reduce")
        ra = rt.make_record(pa, [(gh.RES_SLOT, 0, 0), (gh.AUX_SLOT, 1, 0)], [(2, rows), (3, chunk)], (parts, 1, 1), (256, 1, 1))
        rr = rt.make_record(pr, [(gh.AUX_SLOT, 0, 0), (gh.Y_SLOT, 1, 0)], [(2, parts)], (1, 1, 1), (256, 1, 1))
        assert ctx.interpret_decode(ctx.table([rm, ra, rr])) == 3
        ctx.wait()
        assert int(ctx.read(gh.Y_SLOT, np.int32, 1)[0]) == want[0]


def test_lm_head_argmax_logit_cap(ctx):
    """cap * tanh(v / cap) is applied in fp32 before the fp16/bf16 rounding that forms the key
    (lut_matvec.metal:4194-4199).  The cap compresses the top logits into a few representable
    values, so the winner is checked by value: its capped, rounded logit equals the best capped,
    rounded logit of the oracle (to one output ulp for the exp-vs-tanh formulation), and where
    the oracle's top value is unique by more than that the index is identical."""
    rows, cols, group = 6000, 1024, 64
    for dtype in (fx.F16, fx.BF16):
        w = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=8)
        x = fx.synth_activation(1, cols, dtype, config=1, tensor=34)
        ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype)[0].astype(np.float64)
        cap = float(np.abs(ref).max()) * 0.75
        capped = fx.from_bits(so.narrow((cap * np.tanh(ref / cap)).astype(np.float32), dtype), dtype).astype(np.float64)
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in w]
        ctx.upload_weights(0, wf.image())
        ctx.put(gh.X_SLOT, x)
        grid_w = 96
        ctx.alloc(gh.AUX_SLOT, grid_w * 8)
        ctx.alloc(gh.Y_SLOT, 4)
        p1 = ctx.pipeline(f"affine_matvec_argmax_c{cols}_r{rows}_g{group}_batched" + gh.t_suffix(dtype))
        p2 = ctx.pipeline(f"lm_head_argmax_reduce_r{rows}")
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0)]
        r1 = rt.make_record(p1, bufs, [(5, 1), (6, cap)], (grid_w, 1, 1), (256, 1, 1))
        r2 = rt.make_record(p2, [(gh.AUX_SLOT, 0, 0), (gh.Y_SLOT, 1, 0)], [(2, 1), (3, grid_w)], (1, 1, 1), (256, 1, 1))
        assert ctx.interpret_decode(ctx.table([r1, r2])) == 2
        ctx.wait()
        got = int(ctx.read(gh.Y_SLOT, np.int32, 1)[0])
        top = capped.max()
        ulp = top * (2.0 ** -10 if dtype == fx.F16 else 2.0 ** -7)
        assert 0 <= got < rows and capped[got] >= top - ulp, (got, capped[got], top)
        assert capped[got] < cap * 1.001
        order = np.sort(capped)
        if order[-1] - order[-2] > 2 * ulp:
            assert got == int(np.argmax(capped))


def test_argmax_ties_and_signed_zero(ctx):
    vals = np.zeros(5000, np.float16)
    vals[[17, 400, 4999]] = 3.5                  # ties -> lowest index
    logits = vals.view(np.uint16).copy()
    ctx.put(gh.RES_SLOT, logits)
    ctx.alloc(gh.AUX_SLOT, 64 * 8)
    ctx.alloc(gh.Y_SLOT, 4)
    pa, pr = ctx.pipeline("argmax_fp16_partials"), ctx.pipeline("argmax_key_reduce")

    def run(n):
        ra = rt.make_record(pa, [(gh.RES_SLOT, 0, 0), (gh.AUX_SLOT, 1, 0)], [(2, n), (3, 512)], ((n + 511) // 512, 1, 1), (256, 1, 1))
        rr = rt.make_record(pr, [(gh.AUX_SLOT, 0, 0), (gh.Y_SLOT, 1, 0)], [(2, (n + 511) // 512)], (1, 1, 1), (256, 1, 1))
        ctx.interpret_decode(ctx.table([ra, rr]))
        ctx.wait()
        return int(ctx.read(gh.Y_SLOT, np.int32, 1)[0])

    assert run(5000) == 17
    z = np.full(3000, 0x8000, np.uint16)         # all -0, one +0 later: -0 == +0 -> index 0
    z[1234] = 0x0000
    ctx.write(gh.RES_SLOT, z)
    assert run(3000) == 0 == so.argmax16(z)
    neg = (-np.abs(np.random.default_rng(3).normal(0, 1, 3000)) - 0.1).astype(np.float16).view(np.uint16)
    ctx.write(gh.RES_SLOT, neg)
    assert run(3000) == so.argmax16(neg)


def test_ternary_affine_names_bank4_and_trit5(ctx):
    """The production ternary pipeline names, the four-member projection bank, and the trit5
    encoding of the same logical matrix all give the bits of the plain ternary2 kernel."""
    cols = 5120
    member_rows = [40, 24, 56, 16]
    rows = sum(member_rows)
    codes = fx.synth_signed_codes(fx.TERNARY2, rows, cols, config=3, tensor=2)
    scales = fx.synth_signed_scales(rows, cols, config=3, tensor=2)
    p2 = fx.pack_signed_np(codes, fx.TERNARY2)
    stride5 = (((cols + 4) // 5) + 15) // 16 * 16
    p5 = fx.pack_signed_np(codes, fx.TRIT5, stride5)
    x = fx.synth_activation(1, cols, fx.F16, config=3, tensor=1)
    ref = so.signed_matvec(so.TERNARY2, p2, scales, fx.from_bits(x, fx.F16), rows, cols, cols, 128)
    wf = gh.WeightFile()
    o2, o5, os_ = wf.add(p2), wf.add(p5), wf.add(scales)
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x)
    for s in (gh.Y_SLOT, gh.RES_SLOT, gh.AUX_SLOT, gh.AUX2_SLOT, 6, 7):
        ctx.alloc(s, rows * 2)
    grid = ((rows + 7) // 8, 1, 1)

    def run(name, bufs, consts):
        ctx.encode_decode(rt.make_record(ctx.pipeline(name), bufs, consts, grid, (256, 1, 1)))
        ctx.wait()

    run("signed_ternary_matvec_g128_rows8", [(0, 0, o2), (0, 1, os_), (gh.X_SLOT, 2, 0), (gh.Y_SLOT, 3, 0)], [(4, rows), (5, cols)])
    plain = ctx.read(gh.Y_SLOT, np.uint16, rows)
    gh.check_outputs(plain.reshape(1, rows), ref, fx.F16, "ternary2 plain")
    run("signed_ternary_affine_matvec_g128_rows8",
        [(0, 0, o2), (0, 1, os_), (0, 2, os_), (gh.X_SLOT, 3, 0), (gh.RES_SLOT, 4, 0)], [(5, rows), (6, cols)])
    assert np.array_equal(ctx.read(gh.RES_SLOT, np.uint16, rows), plain)
    run("signed_trit5_matvec_g128_rows8", [(0, 0, o5), (0, 1, os_), (gh.X_SLOT, 2, 0), (gh.RES_SLOT, 3, 0)], [(4, rows), (5, cols)])
    t5 = ctx.read(gh.RES_SLOT, np.uint16, rows)
    # 80-column units sum in a different order than 64-column units: same value to the last ulp
    gh.check_outputs(t5.reshape(1, rows), ref, fx.F16, "trit5 vs oracle")
    assert np.abs(t5.astype(int) - plain.astype(int)).max() <= 1
    outs = [gh.AUX_SLOT, gh.AUX2_SLOT, 6, 7]
    run("signed_ternary_affine_bank4_matvec_g128_rows8",
        [(0, 0, o2), (0, 1, os_), (0, 2, os_), (gh.X_SLOT, 3, 0)] + [(s, 4 + i, 0) for i, s in enumerate(outs)],
        [(8 + i, r) for i, r in enumerate(member_rows)] + [(12, cols)])
    start = 0
    for s, r in zip(outs, member_rows):
        assert np.array_equal(ctx.read(s, np.uint16, r), plain[start:start + r])
        start += r
    # the MLX golden fixtures re-encoded as trit5: every partial sum is exact, so the trit5
    # kernel must reproduce the same bit patterns the ternary2 kernel does
    g = fx.golden_vectors()
    for key in ("ternary_qmv_mlx_k512", "ternary_qmv_mlx_k5120_m3"):
        case = g[key]
        gc, gs, gx = fx.mlx_ternary_fixture(case["rows"], case["cols"], case["batch"], case["scale_unit"])
        st = (((case["cols"] + 4) // 5) + 15) // 16 * 16
        wf = gh.WeightFile()
        oc, os3 = wf.add(fx.pack_signed_np(gc, fx.TRIT5, st)), wf.add(gs)
        ctx.upload_weights(0, wf.image())
        ctx.put(gh.X_SLOT, gx)
        ctx.alloc(gh.Y_SLOT, case["batch"] * case["rows"] * 2)
        ctx.encode_decode(rt.make_record(ctx.pipeline("signed_trit5_matvec_g128_rows8"),
                                         [(0, 0, oc), (0, 1, os3), (gh.X_SLOT, 2, 0), (gh.Y_SLOT, 3, 0)],
                                         [(4, case["rows"]), (5, case["cols"])], (2, case["batch"], 1), (256, 1, 1)))
        ctx.wait()
        want = np.array([int(b, 16) for b in case["expected_bits"]], np.uint16)
        assert np.array_equal(ctx.read(gh.Y_SLOT, np.uint16, want.size), want), key
    # trit5 with K = 17408 (not a multiple of 5; rows padded to 3488 bytes)
    rows2, cols2 = 64, 17408
    codes2 = fx.synth_signed_codes(fx.TERNARY2, rows2, cols2, config=3, tensor=5)
    scales2 = fx.synth_signed_scales(rows2, cols2, config=3, tensor=5)
    stride = (((cols2 + 4) // 5) + 15) // 16 * 16
    assert stride == 3488
    p5b = fx.pack_signed_np(codes2, fx.TRIT5, stride)
    x2 = fx.synth_activation(1, cols2, fx.BF16, config=3, tensor=6)
    ref2 = so.signed_matvec(so.TRIT5, p5b, scales2, fx.from_bits(x2, fx.BF16), rows2, cols2, cols2, 128)
    wf = gh.WeightFile()
    oc, os2 = wf.add(p5b), wf.add(scales2)
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x2)
    ctx.alloc(gh.Y_SLOT, rows2 * 2)
    ctx.encode_decode(rt.make_record(ctx.pipeline("signed_trit5_matvec_g128_rows8@bf16"),
                                     [(0, 0, oc), (0, 1, os2), (gh.X_SLOT, 2, 0), (gh.Y_SLOT, 3, 0)],
                                     [(4, rows2), (5, cols2)], (16, 1, 1), (256, 1, 1)))
    ctx.wait()
    gh.check_outputs(ctx.read(gh.Y_SLOT, np.uint16, rows2).reshape(1, rows2), ref2, fx.BF16, "trit5 K=17408")


def test_bad_records_are_rejected_before_launch(ctx):
    rows, cols, group = 64, 1024, 64
    w = fx.synth_affine(rows, cols, group, fx.F16)
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in w]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, fx.synth_activation(1, cols, fx.F16))
    ctx.alloc(gh.Y_SLOT, rows * 2)
    pipe = ctx.pipeline(f"affine_matvec:{cols}:{group}")
    good = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
    with pytest.raises(rt.SmeltHipError) as e:      # more rows than the output slot holds
        ctx.encode_decode(rt.make_record(pipe, good, [(5, rows * 4)], (8, 1, 1), (256, 1, 1)))
    assert e.value.code == -6
    with pytest.raises(rt.SmeltHipError) as e:      # a binding the kernel does not have
        ctx.encode_decode(rt.make_record(pipe, good + [(gh.Y_SLOT, 9, 0)], [(5, rows)], (8, 1, 1), (256, 1, 1)))
    assert e.value.code == -5
    with pytest.raises(rt.SmeltHipError) as e:      # missing constant
        ctx.encode_decode(rt.make_record(pipe, good, [], (8, 1, 1), (256, 1, 1)))
    assert e.value.code == -5
    with pytest.raises(rt.SmeltHipError) as e:      # output bound to the read-only weights slot
        bad = good[:4] + [(0, 4, 0)]
        ctx.encode_decode(rt.make_record(pipe, bad, [(5, rows)], (8, 1, 1), (256, 1, 1)))
    assert e.value.code == -1
    with pytest.raises(rt.SmeltHipError) as e:      # unknown offset kind is an emitter/runtime mismatch
        bad = good[:3] + [(gh.X_SLOT, 3, 0, 9), (gh.Y_SLOT, 4, 0)]
        ctx.encode_prefill(rt.make_record(pipe, bad, [(5, rows)], (8, 1, 1), (256, 1, 1)), seq_len=1)
    assert e.value.code == -3 and "offsetKind" in e.value.message
    with pytest.raises(rt.SmeltHipError) as e:
        ctx.pipeline("affine_matvec:10x:64")
    assert e.value.code == -3
    with pytest.raises(rt.SmeltHipError) as e:
        ctx.pipeline("causal_gqa_attn_cached_f32")
    assert e.value.code == -4
    # a missing function becomes a fallback-to-previous slot when the package allows it
    idx = ctx.pipeline("rope_apply_f32", allow_missing=True)
    assert not ctx.pipeline_ready(idx)
    # everything still works afterwards
    assert ctx.encode_decode(rt.make_record(pipe, good, [(5, rows)], (8, 1, 1), (256, 1, 1))) == 1
    ctx.wait()


def test_fused_argmax_at_the_largest_vocabulary(ctx):
    """The key holds 18 index bits (lut_matvec.metal:4048-4074): 262 144 rows is the largest table.
    The winning row is planted first at the very last index, then duplicated at an earlier one
    (identical rows give identical logits): the tie must go to the lower index."""
    rows, cols, group, dtype = 1 << 18, 256, 64, fx.F16
    rng = np.random.default_rng(7)
    packed = rng.integers(0, 256, (rows, cols // 2), dtype=np.uint8)
    scales = fx.f16_bits(np.full((rows, cols // group), 0.01, np.float32))
    biases = fx.f16_bits(np.full((rows, cols // group), -0.075, np.float32))
    x = fx.f16_bits(np.abs(rng.normal(0, 1, (1, cols))).astype(np.float32))      # positive activations
    packed[rows - 1] = 0xFF                                                       # largest code everywhere: the unique maximum
    p1 = ctx.pipeline(f"affine_matvec_argmax_c{cols}_r{rows}_g{group}_batched")
    p2 = ctx.pipeline(f"lm_head_argmax_reduce_r{rows}")
    grid_w = 1024
    for dup in (None, 123457):
        if dup is not None:
            packed[dup] = 0xFF
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in (packed, scales, biases)]
        ctx.upload_weights(0, wf.image())
        ctx.put(gh.X_SLOT, x)
        ctx.alloc(gh.AUX_SLOT, grid_w * 8)
        ctx.alloc(gh.Y_SLOT, 4)
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0)]
        r1 = rt.make_record(p1, bufs, [(5, 1), (6, 0.0)], (grid_w, 1, 1), (256, 1, 1))
        r2 = rt.make_record(p2, [(gh.AUX_SLOT, 0, 0), (gh.Y_SLOT, 1, 0)], [(2, 1), (3, grid_w)], (1, 1, 1), (256, 1, 1))
        assert ctx.interpret_decode(ctx.table([r1, r2])) == 2
        ctx.wait()
        assert int(ctx.read(gh.Y_SLOT, np.int32, 1)[0]) == (rows - 1 if dup is None else dup)
    # one row more does not fit the key: the launch is refused, nothing runs
    with pytest.raises(rt.SmeltHipError):
        ctx.pipeline(f"affine_matvec_argmax_c{cols}_r{rows + 8}_g{group}_batched")
        wf = gh.WeightFile()
        offs = [wf.add(np.zeros((rows + 8, cols // 2), np.uint8)), wf.add(np.zeros((rows + 8, 4), np.uint16)), wf.add(np.zeros((rows + 8, 4), np.uint16))]
        ctx.upload_weights(0, wf.image())
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0)]
        ctx.encode_decode(rt.make_record(ctx.pipeline(f"affine_matvec_argmax_c{cols}_r{rows + 8}_g{group}_batched"), bufs,
                                         [(5, 1), (6, 0.0)], (grid_w, 1, 1), (256, 1, 1)))


@pytest.fixture(scope="module")
def auto_ctx():
    c = rt.Context()            # default engine: the ternary qmm record takes the streaming kernel up to 64 tokens
    yield c
    c.close()


def test_ternary_qmm_streaming_kernel_reproduces_the_golden_bits_too(auto_ctx):
    test_ternary_qmm_reproduces_mlx_golden_bits_and_byte_lane_subscales(auto_ctx)
    test_ternary_qmm_matches_per_row_matvec_and_oracle(auto_ctx)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("shape", [(1003, 5120, 14), (40, 512, 6), (200, 17408, 33), (2050, 1536, 64), (96, 1024, 9), (77, 2816, 20)])
def test_ternary_qmm_streaming_kernel_shapes(ctx, auto_ctx, dtype, shape):
    """The streaming ternary qmm against the oracle's per-element fp16 dequantisation and against the token-slab
    kernel (one output step apart at most: the two add up a row in different orders): ragged rows, one to four
    16-token passes, eight and sixteen staged token rows, rows of four, twelve, forty and 136 groups, separate
    bias plane, bf16 rows (converted to fp16 as in the token-slab kernel)."""
    rows, cols, batch = shape
    codes = fx.synth_signed_codes(fx.TERNARY2, rows, cols, config=3, tensor=rows % 7)
    scales = fx.synth_signed_scales(rows, cols, config=3, tensor=rows % 7)
    bias_scales = np.roll(scales, 3, axis=0)
    packed = fx.pack_signed_np(codes, fx.TERNARY2)
    x = fx.synth_activation(batch, cols, dtype, config=3, tensor=batch)
    out = {}
    for name, c in (("stream", auto_ctx), ("slab", ctx)):
        wf = gh.WeightFile()
        oc, os_, ob = wf.add(packed), wf.add(scales), wf.add(bias_scales)
        c.upload_weights(0, wf.image())
        c.put(gh.X_SLOT, x)
        c.alloc(gh.Y_SLOT, batch * rows * 2)
        rec = rt.make_record(c.pipeline("signed_ternary_affine_qmm_g128_bm32_bn32_bk32" + gh.t_suffix(dtype)),
                             [(0, 0, oc), (0, 1, os_), (0, 2, ob), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)],
                             [(5, rows), (6, cols), (7, batch)], ((rows + 63) // 64, (batch + 31) // 32, 1), (256, 1, 1))
        assert c.encode_decode(rec) == 1
        c.wait()
        out[name] = c.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)
        assert np.array_equal(out[name], (c.encode_decode(rec), c.wait(), c.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows))[2])
    gh.check_steps(out["stream"], out["slab"], dtype, f"ternary qmm, streaming against token-slab {shape}", max_steps=1, min_exact=0.9)
    if dtype == fx.F16:
        ref = so.ternary_affine_qmm(packed, scales, x, rows, cols, bias_scales=bias_scales)
        gh.check_outputs(out["stream"], ref, dtype, f"ternary qmm streaming {shape}")


def test_ternary_qmm_streaming_kernel_is_bit_exact_where_the_sums_are(auto_ctx):
    """The MLX fixture of the golden test at 512, 768 and 1024 columns (the golden shape itself, 256 columns, runs on the
    streaming kernel in `test_ternary_qmm_streaming_kernel_reproduces_the_golden_bits_too`): every partial sum is exact,
    so the bits must be the oracle's, with ordinary scales, with scales whose quarter, sixteenth and sixty-fourth round
    in the fp16 subnormal range, and with a separate bias plane."""
    case = fx.golden_vectors()["ternary_qmm_mlx_m14"]
    small = ["1b95", "1797", "1b93", "17ff", "1a01"]
    for cols, rows, batch in ((512, 24, 14), (1024, 40, 37), (768, 19, 9)):
        for scale_bits, separate_bias in ((case["scale_bits"], False), (small, False), (small, True)):
            codes, scales, x = fx.mlx_ternary_qmm_fixture(rows, cols, batch, scale_bits)
            bias_scales = np.roll(scales, 1, axis=0) if separate_bias else scales
            packed = fx.pack_signed_np(codes, fx.TERNARY2)
            ref = so.ternary_affine_qmm(packed, scales, x, rows, cols, bias_scales=bias_scales)
            want = ref.astype(np.float16).view(np.uint16).ravel()
            wf = gh.WeightFile()
            oc, os_, ob = wf.add(packed), wf.add(scales), wf.add(bias_scales)
            auto_ctx.upload_weights(0, wf.image())
            auto_ctx.put(gh.X_SLOT, x)
            auto_ctx.alloc(gh.Y_SLOT, batch * rows * 2)
            auto_ctx.encode_decode(rt.make_record(
                auto_ctx.pipeline("signed_ternary_affine_qmm_g128_bm32_bn32_bk32"),
                [(0, 0, oc), (0, 1, os_), (0, 2, ob), (gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)],
                [(5, rows), (6, cols), (7, batch)], (1, (batch + 31) // 32, 1), (256, 1, 1)))
            auto_ctx.wait()
            assert np.array_equal(auto_ctx.read(gh.Y_SLOT, np.uint16, want.size), want), (cols, scale_bits, separate_bias)
