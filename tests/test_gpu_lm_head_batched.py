"""GPU parity: the lm_head (matvec + argmax) under the default engine, at one token and over several.

At one token, for rows whose 16-byte pieces leave the fused vector kernel's last pass over a row partly empty (1536,
2560, 3072, 5120 columns ...), the record runs the single-pass kernel with the argmax as its epilogue: the eight-row tiles
that share a partial slot meet through the context workspace, and the last to arrive writes the slot.  From two tokens on the fused record runs as two launches: the streaming qmm leaves the rounded logits of every
token in the context workspace and a second kernel forms the partial keys the record's reduce launch reads.  The
result is the argmax of the logits the streaming kernel produced; against the oracle that is the oracle's token, or a
token whose oracle logit is the winner's or one step of the 16-bit type below it (the two sides add up a row in
different orders)."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import runtime as rt
from test_gpu_matvec import run_affine

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = rt.Context()
    yield c
    c.close()


def ordered(bits):
    b = int(bits)
    if (b & 0x7FFF) == 0:
        b = 0
    return 0xFFFF - b if b & 0x8000 else b ^ 0x8000


def run_lm_head(ctx, w, x, rows, cols, group, dtype, batch, grid_w, cap=0.0):
    wf = gh.WeightFile()
    offs = [wf.add(a) for a in w]
    ctx.upload_weights(0, wf.image())
    ctx.put(gh.X_SLOT, x)
    # every partial slot is filled with a key that would win: a slot the launch leaves unwritten shows as token -1
    ctx.put(gh.AUX_SLOT, np.full(batch * grid_w * 2, 0xFFFFFFFF, np.uint32))
    ctx.alloc(gh.Y_SLOT, batch * 4)
    p1 = ctx.pipeline(f"affine_matvec_argmax_c{cols}_r{rows}_g{group}_batched" + gh.t_suffix(dtype))
    p2 = ctx.pipeline(f"lm_head_argmax_reduce_r{rows}")
    bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.AUX_SLOT, 4, 0)]
    bt = 4
    r1 = rt.make_record(p1, bufs, [(5, batch), (6, cap)], (grid_w, (batch + bt - 1) // bt, 1), (256, 1, 1))
    r2 = rt.make_record(p2, [(gh.AUX_SLOT, 0, 0), (gh.Y_SLOT, 1, 0)], [(2, batch), (3, grid_w)], (batch, 1, 1), (256, 1, 1))
    launched = ctx.interpret_decode(ctx.table([r1, r2]))
    ctx.wait()
    return launched, ctx.read(gh.Y_SLOT, np.int32, batch).tolist()


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("batch", [2, 3, 8, 17])
def test_lm_head_over_several_tokens(ctx, dtype, batch):
    rows, cols, group, grid_w = 20000, 1024, 64, 160
    w = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=7)
    x = fx.synth_activation(batch, cols, dtype, config=1, tensor=40 + batch)
    ref_bits = so.narrow(so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype), dtype)
    launched, got = run_lm_head(ctx, w, x, rows, cols, group, dtype, batch, grid_w)
    assert launched == 3      # logits, partial keys, reduce
    exact = 0
    for b in range(batch):
        want = so.argmax16(ref_bits[b])
        assert 0 <= got[b] < rows, (b, got[b])
        assert ordered(ref_bits[b][want]) - ordered(ref_bits[b][got[b]]) <= 1, (b, got[b], want)
        exact += got[b] == want
    print(f"\n  lm_head {rows}x{cols} batch {batch} dtype={dtype}: {exact}/{batch} tokens are the oracle's")
    # the same record on the vector engine (the fused kernel, one launch) picks tokens of the same standing
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)
    try:
        launched_v, got_v = run_lm_head(ctx, w, x, rows, cols, group, dtype, batch, grid_w)
    finally:
        ctx.set_matvec_engine(rt.MATVEC_AUTO)
    assert launched_v == 2
    for b in range(batch):
        assert abs(ordered(ref_bits[b][got_v[b]]) - ordered(ref_bits[b][got[b]])) <= 1


def test_lm_head_with_a_logit_cap_keeps_the_fused_kernel_over_several_tokens(ctx):
    rows, cols, group, grid_w, dtype = 20000, 1024, 64, 160, fx.BF16
    w = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=7)
    x = fx.synth_activation(4, cols, dtype, config=1, tensor=44)
    launched, got = run_lm_head(ctx, w, x, rows, cols, group, dtype, 4, grid_w, cap=30.0)
    assert launched == 2 and all(0 <= t < rows for t in got)


def capped(values, cap):
    v = np.asarray(values, np.float32)
    return (np.float32(cap) * np.tanh(v / np.float32(cap))).astype(np.float32)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
@pytest.mark.parametrize("rows,cols,grid_w", [(20000, 1536, 160), (20000, 2560, 1024), (4099, 5120, 64), (1003, 768, 7),
                                              (1003, 768, 64), (1003, 768, 126), (20000, 1024, 160)])
def test_lm_head_at_one_token_on_the_single_pass_kernel(ctx, dtype, rows, cols, grid_w):
    """Several tiles per partial slot (sixteen, two or three, nine with a ragged last tile, eighteen, one or two, one;
    the last shape has full passes and keeps the fused kernel); three calls in a row with different inputs, so a
    counter the kernel left behind would show; with and without a logit cap; one launch for the record, one for its
    reduce.  The token is the argmax of the logits the same engine stores through the plain matvec record."""
    group = 64
    w = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=11)
    for call, cap in enumerate((0.0, 0.0, 30.0)):
        x = fx.synth_activation(1, cols, dtype, config=1, tensor=60 + call)
        ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype)
        ref_bits = so.narrow(capped(ref, cap) if cap else ref, dtype)[0]
        want = so.argmax16(ref_bits)
        launched, got = run_lm_head(ctx, w, x, rows, cols, group, dtype, 1, grid_w, cap=cap)
        assert launched == 2
        assert 0 <= got[0] < rows, (call, got)
        assert ordered(ref_bits[want]) - ordered(ref_bits[got[0]]) <= 1, (call, got[0], want)
        if not cap:
            logits = run_affine(ctx, *w, x, dtype, f"affine_matvec:{cols}:{group}", generic=True)[0]
            assert got[0] == so.argmax16(logits), (call, got[0])
        ctx.set_matvec_engine(rt.MATVEC_VECTOR)
        try:
            _, got_v = run_lm_head(ctx, w, x, rows, cols, group, dtype, 1, grid_w, cap=cap)
        finally:
            ctx.set_matvec_engine(rt.MATVEC_AUTO)
        assert abs(ordered(ref_bits[got_v[0]]) - ordered(ref_bits[got[0]])) <= 1


def test_lm_head_at_one_token_finds_a_winner_in_any_tile_and_breaks_ties_by_index(ctx):
    """Rows copied from one another tie exactly (same codes, scales and biases): the lowest index wins, whichever tile
    or partial slot holds it; a planted winner in the first, a middle and the last (ragged) tile is found."""
    rows, cols, group, dtype, grid_w = 1003, 768, 64, fx.BF16, 7
    codes, scales, biases = [a.copy() for a in fx.synth_affine(rows, cols, group, dtype, config=1, tensor=12)]
    x = fx.synth_activation(1, cols, dtype, config=1, tensor=70)
    ref = so.affine_matvec(codes, scales, biases, fx.from_bits(x, dtype), rows, cols, group, dtype)
    top = int(np.argmax(ref[0]))
    c2, s2, b2 = codes, scales, biases
    for plant in ([0], [rows - 1], [501, 77, 1002], [8, 9, 15, 1001]):
        cc, ss, bb = c2.copy(), s2.copy(), b2.copy()
        for r in plant:
            cc[r], ss[r], bb[r] = c2[top], s2[top], b2[top]
        launched, got = run_lm_head(ctx, [cc, ss, bb], x, rows, cols, group, dtype, 1, grid_w)
        assert launched == 2
        assert got[0] == min(plant + [top]), (plant, top, got)


def test_lm_head_at_one_token_keeps_the_fused_kernel_when_the_partials_do_not_fit_the_tiles(ctx):
    """More partial slots than tiles (a slot would stay unwritten) and more than 64 tiles per slot: the kernel the
    record names runs, and every slot is written."""
    rows, cols, group, dtype = 1003, 768, 64, fx.BF16
    w = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=9)
    x = fx.synth_activation(1, cols, dtype, config=1, tensor=52)
    ref_bits = so.narrow(so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype), dtype)[0]
    want = so.argmax16(ref_bits)
    for grid_w in (1, 127, 1024):
        launched, got = run_lm_head(ctx, w, x, rows, cols, group, dtype, 1, grid_w)
        assert launched == 2 and 0 <= got[0] < rows
        assert ordered(ref_bits[want]) - ordered(ref_bits[got[0]]) <= 1, grid_w


def test_lm_head_rows_not_a_multiple_of_the_partial_count(ctx):
    """Ragged split of the rows over the partial slots, a winner in the last rows, and slots that get no row."""
    rows, cols, group, dtype, batch = 1003, 512, 64, fx.BF16, 5
    w = list(fx.synth_affine(rows, cols, group, dtype, config=1, tensor=9))
    x = fx.synth_activation(batch, cols, dtype, config=1, tensor=51)
    ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, group, dtype)
    ref_bits = so.narrow(ref, dtype)
    for grid_w in (7, 64, 1024, 1500):
        launched, got = run_lm_head(ctx, w, x, rows, cols, group, dtype, batch, grid_w)
        assert launched == 3
        for b in range(batch):
            want = so.argmax16(ref_bits[b])
            assert 0 <= got[b] < rows and ordered(ref_bits[b][want]) - ordered(ref_bits[b][got[b]]) <= 1, (grid_w, b)
