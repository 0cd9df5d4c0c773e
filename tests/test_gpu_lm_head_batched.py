"""GPU parity: the lm_head (matvec + argmax) over several tokens under the default engine.

From two tokens on the fused record runs as two launches: the streaming qmm leaves the rounded logits of every
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


def test_lm_head_with_a_logit_cap_or_one_token_keeps_the_fused_kernel(ctx):
    rows, cols, group, grid_w, dtype = 20000, 1024, 64, 160, fx.BF16
    w = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=7)
    x = fx.synth_activation(4, cols, dtype, config=1, tensor=44)
    launched, got = run_lm_head(ctx, w, x, rows, cols, group, dtype, 4, grid_w, cap=30.0)
    assert launched == 2 and all(0 <= t < rows for t in got)
    launched, got = run_lm_head(ctx, w, x[:1], rows, cols, group, dtype, 1, grid_w)
    assert launched == 2 and 0 <= got[0] < rows


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
