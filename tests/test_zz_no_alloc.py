"""GPU parity of the allocation-free entry point: smelt_hip_encode_prefill_record_static_scratch
against smelt_hip_encode_prefill_record on the split-K skinny qmm, bit for bit, on two calls in a
row (the second with a smaller input), plus the size limit; and on a token-slab record whose tiles
the token-tile kernel splits along K (its partial sums then live in the same static array)."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import runtime as rt

pytestmark = pytest.mark.gpu


def _run(ctx, encode, w_offs, x_bits, rows, cols, ksplit, pipe_name, nmat_bufs):
    batch = x_bits.shape[0]
    ctx.put(gh.X_SLOT, x_bits)
    ctx.alloc(gh.Y_SLOT, batch * rows * 2)
    pipe = ctx.pipeline(pipe_name)
    nb = len(w_offs)
    bufs = [(0, i, o) for i, o in enumerate(w_offs)] + [(gh.X_SLOT, nb, 0), (gh.Y_SLOT, nb + 1, 0)]
    tiles = (rows + 31) // 32
    rec = rt.make_record(pipe, bufs, [(nb + 2, 0, rt.CONST_SEQ_LEN)], (tiles * ksplit, 32, 1), (256, 1, 1),
                         grid_kinds=(0, rt.GRID_SEQ_LEN_CEIL_DIV, 0))
    assert encode(rec, seq_len=batch) == 1
    ctx.wait()
    return ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows)


def test_static_scratch_matches_allocated_workspace_twice_in_a_row():
    dtype = fx.BF16
    ctx = rt.Context()
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)   # the split-K kernels: the ones that use the scratch
    try:
        # first call: 13 tokens on 416 x 2560 split 4 ways (13 row tiles x 4 partials)
        # second call: 5 tokens on the first 100 rows of a 1536-column matrix split 3 ways
        cases = [(416, 2560, 13, 4, 31), (100, 1536, 5, 3, 32)]
        for rows, cols, batch, ksplit, tensor in cases:
            w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=tensor)
            x = fx.synth_activation(batch, cols, dtype, config=4, tensor=100 + tensor, outlier_frac=0.01)
            wf = gh.WeightFile()
            offs = [wf.add(a) for a in w]
            ctx.upload_weights(0, wf.image())
            name = f"affine_matvec_c{cols}_r{rows}_g64_batched_skinny@bf16"
            print(f"\n  static scratch case rows={rows} cols={cols} batch={batch} ksplit={ksplit}", flush=True)
            want = _run(ctx, ctx.encode_prefill, offs, x, rows, cols, ksplit, name, 1)
            got = _run(ctx, ctx.encode_prefill_static_scratch, offs, x, rows, cols, ksplit, name, 1)
            assert np.array_equal(got, want), (rows, cols, batch, ksplit)
            ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
            gh.check_outputs(got, ref, dtype, f"static-scratch skinny qmm {rows}x{cols} M={batch}")
            again = _run(ctx, ctx.encode_prefill_static_scratch, offs, x, rows, cols, ksplit, name, 1)
            assert np.array_equal(again, want)
    finally:
        ctx.close()


def test_static_scratch_call_allocates_nothing():
    """Free device memory (hipMemGetInfo) is the same before and after calls of the allocation-free entry point,
    and a call launches one kernel: the record's own."""
    dtype = fx.BF16
    ctx = rt.Context()
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)
    try:
        rows, cols, batch, ksplit = 416, 2560, 13, 4
        w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=31)
        x = fx.synth_activation(batch, cols, dtype, config=4, tensor=131)
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in w]
        ctx.upload_weights(0, wf.image())
        ctx.put(gh.X_SLOT, x)
        ctx.alloc(gh.Y_SLOT, batch * rows * 2)
        pipe = ctx.pipeline(f"affine_matvec_c{cols}_r{rows}_g64_batched_skinny@bf16")
        bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
        tiles = (rows + 31) // 32
        rec = rt.make_record(pipe, bufs, [(5, 0, rt.CONST_SEQ_LEN)], (tiles * ksplit, 32, 1), (256, 1, 1),
                             grid_kinds=(0, rt.GRID_SEQ_LEN_CEIL_DIV, 0))
        assert ctx.encode_prefill_static_scratch(rec, seq_len=batch) == 1     # first call: whatever lazy set-up there is
        ctx.wait()
        free_before, _ = ctx.memory_info()
        for _ in range(5):
            assert ctx.encode_prefill_static_scratch(rec, seq_len=batch) == 1
        ctx.wait()
        free_after, _ = ctx.memory_info()
        assert free_after == free_before, (free_before, free_after)
        ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
        gh.check_outputs(ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows), ref, dtype, "static scratch after repeated calls")
    finally:
        ctx.close()


def test_static_scratch_rejects_partials_beyond_its_size():
    dtype = fx.F16
    ctx = rt.Context()
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)
    try:
        # 4096 workgroup partials of 4 KB fit; 140 row tiles x 32 splits = 4480 do not.  The context's
        # own 64 MB workspace takes the same record.
        rows, cols, batch, ksplit = 4480, 2048, 4, 32
        w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=33)
        x = fx.synth_activation(batch, cols, dtype, config=4, tensor=133)
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in w]
        ctx.upload_weights(0, wf.image())
        name = f"affine_matvec_c{cols}_r{rows}_g64_batched_skinny@f16"
        with pytest.raises(rt.SmeltHipError) as err:
            _run(ctx, ctx.encode_prefill_static_scratch, offs, x, rows, cols, ksplit, name, 1)
        assert "exceed the workspace" in err.value.message
        y = _run(ctx, ctx.encode_prefill, offs, x, rows, cols, ksplit, name, 1)
        ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype)
        gh.check_outputs(y, ref, dtype, "allocated workspace takes the larger record")
    finally:
        ctx.close()


def test_static_scratch_holds_the_token_tile_kernels_partials():
    """200 x 9216 at 300 and then 140 tokens: few tiles and long rows, so three workgroups share each
    tile along K; their partials go to the static array in one call and to the context's workspace in
    the other, and the results are the same bits."""
    dtype = fx.BF16
    ctx = rt.Context()
    try:
        rows, cols = 200, 9216
        w = fx.synth_affine(rows, cols, 64, dtype, config=4, tensor=34)
        wf = gh.WeightFile()
        offs = [wf.add(a) for a in w]
        ctx.upload_weights(0, wf.image())
        pipe = ctx.pipeline(f"affine_matvec_c{cols}_r{rows}_g64_batched_full_b64@bf16")
        for batch in (300, 140):
            x = fx.synth_activation(batch, cols, dtype, config=4, tensor=200 + batch)
            ctx.put(gh.X_SLOT, x)
            ctx.alloc(gh.Y_SLOT, batch * rows * 2)
            bufs = [(0, i, o) for i, o in enumerate(offs)] + [(gh.X_SLOT, 3, 0), (gh.Y_SLOT, 4, 0)]
            rec = rt.make_record(pipe, bufs, [(5, 0, rt.CONST_SEQ_LEN)], ((rows + 63) // 64, 64, 1), (256, 1, 1),
                                 grid_kinds=(0, rt.GRID_SEQ_LEN_CEIL_DIV, 0))
            outs = []
            for encode in (ctx.encode_prefill, ctx.encode_prefill_static_scratch, ctx.encode_prefill_static_scratch):
                print(f"\n  token-tile split case batch={batch} via {encode.__name__}", flush=True)
                assert encode(rec, seq_len=batch) == 1
                ctx.wait()
                outs.append(ctx.read(gh.Y_SLOT, np.uint16, batch * rows).reshape(batch, rows))
            assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[1], outs[2])
            ref = so.affine_matvec(*w, fx.from_bits(x, dtype), rows, cols, 64, dtype, threads=True)
            gh.check_outputs(outs[1], ref, dtype, f"static-scratch token-tile qmm M={batch}")
    finally:
        ctx.close()
