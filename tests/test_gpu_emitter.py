"""GPU: records produced by the emitters, interpreted eagerly and replayed as a HIP graph,
reproduce the oracle on a small decode-step-shaped table for each weight family."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from gpu_harness import SIGNED_SWIGLU_STEPS
from oracle import oracle as so
from smelt_amd import compiler as cc
from smelt_amd import runtime as rt

pytestmark = pytest.mark.gpu

H_SLOT, Q_SLOT, FFN_SLOT, OUT_SLOT, KEY_SLOT, TOK_SLOT, RES_SLOT = 1, 2, 3, 4, 5, 6, 7


def build_affine_table(dtype):
    hidden, qdim, ffn, vocab, group = 1024, 512, 3584, 4096, 64
    lay = cc.Layout()
    wq, wg, wu = lay.affine(qdim, hidden, group), lay.affine(ffn, hidden, group), lay.affine(ffn, hidden, group)
    wd, wl = lay.affine(hidden, ffn, group), lay.affine(vocab, hidden, group)
    image = np.zeros(lay.total_bytes, np.uint8)
    tensors = {}
    for i, (name, e) in enumerate((("q", wq), ("gate", wg), ("up", wu), ("down", wd), ("lm_head", wl))):
        t = fx.synth_affine(e.rows, e.cols, group, dtype, config=1, tensor=20 + i)
        if name in ("down", "lm_head"):
            # the chain multiplies magnitudes up; the two deep tensors are scaled by 2^-6 (exact in
            # both 16-bit types) so that every intermediate and every logit stays inside fp16
            t = (t[0], fx.to_bits(fx.from_bits(t[1], dtype) / 64.0, dtype), fx.to_bits(fx.from_bits(t[2], dtype) / 64.0, dtype))
        cc.write_affine(image, e, *t)
        tensors[name] = t
    em = cc.Emitter(rt.ACT_BF16 if dtype == fx.BF16 else rt.ACT_F16)
    em.matvec(0, wq, cc.bind(H_SLOT), cc.bind(Q_SLOT))
    em.gate_up_swiglu(0, wg, wu, cc.bind(H_SLOT), cc.bind(FFN_SLOT))
    em.matvec_add(0, wd, cc.bind(FFN_SLOT), cc.bind(OUT_SLOT), cc.bind(RES_SLOT))
    em.lm_head_argmax(0, wl, cc.bind(OUT_SLOT), cc.bind(KEY_SLOT), cc.bind(TOK_SLOT))
    return em, image, tensors, (hidden, qdim, ffn, vocab, group)


@pytest.mark.filterwarnings("error::RuntimeWarning")   # an fp16 overflow in the reference chain would be one
@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_affine_decode_table_eager_and_graph(dtype):
    em, image, tensors, (hidden, qdim, ffn, vocab, group) = build_affine_table(dtype)
    ctx = rt.Context(act_dtype=rt.ACT_BF16 if dtype == fx.BF16 else rt.ACT_F16)
    try:
        em.install(ctx)
        ctx.upload_weights(0, image)
        x = fx.synth_activation(1, hidden, dtype, config=1, tensor=70)
        res = fx.to_bits(fx.rng_for(1, 71).normal(0, 1, (1, hidden)).astype(np.float32), dtype)
        ctx.put(H_SLOT, x)
        ctx.put(RES_SLOT, res)
        ctx.alloc(Q_SLOT, qdim * 2)
        ctx.alloc(FFN_SLOT, ffn * 2)
        ctx.alloc(OUT_SLOT, hidden * 2)
        ctx.alloc(KEY_SLOT, max(em.argmax_partial_bytes, 8))
        ctx.alloc(TOK_SLOT, 4)
        table = em.records()
        assert ctx.interpret_decode(table) == 5
        ctx.submit()
        ctx.wait()
        assert ctx.last_gpu_ns() > 0

        def outputs():
            return (ctx.read(Q_SLOT, np.uint16, qdim), ctx.read(FFN_SLOT, np.uint16, ffn),
                    ctx.read(OUT_SLOT, np.uint16, hidden), int(ctx.read(TOK_SLOT, np.int32, 1)[0]))

        q, act, out, tok = outputs()
        xf = fx.from_bits(x, dtype)
        gh.check_outputs(q.reshape(1, -1), so.affine_matvec(*tensors["q"], xf, qdim, hidden, group, dtype), dtype, "q")
        g = so.affine_matvec(*tensors["gate"], xf, ffn, hidden, group, dtype)
        u = so.affine_matvec(*tensors["up"], xf, ffn, hidden, group, dtype)
        act_ref = fx.from_bits(so.epilogue_affine_swiglu(g, u, dtype), dtype)
        gh.check_outputs(act.reshape(1, -1), gh.swiglu_unrounded(g, u), dtype, "gate_up")
        # downstream references consume the GPU's own upstream bits, as the next kernel does
        d = so.affine_matvec(*tensors["down"], fx.from_bits(act.reshape(1, -1), dtype), hidden, ffn, group, dtype)
        out_ref = fx.from_bits(so.epilogue_residual_add(d, res, dtype), dtype)
        gh.check_outputs(out.reshape(1, -1), out_ref, dtype, "down+add")
        logits = so.affine_matvec(*tensors["lm_head"], fx.from_bits(out.reshape(1, -1), dtype), vocab, hidden, group, dtype)
        assert tok == so.argmax16(so.narrow(logits, dtype)[0])

        # graph replays: eager work and synchronisation between replays, every replay checked
        graph, launches = ctx.capture_decode(table)
        assert launches == 5
        for i in range(3):
            ctx.write(Q_SLOT, np.zeros(qdim, np.uint16))
            ctx.write(OUT_SLOT, np.zeros(hidden, np.uint16))
            ctx.write(TOK_SLOT, np.full(1, -1, np.int32))
            assert ctx.graph_launch(graph) == 5
            ctx.wait()
            q2, act2, out2, tok2 = outputs()
            assert np.array_equal(q2, q) and np.array_equal(act2, act) and np.array_equal(out2, out) and tok2 == tok, i
        ctx.graph_destroy(graph)
    finally:
        ctx.close()


@pytest.mark.parametrize("wdtype", [cc.BINARY1, cc.TERNARY2, cc.TRIT5])
def test_signed_layer_table_decode_and_prefill(wdtype):
    fmt = {cc.BINARY1: fx.BINARY1, cc.TERNARY2: fx.TERNARY2, cc.TRIT5: fx.TRIT5}[wdtype]
    base = fx.TERNARY2 if fmt == fx.TRIT5 else fmt
    hidden, kv, ffn = 1280, 256, 2048
    lay = cc.Layout()
    wk = lay.signed(kv, hidden, wdtype)
    wg, wu = lay.signed(ffn, hidden, wdtype), lay.signed(ffn, hidden, wdtype)
    wd = lay.signed(hidden, ffn, wdtype)
    image = np.zeros(lay.total_bytes, np.uint8)
    t = {}
    for i, (name, e) in enumerate((("k", wk), ("gate", wg), ("up", wu), ("down", wd))):
        codes = fx.synth_signed_codes(base, e.rows, e.cols, config=2, tensor=30 + i)
        scales = fx.synth_signed_scales(e.rows, e.cols, config=2, tensor=30 + i)
        packed = fx.pack_signed_np(codes, fmt, e.packed_row_stride)
        cc.write_signed(image, e, packed, scales)
        t[name] = (packed, scales)
    ctx = rt.Context()
    try:
        # decode table
        em = cc.Emitter()
        em.matvec(0, wk, cc.bind(H_SLOT), cc.bind(Q_SLOT))
        em.gate_up_swiglu(0, wg, wu, cc.bind(H_SLOT), cc.bind(FFN_SLOT))
        em.matvec_add(0, wd, cc.bind(FFN_SLOT), cc.bind(OUT_SLOT), cc.bind(RES_SLOT))
        # prefill table appended to the same pipeline list: k projection over seqLen tokens
        em.matvec(0, wk, cc.bind(H_SLOT), cc.bind(Q_SLOT), batch=1, dynamic=True)
        em.install(ctx)
        ctx.upload_weights(0, image)
        batch = 9
        x = fx.synth_activation(batch, hidden, fx.F16, config=2, tensor=72)
        res = fx.to_bits(fx.rng_for(2, 73).normal(0, 1, (1, hidden)).astype(np.float32), fx.F16)
        ctx.put(H_SLOT, x)
        ctx.put(RES_SLOT, res)
        ctx.alloc(Q_SLOT, batch * kv * 2)
        ctx.alloc(FFN_SLOT, ffn * 2)
        ctx.alloc(OUT_SLOT, hidden * 2)
        recs = em.records()
        decode = ctx.table(list(recs)[:3])
        assert ctx.interpret_decode(decode) == 3
        ctx.wait()
        xf = fx.from_bits(x, fx.F16)
        ofmt = {fx.BINARY1: so.BINARY1, fx.TERNARY2: so.TERNARY2, fx.TRIT5: so.TRIT5}[fmt]
        k_ref = so.signed_matvec(ofmt, *t["k"], xf, kv, hidden, hidden, 128)
        gh.check_outputs(ctx.read(Q_SLOT, np.uint16, kv).reshape(1, -1), k_ref[:1], fx.F16, "k")
        g = so.narrow(so.signed_matvec(ofmt, *t["gate"], xf[:1], ffn, hidden, hidden, 128), fx.F16)
        u = so.narrow(so.signed_matvec(ofmt, *t["up"], xf[:1], ffn, hidden, hidden, 128), fx.F16)
        act = ctx.read(FFN_SLOT, np.uint16, ffn)
        gh.check_steps(act.reshape(1, -1), so.epilogue_signed_swiglu(g, u, so.F16).reshape(1, -1), fx.F16, "signed gate_up", max_steps=SIGNED_SWIGLU_STEPS)
        d = so.signed_matvec(ofmt, *t["down"], fx.from_bits(act.reshape(1, -1), fx.F16), hidden, ffn, ffn, 128)
        out_ref = fx.from_bits(so.epilogue_residual_add(d, res, so.F16), fx.F16)
        gh.check_outputs(ctx.read(OUT_SLOT, np.uint16, hidden).reshape(1, -1), out_ref, fx.F16, "down+add")
        # prefill records at several sequence lengths (ternary switches QMV -> QMM at 6)
        prefill = ctx.table(list(recs)[3:])
        for seq in (1, 4, 5, 6, 9):
            ctx.write(Q_SLOT, np.zeros(batch * kv, np.uint16))
            assert ctx.interpret_prefill(prefill, seq_len=seq) == 1
            ctx.wait()
            y = ctx.read(Q_SLOT, np.uint16, seq * kv).reshape(seq, kv)
            gh.check_outputs(y, k_ref[:seq], fx.F16, f"prefill seq={seq}")
            rest = ctx.read(Q_SLOT, np.uint16, (batch - seq) * kv, offset=seq * kv * 2) if seq < batch else np.zeros(0)
            assert not rest.any(), "tokens past seqLen must not be written"
    finally:
        ctx.close()


@pytest.mark.parametrize("engine", [rt.MATVEC_VECTOR, rt.MATVEC_MATRIX_CORE])
def test_affine_projection_bank_equals_independent_matvecs(engine):
    """One bank dispatch over q|k|v gives the bits of three independent dispatches (on either engine; AUTO picks
    per matrix size, and the bank is larger than its members)."""
    hidden, group = 1024, 64
    member_rows = [2048, 512, 520]
    lay = cc.Layout()
    members = lay.affine_bank(member_rows, hidden, group)
    lone = lay.affine(64, hidden, group)
    # slabs are contiguous per plane and 128-byte aligned; byte counts are unchanged
    assert members[1].offset == members[0].offset + members[0].size_bytes
    assert members[2].scales_offset == members[1].scales_offset + members[1].scales_size_bytes
    assert members[0].offset % 128 == 0 and members[0].scales_offset % 128 == 0 and members[0].biases_offset % 128 == 0
    image = np.zeros(lay.total_bytes, np.uint8)
    for i, e in enumerate(members):
        cc.write_affine(image, e, *fx.synth_affine(e.rows, e.cols, group, fx.F16, config=1, tensor=40 + i))
    ctx = rt.Context()
    try:
        em = cc.Emitter()
        outs = [cc.bind(2, 0), cc.bind(2, 2048 * 2), cc.bind(2, 2560 * 2)]
        assert em.bank_matvec(0, members, cc.bind(1), outs)
        for e, o in zip(members, [cc.bind(3, 0), cc.bind(3, 2048 * 2), cc.bind(3, 2560 * 2)]):
            em.matvec(0, e, cc.bind(1), o)
        assert not em.bank_matvec(0, [members[0], lone], cc.bind(1), outs[:2])   # not contiguous: no bank
        em.install(ctx)
        ctx.set_matvec_engine(engine)
        ctx.upload_weights(0, image)
        ctx.put(1, fx.synth_activation(1, hidden, fx.F16, config=1, tensor=41))
        total = sum(member_rows)
        ctx.alloc(2, total * 2)
        ctx.alloc(3, total * 2)
        assert ctx.interpret_decode(em.records()) == 4
        ctx.wait()
        a, b = ctx.read(2, np.uint16, total), ctx.read(3, np.uint16, total)
        assert a.any() and np.array_equal(a, b)
    finally:
        ctx.close()


@pytest.mark.parametrize("engine", [rt.MATVEC_VECTOR, rt.MATVEC_MATRIX_CORE])
@pytest.mark.parametrize("fmt,wdtype", [(fx.BINARY1, cc.BINARY1), (fx.TERNARY2, cc.TERNARY2), (fx.TRIT5, cc.TRIT5)])
def test_signed_projection_bank(fmt, wdtype, engine):
    """q|k|v of a signed format laid out as one bank: contiguous code and scale slabs, one dispatch
    (binary, ternary and five-digit-byte members alike); every member against the oracle, on both
    matvec engines."""
    hidden = 1280
    member_rows = [520, 136, 128]
    lay = cc.Layout()
    members = lay.signed_bank(member_rows, hidden, wdtype)
    assert members[1].offset == members[0].offset + members[0].size_bytes
    assert members[2].scales_offset == members[1].scales_offset + members[1].scales_size_bytes
    assert members[0].offset % 128 == 0 and members[0].scales_offset % 128 == 0
    image = np.zeros(lay.total_bytes, np.uint8)
    tensors = []
    for i, e in enumerate(members):
        codes = fx.synth_signed_codes(fmt, e.rows, hidden, config=2 + fmt, tensor=i)
        scales = fx.synth_signed_scales(e.rows, hidden, config=2 + fmt, tensor=i)
        packed = fx.pack_signed_np(codes, fmt, e.packed_row_stride)
        cc.write_signed(image, e, packed, scales)
        tensors.append((packed, scales))
    dtype = fx.BF16
    ctx = rt.Context(act_dtype=rt.ACT_BF16)
    ctx.set_matvec_engine(engine)
    try:
        em = cc.Emitter(rt.ACT_BF16)
        outs = [cc.bind(2, 0), cc.bind(2, 520 * 2), cc.bind(2, 656 * 2)]
        banked = em.bank_matvec(0, members, cc.bind(1), outs)
        assert banked
        if not banked:
            for e, o in zip(members, outs):
                em.matvec(0, e, cc.bind(1), o)
        em.install(ctx)
        ctx.upload_weights(0, image)
        x = fx.synth_activation(1, hidden, dtype, config=2, tensor=43)
        ctx.put(1, x)
        total = sum(member_rows)
        ctx.alloc(2, total * 2)
        assert ctx.interpret_decode(em.records()) == (1 if banked else 3)
        ctx.wait()
        y = ctx.read(2, np.uint16, total)
        at = 0
        for (packed, scales), e in zip(tensors, members):
            ref = so.signed_matvec(fmt, packed, scales, fx.from_bits(x, dtype), e.rows, hidden, hidden, 128)
            gh.check_outputs(y[at:at + e.rows].reshape(1, -1), ref, dtype, f"bank member of {e.rows} rows")
            at += e.rows
    finally:
        ctx.close()


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_lm_head_argmax_full_vocabulary(dtype):
    """The tied lm_head of the decode-step configuration at its real size (151936 x 1024, affine u4
    g64): the token the fused matvec + argmax returns is the oracle's argmax over all 151936 16-bit
    logits.  The two sides sum in different orders, so a token whose oracle logit has the winner's
    16-bit value counts as the tie it is (lowest index wins only among bit-identical logits)."""
    vocab, hidden, group = 151936, 1024, 64
    lay = cc.Layout()
    wl = lay.affine(vocab, hidden, group)
    w = fx.synth_affine(vocab, hidden, group, dtype, config=1, tensor=168)
    image = np.zeros(lay.total_bytes, np.uint8)
    cc.write_affine(image, wl, *w)
    act = rt.ACT_BF16 if dtype == fx.BF16 else rt.ACT_F16
    ctx = rt.Context(act_dtype=act)
    try:
        em = cc.Emitter(act, ctx.device_info()["compute_units"])
        em.lm_head_argmax(0, wl, cc.bind(H_SLOT), cc.bind(KEY_SLOT), cc.bind(TOK_SLOT))
        em.install(ctx)
        ctx.upload_weights(0, image)
        ctx.alloc(KEY_SLOT, max(em.argmax_partial_bytes, 8))
        ctx.alloc(TOK_SLOT, 4)
        for seed in (9000, 9001, 9002):
            x = fx.to_bits(fx.rng_for(1, seed).normal(0, 1, (1, hidden)).astype(np.float32), dtype)
            ctx.put(H_SLOT, x)
            ctx.interpret_decode(em.records())
            ctx.wait()
            tok = int(ctx.read(TOK_SLOT, np.int32, 1)[0])
            logits = so.narrow(so.affine_matvec(*w, fx.from_bits(x, dtype), vocab, hidden, group, dtype, threads=True), dtype)[0]
            want = so.argmax16(logits)
            assert 0 <= tok < vocab
            assert tok == want or logits[tok] == logits[want], (seed, tok, want)
            print(f"\n  lm_head dtype={dtype} seed={seed}: token {tok} (oracle {want})")
    finally:
        ctx.close()
