"""GPU parity of the signed-activation-view path (signed_quant.metal:746-2260): producers bit for
bit against the oracle, consumers (integer popcount dots, exact) within the fp32 summation-order
tolerance of the other matvec kernels, through hand-built dispatch records with the reference's
bindings and launch shapes."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import runtime as rt

pytestmark = pytest.mark.gpu

W, X, PL, AS, Y, RES, X2 = 0, 1, 2, 3, 4, 5, 6


@pytest.fixture(scope="module", params=[fx.F16, fx.BF16], ids=["f16", "bf16"])
def env(request):
    act, odt = (rt.ACT_F16, so.F16) if request.param == fx.F16 else (rt.ACT_BF16, so.BF16)
    c = rt.Context(act_dtype=act)
    yield c, request.param, odt
    c.close()


def bits(values, dtype):
    return fx.f16_bits(values) if dtype == fx.F16 else fx.bf16_bits(values)


def build_view(ctx, x_bits, planes, tokens=1, grid=None, threads=32, name=None):
    cols = x_bits.size // tokens
    groups = cols // 128
    ctx.put(X, x_bits)
    ctx.alloc(PL, tokens * groups * planes * 16)
    ctx.alloc(AS, tokens * groups * 2)
    name = name or f"signed_activation_bitplanes_i{planes}_g128" + ("_batched" if tokens > 1 else "")
    rec = rt.make_record(ctx.pipeline(name), [(X, 0, 0), (PL, 1, 0), (AS, 2, 0)], [(3, cols)],
                         (grid or groups, tokens, 1), (threads, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    return (ctx.read(PL, np.uint32, tokens * groups * planes * 4).reshape(tokens, groups, planes, 4),
            ctx.read(AS, np.uint16, tokens * groups).reshape(tokens, groups))


@pytest.mark.parametrize("planes", [2, 3, 4, 5, 6])
@pytest.mark.parametrize("cols,tokens,grid,threads", [(256, 1, None, 32), (5120, 1, None, 32), (5120, 1, 7, 256), (1024, 3, None, 64)])
def test_activation_view_producers_are_bit_exact(env, planes, cols, tokens, grid, threads):
    ctx, dtype, odt = env
    rng = fx.rng_for(120, planes * 100 + cols)
    x = rng.normal(0, 1.2, (tokens, cols)).astype(np.float32)
    x[0, :128] = 0.0
    x[-1, 200] = 33.0
    xb = bits(x, dtype)
    got_pl, got_sc = build_view(ctx, xb, planes, tokens, grid, threads)
    for t in range(tokens):
        ref_pl, ref_sc, _ = so.activation_bitplanes(xb[t], planes, odt)
        assert np.array_equal(got_sc[t], ref_sc)
        assert np.array_equal(got_pl[t], ref_pl)


def test_fused_producers(env):
    ctx, dtype, odt = env
    cols = 2048
    rng = fx.rng_for(121, 0)
    g, u = bits(rng.normal(0, 2, cols).astype(np.float32), dtype), bits(rng.normal(0, 1, cols).astype(np.float32), dtype)
    groups = cols // 128
    ctx.put(X, g); ctx.put(X2, u); ctx.alloc(PL, groups * 5 * 16); ctx.alloc(AS, groups * 2); ctx.alloc(Y, cols * 2)
    fused = rt.make_record(ctx.pipeline("swiglu_signed_activation_bitplanes_i5_g128"), [(X, 0, 0), (X2, 1, 0), (PL, 2, 0), (AS, 3, 0)],
                           [(4, cols)], (groups, 1, 1), (32, 1, 1))
    ctx.interpret_decode(ctx.table([fused])); ctx.wait()
    fused_pl, fused_sc = ctx.read(PL, np.uint32, groups * 20), ctx.read(AS, np.uint16, groups)
    # staged on the device: swiglu_fused, then the plain i5 producer -> identical bits
    staged = [rt.make_record(ctx.pipeline("swiglu_fused"), [(X, 0, 0), (X2, 1, 0), (Y, 2, 0)], [(3, cols)], (cols, 1, 1), (256, 1, 1), style=rt.STYLE_THREADS),
              rt.make_record(ctx.pipeline("signed_activation_bitplanes_i5_g128"), [(Y, 0, 0), (PL, 1, 0), (AS, 2, 0)], [(3, cols)], (groups, 1, 1), (32, 1, 1))]
    ctx.interpret_decode(ctx.table(staged)); ctx.wait()
    assert np.array_equal(ctx.read(PL, np.uint32, groups * 20), fused_pl) and np.array_equal(ctx.read(AS, np.uint16, groups), fused_sc)
    ref_pl, ref_sc = so.swiglu_activation_bitplanes(g, u, 5, odt)     # exp may differ in its last bit
    assert np.mean(fused_pl == ref_pl.reshape(-1)) > 0.98 and np.mean(fused_sc == ref_sc) > 0.9
    # sigmoid-mul producer (i6): against the plain producer run on the oracle's staged values
    ctx.alloc(PL, groups * 6 * 16)
    rec = rt.make_record(ctx.pipeline("sigmoid_mul_signed_activation_bitplanes_i6_g128"), [(X, 0, 0), (X2, 1, 0), (PL, 2, 0), (AS, 3, 0)],
                         [(4, cols)], (groups, 1, 1), (32, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    sm_pl, sm_sc = ctx.read(PL, np.uint32, groups * 24), ctx.read(AS, np.uint16, groups)
    ref_pl, ref_sc = so.sigmoid_mul_activation_bitplanes(g, u, 6, odt)
    assert np.mean(sm_pl == ref_pl.reshape(-1)) > 0.98 and np.mean(sm_sc == ref_sc) > 0.9
    ctx.put(Y, so.sigmoid_mul(g, u, odt))
    rec = rt.make_record(ctx.pipeline("signed_activation_bitplanes_i6_g128"), [(Y, 0, 0), (PL, 1, 0), (AS, 2, 0)], [(3, cols)], (groups, 1, 1), (32, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    assert np.mean(ctx.read(PL, np.uint32, groups * 24) == sm_pl) > 0.98
    # norm-scale producer: the scale is an input, everything after it is exact
    x, w = bits(rng.normal(0, 1, cols).astype(np.float32), dtype), bits(rng.normal(0, 0.2, cols).astype(np.float32), dtype)
    rs = so.rms_scale(x, 1e-6, odt)
    ctx.put(RES, np.float32([rs])); ctx.put(X, x); ctx.put(X2, w)
    for planes in (2, 3, 4, 5, 6):
        ctx.alloc(PL, groups * planes * 16)
        rec = rt.make_record(ctx.pipeline(f"norm_scale_signed_activation_bitplanes_i{planes}_g128"),
                             [(RES, 0, 0), (X, 1, 0), (X2, 2, 0), (PL, 3, 0), (AS, 4, 0)], [(5, cols)], (groups, 1, 1), (32, 1, 1))
        ctx.interpret_decode(ctx.table([rec])); ctx.wait()
        ref_pl, ref_sc = so.norm_scale_activation_bitplanes(rs, x, w, planes, odt)
        assert np.array_equal(ctx.read(PL, np.uint32, groups * planes * 4), ref_pl.reshape(-1))
        assert np.array_equal(ctx.read(AS, np.uint16, groups), ref_sc)


def signed_weights(seed, rows, cols, fmt):
    rng = fx.rng_for(122, seed)
    codes = rng.integers(0, 2 if fmt == so.BINARY1 else 3, (rows, cols)).astype(np.uint8)
    scales = fx.f16_bits(np.abs(rng.normal(0, 0.02, (rows, cols // 128))).astype(np.float32) + 1e-3)
    return so.signed_pack(codes, fmt), scales


def run_consumer(ctx, name, mats, pl, asc, rows, cols, tokens=1, residual=None, grid=None):
    wf = gh.WeightFile()
    offs = [(wf.add(p), wf.add(s)) for p, s in mats]
    ctx.upload_weights(W, wf.image())
    ctx.put(PL, pl); ctx.put(AS, asc); ctx.alloc(Y, tokens * rows * 2)
    bufs, i = [], 0
    for oc, os_ in offs:
        bufs += [(W, i, oc), (W, i + 1, os_)]
        i += 2
    bufs += [(PL, i, 0), (AS, i + 1, 0), (Y, i + 2, 0)]
    i += 3
    if residual is not None:
        ctx.put(RES, residual)
        bufs.append((RES, i, 0))
        i += 1
    rec = rt.make_record(ctx.pipeline(name), bufs, [(i, rows), (i + 1, cols)], (grid or (rows + 7) // 8, tokens, 1), (256, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    return ctx.read(Y, np.uint16, tokens * rows).reshape(tokens, rows)


@pytest.mark.parametrize("fmt,planes", [(so.BINARY1, 2), (so.BINARY1, 3), (so.BINARY1, 4), (so.BINARY1, 5), (so.BINARY1, 6),
                                        (so.TERNARY2, 4), (so.TERNARY2, 5), (so.TERNARY2, 6)])
@pytest.mark.parametrize("rows,cols,tokens", [(9, 256, 1), (37, 640, 1), (300, 5120, 1), (1024, 1024, 2), (64, 17408, 1)])
def test_bitplane_matvec(env, fmt, planes, rows, cols, tokens):
    ctx, dtype, odt = env
    stem = "binary" if fmt == so.BINARY1 else "ternary"
    packed, ws = signed_weights(rows + cols + planes, rows, cols, fmt)
    x = bits(fx.rng_for(123, cols).normal(0, 1, (tokens, cols)).astype(np.float32), dtype)
    views = [so.activation_bitplanes(x[t], planes, odt) for t in range(tokens)]
    pl = np.stack([v[0] for v in views]); asc = np.stack([v[1] for v in views])
    got = run_consumer(ctx, f"signed_{stem}_bitplane_i{planes}_matvec_g128_rows8", [(packed, ws)], pl, asc, rows, cols, tokens)
    for t in range(tokens):
        ref = so.signed_bitplane_matvec(fmt, packed, ws, views[t][0], views[t][1], rows, cols, odt)
        gh.check_outputs(got[t], ref, dtype, f"{stem} i{planes} {rows}x{cols}")


@pytest.mark.parametrize("fmt,planes", [(so.BINARY1, 3), (so.BINARY1, 5), (so.TERNARY2, 5)])
def test_bitplane_add_and_gate_up(env, fmt, planes):
    ctx, dtype, odt = env
    stem = "binary" if fmt == so.BINARY1 else "ternary"
    rows, cols = 200, 2560
    x = bits(fx.rng_for(124, planes).normal(0, 1, cols).astype(np.float32), dtype)
    pl, asc, _ = so.activation_bitplanes(x, planes, odt)
    a, b = signed_weights(1, rows, cols, fmt), signed_weights(2, rows, cols, fmt)
    res = bits(fx.rng_for(125, 0).normal(0, 1, rows).astype(np.float32), dtype)
    got = run_consumer(ctx, f"signed_{stem}_bitplane_i{planes}_matvec_add_g128_rows8", [a], pl, asc, rows, cols, residual=res)[0]
    acc = so.signed_bitplane_matvec(fmt, a[0], a[1], pl, asc, rows, cols, odt)
    gh.check_outputs(got, so.widen(so.epilogue_residual_add(acc, res, odt), odt), dtype, "bitplane matvec + residual")
    got = run_consumer(ctx, f"signed_{stem}_bitplane_i{planes}_gate_up_swiglu_g128_rows8", [a, b], pl, asc, rows, cols)[0]
    g = so.narrow(acc, odt)
    u = so.narrow(so.signed_bitplane_matvec(fmt, b[0], b[1], pl, asc, rows, cols, odt), odt)
    gh.check_steps(got, so.epilogue_signed_swiglu(g, u, odt).reshape(np.shape(got)), dtype, "bitplane gate+up+SwiGLU", max_steps=gh.SIGNED_SWIGLU_STEPS)


@pytest.mark.parametrize("planes", [2, 3, 4, 5, 6])
def test_reference_fixture_view_then_matvec_against_the_direct_kernel(planes):
    """SignedQuantKernelTests.swift:1523-1650: builder + bit-plane matvec track the direct binary
    matvec as closely as the quantised activations allow, and match the quantised CPU mirror within
    max(0.02, 1 %)."""
    rows, cols = 9, 256
    groups = cols // 128
    r, c = np.meshgrid(np.arange(rows), np.arange(cols), indexing="ij")
    codes = ((r * 13 + c * 7) & 1).astype(np.uint8)
    ws = fx.f16_bits((0.001953125 * ((np.arange(rows * groups) % 7) + 1)).astype(np.float32)).reshape(rows, groups)
    x = fx.f16_bits((np.sin((np.arange(cols) * 17 + 3).astype(np.float32)) * np.float32(0.75)).astype(np.float32))
    packed = so.signed_pack(codes, so.BINARY1)
    ctx = rt.Context()
    try:
        got_pl, got_sc = build_view(ctx, x, planes)
        got = run_consumer(ctx, f"signed_binary_bitplane_i{planes}_matvec_g128_rows8", [(packed, ws)], got_pl[0], got_sc[0], rows, cols)[0]
    finally:
        ctx.close()
    max_q = 1 if planes == 2 else (1 << (planes - 1)) - 1
    a = so.widen(got_sc[0], so.F16).repeat(128)
    xq = np.sign(so.widen(x, so.F16) / a) * np.floor(np.abs(np.clip(so.widen(x, so.F16) / a, -max_q, max_q)) + 0.5)
    sign = np.where(codes == 0, -1.0, 1.0)
    expected = (xq[None, :] * a[None, :] * sign * so.widen(ws, so.F16).repeat(128, axis=1)).sum(axis=1)
    gotf = fx.from_bits(got, fx.F16).astype(np.float64)
    assert np.all(np.abs(gotf - expected) <= np.maximum(0.02, np.abs(expected) * 0.01))


def test_bad_view_records_are_refused(env):
    ctx, dtype, odt = env
    with pytest.raises(rt.SmeltHipError):
        ctx.pipeline("signed_binary_bitplane_i7_matvec_g128_rows8")
    with pytest.raises(rt.SmeltHipError):
        ctx.pipeline("signed_activation_bitplanes_i1_g128")
    ctx.put(X, np.zeros(256, np.uint16)); ctx.alloc(PL, 2 * 4 * 16); ctx.alloc(AS, 2 * 2)
    pipe = ctx.pipeline("signed_activation_bitplanes_i5_g128")      # needs 2 * 5 * 16 bytes of planes
    with pytest.raises(rt.SmeltHipError):
        ctx.interpret_decode(ctx.table([rt.make_record(pipe, [(X, 0, 0), (PL, 1, 0), (AS, 2, 0)], [(3, 256)], (2, 1, 1), (32, 1, 1))]))
    with pytest.raises(rt.SmeltHipError):
        ctx.interpret_decode(ctx.table([rt.make_record(ctx.pipeline("signed_activation_bitplanes_i4_g128"), [(X, 0, 0), (PL, 1, 0), (AS, 2, 0)],
                                                       [(3, 200)], (2, 1, 1), (32, 1, 1))]))


def test_view_emitters_replay_a_signed_layer():
    """One view per projection-bank input, every binary member consumes it: q/k/v from the hidden
    view, gate+up+SwiGLU from the same view, down + residual from the activation's view."""
    from smelt_amd import compiler as cc
    hidden, ffn, planes = 1024, 2560, 5
    ctx = rt.Context()
    try:
        lay = cc.Layout()
        q, k = lay.signed(512, hidden, cc.BINARY1), lay.signed(256, hidden, cc.BINARY1)
        gate, up = lay.signed(ffn, hidden, cc.BINARY1), lay.signed(ffn, hidden, cc.BINARY1)
        down = lay.signed(hidden, ffn, cc.TERNARY2)
        image = np.zeros(lay.total_bytes, np.uint8)
        tensors = {}
        for i, (name, e) in enumerate((("q", q), ("k", k), ("gate", gate), ("up", up), ("down", down))):
            fmt = so.BINARY1 if e.dtype == cc.BINARY1 else so.TERNARY2
            tensors[name] = signed_weights(50 + i, e.rows, e.cols, fmt) + (fmt,)
            cc.write_signed(image, e, tensors[name][0], tensors[name][1])
        H, V0P, V0S, Q, K, ACTB, V1P, V1S, OUT = 1, 2, 3, 4, 5, 6, 7, 8, 9
        ctx.upload_weights(W, image)
        h = fx.f16_bits(fx.rng_for(126, 0).normal(0, 1, hidden).astype(np.float32))
        ctx.put(H, h)
        for slot, size in ((V0P, hidden // 128 * planes * 16), (V0S, hidden // 128 * 2), (Q, 512 * 2), (K, 256 * 2), (ACTB, ffn * 2),
                           (V1P, ffn // 128 * planes * 16), (V1S, ffn // 128 * 2), (OUT, hidden * 2)):
            ctx.alloc(slot, size)
        em = cc.Emitter(rt.ACT_F16, ctx.device_info()["compute_units"])
        em.activation_view(planes, cc.bind(H), cc.bind(V0P), cc.bind(V0S), hidden)
        em.view_matvec(W, q, planes, cc.bind(V0P), cc.bind(V0S), cc.bind(Q))
        em.view_matvec(W, k, planes, cc.bind(V0P), cc.bind(V0S), cc.bind(K))
        em.view_gate_up_swiglu(W, gate, up, planes, cc.bind(V0P), cc.bind(V0S), cc.bind(ACTB))
        em.activation_view(planes, cc.bind(ACTB), cc.bind(V1P), cc.bind(V1S), ffn)
        em.view_matvec(W, down, planes, cc.bind(V1P), cc.bind(V1S), cc.bind(OUT), residual=cc.bind(H))
        assert em.pipelines == ["signed_activation_bitplanes_i5_g128", "signed_binary_bitplane_i5_matvec_g128_rows8",
                                "signed_binary_bitplane_i5_gate_up_swiglu_g128_rows8", "signed_ternary_bitplane_i5_matvec_add_g128_rows8"]
        em.install(ctx)
        assert ctx.interpret_decode(em.records()) == 6
        ctx.wait()
        pl0, sc0, _ = so.activation_bitplanes(h, planes, so.F16)
        mv = lambda n, pl, sc: so.signed_bitplane_matvec(tensors[n][2], tensors[n][0], tensors[n][1], pl, sc, tensors[n][0].shape[0],
                                                         pl.shape[0] * 128, so.F16)
        gh.check_outputs(ctx.read(Q, np.uint16, 512), mv("q", pl0, sc0), fx.F16, "q from the view")
        gh.check_outputs(ctx.read(K, np.uint16, 256), mv("k", pl0, sc0), fx.F16, "k from the view")
        act = ctx.read(ACTB, np.uint16, ffn)
        ref_act = so.epilogue_signed_swiglu(so.narrow(mv("gate", pl0, sc0), so.F16), so.narrow(mv("up", pl0, sc0), so.F16), so.F16)
        gh.check_steps(act, ref_act.reshape(np.shape(act)), fx.F16, "gate+up+SwiGLU from the view", max_steps=gh.SIGNED_SWIGLU_STEPS)
        pl1, sc1, _ = so.activation_bitplanes(act, planes, so.F16)      # the device's own activations feed the second view
        assert np.array_equal(ctx.read(V1P, np.uint32, pl1.size), pl1.reshape(-1)) and np.array_equal(ctx.read(V1S, np.uint16, sc1.size), sc1)
        ref_out = so.epilogue_residual_add(mv("down", pl1, sc1), h, so.F16)
        gh.check_outputs(ctx.read(OUT, np.uint16, hidden), so.widen(ref_out, so.F16), fx.F16, "down + residual from the view")
    finally:
        ctx.close()


def run_bank(ctx, name, mats, inputs, member_rows, cols, dtype):
    """mats: [(packed, scales)] (one slab, or two matrices); inputs: list of arrays bound after them;
    outputs follow, then one row count per output, then cols."""
    wf = gh.WeightFile()
    bufs, i = [], 0
    for p, s in mats:
        bufs += [(W, i, wf.add(p)), (W, i + 1, wf.add(s))]
        i += 2
    ctx.upload_weights(W, wf.image())
    for k, arr in enumerate(inputs):
        ctx.put(10 + k, arr)
        bufs.append((10 + k, i, 0))
        i += 1
    for k, r in enumerate(member_rows):
        ctx.alloc(20 + k, max(r, 1) * 2)
        bufs.append((20 + k, i, 0))
        i += 1
    consts = [(i + k, r) for k, r in enumerate(member_rows)] + [(i + len(member_rows), cols)]
    rec = rt.make_record(ctx.pipeline(name), bufs, consts, ((sum(member_rows) + 15) // 16, 1, 1), (256, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    return [ctx.read(20 + k, np.uint16, r) for k, r in enumerate(member_rows) if r]


@pytest.mark.parametrize("fmt,planes", [(so.BINARY1, 2), (so.BINARY1, 3), (so.TERNARY2, 4), (so.TERNARY2, 6)])
def test_view_bank4(env, fmt, planes):
    ctx, dtype, odt = env
    stem = "binary" if fmt == so.BINARY1 else "ternary"
    member_rows, cols = [130, 37, 37, 64], 1280
    rows = sum(member_rows)
    packed, ws = signed_weights(60 + planes, rows, cols, fmt)
    x = bits(fx.rng_for(127, planes).normal(0, 1, cols).astype(np.float32), dtype)
    pl, asc, _ = so.activation_bitplanes(x, planes, odt)
    outs = run_bank(ctx, f"signed_{stem}_bitplane_i{planes}_bank4_matvec_g128_rows8", [(packed, ws)], [pl, asc], member_rows, cols, dtype)
    ref = so.signed_bitplane_matvec(fmt, packed, ws, pl, asc, rows, cols, odt)
    at = 0
    for got, r in zip(outs, member_rows):
        gh.check_outputs(got, ref[at:at + r], dtype, f"{stem} view bank member at row {at}")
        at += r


def test_binary_packed_banks_and_two_matrix_banks(env):
    ctx, dtype, odt = env
    cols = 2560
    x = bits(fx.rng_for(128, 0).normal(0, 1, cols).astype(np.float32), dtype)
    xf = so.widen(x, odt)
    for name, member_rows in (("signed_binary_packed_bank_matvec_g128_rows8", [200, 77]),
                              ("signed_binary_packed_bank4_matvec_g128_rows8", [64, 3, 129, 40])):
        rows = sum(member_rows)
        packed, ws = signed_weights(70 + rows, rows, cols, so.BINARY1)
        outs = run_bank(ctx, name, [(packed, ws)], [x], member_rows, cols, dtype)
        ref = so.signed_matvec(so.BINARY1, packed, ws, xf, rows, cols, cols, 128)[0]
        at = 0
        for got, r in zip(outs, member_rows):
            gh.check_outputs(got, ref[at:at + r], dtype, f"{name} member at row {at}")
            at += r
    # two physical matrices, one row space: the boundary falls inside a row tile
    for name in ("signed_binary_dual_matvec_g128_rows8", "signed_binary_virtual_bank_matvec_g128_rows8"):
        for rows1, rows2 in ((37, 91), (128, 5), (1, 300)):
            a, b = signed_weights(80 + rows1, rows1, cols, so.BINARY1), signed_weights(81 + rows2, rows2, cols, so.BINARY1)
            outs = run_bank(ctx, name, [a, b], [x], [rows1, rows2], cols, dtype)
            gh.check_outputs(outs[0], so.signed_matvec(so.BINARY1, a[0], a[1], xf, rows1, cols, cols, 128)[0], dtype, f"{name} first")
            gh.check_outputs(outs[1], so.signed_matvec(so.BINARY1, b[0], b[1], xf, rows2, cols, cols, 128)[0], dtype, f"{name} second")


@pytest.mark.parametrize("tile,planes,batch", [(4, 5, 3), (4, 2, 9), (8, 4, 13), (16, 6, 16)])
def test_view_matvec_over_prompt_rows(env, tile, planes, batch):
    """signed_binary_bitplane_i{N}_matvec_g128_rows8_batched_b{4,8,16}: bit-exact with independent rows
    (SignedQuantKernelTests.swift:664-860 checks the same property)."""
    ctx, dtype, odt = env
    rows, cols = 123, 1536
    packed, ws = signed_weights(90 + tile, rows, cols, so.BINARY1)
    x = bits(fx.rng_for(129, batch).normal(0, 1, (batch, cols)).astype(np.float32), dtype)
    views = [so.activation_bitplanes(x[t], planes, odt) for t in range(batch)]
    pl = np.stack([v[0] for v in views]); asc = np.stack([v[1] for v in views])
    wf = gh.WeightFile()
    a, b = wf.add(packed), wf.add(ws)
    ctx.upload_weights(W, wf.image())
    ctx.put(PL, pl); ctx.put(AS, asc); ctx.alloc(Y, batch * rows * 2); ctx.alloc(RES, batch * rows * 2)
    rec = rt.make_record(ctx.pipeline(f"signed_binary_bitplane_i{planes}_matvec_g128_rows8_batched_b{tile}"),
                         [(W, 0, a), (W, 1, b), (PL, 2, 0), (AS, 3, 0), (Y, 4, 0)], [(5, rows), (6, cols), (7, batch)],
                         ((rows + 7) // 8, (batch + tile - 1) // tile, 1), (256, 1, 1))
    single = rt.make_record(ctx.pipeline(f"signed_binary_bitplane_i{planes}_matvec_g128_rows8"),
                            [(W, 0, a), (W, 1, b), (PL, 2, 0), (AS, 3, 0), (RES, 4, 0)], [(5, rows), (6, cols)],
                            ((rows + 7) // 8, batch, 1), (256, 1, 1))
    ctx.interpret_decode(ctx.table([rec, single])); ctx.wait()
    got = ctx.read(Y, np.uint16, batch * rows).reshape(batch, rows)
    assert np.array_equal(got, ctx.read(RES, np.uint16, batch * rows).reshape(batch, rows))
    for t in (0, batch - 1):
        gh.check_outputs(got[t], so.signed_bitplane_matvec(so.BINARY1, packed, ws, views[t][0], views[t][1], rows, cols, odt), dtype, "batched view matvec")
