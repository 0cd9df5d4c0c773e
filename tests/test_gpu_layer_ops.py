"""GPU parity of the layer ops between the matvecs (RMS norms, staged SwiGLU, elementwise add) and a
whole-layer record list replayed eagerly and as a graph, against the CPU oracle.

Tolerance: elementwise ops and the staged SwiGLU are compared bit for bit up to the last bit of
`exp`; the norms sum squares in a different (parallel) order than the oracle's running sum, so
their 16-bit outputs may differ in the last place: |got - ref| <= 1 ulp of the output type (2 for
the generic kernel, which rounds x * rs before it multiplies by 1 + w), with at least 98% of the
elements identical."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import compiler as cc
from smelt_amd import runtime as rt

pytestmark = pytest.mark.gpu

DT = {fx.F16: (rt.ACT_F16, so.F16, "f16"), fx.BF16: (rt.ACT_BF16, so.BF16, "bf16")}


def ulps_apart(got_bits, ref_bits, dtype):
    g = fx.from_bits(got_bits, dtype).astype(np.float64)
    r = fx.from_bits(ref_bits, dtype).astype(np.float64)
    return np.abs(g - r) / gh.ulp_of(np.where(r == 0, 1e-30, r), dtype)


def assert_last_place(got_bits, ref_bits, dtype, what, exact_fraction=0.98, max_ulps=1.0):
    d = ulps_apart(got_bits, ref_bits, dtype)
    assert d.max() <= max_ulps, f"{what}: {d.max()} ulps apart at {d.argmax()}"
    same = np.mean(np.asarray(got_bits) == np.asarray(ref_bits))
    assert same >= exact_fraction, f"{what}: only {same:.4f} of the elements identical"


@pytest.fixture(scope="module", params=[fx.F16, fx.BF16], ids=["f16", "bf16"])
def env(request):
    act, odt, tag = DT[request.param]
    c = rt.Context(act_dtype=act)
    yield c, request.param, odt
    c.close()


def bits(values, dtype):
    return fx.f16_bits(values) if dtype == fx.F16 else fx.bf16_bits(values)


@pytest.mark.parametrize("name,dim,tokens,threads", [
    ("rms_norm_1pw", 1024, 1, 1024), ("rms_norm_1pw", 1000, 1, 256), ("rms_norm_1pw", 77, 1, 64),
    ("rms_norm_1pw_batched", 2560, 5, 1024), ("rms_norm_1pw_d1024", 1024, 1, 128),
    ("rms_norm_1pw_d2048", 2048, 1, 256), ("rms_norm_1pw_d1536_batched", 1536, 7, 192),
    ("rms_norm_1pw_d2560", 2560, 1, 320)])
def test_rms_norm_1pw(env, name, dim, tokens, threads):
    ctx, dtype, odt = env
    rng = fx.rng_for(95, dim + tokens)
    x = bits(rng.normal(0, 1.5, (tokens, dim)).astype(np.float32), dtype)
    w = bits(rng.normal(0, 0.2, dim).astype(np.float32), dtype)
    ctx.put(1, x); ctx.put(2, w); ctx.alloc(3, tokens * dim * 2)
    generic = "_d" not in name
    consts = [(3, dim), (4, 1e-6)] if generic else []
    rec = rt.make_record(ctx.pipeline(name), [(1, 0, 0), (2, 1, 0), (3, 2, 0)], consts, (tokens, 1, 1), (threads, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    got = ctx.read(3, np.uint16, tokens * dim).reshape(tokens, dim)
    for t in range(tokens):
        ref = so.rms_norm_1pw(x[t], w, 1e-6, odt, generic)
        # the two-step form multiplies a last-place difference of the rounded x * rs by (1 + w)
        assert_last_place(got[t], ref, dtype, f"{name} token {t}", max_ulps=2.0 if generic else 1.0)
        if dtype == fx.F16:     # one bf16 ulp is already 4e-3 of the value; the ulp bound above is the test there
            gh.check_outputs(got[t], so.widen(ref, odt), dtype, name)


@pytest.mark.parametrize("name,dim,tokens", [("rms_norm_1pw_d1536_add", 1536, 1), ("rms_norm_1pw_d2560_add_batched", 2560, 4),
                                             ("rms_norm_1pw_d256_add", 256, 1)])
def test_rms_norm_1pw_add_including_in_place(env, name, dim, tokens):
    ctx, dtype, odt = env
    rng = fx.rng_for(96, dim)
    x = bits(rng.normal(0, 1.5, (tokens, dim)).astype(np.float32), dtype)
    w = bits(rng.normal(0, 0.2, dim).astype(np.float32), dtype)
    res = bits(rng.normal(0, 1.0, (tokens, dim)).astype(np.float32), dtype)
    ctx.put(1, x); ctx.put(2, w); ctx.put(3, res); ctx.alloc(4, tokens * dim * 2)
    pipe = ctx.pipeline(name)
    for out_slot in (4, 3):      # second pass writes over the residual (the reference allows the alias)
        rec = rt.make_record(pipe, [(1, 0, 0), (2, 1, 0), (3, 2, 0), (out_slot, 3, 0)], [], (tokens, 1, 1), (256, 1, 1))
        ctx.interpret_decode(ctx.table([rec])); ctx.wait()
        got = ctx.read(out_slot, np.uint16, tokens * dim).reshape(tokens, dim)
        for t in range(tokens):
            ref = so.rms_norm_1pw(x[t], w, 1e-6, odt, False, res[t])
            # a last-place difference of the norm survives the add at the norm's magnitude (the
            # sum itself may be much smaller), plus the rounding of the sum
            normed = so.widen(so.rms_norm_1pw(x[t], w, 1e-6, odt, False), odt).astype(np.float64)
            g, r = fx.from_bits(got[t], dtype).astype(np.float64), so.widen(ref, odt).astype(np.float64)
            bound = gh.ulp_of(np.where(normed == 0, 1e-30, normed), dtype) + gh.ulp_of(np.where(r == 0, 1e-30, r), dtype)
            assert np.all(np.abs(g - r) <= bound), name
            assert np.mean(got[t] == ref) >= 0.97, name


@pytest.mark.parametrize("name,dim,tokens,eps", [("rms_norm_scale_only", 3000, 1, 1e-6), ("rms_norm_scale_only_precise", 1024, 1, 1e-5),
                                                 ("rms_norm_scale_only_d1536", 1536, 1, 1e-6),
                                                 ("rms_norm_scale_only_d2048_eps1e5_batched", 2048, 6, 1e-5)])
def test_rms_norm_scale_only(env, name, dim, tokens, eps):
    ctx, dtype, odt = env
    x = bits(fx.rng_for(97, dim).normal(0, 3, (tokens, dim)).astype(np.float32), dtype)
    ctx.put(1, x); ctx.alloc(2, tokens * 4)
    consts = [(2, dim), (3, float(eps))] if "_d" not in name else []
    rec = rt.make_record(ctx.pipeline(name), [(1, 0, 0), (2, 1, 0)], consts, (tokens, 1, 1), (256, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    got = ctx.read(2, np.float32, tokens)
    ref = np.float32([so.rms_scale(x[t], eps, odt) for t in range(tokens)])
    assert np.all(np.abs(got - ref) <= 5e-6 * ref)            # the oracle's running fp32 sum drifts by a few 1e-6
    exact = np.array([1.0 / np.sqrt(np.mean(fx.from_bits(x[t], dtype).astype(np.float64) ** 2) + eps) for t in range(tokens)])
    assert np.all(np.abs(got - exact) <= 1e-6 * exact)        # the pairwise device sum does not


def test_residual_add_then_scale(env):
    ctx, dtype, odt = env
    dim = 2560
    rng = fx.rng_for(98, 0)
    a, b = bits(rng.normal(0, 1, dim).astype(np.float32), dtype), bits(rng.normal(0, 1, dim).astype(np.float32), dtype)
    ctx.put(1, a); ctx.put(2, b); ctx.alloc(3, dim * 2); ctx.alloc(4, 4)
    rec = rt.make_record(ctx.pipeline("residual_add_rms_norm_scale_only_precise"), [(1, 0, 0), (2, 1, 0), (3, 2, 0), (4, 3, 0)],
                         [(4, dim), (5, 1e-6)], (1, 1, 1), (1024, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    summed = so.elementwise(a, b, odt)
    assert np.array_equal(ctx.read(3, np.uint16, dim), summed)
    ref = so.rms_scale(summed, 1e-6, odt)
    assert abs(ctx.read(4, np.float32, 1)[0] - ref) <= 5e-6 * ref


@pytest.mark.parametrize("count", [1, 9, 3584, 100003])
def test_staged_swiglu_and_elementwise(env, count):
    ctx, dtype, odt = env
    rng = fx.rng_for(99, count)
    g = bits(rng.normal(0, 3, count).astype(np.float32), dtype)
    u = bits(rng.normal(0, 1, count).astype(np.float32), dtype)
    ctx.put(1, g); ctx.put(2, u); ctx.alloc(3, count * 2)
    for name, ref, exact in (("swiglu_fused", so.swiglu_fused(g, u, odt), False),
                             ("elementwise_add", so.elementwise(g, u, odt), True),
                             ("elementwise_mul", so.elementwise(g, u, odt, True), True)):
        # dispatchThreads style: the grid counts threads, the ragged edge is bounds-checked
        rec = rt.make_record(ctx.pipeline(name), [(1, 0, 0), (2, 1, 0), (3, 2, 0)], [(3, count)], (count, 1, 1),
                             (min(count, 256), 1, 1), style=rt.STYLE_THREADS)
        ctx.interpret_decode(ctx.table([rec])); ctx.wait()
        got = ctx.read(3, np.uint16, count)
        if exact:
            assert np.array_equal(got, ref), name
        else:
            assert_last_place(got, ref, dtype, name, 0.99)
    rec = rt.make_record(ctx.pipeline("buffer_copy"), [(1, 0, 0), (3, 1, 0)], [(2, count)], (count, 1, 1), (min(count, 64), 1, 1),
                         style=rt.STYLE_THREADS)
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    assert np.array_equal(ctx.read(3, np.uint16, count), g)


def test_fused_gate_up_equals_staged_matvecs_plus_swiglu_bit_for_bit():
    """SignedQuantKernelTests.swift:200-330: the fused gate+up+SwiGLU kernel and the staged path
    (two matvecs, then swiglu_fused) give the same bits."""
    rows, cols = 9, 5120
    groups = cols // 128
    r, c = np.meshgrid(np.arange(rows), np.arange(cols), indexing="ij")
    gate_codes = ((r * 13 + c * 7) % 3).astype(np.uint8)
    up_codes = ((r * 5 + c * 11 + 1) % 3).astype(np.uint8)
    gs = fx.f16_bits((0.00390625 * ((np.arange(rows * groups) % 5) + 1)).astype(np.float32)).reshape(rows, groups)
    us = fx.f16_bits((0.0029296875 * ((np.arange(rows * groups) % 7) + 1)).astype(np.float32)).reshape(rows, groups)
    x = fx.f16_bits((((np.arange(cols) * 17 + 3) % 31 - 15) / 16).astype(np.float32))
    wf = gh.WeightFile()
    og, ogs = wf.add(so.signed_pack(gate_codes, so.TERNARY2)), wf.add(gs)
    ou, ous = wf.add(so.signed_pack(up_codes, so.TERNARY2)), wf.add(us)
    ctx = rt.Context()
    try:
        ctx.upload_weights(0, wf.image())
        ctx.put(1, x)
        for s in (2, 3, 4, 5):
            ctx.alloc(s, rows * 2)
        mv = ctx.pipeline("signed_ternary_affine_matvec_g128_rows8")
        sw = ctx.pipeline("swiglu_fused")
        fused = ctx.pipeline("signed_ternary_affine_gate_up_swiglu_g128_rows8")
        def matvec(codes, scales, out):
            return rt.make_record(mv, [(0, 0, codes), (0, 1, scales), (0, 2, scales), (1, 3, 0), (out, 4, 0)],
                                  [(5, rows), (6, cols)], ((rows + 7) // 8, 1, 1), (256, 1, 1))
        recs = [matvec(og, ogs, 2), matvec(ou, ous, 3),
                rt.make_record(sw, [(2, 0, 0), (3, 1, 0), (4, 2, 0)], [(3, rows)], (rows, 1, 1), (rows, 1, 1), style=rt.STYLE_THREADS),
                rt.make_record(fused, [(0, 0, og), (0, 1, ogs), (0, 2, ogs), (0, 3, ou), (0, 4, ous), (0, 5, ous), (1, 6, 0), (5, 7, 0)],
                               [(8, rows), (9, cols)], ((rows + 7) // 8, 1, 1), (256, 1, 1))]
        ctx.interpret_decode(ctx.table(recs)); ctx.wait()
        staged, one = ctx.read(4, np.uint16, rows), ctx.read(5, np.uint16, rows)
        assert np.array_equal(staged, one)
        assert np.abs(fx.from_bits(staged, fx.F16)).max() > 0
    finally:
        ctx.close()


def test_whole_layer_record_list_eager_and_graph():
    """norm -> q/k/v bank -> (attention output stands in) -> o projection + residual -> norm ->
    gate+up+SwiGLU -> down projection + residual, replayed from one record table."""
    dtype, odt = fx.BF16, so.BF16
    hidden, ffn, group = 1024, 3584, 64
    ctx = rt.Context(act_dtype=rt.ACT_BF16)
    try:
        cus = ctx.device_info()["compute_units"]
        lay = cc.Layout()
        q, k, v = lay.affine_bank([2048, 512, 512], hidden, group)
        o = lay.affine(hidden, 2048, group)
        gate, up = lay.affine(ffn, hidden, group), lay.affine(ffn, hidden, group)
        down = lay.affine(hidden, ffn, group)
        n1, n2 = lay.dense(1, hidden, cc.BF16), lay.dense(1, hidden, cc.BF16)
        image = np.zeros(lay.total_bytes, np.uint8)
        rng = fx.rng_for(100, 0)
        tensors = {}
        for name, e in (("q", q), ("k", k), ("v", v), ("o", o), ("gate", gate), ("up", up), ("down", down)):
            w = rng.normal(0, 0.03, (e.rows, e.cols)).astype(np.float32)
            tensors[name] = so.affine_quantize(w, group, 0, None, odt)
            cc.write_affine(image, e, *tensors[name])
        norm_w = [fx.bf16_bits(rng.normal(0, 0.1, hidden).astype(np.float32)) for _ in range(2)]
        for e, w in zip((n1, n2), norm_w):
            image[e.offset:e.offset + hidden * 2] = w.view(np.uint8)
        W, H, N, QKV, ATT, ACT = 0, 1, 2, 3, 4, 5
        ctx.upload_weights(W, image)
        h0 = fx.bf16_bits(rng.normal(0, 1, hidden).astype(np.float32))
        att = fx.bf16_bits(rng.normal(0, 0.5, 2048).astype(np.float32))
        ctx.put(ATT, att); ctx.alloc(N, hidden * 2); ctx.alloc(QKV, 3072 * 2); ctx.alloc(ACT, ffn * 2)
        em = cc.Emitter(rt.ACT_BF16, cus)
        em.rms_norm_1pw(cc.bind(H), cc.bind(W, n1.offset), cc.bind(N), hidden)
        em.bank_matvec(W, [q, k, v], cc.bind(N), [cc.bind(QKV, 0), cc.bind(QKV, 4096), cc.bind(QKV, 5120)])
        em.matvec_add(W, o, cc.bind(ATT), cc.bind(H), cc.bind(H))
        em.rms_norm_1pw(cc.bind(H), cc.bind(W, n2.offset), cc.bind(N), hidden)
        em.gate_up_swiglu(W, gate, up, cc.bind(N), cc.bind(ACT))
        em.matvec_add(W, down, cc.bind(ACT), cc.bind(H), cc.bind(H))
        assert em.pipelines[0] == "rms_norm_1pw_d1024@bf16"
        em.install(ctx)
        table = em.records()

        def reference():
            f = lambda b: so.widen(b, odt)
            normed = so.rms_norm_1pw(h0, norm_w[0], 1e-6, odt, False)
            qkv = np.concatenate([so.narrow(so.affine_matvec(*tensors[n], f(normed), e.rows, hidden, group, odt)[0], odt)
                                  for n, e in (("q", q), ("k", k), ("v", v))])
            proj = so.affine_matvec(*tensors["o"], f(att), hidden, 2048, group, odt)[0]
            h1 = so.epilogue_residual_add(proj, h0, odt)
            normed2 = so.rms_norm_1pw(h1, norm_w[1], 1e-6, odt, False)
            g = so.affine_matvec(*tensors["gate"], f(normed2), ffn, hidden, group, odt)[0]
            u = so.affine_matvec(*tensors["up"], f(normed2), ffn, hidden, group, odt)[0]
            act = so.epilogue_affine_swiglu(g, u, odt)
            dn = so.affine_matvec(*tensors["down"], f(act), hidden, ffn, group, odt)[0]
            return qkv, so.epilogue_residual_add(dn, h1, odt)

        ref_qkv, ref_h = reference()
        ctx.put(H, h0)
        assert ctx.interpret_decode(table) == 6
        ctx.wait()
        eager_h, eager_qkv = ctx.read(H, np.uint16, hidden), ctx.read(QKV, np.uint16, 3072)
        # the normed row feeding q/k/v can sit one step of the 16-bit type from the oracle's (sum of squares in another order)
        gh.check_steps(eager_qkv, np.asarray(ref_qkv).reshape(np.shape(eager_qkv)), dtype, "layer q/k/v", max_steps=2, min_exact=0.9)
        # six chained kernels with bf16 values between them: a last-place flip of one activation
        # moves every downstream sum a little, so the end of the chain is compared in norm
        gh_, rh = fx.from_bits(eager_h, dtype).astype(np.float64), so.widen(ref_h, odt).astype(np.float64)
        assert np.linalg.norm(gh_ - rh) <= 4e-3 * np.linalg.norm(rh)
        assert np.abs(gh_ - rh).max() <= 2e-2 * np.abs(rh).max()
        graph, n = ctx.capture_decode(table)
        assert n == 6
        for _ in range(3):
            ctx.put(H, h0)
            ctx.graph_launch(graph); ctx.wait()
            assert np.array_equal(ctx.read(H, np.uint16, hidden), eager_h)
            assert np.array_equal(ctx.read(QKV, np.uint16, 3072), eager_qkv)
        ctx.graph_destroy(graph)
    finally:
        ctx.close()


def test_norm_variants(env):
    """rms_norm_1pw_d256_add_scalar_weight (norms.metal:218-260), rms_norm_1pw_from_fp32[_batched]
    (norms_fp32.metal:50-130) and rms_norm_gated (norms.metal:1093-1153) against the oracle: last-place
    agreement (the sum of squares is formed in another order), at least 97 % of the elements identical."""
    ctx, dtype, odt = env
    rng = fx.rng_for(97, 3)
    x = bits(rng.normal(0, 1.5, 256).astype(np.float32), dtype)
    w = bits(rng.normal(0, 0.2, 256).astype(np.float32), dtype)
    res = bits(rng.normal(0, 1.0, 256).astype(np.float32), dtype)
    scalar = bits(np.float32([0.75]), dtype)
    ctx.put(1, x); ctx.put(2, w); ctx.put(3, res); ctx.put(4, scalar); ctx.alloc(5, 512)
    rec = rt.make_record(ctx.pipeline("rms_norm_1pw_d256_add_scalar_weight"), [(1, 0, 0), (2, 1, 0), (3, 2, 0), (4, 3, 0), (5, 4, 0)],
                         [], (1, 1, 1), (256, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    got = ctx.read(5, np.uint16, 256)
    ref = so.rms_norm_1pw_add_scalar(x, w, res, int(scalar[0]), 1e-6, odt)
    normed = so.widen(so.rms_norm_1pw(x, w, 1e-6, odt, 2), odt).astype(np.float64)
    g, r = fx.from_bits(got, dtype).astype(np.float64), so.widen(ref, odt).astype(np.float64)
    bound = gh.ulp_of(np.where(normed == 0, 1e-30, normed), dtype) + 2 * gh.ulp_of(np.where(r == 0, 1e-30, r), dtype)
    assert np.all(np.abs(g - r) <= bound) and np.mean(got == ref) >= 0.97
    # the plain d256 add kernel now multiplies left to right as the reference's does
    ctx.alloc(5, 512)
    rec = rt.make_record(ctx.pipeline("rms_norm_1pw_d256_add"), [(1, 0, 0), (2, 1, 0), (3, 2, 0), (5, 3, 0)], [], (1, 1, 1), (256, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    assert np.mean(ctx.read(5, np.uint16, 256) == so.rms_norm_1pw(x, w, 1e-6, odt, 2, res)) >= 0.97

    tokens, dim = 3, 1536
    x32 = rng.normal(0, 3, (tokens, dim)).astype(np.float32)
    x32[1, 7] = 3.0e5                                  # one row whose product clamps at the fp16 limit
    w = bits(rng.normal(0, 0.2, dim).astype(np.float32), dtype)
    ctx.put(1, x32); ctx.put(2, w); ctx.alloc(3, tokens * dim * 2)
    rec = rt.make_record(ctx.pipeline("rms_norm_1pw_from_fp32_batched"), [(1, 0, 0), (2, 1, 0), (3, 2, 0)], [(3, dim), (4, 1e-6)],
                         (tokens, 1, 1), (256, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    got = ctx.read(3, np.uint16, tokens * dim).reshape(tokens, dim)
    for t in range(tokens):
        assert_last_place(got[t], so.rms_norm_1pw_from_fp32(x32[t], w, 1e-6, odt), dtype, f"from_fp32 token {t}", exact_fraction=0.97)
    assert fx.from_bits(got[1], dtype).max() <= 65504.0

    heads, d = 16, 128
    xh = bits((rng.normal(0, 1, (heads, d)) * rng.uniform(0.1, 8, (heads, 1))).astype(np.float32), dtype)
    gate = bits(rng.normal(0, 2, (heads, d)).astype(np.float32), dtype)
    wg = bits((1.0 + rng.normal(0, 0.1, d)).astype(np.float32), dtype)
    ctx.put(1, xh); ctx.put(2, gate); ctx.put(3, wg); ctx.alloc(4, heads * d * 2)
    rec = rt.make_record(ctx.pipeline("rms_norm_gated"), [(1, 0, 0), (2, 1, 0), (3, 2, 0), (4, 3, 0)], [(4, d), (5, 1e-6)],
                         (heads, 1, 1), (64, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    got = ctx.read(4, np.uint16, heads * d)
    ref = so.rms_norm_gated(xh.ravel(), gate.ravel(), wg, heads, d, 1e-6, odt)
    assert_last_place(got, ref, dtype, "rms_norm_gated", exact_fraction=0.97)


@pytest.mark.parametrize("threads", [32, 128])
def test_gated_norm_precise_batched_and_view(env, threads):
    """rms_norm_gated_d128[_batched] (norms_gated_precise.metal:20-88) and the fused gated-norm -> i6 view
    (signed_quant.metal:1149-1173), which takes the precise arithmetic exactly when launched with 32
    threads per 128-value head, as the reference's does."""
    ctx, dtype, odt = env
    rng = fx.rng_for(98, threads)
    tokens, heads, d = 2, 8, 128
    x = bits((rng.normal(0, 1, (tokens * heads, d)) * rng.uniform(0.2, 5, (tokens * heads, 1))).astype(np.float32), dtype)
    gate = bits(rng.normal(0, 2, (tokens * heads, d)).astype(np.float32), dtype)
    w = bits((1.0 + rng.normal(0, 0.1, d)).astype(np.float32), dtype)
    ctx.put(1, x); ctx.put(2, gate); ctx.put(3, w); ctx.alloc(4, x.size * 2)
    rec = rt.make_record(ctx.pipeline("rms_norm_gated_d128_batched"), [(1, 0, 0), (2, 1, 0), (3, 2, 0), (4, 3, 0)], [(4, heads)],
                         (heads, tokens, 1), (threads, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    got = ctx.read(4, np.uint16, x.size)
    ref = so.rms_norm_gated(x.ravel(), gate.ravel(), w, tokens * heads, d, 1e-6, odt, precise=True)
    assert_last_place(got, ref, dtype, "rms_norm_gated_d128_batched", exact_fraction=0.97, max_ulps=2.0)
    ctx.alloc(4, heads * d * 2)
    rec = rt.make_record(ctx.pipeline("rms_norm_gated_d128"), [(1, 0, 0), (2, 1, 0), (3, 2, 0), (4, 3, 0)], [], (heads, 1, 1), (threads, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    assert np.array_equal(ctx.read(4, np.uint16, heads * d), got[:heads * d])          # token 0 of the batched run
    # fused view: equal to the plain i6 producer run on this backend's own norm output of the same arithmetic
    n = tokens * heads
    ctx.alloc(5, n * 6 * 16); ctx.alloc(6, n * 2); ctx.alloc(7, x.size * 2)
    rec = rt.make_record(ctx.pipeline("rms_norm_gated_d128_signed_activation_bitplanes_i6_g128"),
                         [(1, 0, 0), (2, 1, 0), (3, 2, 0), (5, 3, 0), (6, 4, 0)], [(5, d), (6, 1e-6)], (n, 1, 1), (threads, 1, 1))
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    fused_pl, fused_sc = ctx.read(5, np.uint32, n * 24), ctx.read(6, np.uint16, n)
    norm_name, consts = ("rms_norm_gated_d128", []) if threads == 32 else ("rms_norm_gated", [(4, d), (5, 1e-6)])
    staged = [rt.make_record(ctx.pipeline(norm_name), [(1, 0, 0), (2, 1, 0), (3, 2, 0), (7, 3, 0)], consts, (n, 1, 1), (threads, 1, 1)),
              rt.make_record(ctx.pipeline("signed_activation_bitplanes_i6_g128"), [(7, 0, 0), (5, 1, 0), (6, 2, 0)], [(3, n * d)], (n, 1, 1), (32, 1, 1))]
    ctx.alloc(5, n * 6 * 16); ctx.alloc(6, n * 2)
    ctx.interpret_decode(ctx.table(staged)); ctx.wait()
    assert np.array_equal(ctx.read(5, np.uint32, n * 24), fused_pl) and np.array_equal(ctx.read(6, np.uint16, n), fused_sc)
    ref_pl, ref_sc = so.rms_norm_gated_activation_bitplanes(x.ravel(), gate.ravel(), w, n, 1e-6, odt, threads == 32)
    assert np.mean(fused_pl == ref_pl.reshape(-1)) > 0.97 and np.mean(fused_sc == ref_sc) > 0.85


def test_pointwise_activations(env):
    """silu / sigmoid_kernel / softplus / scalar_mul / scalar_mul_weight / logit_cap / sigmoid_mul /
    geglu_fused (activations.metal, activations_precise.metal:26-38) against the oracle: identical up to the
    last bit of exp / tanh / log; scalar multiplies bit for bit."""
    ctx, dtype, odt = env
    rng = fx.rng_for(99, 1)
    n = 5000
    x = bits(rng.normal(0, 4, n).astype(np.float32), dtype)
    y = bits(rng.normal(0, 2, n).astype(np.float32), dtype)
    ctx.put(1, x); ctx.put(2, y); ctx.alloc(3, n * 2)
    grid, tg = ((n + 255) // 256 * 256, 1, 1), (256, 1, 1)

    def run(name, bufs, consts):
        ctx.alloc(3, n * 2)
        ctx.interpret_decode(ctx.table([rt.make_record(ctx.pipeline(name), bufs, consts, grid, tg, style=rt.STYLE_THREADS)])); ctx.wait()
        return ctx.read(3, np.uint16, n)

    for name in ("silu", "sigmoid_kernel", "softplus"):
        assert_last_place(run(name, [(1, 0, 0), (3, 1, 0)], [(2, n)]), so.unary(name, x, odt), dtype, name, exact_fraction=0.97)
    assert_last_place(run("logit_cap", [(1, 0, 0), (3, 1, 0)], [(2, n), (3, 30.0)]), so.unary("logit_cap", x, odt, 30.0), dtype,
                      "logit_cap", exact_fraction=0.97)
    assert np.array_equal(run("scalar_mul", [(1, 0, 0), (3, 1, 0)], [(2, 0.37), (3, n)]), so.unary("scalar_mul", x, odt, 0.37))
    scalar = bits(np.float32([0.75]), dtype)
    ctx.put(4, scalar)
    assert np.array_equal(run("scalar_mul_weight", [(1, 0, 0), (4, 1, 0), (3, 2, 0)], [(3, n)]),
                          so.unary("scalar_mul", x, odt, float(fx.from_bits(scalar, dtype)[0])))
    assert_last_place(run("sigmoid_mul", [(1, 0, 0), (2, 1, 0), (3, 2, 0)], [(3, n)]), so.sigmoid_mul(x, y, odt), dtype, "sigmoid_mul",
                      exact_fraction=0.97)
    got = run("geglu_fused", [(1, 0, 0), (2, 1, 0), (3, 2, 0)], [(3, n)])
    ref = so.epilogue_geglu(so.widen(x, odt), so.widen(y, odt), odt)
    # 1 + tanh cancels for negative gates: absolute slack of 2^-22 |g u| beside the last place
    g, r = fx.from_bits(got, dtype).astype(np.float64), so.widen(ref, odt).astype(np.float64)
    slack = np.abs(so.widen(x, odt).astype(np.float64) * so.widen(y, odt).astype(np.float64)) * 2.0 ** -21
    assert np.all(np.abs(g - r) <= gh.ulp_of(np.where(r == 0, 1e-30, r), dtype) + slack) and np.mean(got == ref) > 0.95
    # fused sigmoid-mul view == sigmoid_mul then the plain i6 view, bit for bit on the device
    cols = 4096
    groups = cols // 128
    ctx.alloc(5, groups * 6 * 16); ctx.alloc(6, groups * 2)
    fused = rt.make_record(ctx.pipeline("sigmoid_mul_signed_activation_bitplanes_i6_g128"), [(1, 0, 0), (2, 1, 0), (5, 2, 0), (6, 3, 0)],
                           [(4, cols)], (groups, 1, 1), (32, 1, 1))
    ctx.interpret_decode(ctx.table([fused])); ctx.wait()
    f_pl, f_sc = ctx.read(5, np.uint32, groups * 24), ctx.read(6, np.uint16, groups)
    staged = [rt.make_record(ctx.pipeline("sigmoid_mul"), [(1, 0, 0), (2, 1, 0), (3, 2, 0)], [(3, cols)], (cols, 1, 1), (256, 1, 1), style=rt.STYLE_THREADS),
              rt.make_record(ctx.pipeline("signed_activation_bitplanes_i6_g128"), [(3, 0, 0), (5, 1, 0), (6, 2, 0)], [(3, cols)], (groups, 1, 1), (32, 1, 1))]
    ctx.alloc(5, groups * 6 * 16); ctx.alloc(6, groups * 2)
    ctx.interpret_decode(ctx.table(staged)); ctx.wait()
    assert np.array_equal(ctx.read(5, np.uint32, groups * 24), f_pl) and np.array_equal(ctx.read(6, np.uint16, groups), f_sc)


def test_batched_geglu_with_strided_up_and_batched_bias_add(env):
    """geglu_fused_strided_batched (activations.metal:142-163): token b reads gate[b, :count] and
    up[b * upStride : b * upStride + count]; it must equal the single-row geglu_fused applied to those
    slices bit for bit on the device and stay within the last place of the oracle.
    projection_bias_add_batched (activations.metal:69-82): bit-exact row-broadcast add."""
    ctx, dtype, odt = env
    rng = fx.rng_for(99, 7)
    count, stride, batch = 1000, 1536, 5
    gate = bits(rng.normal(0, 3, (batch, count)).astype(np.float32), dtype)
    up = bits(rng.normal(0, 2, (batch, stride)).astype(np.float32), dtype)
    ctx.put(1, gate); ctx.put(2, up); ctx.alloc(3, batch * count * 2)
    grid, tg = ((count + 255) // 256 * 256, batch, 1), (256, 1, 1)
    rec = rt.make_record(ctx.pipeline("geglu_fused_strided_batched"), [(1, 0, 0), (2, 1, 0), (3, 2, 0)],
                         [(3, count), (4, stride)], grid, tg, style=rt.STYLE_THREADS)
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    got = ctx.read(3, np.uint16, batch * count).reshape(batch, count)
    ref = so.epilogue_geglu(so.widen(gate, odt).ravel(), so.widen(up[:, :count], odt).ravel(), odt).reshape(batch, count)
    g, r = fx.from_bits(got, dtype).astype(np.float64), so.widen(ref, odt).astype(np.float64)
    slack = np.abs(so.widen(gate, odt).astype(np.float64) * so.widen(up[:, :count], odt).astype(np.float64)) * 2.0 ** -21
    assert np.all(np.abs(g - r) <= gh.ulp_of(np.where(r == 0, 1e-30, r), dtype) + slack) and np.mean(got == ref) > 0.95
    one = ctx.pipeline("geglu_fused")
    for b in (0, batch - 1):
        ctx.alloc(4, count * 2)
        ctx.interpret_decode(ctx.table([rt.make_record(one, [(1, 0, b * count * 2), (2, 1, b * stride * 2), (4, 2, 0)], [(3, count)],
                                                       ((count + 255) // 256 * 256, 1, 1), tg, style=rt.STYLE_THREADS)]))
        ctx.wait()
        assert np.array_equal(ctx.read(4, np.uint16, count), got[b])
    # a stride shorter than the last row needs is caught before launch
    ctx.alloc(5, ((batch - 1) * stride + count) * 2 - 2)
    bad = rt.make_record(ctx.pipeline("geglu_fused_strided_batched"), [(1, 0, 0), (5, 1, 0), (3, 2, 0)],
                         [(3, count), (4, stride)], grid, tg, style=rt.STYLE_THREADS)
    with pytest.raises(rt.SmeltHipError):
        ctx.interpret_decode(ctx.table([bad]))

    rows = 777
    x = bits(rng.normal(0, 4, (batch, rows)).astype(np.float32), dtype)
    bias = bits(rng.normal(0, 1, rows).astype(np.float32), dtype)
    ctx.put(1, x); ctx.put(2, bias); ctx.alloc(3, batch * rows * 2)
    rec = rt.make_record(ctx.pipeline("projection_bias_add_batched"), [(1, 0, 0), (2, 1, 0), (3, 2, 0)], [(3, rows)],
                         ((rows + 255) // 256 * 256, batch, 1), tg, style=rt.STYLE_THREADS)
    ctx.interpret_decode(ctx.table([rec])); ctx.wait()
    want = so.elementwise(x.ravel(), np.tile(bias, batch), odt)
    assert np.array_equal(ctx.read(3, np.uint16, batch * rows), want)

