"""Pins of the oracle's layer ops (RMS norm with the 1 + weight convention, staged SwiGLU,
elementwise add / multiply): closed forms, invariants and an independent restatement in numpy's
own float16 arithmetic, chosen so that a dropped eps, a missing "1 +", a wrong mean or a moved
rounding point fails at least one of them."""
import numpy as np

import fixtures as fx
from oracle import oracle as so


def f16(v):
    return so.narrow(np.asarray(v, np.float32), so.F16)


def test_rms_scale_closed_forms():
    assert so.rms_scale(f16(np.ones(64)), 0.0, so.F16) == 1.0
    assert so.rms_scale(f16(np.full(48, -4.0)), 0.0, so.F16) == 0.25                 # 1 / sqrt(mean(16))
    x = np.zeros(100, np.float32); x[0] = 10.0                                       # mean = 100 / 100
    assert so.rms_scale(f16(x), 0.0, so.F16) == 1.0
    assert so.rms_scale(f16(np.zeros(8)), 0.25, so.F16) == 2.0                       # eps is under the root
    assert abs(so.rms_scale(f16(np.ones(8)), 3.0, so.F16) - 0.5) < 1e-7              # ... and added to the mean
    assert so.rms_scale(so.narrow(np.full(16, 2.0, np.float32), so.BF16), 0.0, so.BF16) == 0.5


def test_rms_norm_closed_forms_and_invariants():
    n = 256
    x = np.where(np.arange(n) % 2 == 0, 0.5, -0.5).astype(np.float32)
    zero = f16(np.zeros(n))
    for two_step in (False, True):
        out = so.widen(so.rms_norm_1pw(f16(x), zero, 0.0, so.F16, two_step), so.F16)
        assert np.array_equal(out, np.sign(x))                                       # unit RMS, weight 1 + 0
        out = so.widen(so.rms_norm_1pw(f16(x), f16(np.ones(n)), 0.0, so.F16, two_step), so.F16)
        assert np.array_equal(out, 2 * np.sign(x))                                   # the stored weight is a delta from 1
        out = so.widen(so.rms_norm_1pw(f16(x), f16(np.full(n, -1.0)), 0.0, so.F16, two_step), so.F16)
        assert not out.any()
        rng = fx.rng_for(90, int(two_step))
        r = rng.normal(0, 1, n).astype(np.float32)
        w = rng.normal(0, 0.2, n).astype(np.float32)
        a = so.rms_norm_1pw(f16(r), f16(w), 0.0, so.F16, two_step)
        b = so.rms_norm_1pw(f16(4 * so.widen(f16(r), so.F16)), f16(w), 0.0, so.F16, two_step)
        assert np.array_equal(a, b)                                                  # scale invariance for powers of two
        res = f16(rng.normal(0, 1, n))
        with_res = so.rms_norm_1pw(f16(r), f16(w), 1e-6, so.F16, two_step, res)
        plain = so.rms_norm_1pw(f16(r), f16(w), 1e-6, so.F16, two_step)
        assert np.array_equal(with_res.view(np.float16), (plain.view(np.float16) + res.view(np.float16)))


def test_rms_norm_against_numpy_float16_arithmetic():
    """Independent restatement: numpy's float16 type performs the half multiplies and roundings."""
    rng = fx.rng_for(91, 0)
    for n in (64, 1000, 2560):
        xb, wb = f16(rng.normal(0, 2, n)), f16(rng.normal(0, 0.3, n))
        x32, w32 = xb.view(np.float16).astype(np.float32), wb.view(np.float16).astype(np.float32)
        rs = np.float32(so.rms_scale(xb, 1e-6, so.F16))
        exact = 1.0 / np.sqrt(np.mean(x32.astype(np.float64) ** 2) + 1e-6)
        assert abs(float(rs) - exact) <= 2e-6 * exact                             # fp32 running sum
        two = (np.float32(1.0) + w32).astype(np.float16) * (x32 * rs).astype(np.float16)
        assert np.array_equal(so.rms_norm_1pw(xb, wb, 1e-6, so.F16, True), two.view(np.uint16))
        one = (x32 * (rs * (np.float32(1.0) + w32))).astype(np.float16)
        assert np.array_equal(so.rms_norm_1pw(xb, wb, 1e-6, so.F16, False), one.view(np.uint16))
        # the two rounding conventions stay within two 16-bit ulps of each other
        d = np.abs(two.astype(np.float64) - one.astype(np.float64))
        assert np.all(d <= 2 * np.spacing(np.abs(one).astype(np.float16)).astype(np.float64))


def test_swiglu_fused_closed_forms_and_numpy_float16():
    assert so.swiglu_fused(f16([0.0]), f16([3.0]), so.F16)[0] == 0                    # silu(0) = 0
    big = so.widen(so.swiglu_fused(f16([12.0, -12.0]), f16([0.5, 0.5]), so.F16), so.F16)
    assert big[0] == 6.0 and abs(big[1]) < 1e-3                                      # sigmoid saturates to 1 / ~0
    one = so.widen(so.swiglu_fused(f16([1.0]), f16([1.0]), so.F16), so.F16)[0]
    assert abs(one - 0.7310585786) < 1e-3                                            # 1 * sigmoid(1)
    rng = fx.rng_for(92, 0)
    g, u = f16(rng.normal(0, 3, 4096)), f16(rng.normal(0, 1, 4096))
    gh, uh = g.view(np.float16), u.view(np.float16)
    h1 = np.float16(1.0)
    tail = h1 / (h1 + np.exp(np.abs(gh)))            # float16 in, float16 out at every step
    sig = np.where(gh < 0, tail, h1 - tail).astype(np.float16)
    ref = ((gh * sig).astype(np.float16) * uh).astype(np.float16)
    got = so.swiglu_fused(g, u, so.F16).view(np.float16)
    ulp = np.spacing(np.abs(ref)).astype(np.float64)
    assert np.all(np.abs(got.astype(np.float64) - ref.astype(np.float64)) <= ulp)    # exp may differ in its last bit
    assert np.mean(got.view(np.uint16) == ref.view(np.uint16)) > 0.995


def test_elementwise_matches_numpy_float16():
    rng = fx.rng_for(93, 0)
    a, b = f16(rng.normal(0, 100, 5000)), f16(rng.normal(0, 0.01, 5000))
    assert np.array_equal(so.elementwise(a, b, so.F16).view(np.float16), a.view(np.float16) + b.view(np.float16))
    assert np.array_equal(so.elementwise(a, b, so.F16, True).view(np.float16), a.view(np.float16) * b.view(np.float16))


def test_norm_scale_input_closed_forms_and_rounding_order():
    """x_norm = half((x * rs) * (1 + w)): products left to right, each rounded to fp32, one final
    narrowing (lut_matvec.metal:1347-1379)."""
    x = f16([1.0, -2.0, 0.5, 3.0])
    zero = f16(np.zeros(4))
    assert np.array_equal(so.norm_scale_input(x, 1.0, zero, so.F16), x)                          # rs = 1, w = 0: identity
    assert np.array_equal(so.norm_scale_input(x, 0.25, zero, so.F16), f16([0.25, -0.5, 0.125, 0.75]))
    assert np.array_equal(so.norm_scale_input(x, 0.5, f16([1.0, 3.0, -1.0, -0.5]), so.F16), f16([1.0, -4.0, 0.0, 0.75]))
    # a product that lands exactly on an fp16 tie after its fp32 rounding, while the exact product lies
    # below the tie: narrowing the fp32 value gives 0x2670, a single rounding of the exact product 0x266F
    xt = np.array([np.float16(0.043273926)], np.float16).view(np.uint16)
    wt = np.array([np.float16(0.15661621)], np.float16).view(np.uint16)
    rs = float(np.float32(0.5022615))
    exact = float(xt.view(np.float16)[0]) * rs * (1.0 + float(wt.view(np.float16)[0]))
    assert np.float16(exact).view(np.uint16) == 0x266F
    assert so.norm_scale_input(xt, rs, wt, so.F16)[0] == 0x2670
    # against float64 on random data: never more than one 16-bit ulp away, almost always identical
    rng = fx.rng_for(97, 0)
    for dt, npdt in ((so.F16, np.float16),):
        xb, wb = f16(rng.normal(0, 2, 8192)), f16(rng.normal(0, 0.3, 8192))
        got = so.widen(so.norm_scale_input(xb, 0.7371, wb, dt), dt).astype(np.float64)
        ref = so.widen(xb, dt).astype(np.float64) * float(np.float32(0.7371)) * (1.0 + so.widen(wb, dt).astype(np.float64))
        ulp = np.spacing(np.abs(ref).astype(npdt)).astype(np.float64)
        assert np.all(np.abs(got - ref) <= ulp)
        assert np.mean(got == ref.astype(npdt).astype(np.float64)) > 0.995
    # bf16: same formula in the wider-exponent type; the staged norm of the same row agrees within an ulp
    xb, wb = so.narrow(rng.normal(0, 2, 2048).astype(np.float32), so.BF16), so.narrow(rng.normal(0, 0.3, 2048).astype(np.float32), so.BF16)
    rs = so.rms_scale(xb, 1e-6, so.BF16)
    a = so.widen(so.norm_scale_input(xb, rs, wb, so.BF16), so.BF16).astype(np.float64)
    b = so.widen(so.rms_norm_1pw(xb, wb, 1e-6, so.BF16, False), so.BF16).astype(np.float64)
    assert np.all(np.abs(a - b) <= 2.0 ** (np.floor(np.log2(np.maximum(np.abs(b), 1e-30))) - 7))


def test_geglu_closed_forms_clamps_and_float64():
    """lut_matvec.metal:2235-2243."""
    def geglu(g, u, dt=so.F16):
        return so.widen(so.epilogue_geglu(np.float32(g), np.float32(u), dt), dt)
    assert geglu([0.0], [5.0])[0] == 0.0                                   # gelu(0) = 0
    assert geglu([10.0], [0.5])[0] == 5.0                                  # tanh saturates: gelu(g) = g
    assert geglu([-10.0], [3.0])[0] == 0.0                                 # ... and gelu(-g) = 0
    assert geglu([100.0], [1000.0])[0] == 65504.0 and geglu([100.0], [-1000.0])[0] == -65504.0   # product clamp
    assert geglu([1.0 + 2.0 ** -12], [1.0])[0] == geglu([1.0], [1.0])[0]   # inputs are rounded to the 16-bit type first
    assert abs(float(geglu([1.0], [1.0])[0]) - 0.8411919906) < 1e-3        # 0.5 * (1 + tanh(0.79788 * 1.044715))
    rng = fx.rng_for(98, 0)
    g = rng.normal(0, 3, 4096).astype(np.float32)
    u = rng.normal(0, 2, 4096).astype(np.float32)
    gh_, uh = g.astype(np.float16).astype(np.float64), u.astype(np.float16).astype(np.float64)
    inner = np.clip(float(np.float32(0.7978845608)) * (gh_ + float(np.float32(0.044715)) * gh_ ** 3), -20, 20)
    ref = np.clip(0.5 * gh_ * (1 + np.tanh(inner)) * uh, -65504, 65504)
    got = geglu(g, u).astype(np.float64)
    # 1 + tanh(inner) is formed in fp32: for negative gates its rounding error (2^-24 of 1) is scaled by g * u / 2
    tol = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64) + np.abs(gh_ * uh) * 2.0 ** -22
    assert np.all(np.abs(got - ref) <= tol)
    assert np.mean(got == ref.astype(np.float16).astype(np.float64)) > 0.94


def test_norm_variants_closed_forms():
    """d256 left-to-right norm + residual + scalar (norms.metal:218-260), the fp32-input norm
    (norms_fp32.metal:50-88) and the gated norm (norms.metal:1093-1153)."""
    rng = fx.rng_for(99, 0)
    # from_fp32: unit weight (w = 0) on a constant row is +-1; large rows clamp at the fp16 limit
    assert np.array_equal(so.widen(so.rms_norm_1pw_from_fp32(np.full(64, -3.0, np.float32), f16(np.zeros(64)), 0.0, so.F16), so.F16),
                          np.full(64, -1.0, np.float32))
    big = np.zeros(16, np.float32); big[0] = 1.0
    out = so.widen(so.rms_norm_1pw_from_fp32(big, f16(np.full(16, 60000.0)), 0.0, so.F16), so.F16)
    assert out[0] == 65504.0 and np.all(out[1:] == 0)                                  # 4 * (1 + 60000) clamps
    x32 = rng.normal(0, 3, 1536).astype(np.float32)
    w = f16(rng.normal(0, 0.2, 1536))
    got = so.widen(so.rms_norm_1pw_from_fp32(x32, w, 1e-6, so.F16), so.F16).astype(np.float64)
    rs = 1.0 / np.sqrt(np.mean(x32.astype(np.float64) ** 2) + 1e-6)
    ref = x32.astype(np.float64) * rs * (1.0 + so.widen(w, so.F16).astype(np.float64))
    assert np.all(np.abs(got - ref) <= np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64))
    # fp16 input given as fp32 equals the left-to-right 16-bit norm when nothing clamps
    x = f16(rng.normal(0, 1.5, 256))
    assert np.mean(so.rms_norm_1pw_from_fp32(so.widen(x, so.F16), w[:256], 1e-6, so.F16) == so.rms_norm_1pw(x, w[:256], 1e-6, so.F16, 2)) > 0.99
    # left-to-right against scale-first: same value up to the last place
    a = so.widen(so.rms_norm_1pw(x, w[:256], 1e-6, so.F16, 2), so.F16).astype(np.float64)
    b = so.widen(so.rms_norm_1pw(x, w[:256], 1e-6, so.F16, 0), so.F16).astype(np.float64)
    assert np.all(np.abs(a - b) <= np.spacing(np.abs(b).astype(np.float16)).astype(np.float64)) and np.mean(a == b) > 0.9
    # + residual, * scalar: scalar 1 is the add form, scalar 0.5 halves it exactly, scalar 0 gives zeros
    res = f16(rng.normal(0, 1, 256))
    added = so.rms_norm_1pw(x, w[:256], 1e-6, so.F16, 2, res)
    assert np.array_equal(so.rms_norm_1pw_add_scalar(x, w[:256], res, int(f16([1.0])[0]), 1e-6, so.F16), added)
    half = so.widen(so.rms_norm_1pw_add_scalar(x, w[:256], res, int(f16([0.5])[0]), 1e-6, so.F16), so.F16)
    assert np.array_equal(half[np.abs(half) > 1e-3], (so.widen(added, so.F16) * 0.5)[np.abs(half) > 1e-3])
    assert not so.widen(so.rms_norm_1pw_add_scalar(x, w[:256], res, 0, 1e-6, so.F16), so.F16).any()
    # gated: gate 0 -> 0; large gate -> w * x * rs * gate; heads are normalised separately
    heads, d = 3, 128
    xh = f16(rng.normal(0, 1, heads * d) * np.repeat([1.0, 10.0, 0.1], d))
    wg = f16(1.0 + rng.normal(0, 0.1, d))
    assert not so.widen(so.rms_norm_gated(xh, f16(np.zeros(heads * d)), wg, heads, d, 1e-6, so.F16), so.F16).any()
    gate = f16(rng.normal(0, 2, heads * d))
    got = so.widen(so.rms_norm_gated(xh, gate, wg, heads, d, 1e-6, so.F16), so.F16).astype(np.float64)
    xf, gf = so.widen(xh, so.F16).astype(np.float64).reshape(heads, d), so.widen(gate, so.F16).astype(np.float64).reshape(heads, d)
    rs = 1.0 / np.sqrt((xf ** 2).mean(axis=1, keepdims=True) + 1e-6)
    ref = (so.widen(wg, so.F16).astype(np.float64)[None, :] * xf * rs * gf / (1.0 + np.exp(-gf))).ravel()
    assert np.all(np.abs(got - ref) <= np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64) + 1e-7)
    assert np.mean(got == ref.astype(np.float16).astype(np.float64)) > 0.98


def test_gated_norm_precise_form_and_its_view():
    """rms_norm_gated_d128 (norms_gated_precise.metal:7-52): half(w) * half(x * rs) is a 16-bit product
    before the fp32 SiLU; restated in numpy float16, and the fused view is the plain i6 view of it."""
    rng = fx.rng_for(100, 0)
    heads, d = 4, 128
    x = f16(rng.normal(0, 1, heads * d) * np.repeat([1.0, 6.0, 0.2, 1.0], d))
    gate = f16(rng.normal(0, 2, heads * d))
    w = f16(1.0 + rng.normal(0, 0.1, d))
    got = so.rms_norm_gated(x, gate, w, heads, d, 1e-6, so.F16, precise=True).view(np.float16)
    xf = so.widen(x, so.F16).reshape(heads, d)
    rs = np.array([so.rms_scale(x[h * d:(h + 1) * d], 1e-6, so.F16) for h in range(heads)], np.float32)[:, None]
    normalized = (w.view(np.float16)[None, :] * (xf * rs).astype(np.float16)).astype(np.float16)      # float16 x float16
    g = so.widen(gate, so.F16).reshape(heads, d)
    tail = np.float32(1) / (np.float32(1) + np.exp(np.abs(g), dtype=np.float32))
    sig = np.where(g < 0, tail, np.float32(1) - tail).astype(np.float32)
    ref = (normalized.astype(np.float32) * (g * sig)).astype(np.float16).ravel()
    ulp = np.spacing(np.abs(ref)).astype(np.float64)
    assert np.all(np.abs(got.astype(np.float64) - ref.astype(np.float64)) <= ulp)          # exp may differ in its last bit
    assert np.mean(got.view(np.uint16) == ref.view(np.uint16)) > 0.99
    # the two arithmetic forms agree to a couple of 16-bit ulps and are not the same function
    generic = so.rms_norm_gated(x, gate, w, heads, d, 1e-6, so.F16).view(np.float16)
    assert np.all(np.abs(generic.astype(np.float64) - got.astype(np.float64)) <= 3 * np.spacing(np.abs(got)).astype(np.float64) + 1e-7)
    assert np.any(generic.view(np.uint16) != got.view(np.uint16))
    for precise in (False, True):
        staged = so.activation_bitplanes(so.rms_norm_gated(x, gate, w, heads, d, 1e-6, so.F16, precise), 6, so.F16)
        fused = so.rms_norm_gated_activation_bitplanes(x, gate, w, heads, 1e-6, so.F16, precise)
        assert np.array_equal(staged[0], fused[0]) and np.array_equal(staged[1], fused[1])


def test_pointwise_activations_closed_forms_and_float64():
    """activations.metal:5-40, 98-108, 166-177."""
    one = lambda name, v, p=0.0: float(so.widen(so.unary(name, f16([v]), so.F16, p), so.F16)[0])
    assert one("silu", 0.0) == 0.0 and one("sigmoid_kernel", 0.0) == 0.5
    assert one("softplus", 25.0) == 25.0 and abs(one("softplus", 0.0) - np.log(2)) < 1e-3      # x itself above 20
    assert one("scalar_mul", 3.0, 0.25) == 0.75
    assert abs(one("logit_cap", 0.01, 30.0) - 0.01) < 1e-5 and abs(one("logit_cap", 1000.0, 30.0) - 30.0) < 1e-2
    rng = fx.rng_for(101, 0)
    x = f16(rng.normal(0, 4, 4096))
    xf = so.widen(x, so.F16).astype(np.float64)
    refs = {"silu": xf / (1 + np.exp(-xf)), "sigmoid_kernel": 1 / (1 + np.exp(-xf)),
            "softplus": np.where(xf > 20, xf, np.log1p(np.exp(xf))), "scalar_mul": xf * float(np.float32(0.37)),
            "logit_cap": 30.0 * np.tanh(xf / 30.0)}
    for name, ref in refs.items():
        got = so.widen(so.unary(name, x, so.F16, 0.37 if name == "scalar_mul" else 30.0), so.F16).astype(np.float64)
        ulp = np.spacing(np.abs(ref).astype(np.float16)).astype(np.float64)
        assert np.all(np.abs(got - ref) <= ulp + 1e-7 * np.abs(xf)), name
        assert np.mean(got == ref.astype(np.float16).astype(np.float64)) > 0.97, name
