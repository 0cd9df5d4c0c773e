"""Pins the CPU oracle before anything is compared against it.

Each test checks an oracle function against something independent of the oracle's
own source: a known-answer vector held by the reference's tests, numpy's IEEE
conversions, an exact-rational recomputation, or a brute-force closed form.
"""
from fractions import Fraction

import numpy as np
import pytest

import fixtures as fx
from oracle import oracle as so

FMT = {"binary1": so.BINARY1, "ternary2": so.TERNARY2}


# ---------------------------------------------------------------------------
# conversions: exhaustive / dense against numpy's independent implementation
# ---------------------------------------------------------------------------

def test_f16_widening_exhaustive_matches_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    ours = so.f16_bits_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    both_nan = np.isnan(ours) & np.isnan(ref)
    assert np.array_equal(ours.view(np.uint32)[~both_nan], ref.view(np.uint32)[~both_nan])


def test_f16_narrowing_matches_numpy_on_ties_edges_and_random():
    rng = np.random.default_rng(1)
    # every fp16 value, every midpoint between neighbours, and one ulp32 either side
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = (h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2
    mids32 = mids.astype(np.float32)
    cand = np.concatenate([
        h, mids32, np.nextafter(mids32, np.float32(np.inf)), np.nextafter(mids32, np.float32(-np.inf)),
        np.array([65504, 65519.99, 65520, 65536, 1e9, np.inf, 2**-24, 2**-25, 2**-25 * 1.0001,
                  2**-26, 0.0, 5.96e-8, 6.1e-5, 6.097e-5], np.float32),
        rng.normal(0, 1, 20000).astype(np.float32),
        (rng.normal(0, 1, 20000) * 10.0 ** rng.integers(-9, 6, 20000)).astype(np.float32),
    ])
    cand = np.concatenate([cand, -cand]).astype(np.float32)
    with np.errstate(over="ignore"):
        ref = cand.astype(np.float16).view(np.uint16)
    ours = so.f32_to_f16_bits(cand)
    assert np.array_equal(ours, ref)


def test_bf16_matches_closed_form_and_numpy_helpers():
    rng = np.random.default_rng(2)
    v = (rng.normal(0, 1, 5000) * 10.0 ** rng.integers(-20, 20, 5000)).astype(np.float32)
    l = so.lib()
    ours = np.array([l.so_f32_to_bf16(float(x)) for x in v], np.uint16)
    # independent: nearest of the two bracketing bf16 values in exact arithmetic, ties to even
    for x, o in zip(v[:600], ours[:600]):
        b = int(np.float32(x).view(np.uint32))
        lo = b & 0xFFFF0000
        hi = lo + 0x10000
        flo = Fraction(float(np.uint32(lo).view(np.float32)))
        fhi = Fraction(float(np.uint32(hi & 0xFFFFFFFF).view(np.float32)))
        fx_ = Fraction(float(x))
        dlo, dhi = abs(fx_ - flo), abs(fhi - fx_)
        want = lo if dlo < dhi else hi if dhi < dlo else (lo if ((lo >> 16) & 1) == 0 else hi)
        assert o == (want >> 16) & 0xFFFF
    assert np.array_equal(so.narrow(v, so.BF16), ours)
    assert np.array_equal(so.widen(ours, so.BF16),
                          np.array([l.so_bf16_to_f32(int(b)) for b in ours], np.float32))


# ---------------------------------------------------------------------------
# signed codec known answers (SmeltSignedQuantCodecTests.swift)
# ---------------------------------------------------------------------------

def test_signed_codec_geometry_and_known_rows():
    g = fx.golden_vectors()["signed_codec"]
    l = so.lib()
    for n, fmt, want in g["packed_byte_count"]:
        assert l.so_signed_packed_byte_count(n, FMT[fmt]) == want
    for pc, gs, want in g["groups_per_row_ok"]:
        assert l.so_signed_groups_per_row(pc, gs) == want
    for pc, gs in g["groups_per_row_throws"]:
        assert l.so_signed_groups_per_row(pc, gs) == so.ERR_GEOMETRY
    for name, fmt in (("binary", so.BINARY1), ("ternary", so.TERNARY2)):
        case = g[name]
        codes = np.array([case["codes"]], np.uint8)
        scales = fx.f16_bits(case["scales_f32"]).reshape(1, -1)
        out = so.signed_dequantize(fmt, codes, scales, case["cols"], case["cols"], case["group"])
        assert out[0].tolist() == [float(v) for v in case["expected"]]
        out16 = np.zeros(case["cols"], np.uint16)
        rc = l.so_signed_dequantize_row_f16(fmt, codes.ctypes.data, codes.size, scales.ctypes.data,
                                            scales.size * 2, case["cols"], case["cols"],
                                            case["group"], out16.ctypes.data)
        assert rc == so.OK
        assert out16.view(np.float16).astype(np.float32).tolist() == out[0].tolist()


def test_signed_codec_rejects_ternary_code_three():
    case = fx.golden_vectors()["signed_codec"]["ternary_code3"]
    codes = np.array(case["codes"], np.uint8)
    import ctypes
    bad = ctypes.c_int64(-1)
    rc = so.lib().so_signed_validate_codes(codes.ctypes.data, codes.size, case["logical_count"],
                                           so.TERNARY2, ctypes.byref(bad))
    assert rc == so.ERR_INVALID_CODE and bad.value == case["bad_index"]


def test_mlx_scale_normalisation_known_answers():
    g = fx.golden_vectors()["mlx_scale_normalisation"]
    l = so.lib()
    import ctypes
    out = ctypes.c_uint16(0)
    for fmt, s, b, want in g["ok_f32"]:
        rc = l.so_signed_canonical_mlx_scale_bits(FMT[fmt], int(fx.f16_bits([s])[0]),
                                                  int(fx.f16_bits([b])[0]), ctypes.byref(out))
        assert rc == so.OK and out.value == int(fx.f16_bits([want])[0])
    for fmt, s, b in g["reject_f32"]:
        rc = l.so_signed_canonical_mlx_scale_bits(FMT[fmt], int(fx.f16_bits([s])[0]),
                                                  int(fx.f16_bits([b])[0]), ctypes.byref(out))
        assert rc == so.ERR_MLX_BIAS
    for fmt, s, b, want in g["ok_bits"]:
        rc = l.so_signed_canonical_mlx_scale_bits(FMT[fmt], s, b, ctypes.byref(out))
        assert rc == so.OK and out.value == want
    for fmt, s, b in g["reject_bits"]:
        assert l.so_signed_canonical_mlx_scale_bits(FMT[fmt], s, b, ctypes.byref(out)) == so.ERR_MLX_BIAS
    # negative / non-finite source scale is an invalid-scale error
    assert l.so_signed_canonical_mlx_scale_bits(so.BINARY1, 0xBC00, 0x3800, ctypes.byref(out)) == so.ERR_MLX_SCALE
    assert l.so_signed_canonical_mlx_scale_bits(so.TERNARY2, 0x7C00, 0xFC00, ctypes.byref(out)) == so.ERR_MLX_SCALE


def test_signed_code_extraction_brute_force_all_bytes():
    l = so.lib()
    for byte in range(256):
        arr = np.array([byte], np.uint8)
        for i in range(8):
            assert l.so_signed_code_at(i, arr.ctypes.data, 1, so.BINARY1) == (byte >> i) & 1
        for i in range(4):
            assert l.so_signed_code_at(i, arr.ctypes.data, 1, so.TERNARY2) == (byte >> (2 * i)) & 3
        if byte < 243:
            digits = [(byte // 3 ** i) % 3 for i in range(5)]
            for i in range(5):
                assert l.so_signed_code_at(i, arr.ctypes.data, 1, so.TRIT5) == digits[i]
        else:
            assert l.so_signed_code_at(0, arr.ctypes.data, 1, so.TRIT5) == so.ERR_INVALID_CODE


def test_trit5_lut_exhaustive_and_agrees_with_ternary2():
    lut = so.trit5_lut()
    for b in range(243):
        digits = [(b // 3 ** i) % 3 for i in range(5)]
        assert lut[b] == sum(d << (2 * i) for i, d in enumerate(digits))
        assert sum(d * 3 ** i for i, d in enumerate(digits)) == b
    assert all(lut[b] == 0xFFFF for b in range(243, 256))
    # same logical matrix through both encodings dequantises identically; K not a multiple of 5
    rng = np.random.default_rng(5)
    rows, cols = 7, 384
    codes = rng.integers(0, 3, size=(rows, cols), dtype=np.uint8)
    scales = fx.f16_bits(np.abs(rng.normal(0, 0.02, (rows, cols // 128))))
    p2 = so.signed_pack(codes, so.TERNARY2)
    p5 = so.signed_pack(codes, so.TRIT5)
    assert p5.shape[1] == (cols + 4) // 5
    assert np.array_equal(p2, fx.pack_signed_np(codes, fx.TERNARY2))
    assert np.array_equal(p5, fx.pack_signed_np(codes, fx.TRIT5))
    d2 = so.signed_dequantize(so.TERNARY2, p2, scales, cols, cols, 128)
    d5 = so.signed_dequantize(so.TRIT5, p5, scales, cols, cols, 128)
    assert np.array_equal(d2, d5)
    want = (codes.astype(np.float32) - 1) * np.repeat(fx.from_bits(scales, fx.F16), 128, axis=1)
    assert np.array_equal(d2, want)
    # the tail digits of the last byte encode semantic zero
    tail = int(p5[0, -1])
    assert [(tail // 3 ** i) % 3 for i in range(5)][cols % 5:] == [1] * (5 - cols % 5)


def test_binary_pack_matches_numpy_packbits():
    rng = np.random.default_rng(6)
    codes = rng.integers(0, 2, size=(3, 256), dtype=np.uint8)
    assert np.array_equal(so.signed_pack(codes, so.BINARY1), np.packbits(codes, axis=1, bitorder="little"))
    assert np.array_equal(fx.pack_signed_np(codes, fx.BINARY1), np.packbits(codes, axis=1, bitorder="little"))


# ---------------------------------------------------------------------------
# affine u4 known answers (SmeltAffineU4Tests.swift)
# ---------------------------------------------------------------------------

def test_affine_exact_packing_layout_and_constant_group():
    g = fx.golden_vectors()["affine_u4"]
    cols, group = g["ramp"]["cols"], g["ramp"]["group"]
    w = np.arange(cols, dtype=np.float32)[None, :]
    packed, scales, biases = so.affine_quantize(w, group)
    assert packed.shape == (1, 8)
    for i in range(8):
        assert packed[0, i] == (((2 * i + 1) << 4) | (2 * i))
    assert scales[0, 0] == 0x3C00 and biases[0, 0] == 0
    assert np.array_equal(so.affine_dequantize(packed, scales, biases, cols, group), w)

    c = g["constant"]
    w = np.full((1, c["cols"]), c["value"], np.float32)
    packed, scales, biases = so.affine_quantize(w, c["group"])
    deq = so.affine_dequantize(packed, scales, biases, c["cols"], c["group"])
    assert scales[0, 0] == 0x3C00
    assert np.all(deq == np.float32(np.float16(c["value"])))


def _lcg_gaussian(n, scale):
    """SmeltAffineU4Tests.swift:9-27 — LCG + Box-Muller test data."""
    state = 0x9E3779B97F4A7C15
    out = np.zeros(n, np.float32)
    mask = (1 << 64) - 1

    def nxt():
        nonlocal state
        state = (state * 6364136223846793005 + 1442695040888963407) & mask
        return np.float32(state >> 40) / np.float32(1 << 24)

    i = 0
    while i < n:
        u1 = max(nxt(), np.float32(1e-7))
        u2 = nxt()
        r = np.sqrt(np.float32(-2.0) * np.log(u1, dtype=np.float32), dtype=np.float32)
        out[i] = r * np.cos(np.float32(2 * np.pi) * u2, dtype=np.float32) * np.float32(scale)
        if i + 1 < n:
            out[i + 1] = r * np.sin(np.float32(2 * np.pi) * u2, dtype=np.float32) * np.float32(scale)
        i += 2
    return out


def test_affine_quantize_invariants_from_reference_tests():
    rows, cols, g = 64, 2048, 64
    w = _lcg_gaussian(rows * cols, 0.02).reshape(rows, cols)
    packed, scales, biases = so.affine_quantize(w, g)
    deq = so.affine_dequantize(packed, scales, biases, cols, g)
    rl2 = np.linalg.norm(deq - w) / np.linalg.norm(w)
    cos = float((deq * w).sum() / (np.linalg.norm(deq) * np.linalg.norm(w)))
    assert rl2 < 0.10 and cos > 0.995          # SmeltAffineU4Tests.swift:43-64
    w2 = _lcg_gaussian(32 * 1024, 0.05).reshape(32, 1024)
    e = {}
    for gs in (64, 32):
        p, s, b = so.affine_quantize(w2, gs)
        e[gs] = np.linalg.norm(so.affine_dequantize(p, s, b, 1024, gs) - w2) / np.linalg.norm(w2)
    assert e[32] <= e[64] + 1e-6               # :57-64
    # mseOptimal never worse than minMax (:82-100)
    wm = w[:16].copy()
    wm[:, ::37] = 0.5
    pm, sm, bm = so.affine_quantize(wm, g, clip=0)
    po, so_, bo = so.affine_quantize(wm, g, clip=1)
    em = np.linalg.norm(so.affine_dequantize(pm, sm, bm, cols, g) - wm)
    eo = np.linalg.norm(so.affine_dequantize(po, so_, bo, cols, g) - wm)
    assert eo <= em + 1e-6


def test_affine_dequant_exhaustive_over_nibbles_is_two_rounded_flops():
    rng = np.random.default_rng(7)
    sb = rng.integers(0, 0x7C00, size=(400, 2)).astype(np.uint16)
    sb[:, 1] |= (rng.integers(0, 2, 400) << 15).astype(np.uint16)
    for dtype in (so.F16, so.BF16):
        for s_bits, b_bits in sb[:200]:
            packed = np.array([[(2 * i + 1) << 4 | (2 * i) for i in range(8)]], np.uint8)
            out = so.affine_dequantize(packed, np.array([[s_bits]], np.uint16),
                                       np.array([[b_bits]], np.uint16), 16, 16, dtype)
            s = fx.from_bits(np.array([s_bits], np.uint16), dtype)[0]
            b = fx.from_bits(np.array([b_bits], np.uint16), dtype)[0]
            with np.errstate(over="ignore", invalid="ignore"):
                want = (np.arange(16, dtype=np.float32) * s).astype(np.float32) + b
            assert np.array_equal(out[0].view(np.uint32), want.astype(np.float32).view(np.uint32))


def test_affine_narrow_row_equals_rounded_wide_row():
    packed, scales, biases, _, _ = fx.affine_synthetic_fixture(4, 256, 64, seed=3)
    wide = so.affine_dequantize(packed, scales, biases, 256, 64)
    narrow = so.affine_dequantize_narrow(packed, scales, biases, 256, 64)
    assert np.array_equal(narrow, wide.astype(np.float16).view(np.uint16))


# ---------------------------------------------------------------------------
# matvec references
# ---------------------------------------------------------------------------

def test_ternary_affine_qmv_reproduces_mlx_golden_bits():
    g = fx.golden_vectors()
    for key in ("ternary_qmv_mlx_k512", "ternary_qmv_mlx_k5120_m3"):
        case = g[key]
        codes, scales, x = fx.mlx_ternary_fixture(case["rows"], case["cols"], case["batch"], case["scale_unit"])
        packed = so.signed_pack(codes, so.TERNARY2)
        out = so.ternary_affine_qmv(packed, scales, x, case["rows"], case["cols"])
        want = np.array([int(b, 16) for b in case["expected_bits"]], np.uint16)
        assert np.array_equal(out.ravel(), want), key
        # the same fixture through the plain signed reference (fp32, sequential) and an exact
        # rational recomputation: all partial sums are dyadic and exact, so one final RNE agrees
        ref = so.signed_matvec(so.TERNARY2, packed, scales, fx.from_bits(x, fx.F16), case["rows"],
                               case["cols"], case["cols"], 128)
        assert np.array_equal(ref.astype(np.float16).view(np.uint16).ravel(), want)
        sc = fx.from_bits(scales, fx.F16)
        xv = fx.from_bits(x, fx.F16)
        for b in range(case["batch"]):
            for r in range(case["rows"]):
                acc = Fraction(0)
                for c in range(case["cols"]):
                    acc += Fraction(float(xv[b, c])) * (int(codes[r, c]) - 1) * Fraction(float(sc[r, c // 128]))
                assert np.float16(float(acc)).view(np.uint16) == want[b * case["rows"] + r]


def _exact_qmm_bits(w_bits, x_bits):
    """fp16 outputs [batch, rows] of fp16 weights times fp16 activations with an exact
    rational sum and one rounding to half."""
    w = w_bits.view(np.float16)
    x = x_bits.view(np.float16)
    out = np.zeros((x.shape[0], w.shape[0]), np.uint16)
    for b in range(x.shape[0]):
        for r in range(w.shape[0]):
            acc = sum((Fraction(float(a)) * Fraction(float(v)) for a, v in zip(x[b], w[r])), Fraction(0))
            # float(acc) is exact here: every product is a multiple of 2^-28 and |acc| < 2
            assert Fraction(float(acc)) == acc
            out[b, r] = np.float16(float(acc)).view(np.uint16)
    return out


def test_ternary_affine_qmm_reproduces_mlx_golden_bits():
    """The 112 bit patterns MLX's affine_qmm_t produced (SignedQuantKernelTests.swift:549-568).
    Every fp32 partial sum of this fixture is exact, so the unspecified order inside the matrix
    unit does not matter and one rounding of the exact sum must give the same bits."""
    case = fx.golden_vectors()["ternary_qmm_mlx_m14"]
    rows, cols, batch = case["rows"], case["cols"], case["batch"]
    codes, scales, x = fx.mlx_ternary_qmm_fixture(rows, cols, batch, case["scale_bits"])
    packed = so.signed_pack(codes, so.TERNARY2)
    want = np.array([int(b, 16) for b in case["expected_bits"]], np.uint16).reshape(batch, rows)
    w = so.ternary_affine_qmm_weights(packed, scales, rows, cols)
    assert np.array_equal(_exact_qmm_bits(w, x), want)
    out = so.ternary_affine_qmm(packed, scales, x, rows, cols)
    assert np.array_equal(out.astype(np.float16).view(np.uint16), want)


def test_ternary_affine_qmm_weight_tile_uses_rounded_byte_lane_subscales():
    """signed_quant_precise.metal:407-439 against an independent numpy float16 evaluation, on
    scales whose /16 and /64 fall into the fp16 subnormal range with bits to lose: there the
    tile is not (code - 1) * scale, and a zero code does not dequantise to exactly zero."""
    rows, cols = 8, 256
    scale_bits = ["1b95", "1797", "0c01", "13ff", "2057", "0801"]
    codes, scales, _ = fx.mlx_ternary_qmm_fixture(rows, cols, 1, scale_bits)
    packed = so.signed_pack(codes, so.TERNARY2)
    got = so.ternary_affine_qmm_weights(packed, scales, rows, cols)
    s = np.repeat(scales.view(np.float16), 128, axis=1)
    lane = (np.arange(cols) & 3)[None, :]
    sub = s.copy()
    for k in (1, 2, 3):
        sub = np.where(lane == k, s / np.float16(4 ** k), sub)       # float16 division: rounds once
    assert sub.dtype == np.float16
    shifted = (codes.astype(np.int32) << (2 * lane)).astype(np.float16)
    prod = sub * shifted                                             # exact for fields 0, 1, 2
    assert np.array_equal(prod.astype(np.float64), sub.astype(np.float64) * shifted.astype(np.float64))
    want = (prod.astype(np.float64) - s.astype(np.float64)).astype(np.float16)  # exact sum, one rounding
    assert np.array_equal(got, want.view(np.uint16))
    naive = ((codes.astype(np.float32) - 1) * s.astype(np.float32)).astype(np.float16)
    differs = got != naive.view(np.uint16)
    assert differs.any() and not differs[:, lane[0] == 0].any()
    assert (got.view(np.float16)[codes == 1] != 0).any()
    # a separate bias buffer is honoured (binding 2 of the reference kernel)
    other = np.roll(scales, 1, axis=1)
    got2 = so.ternary_affine_qmm_weights(packed, scales, rows, cols, bias_scales=other)
    want2 = (prod.astype(np.float64) - np.repeat(other.view(np.float16), 128, axis=1).astype(np.float64))
    assert np.array_equal(got2, want2.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("fmt", [so.BINARY1, so.TERNARY2, so.TRIT5])
def test_signed_matvec_against_numpy_dequant_dot(fmt):
    base = fx.TERNARY2 if fmt == so.TRIT5 else fmt
    codes, scales, x = fx.signed_synthetic_fixture(base)
    rows, cols = codes.shape
    packed = so.signed_pack(codes, fmt)
    xf = fx.from_bits(x, fx.F16)
    out = so.signed_matvec(fmt, packed, scales, xf, rows, cols, cols, 128)
    sem = np.where(codes == 0, -1.0, 1.0) if base == fx.BINARY1 else codes.astype(np.float64) - 1
    w = sem * np.repeat(fx.from_bits(scales, fx.F16).astype(np.float64), 128, axis=1)
    want = xf.astype(np.float64) @ w.T
    assert np.allclose(out, want, rtol=0, atol=2e-5)
    f64 = so.signed_matvec_f64(fmt, packed, scales, xf, rows, cols, cols, 128)
    assert np.allclose(f64, want, rtol=1e-12, atol=1e-12)
    # dropping the sign map (binary 0 -> 0 instead of -1) or the scale index would show here
    wrong = xf.astype(np.float64) @ (codes.astype(np.float64) * np.repeat(
        fx.from_bits(scales, fx.F16).astype(np.float64), 128, axis=1)).T
    assert not np.allclose(out, wrong, atol=1e-3)


@pytest.mark.parametrize("dtype", [so.F16, so.BF16])
def test_affine_matvec_groupwise_form_matches_dequant_dot(dtype):
    rows, cols, group = 24, 512, 64
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=0, tensor=1)
    x = fx.from_bits(fx.synth_activation(2, cols, dtype), dtype)
    out = so.affine_matvec(packed, scales, biases, x, rows, cols, group, dtype)
    f64 = so.affine_matvec_f64(packed, scales, biases, x, rows, cols, group, dtype)
    # independent numpy: per-element dequant (mul then add in fp32) then float64 dot
    nib = np.stack([packed & 0xF, packed >> 4], axis=2).reshape(rows, cols).astype(np.float32)
    s = np.repeat(fx.from_bits(scales, dtype), group, axis=1)
    b = np.repeat(fx.from_bits(biases, dtype), group, axis=1)
    w = (nib * s).astype(np.float32) + b
    want = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.allclose(f64, want, rtol=1e-12, atol=1e-12)
    assert np.allclose(out, want, rtol=0, atol=5e-5 * np.abs(want).max())


def test_affine_matvec_exact_on_dyadic_fixture():
    """KernelLab.swift:2829-2855 buffers: scale 2^-4, bias 0, x in {0.5,-0.25}: every partial
    sum is an exact dyadic, so the fp32 result equals the exact rational value."""
    rows, cols, group, batch = 8, 256, 64, 3
    packed, scales, biases, x = fx.kernel_lab_qmm_fixture(rows, cols, group, batch)
    xf = fx.from_bits(x, fx.F16)
    out = so.affine_matvec(packed, scales, biases, xf, rows, cols, group)
    for b in range(batch):
        for r in range(rows):
            acc = Fraction(0)
            for c in range(cols):
                byte = int(packed[r, c // 2])
                nib = (byte & 15) if c % 2 == 0 else (byte >> 4)
                acc += Fraction(nib, 16) * Fraction(float(xf[b, c]))
            assert Fraction(float(out[b, r])) == acc


# ---------------------------------------------------------------------------
# argmax key and epilogues
# ---------------------------------------------------------------------------

def test_argmax_special_cases_and_brute_force():
    f = fx.f16_bits
    assert so.argmax16(f([1.0, 2.0, 2.0, -3.0])) == 1                 # ties -> lowest index
    assert so.argmax16(np.array([0x8000, 0x0000], np.uint16)) == 0     # -0 == +0
    assert so.argmax16(np.array([0x0000, 0x8000], np.uint16)) == 0
    assert so.argmax16(f([-5, -2, -2, -9])) == 1
    assert so.argmax16(np.array([0x8001, 0x8000], np.uint16)) == 1     # -tiny < 0
    rng = np.random.default_rng(11)
    for _ in range(50):
        v = rng.normal(0, 3, 300).astype(np.float16)
        v[rng.integers(0, 300, 40)] = v[rng.integers(0, 300)]
        assert so.argmax16(v.view(np.uint16)) == int(np.argmax(v.astype(np.float32)))
    l = so.lib()
    # ordered key is strictly monotone over all finite fp16 values
    vals = np.arange(0x10000, dtype=np.uint32).astype(np.uint16)
    finite = vals[(vals & 0x7C00) != 0x7C00]
    fl = finite.view(np.float16).astype(np.float32)
    keys = np.array([l.so_argmax_ordered_key16(int(b)) for b in finite])
    order = np.argsort(fl, kind="stable")
    ks, fs = keys[order], fl[order]
    assert np.all((np.diff(ks) > 0) == (np.diff(fs) > 0))
    assert (l.so_argmax_pack_key(0x3C00, 5) & 0xFFFFFFFF) == (1 << 18) - 1 - 5


def test_epilogues_against_numpy_half_arithmetic():
    rng = np.random.default_rng(12)
    acc = rng.normal(0, 2, 200).astype(np.float32)
    res = rng.normal(0, 1, 200).astype(np.float16)
    got = so.epilogue_residual_add(acc, res.view(np.uint16), so.F16)
    want = (acc.astype(np.float16) + res).astype(np.float16)          # numpy half add is RNE
    assert np.array_equal(got, want.view(np.uint16))
    g = rng.normal(0, 3, 200).astype(np.float32)
    u = rng.normal(0, 3, 200).astype(np.float32)
    got = so.epilogue_affine_swiglu(g, u, so.F16)
    want = (g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u).astype(np.float16)
    diff = np.abs(got.view(np.float16).astype(np.float32) - want.astype(np.float32))
    assert np.all(diff <= np.spacing(np.abs(want)).astype(np.float32))
    gh, uh = g.astype(np.float16), u.astype(np.float16)
    got = so.epilogue_signed_swiglu(gh.view(np.uint16), uh.view(np.uint16), so.F16)
    one = np.float16(1)
    e = np.exp(np.abs(gh).astype(np.float32)).astype(np.float16)
    tail = (one / (one + e).astype(np.float16)).astype(np.float16)
    sig = np.where(gh < 0, tail, (one - tail).astype(np.float16)).astype(np.float16)
    want = ((gh * sig).astype(np.float16) * uh).astype(np.float16)
    assert np.array_equal(got, want.view(np.uint16))
