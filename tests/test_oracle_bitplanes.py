"""Pins of the oracle's signed-activation-view functions: the plane encoding is decoded back to the
integers it must hold, the popcount dot is checked against a brute-force integer dot, scales and
rounding against numpy, and the whole matvec against the CPU mirror inside the reference's own
test (SignedQuantKernelTests.swift:1523-1650) on that test's fixture."""
import numpy as np
import pytest

import fixtures as fx
from oracle import oracle as so


def decode_planes(planes):
    groups, n, _ = planes.shape
    bits = ((planes[:, :, :, None] >> np.arange(32, dtype=np.uint32)) & 1).reshape(groups, n, 128).astype(np.int64)
    mag = sum(bits[:, p, :] << p for p in range(n - 1))
    return (np.where(bits[:, n - 1, :] == 1, -mag, mag)).reshape(-1)


def round_half_away(v):
    return np.sign(v) * np.floor(np.abs(v) + 0.5)


@pytest.mark.parametrize("planes", [2, 3, 4, 5, 6])
@pytest.mark.parametrize("dtype", [so.F16, so.BF16])
def test_activation_view_encodes_the_rounded_quotients(planes, dtype):
    rng = fx.rng_for(110, planes)
    x = rng.normal(0, 1.3, 1024).astype(np.float32)
    x[128:256] = 0.0                                  # an all-zero group
    x[300] = 40.0                                     # an outlier that sets its group's scale
    bits = so.narrow(x, dtype)
    pl, scales, q = so.activation_bitplanes(bits, planes, dtype)
    max_q = {2: 1, 3: 3, 4: 7, 5: 15, 6: 31}[planes]
    assert so.lib().so_bitplane_max_q(planes) == max_q
    assert np.array_equal(decode_planes(pl), q)                        # sign-magnitude planes hold q exactly
    assert np.abs(q).max() == max_q and np.abs(q).max() <= max_q
    xv = so.widen(bits, dtype).reshape(-1, 128)
    max_abs = np.abs(xv).max(axis=1)
    producer = np.where(max_abs > 0, max_abs / np.float32(max_q), np.float32(1.0)).astype(np.float32)
    assert np.array_equal(scales, so.narrow(producer, dtype))          # stored scale = rounded max / max_q, 1 for zeros
    assert scales[1] == so.narrow(np.float32([1.0]), dtype)[0] and not q[128:256].any()
    used = so.widen(scales, dtype) if planes >= 4 else producer        # i2 / i3 quantise with the unrounded scale
    want = round_half_away(np.clip((xv / used[:, None]).astype(np.float32), -max_q, max_q)).reshape(-1)
    assert np.array_equal(q, want.astype(np.int64))
    assert np.all(q[np.abs(xv.reshape(-1)) == max_abs.repeat(128)][max_abs.repeat(128)[np.abs(xv.reshape(-1)) == max_abs.repeat(128)] > 0] != 0)


def brute_dot(sem, q, rows, cols):
    return (sem.reshape(rows, cols // 128, 128).astype(np.int64) * q.reshape(1, cols // 128, 128)).sum(axis=2)


@pytest.mark.parametrize("fmt,planes", [(so.BINARY1, 2), (so.BINARY1, 4), (so.BINARY1, 6), (so.TERNARY2, 4), (so.TERNARY2, 5)])
def test_bitplane_matvec_is_the_integer_dot_times_both_scales(fmt, planes):
    rows, cols = 11, 640
    rng = fx.rng_for(111, planes + 10 * fmt)
    codes = rng.integers(0, 2 if fmt == so.BINARY1 else 3, (rows, cols)).astype(np.uint8)
    sem = codes.astype(np.int64) * 2 - 1 if fmt == so.BINARY1 else codes.astype(np.int64) - 1
    packed = so.signed_pack(codes, fmt)
    ws = so.narrow(np.abs(rng.normal(0, 0.02, (rows, cols // 128))).astype(np.float32) + 1e-3, so.F16)
    x = so.narrow(rng.normal(0, 1, cols).astype(np.float32), so.F16)
    pl, asc, q = so.activation_bitplanes(x, planes, so.F16)
    got = so.signed_bitplane_matvec(fmt, packed, ws, pl, asc, rows, cols, so.F16)
    dots = brute_dot(sem, q, rows, cols)
    exact = (dots * so.widen(asc, so.F16).astype(np.float64)[None, :] * so.widen(ws, so.F16).astype(np.float64)).sum(axis=1)
    assert np.all(np.abs(got - exact) <= 1e-6 * np.abs(exact).max() + 1e-9)
    # a single weight flip moves the result by exactly 2 |q| as ws (binary): the dot really reads the codes
    if fmt == so.BINARY1:
        codes2 = codes.copy(); codes2[3, 200] ^= 1
        got2 = so.signed_bitplane_matvec(fmt, so.signed_pack(codes2, fmt), ws, pl, asc, rows, cols, so.F16)
        step = 2 * abs(int(q[200])) * float(so.widen(asc, so.F16)[1]) * float(so.widen(ws, so.F16)[3, 1])
        assert abs(abs(got2[3] - got[3]) - step) <= 2e-6 * max(abs(got[3]), abs(got2[3]), step) and np.array_equal(np.delete(got2, 3), np.delete(got, 3))


@pytest.mark.parametrize("planes", [2, 3, 4, 5, 6])
def test_reference_test_fixture_and_its_cpu_mirror(planes):
    """SignedQuantKernelTests.swift:1523-1650: rows 9, cols 256, codes (13 r + 7 c) & 1, scales
    0.001953125 (i % 7 + 1), input sin(17 i + 3) * 0.75; the mirror re-quantises with the stored
    activation scale and accepts max(0.02, 1 %)."""
    rows, cols = 9, 256
    groups = cols // 128
    r, c = np.meshgrid(np.arange(rows), np.arange(cols), indexing="ij")
    codes = ((r * 13 + c * 7) & 1).astype(np.uint8)
    ws = fx.f16_bits((0.001953125 * ((np.arange(rows * groups) % 7) + 1)).astype(np.float32)).reshape(rows, groups)
    x = fx.f16_bits((np.sin((np.arange(cols) * 17 + 3).astype(np.float32)) * np.float32(0.75)).astype(np.float32))
    pl, asc, _ = so.activation_bitplanes(x, planes, so.F16)
    got = so.widen(so.narrow(so.signed_bitplane_matvec(so.BINARY1, so.signed_pack(codes, so.BINARY1), ws, pl, asc, rows, cols, so.F16), so.F16), so.F16)
    max_q = 1 if planes == 2 else (1 << (planes - 1)) - 1
    a = so.widen(asc, so.F16).repeat(128)
    xq = round_half_away(np.clip(so.widen(x, so.F16) / a, -max_q, max_q)).astype(np.float32)
    sign = np.where(codes == 0, -1.0, 1.0).astype(np.float32)
    expected = (xq[None, :] * a[None, :] * sign * so.widen(ws, so.F16).repeat(128, axis=1)).astype(np.float64).sum(axis=1)
    assert np.all(np.abs(got - expected) <= np.maximum(0.02, np.abs(expected) * 0.01))


def test_fused_producers_equal_their_staged_forms():
    rng = fx.rng_for(112, 0)
    n = 512
    g, u = so.narrow(rng.normal(0, 2, n).astype(np.float32), so.F16), so.narrow(rng.normal(0, 1, n).astype(np.float32), so.F16)
    staged = so.activation_bitplanes(so.swiglu_fused(g, u, so.F16), 5, so.F16)
    fused = so.swiglu_activation_bitplanes(g, u, 5, so.F16)
    assert np.array_equal(staged[0], fused[0]) and np.array_equal(staged[1], fused[1])
    x, w = so.narrow(rng.normal(0, 1, n).astype(np.float32), so.F16), so.narrow(rng.normal(0, 0.2, n).astype(np.float32), so.F16)
    rs = so.rms_scale(x, 1e-6, so.F16)
    for planes in (2, 4, 6):
        staged = so.activation_bitplanes(so.rms_norm_1pw(x, w, 1e-6, so.F16, True), planes, so.F16)
        fused = so.norm_scale_activation_bitplanes(rs, x, w, planes, so.F16)
        assert np.array_equal(staged[0], fused[0]) and np.array_equal(staged[1], fused[1])


def test_sigmoid_mul_producer_closed_forms_and_numpy_float16():
    """sigmoid_mul_signed_activation_bitplanes_i6_g128 (signed_quant.metal:985-1027): a * sigmoid(b)
    with the sigmoid staged in the 16-bit type, then the i6 view of those values."""
    h = lambda v: so.narrow(np.asarray(v, np.float32), so.F16)
    val = lambda a, b: so.widen(so.sigmoid_mul(h(a), h(b), so.F16), so.F16)
    assert val([3.0], [0.0])[0] == 1.5                                     # sigmoid(0) = 1/2
    assert val([3.0], [12.0])[0] == 3.0 and abs(val([3.0], [-12.0])[0]) < 1e-4   # saturates to 1 and ~0
    assert val([-2.0], [1.0])[0] == -val([2.0], [1.0])[0]                  # odd in a
    rng = fx.rng_for(113, 0)
    a, b = h(rng.normal(0, 2, 4096)), h(rng.normal(0, 3, 4096))
    af, bf = a.view(np.float16), b.view(np.float16)
    one = np.float16(1.0)
    tail = one / (one + np.exp(np.abs(bf)))                                 # float16 at every step
    sig = np.where(bf < 0, tail, one - tail).astype(np.float16)
    ref = (af * sig).astype(np.float16)
    got = so.sigmoid_mul(a, b, so.F16).view(np.float16)
    ulp = np.spacing(np.abs(ref)).astype(np.float64)
    assert np.all(np.abs(got.astype(np.float64) - ref.astype(np.float64)) <= ulp)   # exp may differ in its last bit
    assert np.mean(got.view(np.uint16) == ref.view(np.uint16)) > 0.995
    # the fused producer is the plain i6 producer applied to those values
    staged = so.activation_bitplanes(so.sigmoid_mul(a, b, so.F16), 6, so.F16)
    fused = so.sigmoid_mul_activation_bitplanes(a, b, 6, so.F16)
    assert np.array_equal(staged[0], fused[0]) and np.array_equal(staged[1], fused[1])
