"""How many bits a dequantised weight tile must keep for a matrix-core qmm to meet the parity bar.

A qmm that stages weights for the matrix cores has three ways to hold them: one 16-bit float per weight
(bf16 or fp16 of scale * code + bias), a 16-bit pair (the rounding and its remainder), or the 4-bit code
itself with the scale and bias applied to the sums in fp32.  This test carries out each in numpy on the
benchmark's fourth configuration (4B FFN shapes, u4 g64, bf16 activations, seeded tensors) and holds the
result to the criterion every GPU parity test uses (gpu_harness.check_outputs: 2e-3 relative, the
denominator floored at 2^-6 of the largest output).  A single 16-bit tile fails it, by about an order of
magnitude on the outputs near zero; the pair and the exact codes pass.  The kernels of the library
therefore never round a weight: the token-tile qmm multiplies exact (base + code) operands, the
streaming kernels apply scale and bias to fp32 sums (qmm_stream.hpp, qmm_skinny.hpp, mm1_matvec.hpp).
"""
import numpy as np
import pytest

import fixtures as fx
from oracle import oracle as so

REL_TOL, FLOOR_FRAC = 2e-3, 2.0 ** -6     # gpu_harness.REL_TOL / FLOOR_FRAC (that module needs the library)

ROWS, COLS, GROUP, TOKENS = 512, 2560, 64, 8


def worst_error(got: np.ndarray, ref: np.ndarray) -> float:
    """max |got - ref| / max(|ref|, floor), as check_outputs computes it (no storage rounding: fp32 results)."""
    floor = FLOOR_FRAC * np.abs(ref).max()
    return float((np.abs(got - ref) / np.maximum(np.abs(ref), floor)).max())


def round_to(values: np.ndarray, dtype: int) -> np.ndarray:
    return fx.from_bits(fx.to_bits(values.astype(np.float32), dtype), dtype).astype(np.float64)


@pytest.fixture(scope="module")
def case():
    packed, scales, biases = fx.synth_affine(ROWS, COLS, GROUP, fx.BF16, config=4, tensor=1)
    x = fx.from_bits(fx.synth_activation(TOKENS, COLS, fx.BF16, config=4, tensor=2), fx.BF16).astype(np.float64)
    codes = np.empty((ROWS, COLS), np.float64)
    codes[:, 0::2] = packed & 15
    codes[:, 1::2] = packed >> 4
    s = np.repeat(fx.from_bits(scales, fx.BF16).astype(np.float64), GROUP, axis=1)
    b = np.repeat(fx.from_bits(biases, fx.BF16).astype(np.float64), GROUP, axis=1)
    w = s * codes + b                                   # the weights, exact in float64
    ref = x @ w.T
    # the restatement the GPU tests compare with agrees with this float64 product far inside the tolerance
    oracle = np.stack([so.affine_matvec(packed, scales, biases, x[t].astype(np.float32), ROWS, COLS, GROUP, fx.BF16)
                       for t in range(TOKENS)]).reshape(TOKENS, ROWS)
    assert worst_error(oracle.astype(np.float64), ref) < 1e-4
    return dict(codes=codes, s=s, b=b, w=w, x=x, ref=ref)


@pytest.mark.parametrize("dtype,name", [(fx.BF16, "bf16"), (fx.F16, "fp16")])
def test_single_16bit_tile_misses_the_bar(case, dtype, name):
    w16 = round_to(case["w"], dtype)
    got = case["x"] @ w16.T                            # exact products and sums: only the tile is rounded
    worst = worst_error(got, case["ref"])
    print(f"\n  single {name} tile: max rel err {worst:.2e} (bar {REL_TOL})")
    assert worst > REL_TOL, f"a single {name} tile would pass: {worst:.2e}"
    if dtype == fx.BF16:
        assert worst > 4 * REL_TOL                     # not a near miss: 8 mantissa bits against the ~14 needed


def test_bf16_pair_meets_the_bar(case):
    hi = round_to(case["w"], fx.BF16)
    lo = round_to(case["w"] - hi, fx.BF16)
    got = case["x"] @ (hi + lo).T
    worst = worst_error(got, case["ref"])
    print(f"\n  bf16 hi+lo tile: max rel err {worst:.2e}")
    assert worst < REL_TOL / 10


def test_exact_codes_with_fp32_scale_meet_the_bar(case):
    # per group: sum(code * x) and sum(x) in fp32, then scale and bias in fp32, groups added in fp32
    codes, x = case["codes"], case["x"]
    gpr = COLS // GROUP
    cg = codes.reshape(ROWS, gpr, GROUP)
    xg = x.reshape(TOKENS, gpr, GROUP)
    dots = np.einsum("rgk,tgk->trg", cg, xg).astype(np.float32)         # exact integers times bf16, fp32 sums
    sums = xg.sum(axis=2).astype(np.float32)                             # [t, g]
    s = case["s"][:, ::GROUP].astype(np.float32)
    b = case["b"][:, ::GROUP].astype(np.float32)
    got = np.zeros((TOKENS, ROWS), np.float32)
    for g in range(gpr):
        got += s[None, :, g] * dots[:, :, g] + b[None, :, g] * sums[:, None, g]
    worst = worst_error(got.astype(np.float64), case["ref"])
    print(f"\n  exact codes, fp32 scale: max rel err {worst:.2e}")
    assert worst < REL_TOL / 10
