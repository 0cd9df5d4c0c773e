"""Helpers for the GPU parity tests: lay tensors out the way weights.bin does, bind slots,
build dispatch records, and compare with the oracle under the stated tolerance."""
from __future__ import annotations

import numpy as np

import fixtures as fx
from smelt_amd import runtime as rt

WEIGHTS_SLOT = 0
X_SLOT, Y_SLOT, RES_SLOT, AUX_SLOT, AUX2_SLOT = 1, 2, 3, 4, 5

REL_TOL = 2e-3          # max-rel-err on outputs (fp32 accumulation)
FLOOR_FRAC = 2.0 ** -6  # |ref| is floored at this fraction of max|ref| in the denominator
# Epilogues that keep every intermediate in the 16-bit type (signed_quant.metal:15-20): gate and up can each sit one
# step from the oracle's (other summation order), and the chain exp -> 1 + e -> 1 / d -> g * s -> * u rounds five
# more times, so the result is held to a few output steps rather than to a relative bound below one bf16 ulp.
SIGNED_SWIGLU_STEPS = 4
GEGLU_STEPS = 2


def align(v: int, a: int) -> int:
    return (v + a - 1) // a * a


class WeightFile:
    """Byte image laid out like weights.bin: every region 128-byte aligned
    (SmeltWeightPacker.swift:788-862)."""

    def __init__(self):
        self.chunks: list[tuple[int, np.ndarray]] = []
        self.size = 0

    def add(self, arr: np.ndarray) -> int:
        off = align(self.size, 128)
        a = np.ascontiguousarray(arr).view(np.uint8).ravel()
        self.chunks.append((off, a))
        self.size = off + a.size
        return off

    def image(self) -> np.ndarray:
        img = np.zeros(align(self.size, 128), np.uint8)
        for off, a in self.chunks:
            img[off:off + a.size] = a
        return img


def ulp_of(ref: np.ndarray, dtype: int) -> np.ndarray:
    mant = 7 if dtype == fx.BF16 else 10
    a = np.maximum(np.abs(ref.astype(np.float64)), 2.0 ** -14 if dtype == fx.F16 else 2.0 ** -126)
    return 2.0 ** (np.floor(np.log2(a)) - mant)


def check_outputs(got_bits: np.ndarray, ref_f32: np.ndarray, dtype: int, what: str,
                  rel_tol: float = REL_TOL) -> float:
    """|got - ref| <= rel_tol * max(|ref|, floor) + half an output ulp (storage rounding)."""
    got = fx.from_bits(got_bits, dtype).astype(np.float64).reshape(ref_f32.shape)
    ref = ref_f32.astype(np.float64)
    floor = FLOOR_FRAC * np.abs(ref).max()
    denom = np.maximum(np.abs(ref), floor)
    excess = np.abs(got - ref) - 0.5 * ulp_of(ref, dtype)
    rel = np.maximum(excess, 0) / denom
    worst = float(rel.max())
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    assert np.abs(got).max() > 0, f"{what}: output is all zero"
    assert worst <= rel_tol, f"{what}: max rel err {worst:.3e} > {rel_tol} at {np.unravel_index(rel.argmax(), rel.shape)}"
    return worst


def swiglu_unrounded(gate_f32: np.ndarray, up_f32: np.ndarray) -> np.ndarray:
    """silu(gate) * up in float64 from the oracle's fp32 sums: what a fused affine gate+up kernel rounds ONCE.
    Comparing against this (not against its 16-bit rounding) keeps the stated tolerance meaningful: a
    reference that is already rounded sits up to half an output ulp away from the exact value, which for
    bf16 (2^-9 relative) is as large as the tolerance itself."""
    g = gate_f32.astype(np.float64)
    return (g / (1.0 + np.exp(-g)) * up_f32.astype(np.float64)).astype(np.float32)


def check_steps(got_bits: np.ndarray, ref_bits: np.ndarray, dtype: int, what: str, max_steps: int = 1,
                min_exact: float = 0.0) -> float:
    """For epilogues that round more than once (signed SwiGLU, GeGLU, a fused kernel against its staged pair
    on another summation order): a sum that lands on the other side of a 16-bit rounding boundary moves the
    result by whole steps of the output type, so the bound is counted in those: |got - ref| <= max_steps ulp,
    the ulp taken at max(|ref|, 2^-6 max|ref|); at least `min_exact` of the elements identical."""
    got = fx.from_bits(got_bits, dtype).astype(np.float64).reshape(np.shape(ref_bits))
    ref = fx.from_bits(ref_bits, dtype).astype(np.float64)
    floor = FLOOR_FRAC * np.abs(ref).max()
    steps = np.abs(got - ref) / ulp_of(np.maximum(np.abs(ref), floor), dtype)
    worst = float(steps.max())
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    assert np.abs(got).max() > 0, f"{what}: output is all zero"
    assert worst <= max_steps + 1e-9, f"{what}: {worst:.2f} output steps > {max_steps} at {np.unravel_index(steps.argmax(), steps.shape)}"
    exact = float(np.mean(np.asarray(got_bits).reshape(np.shape(ref_bits)) == np.asarray(ref_bits)))
    assert exact >= min_exact, f"{what}: only {exact:.3f} of the elements identical (< {min_exact})"
    return worst


def t_suffix(dtype: int) -> str:
    return "@bf16" if dtype == fx.BF16 else "@f16"
