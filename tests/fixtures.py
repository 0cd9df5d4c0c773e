"""Closed-form and seeded fixtures shared by the oracle tests and the GPU parity tests.

The closed-form generators restate the formulas the reference's tests use to build
their inputs (file:line cited per function); they carry no reference code, only the
arithmetic that defines the data.
"""
from __future__ import annotations

import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

F16, BF16 = 0, 1
BINARY1, TERNARY2, TRIT5 = 0, 1, 2


def golden_vectors() -> dict:
    with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
        return json.load(f)


def f16_bits(values) -> np.ndarray:
    return np.asarray(values, dtype=np.float32).astype(np.float16).view(np.uint16)


def bf16_bits(values) -> np.ndarray:
    b = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def to_bits(values, dtype: int) -> np.ndarray:
    return bf16_bits(values) if dtype == BF16 else f16_bits(values)


def from_bits(bits, dtype: int) -> np.ndarray:
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    if dtype == BF16:
        return (bits.astype(np.uint32) << 16).view(np.float32)
    return bits.view(np.float16).astype(np.float32)


# ---------------------------------------------------------------------------
# closed-form fixtures from the reference's tests
# ---------------------------------------------------------------------------

def mlx_ternary_fixture(rows: int, cols: int, batch: int, scale_unit: float):
    """SignedQuantKernelTests.swift:87-106 / :143-163 — codes (13r+7c)%3, scales
    unit*(i%5+1), x[i] = ((17i+3)%31-15)/16 over batch*cols indices."""
    r = np.arange(rows)[:, None]
    c = np.arange(cols)[None, :]
    codes = ((13 * r + 7 * c) % 3).astype(np.uint8)
    groups = cols // 128
    i = np.arange(rows * groups)
    scales = f16_bits(scale_unit * ((i % 5) + 1).astype(np.float32)).reshape(rows, groups)
    j = np.arange(batch * cols)
    x = f16_bits((((17 * j + 3) % 31) - 15).astype(np.float32) / 16.0).reshape(batch, cols)
    return codes, scales, x


def mlx_ternary_qmm_fixture(rows: int, cols: int, batch: int, scale_bits):
    """SignedQuantKernelTests.swift:527-546 — same codes and activations as above, scales
    cycling through a list of fp16 bit patterns."""
    codes, _, x = mlx_ternary_fixture(rows, cols, batch, 1.0)
    groups = cols // 128
    pool = np.array([int(b, 16) if isinstance(b, str) else int(b) for b in scale_bits], np.uint16)
    scales = pool[np.arange(rows * groups) % pool.size].reshape(rows, groups)
    return codes, scales, x


def signed_synthetic_fixture(fmt: int, rows=5, cols=256, batch=5):
    """SignedQuantKernelTests.swift:989-1016 — binary (13r+7c)&1, ternary (13r+7c)%3,
    scales 0.03125*(i%5+1), x[i] = sin(17i+3)*0.75 (fp32 sin, rounded to fp16)."""
    r = np.arange(rows)[:, None]
    c = np.arange(cols)[None, :]
    v = 13 * r + 7 * c
    codes = ((v & 1) if fmt == BINARY1 else (v % 3)).astype(np.uint8)
    groups = cols // 128
    i = np.arange(rows * groups)
    scales = f16_bits(0.03125 * ((i % 5) + 1).astype(np.float32)).reshape(rows, groups)
    j = np.arange(batch * cols, dtype=np.float32)
    x = f16_bits(np.sin(j * np.float32(17) + np.float32(3), dtype=np.float32) * np.float32(0.75))
    return codes, scales, x.reshape(batch, cols)


def affine_synthetic_fixture(rows: int, cols: int, group: int, seed: int = 0, batch: int = 1):
    """PrefillKernelTests.swift:220-264 / MetalKernelTestSupport.swift:361-388 —
    W[i] = u8(17i+23+131*seed); S[i] = h(0.01+0.04*(0.5+0.5*sin((i+7919*seed)*0.0071)));
    B[i] = h(cos((i+6869*seed)*0.0113)*0.03); x[i] = h(sin((i+6151*seed)*0.0137)*0.5);
    residual[i] = h(cos((i+4817*seed)*0.0091)*0.25)."""
    f = np.float32
    nbytes = rows * cols // 2
    i = np.arange(nbytes, dtype=np.int64)
    packed = ((i * 17 + 23 + seed * 131) & 0xFF).astype(np.uint8).reshape(rows, cols // 2)
    gpr = cols // group
    k = np.arange(rows * gpr, dtype=np.float32)
    scales = f16_bits(f(0.01) + f(0.04) * (f(0.5) + f(0.5) * np.sin((k + f(seed * 7919)) * f(0.0071), dtype=f)))
    biases = f16_bits(np.cos((k + f(seed * 6869)) * f(0.0113), dtype=f) * f(0.03))
    j = np.arange(batch * cols, dtype=np.float32)
    x = f16_bits(np.sin((j + f(seed * 6151)) * f(0.0137), dtype=f) * f(0.5)).reshape(batch, cols)
    m = np.arange(batch * rows, dtype=np.float32)
    residual = f16_bits(np.cos((m + f(seed * 4817)) * f(0.0091), dtype=f) * f(0.25)).reshape(batch, rows)
    return packed, scales.reshape(rows, gpr), biases.reshape(rows, gpr), x, residual


def kernel_lab_qmm_fixture(rows: int, cols: int, group: int, batch: int):
    """KernelLab.swift:2829-2855 — W[i] = u8(73i+19), scales 0x2c00, biases 0,
    input/residual 0x3800 where i%3==0 else 0xb400."""
    i = np.arange(rows * cols // 2, dtype=np.int64)
    packed = ((i * 73 + 19) & 0xFF).astype(np.uint8).reshape(rows, cols // 2)
    gpr = cols // group
    scales = np.full((rows, gpr), 0x2C00, np.uint16)
    biases = np.zeros((rows, gpr), np.uint16)
    j = np.arange(batch * cols)
    x = np.where(j % 3 == 0, 0x3800, 0xB400).astype(np.uint16).reshape(batch, cols)
    return packed, scales, biases, x


# ---------------------------------------------------------------------------
# seeded synthetic tensors for the benchmark configurations
# ---------------------------------------------------------------------------

def rng_for(config: int, tensor: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(0xC0FFEE + config * 1000 + tensor))


def synth_affine(rows, cols, group, dtype, config=0, tensor=0):
    """u4 uniform 0..15, scale ~|N(0,0.02)|, bias ~N(0,0.01) in `dtype` (fp16 or bf16)."""
    g = rng_for(config, tensor)
    packed = g.integers(0, 256, size=(rows, cols // 2), dtype=np.uint8)
    gpr = cols // group
    scales = to_bits(np.abs(g.normal(0, 0.02, size=(rows, gpr))).astype(np.float32), dtype)
    biases = to_bits(g.normal(0, 0.01, size=(rows, gpr)).astype(np.float32), dtype)
    return packed, scales, biases


def synth_activation(batch, cols, dtype, config=0, tensor=99, outlier_frac=0.0):
    g = rng_for(config, tensor)
    x = g.normal(0, 1, size=(batch, cols)).astype(np.float32)
    if outlier_frac > 0:
        n = max(1, int(round(cols * outlier_frac)))
        ch = g.choice(cols, size=n, replace=False)
        x[:, ch] *= 10.0
    return to_bits(x, dtype)


def synth_signed_codes(fmt, rows, cols, config=2, tensor=0):
    g = rng_for(config, tensor)
    if fmt == BINARY1:
        return g.integers(0, 2, size=(rows, cols), dtype=np.uint8)
    return g.choice(np.array([0, 1, 2], np.uint8), size=(rows, cols), p=[0.3, 0.4, 0.3])


def synth_signed_scales(rows, cols, group=128, config=2, tensor=0):
    g = rng_for(config, tensor + 500)
    return f16_bits(np.abs(g.normal(0, 0.02, size=(rows, cols // group))).astype(np.float32))


def pack_signed_np(codes: np.ndarray, fmt: int, row_stride: int | None = None) -> np.ndarray:
    """Vectorised packer (independent of the oracle's scalar packer; the two are
    checked against each other in the oracle tests)."""
    rows, cols = codes.shape
    if fmt == TRIT5:
        nb = (cols + 4) // 5
        pad = np.ones((rows, nb * 5), np.uint8)
        pad[:, :cols] = codes
        d = pad.reshape(rows, nb, 5).astype(np.uint16)
        out = (d * np.array([1, 3, 9, 27, 81], np.uint16)).sum(axis=2).astype(np.uint8)
    else:
        bits = 1 if fmt == BINARY1 else 2
        per = 8 // bits
        nb = (cols * bits + 7) // 8
        pad = np.zeros((rows, nb * per), np.uint8)
        pad[:, :cols] = codes
        d = pad.reshape(rows, nb, per).astype(np.uint16)
        shifts = (np.arange(per) * bits).astype(np.uint16)
        out = (d << shifts).sum(axis=2).astype(np.uint8)
    if row_stride is not None and row_stride != out.shape[1]:
        full = np.zeros((rows, row_stride), np.uint8)
        if fmt == TRIT5:
            full[:] = 121  # five semantic zeros: 1+3+9+27+81
        full[:, : out.shape[1]] = out
        out = full
    return np.ascontiguousarray(out)
