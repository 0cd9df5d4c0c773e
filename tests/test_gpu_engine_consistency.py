"""What the default (AUTO) engine choice does to the invariants the single-engine tests pin bit for bit.

Under AUTO a step mixes two summation orders: plain, +residual, gate+up and bank matvecs of 1M weights and
more run the single-pass matrix-core kernel, while the norm-scale, dual, GeGLU and every `_batched*` form
(the 4-token verify pass included) stay on the vector kernels.  "Fused == staged" and "batched per-token bits
== M = 1 bits" therefore hold bit for bit only on one engine (tests/test_gpu_matvec.py,
tests/test_gpu_norm_scale.py under VECTOR); across engines they hold to the output tolerance.  This file
runs the default engine at a shape above the threshold and measures how far apart the two are."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import runtime as rt
from test_gpu_matvec import run_affine

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = rt.Context()      # AUTO engine: what a package gets
    yield c
    c.close()


def steps_between(a_bits, b_bits, dtype):
    a = fx.from_bits(a_bits, dtype).astype(np.float64)
    b = fx.from_bits(b_bits, dtype).astype(np.float64)
    floor = gh.FLOOR_FRAC * np.abs(b).max()
    return np.abs(a - b) / gh.ulp_of(np.maximum(np.abs(b), floor), dtype)


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_auto_engine_decode_against_verify_b4_and_staged(ctx, dtype):
    rows, cols, group = 2048, 1024, 64          # 2M weights: above the 1M threshold of the matrix-core matvec
    assert rows * cols >= (1 << 20)
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=31)
    x = fx.synth_activation(4, cols, dtype, config=1, tensor=32)
    xf = fx.from_bits(x, dtype)
    ref = so.affine_matvec(packed, scales, biases, xf, rows, cols, group, dtype)
    # decode: one token per launch on the engine AUTO picks (matrix core)
    decode = np.concatenate([run_affine(ctx, packed, scales, biases, x[t:t + 1], dtype, f"affine_matvec:{cols}:{group}", generic=True)
                             for t in range(4)])
    # verify pass: the generated four-token form (vector kernels)
    verify = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec_c{cols}_r{rows}_g{group}_batched_verify_b4", batched=True, batch_tile=4)
    gh.check_outputs(decode, ref, dtype, "AUTO decode")
    gh.check_outputs(verify, ref, dtype, "AUTO verify_b4")
    s = steps_between(decode, verify, dtype)
    same = float(np.mean(decode == verify))
    print(f"\n  decode vs verify_b4 under AUTO: max {s.max():.2f} output steps, {same:.4f} identical")
    assert s.max() <= 1.0 + 1e-9      # both within half a step of the exact sum plus the fp32 order difference
    assert same >= 0.95     # measured: 0.975 (fp16), 0.998 (bf16)
    # fused residual add against the staged pair (matvec on the matrix core, add on the host in the same rounding order)
    res = fx.to_bits(fx.rng_for(1, 33).normal(0, 1, (1, rows)).astype(np.float32), dtype)
    fused = run_affine(ctx, packed, scales, biases, x[:1], dtype, f"fused_affine_matvec_add:{cols}:{group}", residual=res, generic=True)
    staged = so.narrow(fx.from_bits(decode[:1], dtype) + fx.from_bits(res, dtype), dtype)
    assert np.array_equal(fused, staged)     # same engine on both sides: bit for bit
    # on one engine the four-token form reproduces the single-token bits exactly
    ctx.set_matvec_engine(rt.MATVEC_VECTOR)
    try:
        d1 = np.concatenate([run_affine(ctx, packed, scales, biases, x[t:t + 1], dtype, f"affine_matvec:{cols}:{group}", generic=True)
                             for t in range(4)])
        v4 = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec_c{cols}_r{rows}_g{group}_batched_verify_b4", batched=True, batch_tile=4)
        assert np.array_equal(d1, v4)
    finally:
        ctx.set_matvec_engine(rt.MATVEC_AUTO)
