"""GPU parity at the full 27B-layer shapes (hidden 5120, FFN 17408): every weight format through the
kernel a package gets by default (AUTO engine: the single-pass matrix-core matvec for affine u4, binary,
ternary and trit5) against the OpenMP oracle, plain matvec, +residual and fused gate+up where the shape
has one.  Seeded tensors as the benchmark's configurations 2 and 3 draw them."""
import numpy as np
import pytest

import fixtures as fx
import gpu_harness as gh
from oracle import oracle as so
from smelt_amd import runtime as rt
from test_gpu_matvec import run_affine, run_signed

pytestmark = pytest.mark.gpu

H, F = 5120, 17408


@pytest.fixture(scope="module")
def ctx():
    c = rt.Context()
    yield c
    c.close()


@pytest.mark.parametrize("shape", [(F, H), (H, F), (H, H), (1024, H)])
def test_affine_u4_27b_shapes(ctx, shape):
    rows, cols = shape
    dtype = fx.BF16
    rng = fx.rng_for(1, rows % 1000 + cols % 7)
    packed = rng.integers(0, 256, size=(rows, cols // 2), dtype=np.uint8)
    scales = fx.bf16_bits(np.abs(rng.normal(0, 0.02, size=(rows, cols // 64))).astype(np.float32))
    biases = fx.bf16_bits(rng.normal(0, 0.01, size=(rows, cols // 64)).astype(np.float32))
    x = fx.synth_activation(1, cols, dtype, config=1, tensor=5)
    ref = so.affine_matvec(packed, scales, biases, fx.from_bits(x, dtype), rows, cols, 64, dtype, threads=True)
    y = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec:{cols}:64", generic=True)
    worst = gh.check_outputs(y, ref, dtype, f"affine u4 {shape}")
    print(f"\n  u4 {shape} max rel err {worst:.2e}")
    if shape == (H, F):   # the down projection carries the residual
        res = fx.to_bits(fx.rng_for(1, 77).normal(0, 1, (1, rows)).astype(np.float32), dtype)
        fused = run_affine(ctx, packed, scales, biases, x, dtype, f"fused_affine_matvec_add:{cols}:64", residual=res, generic=True)
        assert np.array_equal(fused, so.narrow(fx.from_bits(y, dtype) + fx.from_bits(res, dtype), dtype))


def signed_tensor(fmt, rows, cols, seed):
    rng = fx.rng_for(2 + fmt, seed)
    if fmt == fx.BINARY1:
        packed = rng.integers(0, 256, size=(rows, cols // 8), dtype=np.uint8)
    else:
        u = rng.random(size=(rows, cols), dtype=np.float32)
        codes = (u >= 0.3).astype(np.uint8) + (u >= 0.7).astype(np.uint8)
        stride = cols // 4 if fmt == fx.TERNARY2 else (((cols + 4) // 5) + 15) // 16 * 16
        packed = fx.pack_signed_np(codes, fmt, stride)
    scales = fx.f16_bits(np.abs(rng.normal(0, 0.02, size=(rows, cols // 128))).astype(np.float32))
    return packed, scales


@pytest.mark.parametrize("fmt,name", [(fx.BINARY1, "binary"), (fx.TERNARY2, "ternary"), (fx.TRIT5, "trit5")])
@pytest.mark.parametrize("shape", [(F, H), (H, F)])
def test_signed_27b_shapes(ctx, fmt, name, shape):
    rows, cols = shape
    dtype = fx.BF16
    packed, scales = signed_tensor(fmt, rows, cols, 1)
    x = fx.synth_activation(1, cols, dtype, config=2 + fmt, tensor=3)
    xf = fx.from_bits(x, dtype)
    ref = so.signed_matvec(fmt, packed, scales, xf, rows, cols, cols, 128, threads=True)
    y = run_signed(ctx, name, packed, scales, x, dtype, rows, cols)
    worst = gh.check_outputs(y, ref, dtype, f"{name} {shape}")
    print(f"\n  {name} {shape} max rel err {worst:.2e}")
    if shape == (F, H):   # gate and up share the input: the fused SwiGLU form
        up = signed_tensor(fmt, rows, cols, 2)
        u_ref = so.signed_matvec(fmt, *up, xf, rows, cols, cols, 128, threads=True)
        u = run_signed(ctx, name, *up, x, dtype, rows, cols)
        gh.check_outputs(u, u_ref, dtype, f"{name} {shape} up")
        fused = run_signed(ctx, name, packed, scales, x, dtype, rows, cols, kind="gate_up", second=up)
        # the fused kernel rounds gate and up to the activation type and applies SwiGLU to those bits
        staged = so.epilogue_signed_swiglu(y, u, so.BF16)
        steps = np.abs(fused.astype(np.int32) - staged.astype(np.int32))
        assert steps.max() <= 1, int(steps.max())   # the low-precision exp() is not pinned bit-exactly


@pytest.mark.parametrize("act", ["swiglu", "geglu"])
def test_affine_norm_scale_gate_up_27b_shape(ctx, act):
    """The fused forms a real layer's record list holds in front of the FFN: RMS-norm scale prologue + gate+up with
    SwiGLU / GeGLU at 2 x 17408 x 5120 (matrix-core kernel under AUTO), against the oracle on the normalised row."""
    import oracle.oracle as oo
    from test_gpu_norm_scale import norm_inputs, run_gate_up
    rows, cols, group, dtype = F, H, 64, fx.BF16
    rng = fx.rng_for(1, 91)

    def tensor():
        packed = rng.integers(0, 256, size=(rows, cols // 2), dtype=np.uint8)
        scales = fx.bf16_bits(np.abs(rng.normal(0, 0.02, size=(rows, cols // 64))).astype(np.float32))
        biases = fx.bf16_bits(rng.normal(0, 0.01, size=(rows, cols // 64)).astype(np.float32))
        return packed, scales, biases

    gw, uw = tensor(), tensor()
    x, w, rs = norm_inputs(1, cols, dtype, seed=5)
    xn = oo.norm_scale_input(x[0], rs[0], w, dtype).reshape(1, cols)
    fused = run_gate_up(ctx, gw, uw, dtype, f"norm_scale_affine_gate_up_{act}:{cols}:{group}", [(10, rows)], x, norm=(w, rs))
    staged = run_gate_up(ctx, gw, uw, dtype, f"fused_affine_gate_up_{act}:{cols}:{group}", [(8, rows)], xn)
    assert np.array_equal(fused, staged)
    xf = fx.from_bits(xn, dtype)
    g = so.affine_matvec(*gw, xf, rows, cols, group, dtype, threads=True)
    u = so.affine_matvec(*uw, xf, rows, cols, group, dtype, threads=True)
    if act == "swiglu":
        gh.check_outputs(fused, gh.swiglu_unrounded(g, u), dtype, "27B norm-scale gate+up swiglu")
    else:
        gh.check_steps(fused, so.epilogue_geglu(g, u, dtype).reshape(np.shape(fused)), dtype, "27B norm-scale gate+up geglu",
                       max_steps=gh.GEGLU_STEPS)
