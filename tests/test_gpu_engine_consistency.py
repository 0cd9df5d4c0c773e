"""What the default (AUTO) engine choice does to the invariants the single-engine tests pin bit for bit.

Under AUTO a step mixes two summation orders: single-token affine matvecs (plain, +residual,
gate+up, banks, dual, GeGLU, norm-scale forms) run the single-pass matrix-core kernel, while every `_batched*`
form (the 4-token verify pass included) and the `atomic_norm_*` forms stay on the vector kernels.  "Fused == staged" and "batched per-token bits
== M = 1 bits" therefore hold bit for bit only on one engine (tests/test_gpu_matvec.py,
tests/test_gpu_norm_scale.py under VECTOR); across engines they hold to the output tolerance.  This file
runs the default engine and measures how far apart the two are."""
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
@pytest.mark.parametrize("shape", [(2048, 1024), (1000, 2560), (512, 1024)])
def test_auto_engine_small_matrices_verify_b4_is_decode_bit_for_bit(ctx, dtype, shape):
    """While tokens x weights stay below about 20M the per-token small-batch forms run the single-token kernel with a
    grid row per token: the verify pass then reproduces the decode rows bit for bit under AUTO as well (plain and
    gate+up+SwiGLU forms, two to four tokens)."""
    rows, cols = shape
    group = 64
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=41)
    x = fx.synth_activation(4, cols, dtype, config=1, tensor=42)
    decode = np.concatenate([run_affine(ctx, packed, scales, biases, x[t:t + 1], dtype, f"affine_matvec:{cols}:{group}", generic=True)
                             for t in range(4)])
    for batch in (2, 3, 4):
        verify = run_affine(ctx, packed, scales, biases, x[:batch], dtype, f"affine_matvec_c{cols}_r{rows}_g{group}_batched_verify_b4", batched=True, batch_tile=4)
        assert np.array_equal(verify, decode[:batch]), batch
    tile4 = run_affine(ctx, packed, scales, biases, x, dtype, f"affine_matvec_c{cols}_r{rows}_g{group}_batched_tile4", batched=True, batch_tile=4)
    assert np.array_equal(tile4, decode)
    gh.check_outputs(decode, so.affine_matvec(packed, scales, biases, fx.from_bits(x, dtype), rows, cols, group, dtype), dtype, "decode")


@pytest.mark.parametrize("dtype", [fx.F16, fx.BF16])
def test_auto_engine_decode_against_verify_b4_and_staged(ctx, dtype):
    rows, cols, group = 4096, 2560, 64          # AUTO: single-pass kernel at one token, streaming kernel at four (42M token-weights)
    packed, scales, biases = fx.synth_affine(rows, cols, group, dtype, config=1, tensor=31)
    x = fx.synth_activation(4, cols, dtype, config=1, tensor=32)
    xf = fx.from_bits(x, dtype)
    ref = so.affine_matvec(packed, scales, biases, xf, rows, cols, group, dtype)
    # decode: one token per launch on the engine AUTO picks (matrix core)
    decode = np.concatenate([run_affine(ctx, packed, scales, biases, x[t:t + 1], dtype, f"affine_matvec:{cols}:{group}", generic=True)
                             for t in range(4)])
    # verify pass: the generated four-token form (streaming kernel)
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


def _time_record(ctx, rec):
    """Median GPU time of one launch of the record (microseconds), whichever kernel the engine routes it to."""
    return float(np.median(ctx.benchmark_record(rec, warmup=20, iters=120)))


def _affine_record(ctx, rows, cols, group, dtype, kind):
    nmat = 2 if kind == "gate_up" else 1
    rng = np.random.default_rng(rows * 7 + cols)
    wf = gh.WeightFile()
    bufs = []
    for m in range(nmat):
        packed = rng.integers(0, 256, size=(rows, cols // 2), dtype=np.uint8)
        scales = fx.to_bits(np.abs(rng.normal(0, 0.02, (rows, cols // group))).astype(np.float32), dtype)
        biases = fx.to_bits(rng.normal(0, 0.01, (rows, cols // group)).astype(np.float32), dtype)
        bufs += [(0, 3 * m + i, wf.add(a)) for i, a in enumerate((packed, scales, biases))]
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, fx.to_bits(rng.normal(0, 1, (1, cols)).astype(np.float32), dtype))
    ctx.alloc(gh.Y_SLOT, rows * 2)
    n = 3 * nmat
    bufs += [(gh.X_SLOT, n, 0), (gh.Y_SLOT, n + 1, 0)]
    if kind == "argmax":
        # the lm_head record at one token: partial keys (one per grid column) where the other kinds write y
        ctx.alloc(gh.Y_SLOT, 1024 * 8)
        pipe = ctx.pipeline(f"affine_matvec_argmax_c{cols}_r{rows}_g{group}_batched" + gh.t_suffix(dtype))
        return rt.make_record(pipe, bufs, [(5, 1), (6, 0.0)], (1024, 1, 1), (256, 1, 1))
    entry = {"matvec": "affine_matvec", "gate_up": "fused_affine_gate_up_swiglu"}[kind] + f":{cols}:{group}"
    pipe = ctx.pipeline(entry + gh.t_suffix(dtype))
    return rt.make_record(pipe, bufs, [(n + 2, rows)], (min(1024, (rows + 7) // 8), 1, 1), (256, 1, 1))


def _signed_record(ctx, fmt, name, rows, cols, dtype):
    rng = np.random.default_rng(rows * 5 + cols)
    stride = {fx.BINARY1: cols // 8, fx.TERNARY2: cols // 4}.get(fmt, (((cols + 4) // 5) + 15) // 16 * 16)
    packed = rng.integers(0, 243 if fmt == fx.TRIT5 else 256, size=(rows, stride), dtype=np.uint8)
    # (timing only: a ternary byte may hold the unused code 3 here; nothing is compared)
    scales = fx.f16_bits(np.abs(rng.normal(0, 0.02, (rows, cols // 128))).astype(np.float32))
    wf = gh.WeightFile()
    oc, os_ = wf.add(packed), wf.add(scales)
    ctx.upload_weights(gh.WEIGHTS_SLOT, wf.image())
    ctx.put(gh.X_SLOT, fx.to_bits(rng.normal(0, 1, (1, cols)).astype(np.float32), dtype))
    ctx.alloc(gh.Y_SLOT, rows * 2)
    pipe = ctx.pipeline(f"signed_{name}_matvec_g128_rows8" + gh.t_suffix(dtype))
    bufs = [(0, 0, oc), (0, 1, os_), (gh.X_SLOT, 2, 0), (gh.Y_SLOT, 3, 0)]
    return rt.make_record(pipe, bufs, [(4, rows), (5, cols)], (min(1024, (rows + 7) // 8), 1, 1), (256, 1, 1))


# (the second rows: one shape of each size class of the launch plan: below 1M weights, 8M-24M, from 24M with eight
# and twelve waves, a row beyond 24576 columns, a tall matrix of short rows, a tall matrix with two waves per tile;
# the lm_head record at one token with partly empty and with full vector passes)
AFFINE_SWEEP = [(4096, 4096, 64, "matvec"), (11008, 4096, 128, "matvec"), (4096, 11008, 64, "matvec"), (1536, 8960, 64, "matvec"),
                (32000, 4096, 32, "matvec"), (1024, 1024, 64, "matvec"), (6912, 2304, 64, "gate_up"), (14336, 4096, 128, "gate_up"),
                (512, 1024, 64, "matvec"), (9216, 2560, 64, "matvec"), (8192, 8192, 64, "matvec"), (4096, 14336, 64, "matvec"),
                (4096, 28672, 64, "matvec"), (32768, 2048, 64, "matvec"), (131072, 3072, 64, "matvec"),
                (65536, 2560, 64, "argmax"), (32000, 5120, 64, "argmax"), (65536, 1024, 64, "argmax")]
SIGNED_SWEEP = [(fx.BINARY1, "binary", 8192, 8192), (fx.BINARY1, "binary", 4096, 14336), (fx.BINARY1, "binary", 2048, 2048),
                (fx.TERNARY2, "ternary", 14336, 4096), (fx.TERNARY2, "ternary", 8192, 2048), (fx.TRIT5, "trit5", 8192, 4096),
                (fx.TRIT5, "trit5", 2560, 10240),
                (fx.BINARY1, "binary", 512, 1024), (fx.TERNARY2, "ternary", 1024, 1024), (fx.TRIT5, "trit5", 1024, 1280)]


def test_auto_engine_is_not_the_slower_one(ctx):
    """AUTO's launch plans were fitted on a handful of shapes.  On a sweep of other shapes (Llama- and Gemma-like
    projections, a short-and-wide and a tall-and-narrow matrix, one shape of every size class of the plan) the
    kernel AUTO picks must not lose to the vector kernel by more than run-to-run noise: warm single launches,
    medians of 120, AUTO <= 1.10 x VECTOR + 0.3 us.  Where AUTO keeps the vector kernel the two times are the same
    measurement."""
    dtype = fx.BF16
    lines, worst = [], 0.0

    def both(rec, what):
        nonlocal worst
        t = {}
        for eng in (rt.MATVEC_AUTO, rt.MATVEC_VECTOR):
            ctx.set_matvec_engine(eng)
            t[eng] = _time_record(ctx, rec)
        ctx.set_matvec_engine(rt.MATVEC_AUTO)
        lines.append(f"  {what:34s} auto {t[rt.MATVEC_AUTO]:6.2f} us   vector {t[rt.MATVEC_VECTOR]:6.2f} us")
        worst = max(worst, t[rt.MATVEC_AUTO] / t[rt.MATVEC_VECTOR])
        assert t[rt.MATVEC_AUTO] <= 1.10 * t[rt.MATVEC_VECTOR] + 0.3, lines[-1]

    try:
        for rows, cols, group, kind in AFFINE_SWEEP:
            both(_affine_record(ctx, rows, cols, group, dtype, kind), f"u4 g{group} {kind} {rows}x{cols}")
        for fmt, name, rows, cols in SIGNED_SWEEP:
            both(_signed_record(ctx, fmt, name, rows, cols, dtype), f"{name} {rows}x{cols}")
    finally:
        ctx.set_matvec_engine(rt.MATVEC_AUTO)
        print("\n" + "\n".join(lines) + f"\n  worst auto / vector: {worst:.2f}")
