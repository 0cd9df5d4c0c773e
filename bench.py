#!/usr/bin/env python3
"""Benchmark of the quantized matvec hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass over the decode-step matvec set of a 24-layer Qwen3.5-0.8B-shaped stack
(BASELINE configs[1]): the q/k/v projection bank, o, fused gate+up, down (+residual) per layer and
the tied lm_head with fused argmax; all affine 4-bit g64 weights, bf16 activations, seeded synthetic
tensors resident in HBM before the timed region.  The records are emitted by the library's own
emitters, captured once into a HIP graph and replayed; `value` is weight bytes (packed codes +
scales + biases, counted once per step) divided by the step time.

Prints one JSON line (see the fields at the bottom).  Nothing here runs on the CPU except the
`cpu_baseline` leg, which times the scalar oracle on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth


def synth_affine(rng, rows, cols, group, bf16):
    packed = rng.integers(0, 256, size=(rows, cols // 2), dtype=np.uint8)
    gpr = cols // group
    s = np.abs(rng.normal(0, 0.02, size=(rows, gpr))).astype(np.float32)
    b = rng.normal(0, 0.01, size=(rows, gpr)).astype(np.float32)
    return packed, bf16(s), bf16(b)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the 27B-layer and qmm side measurements")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path has no cross-GPU part in this build "
              f"(--gpus {args.gpus} is not supported; run with --gpus 1)", file=sys.stderr)
        return 2

    import fixtures as fx
    from smelt_amd import compiler as cc
    from smelt_amd import runtime as rt

    ctx = rt.Context(act_dtype=rt.ACT_BF16)
    info = ctx.device_info()
    cus = info["compute_units"]
    dtype = fx.BF16
    group, hidden, ffn, vocab, layers = 64, 1024, 3584, 151936, 24

    # ---- weights.bin image of the workload ----------------------------------------------------
    lay = cc.Layout()
    per_layer = []
    for _ in range(layers):
        q, k, v = lay.affine_bank([2048, 512, 512], hidden, group)  # same-input projection bank
        per_layer.append({
            "q": q, "k": k, "v": v, "o": lay.affine(1024, hidden, group),
            "gate": lay.affine(ffn, hidden, group), "up": lay.affine(ffn, hidden, group),
            "down": lay.affine(hidden, ffn, group)})
    lm_copies = 4  # copy 0 belongs to the step; 1..3 only rotate under the roofline measurement
    lm_heads = [lay.affine(vocab, hidden, group) for _ in range(lm_copies)]
    image = np.zeros(lay.total_bytes, np.uint8)
    weight_bytes = 0
    tensor = 0
    for L in per_layer:
        for e in L.values():
            t = synth_affine(fx.rng_for(1, tensor), e.rows, e.cols, group, fx.bf16_bits)
            cc.write_affine(image, e, *t)
            weight_bytes += e.size_bytes + e.scales_size_bytes + e.biases_size_bytes
            tensor += 1
    lm_t = synth_affine(fx.rng_for(1, tensor), vocab, hidden, group, fx.bf16_bits)
    for e in lm_heads:
        cc.write_affine(image, e, *lm_t)
    lm_bytes = lm_heads[0].size_bytes + lm_heads[0].scales_size_bytes + lm_heads[0].biases_size_bytes
    weight_bytes += lm_bytes

    # ---- slots and records -----------------------------------------------------------------------
    W, H0, H1, QKV, ATT, ACT, KEYS, TOK = 0, 1, 2, 3, 4, 5, 6, 7
    em = cc.Emitter(rt.ACT_BF16, cus)
    for L in per_layer:
        # cur = hidden state in, alt = hidden state out; swapped after every layer
        banked = em.bank_matvec(W, [L["q"], L["k"], L["v"]], cc.bind(rt.SLOT_CUR),
                                [cc.bind(QKV, 0), cc.bind(QKV, 2048 * 2), cc.bind(QKV, 2560 * 2)])
        assert banked
        em.matvec(W, L["o"], cc.bind(ATT), cc.bind(rt.SLOT_ALT))
        em.gate_up_swiglu(W, L["gate"], L["up"], cc.bind(rt.SLOT_ALT), cc.bind(ACT))
        em.matvec_add(W, L["down"], cc.bind(ACT), cc.bind(rt.SLOT_ALT), cc.bind(rt.SLOT_CUR))
        em.swap()
    em.lm_head_argmax(W, lm_heads[0], cc.bind(rt.SLOT_CUR), cc.bind(KEYS), cc.bind(TOK))
    step_records = len(em.records())
    # roofline records: the lm_head kernel over rotating weight copies (4 x 87.5 MB > the 256 MB
    # Infinity Cache, so every launch streams from HBM)
    for e in lm_heads:
        em.lm_head_argmax(W, e, cc.bind(H0), cc.bind(KEYS), cc.bind(TOK))
    em.install(ctx)
    ctx.upload_weights(W, image)
    del image
    x = fx.bf16_bits(fx.rng_for(1, 9000).normal(0, 1, hidden).astype(np.float32))
    ctx.put(H0, x)
    ctx.put(H1, x)
    ctx.put(ATT, fx.bf16_bits(fx.rng_for(1, 9001).normal(0, 1, hidden).astype(np.float32)))
    ctx.alloc(QKV, 3072 * 2)
    ctx.alloc(ACT, ffn * 2)
    ctx.alloc(KEYS, max(em.argmax_partial_bytes, 8))
    ctx.alloc(TOK, 4)
    records = list(em.records())
    step_table = ctx.table(records[:step_records])
    launches_per_step = sum(1 for r in step_table if r.op_kind == 0)

    # ---- timed region: K graph replays bracketed by synchronisation --------------------------------
    graph, launched = ctx.capture_decode(step_table, cur=H0, alt=H1)
    assert launched == launches_per_step
    for _ in range(max(args.warmup, 1)):
        ctx.graph_launch(graph)
    ctx.wait()
    t0 = time.perf_counter()
    gpu_us = ctx.graph_time(graph, args.steps)  # events on the launch stream around exactly K replays
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = gpu_us / 1e3 / args.steps
    value = weight_bytes / (ms_per_step * 1e-3) / 1e9
    token = int(ctx.read(TOK, np.int32, 1)[0])
    ctx.graph_destroy(graph)

    # ---- roofline of the dominant kernel (lm_head matvec + argmax, 30% of the step's bytes) ----------
    rl_table = ctx.table([r for r in records[step_records:] if True])
    # keep only the matvec+argmax records (every second record is the tiny key reduce)
    # (eight rounds over the four copies per replay, so that the cost of starting a graph is spread
    # over 32 launches and the figure is the kernel's own back-to-back cadence)
    rl_only = ctx.table([r for i, r in enumerate(records[step_records:]) if i % 2 == 0] * 8)
    g2, n2 = ctx.capture_decode(rl_only, cur=H0, alt=H1)
    ctx.graph_time(g2, 5)
    reps = 10
    # five timed series of ten replays each; the median series is reported (clock ramps and other
    # tenants of the memory system move single series by a few percent)
    series = sorted(ctx.graph_time(g2, reps) / (reps * n2) for _ in range(5))
    lm_us = series[2]
    ctx.graph_destroy(g2)
    achieved = lm_bytes / lm_us / 1e3
    roofline = {"bound": "hbm", "kernel": "smelt_affine_matvec_argmax_single_bf16 (lm_head 151936x1024 u4 g64, fused argmax)",
                "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                "bytes_per_launch": int(lm_bytes), "us_per_launch": round(lm_us, 3),
                "us_per_launch_series": [round(v, 3) for v in series]}
    del rl_table
    roofline["traffic"] = committed_traffic()

    # One plain copy of known size: the calibration dispatch for HBM traffic counters (a counter
    # run of this same command scales FETCH_SIZE / WRITE_SIZE of the lm_head kernel by what they
    # read for this copy).
    CAL_SRC, CAL_DST, cal_bytes = 8, 9, 256 << 20
    ctx.alloc(CAL_SRC, cal_bytes)
    ctx.alloc(CAL_DST, cal_bytes)
    cp = ctx.pipeline("copy_u128")
    cal = rt.make_record(cp, [(CAL_SRC, 0, 0), (CAL_DST, 1, 0)], [(2, cal_bytes // 16)], (cus * 16, 1, 1), (256, 1, 1))
    for _ in range(2):
        ctx.interpret_decode(ctx.table([cal]))
    ctx.wait()

    extra = {}
    if not args.no_extra:
        extra = side_measurements(ctx, fx, cc, rt, cus)

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(fx, per_layer, lm_heads[0], group)

    out = {
        "metric": "qmatvec effective weight GB/s at M=1 (decode-step matvec set)",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: 24-layer Qwen3.5-0.8B-shaped decode matvec set + 151936x1024 lm_head, "
                               "affine u4 g64, bf16 activations/scales, fp32 accumulate, M=1",
                   "weight_bytes_per_step": int(weight_bytes), "launches_per_step": launches_per_step,
                   "replay": "hip graph", "device": info["name"].strip(), "compute_units": cus},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "wall_ms_timed_region": round(wall_ms, 3), "argmax_token": token,
        "roofline": roofline, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(out))
    ctx.close()
    return 0


def committed_traffic():
    """HBM bytes per lm_head launch from the committed counter summary (two rocprofv3 --pmc runs of
    this command, scaled by the copy calibration); None when no summary is present."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "lm_head_argmax_bf16_hbm_traffic.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch"):
                return int(line.split("=")[1].split()[0])
    except OSError:
        pass
    return None


def side_measurements(ctx, fx, cc, rt, cus) -> dict:
    """27B-layer binary / ternary / trit5 matvec sets, the 4B FFN qmm at M in {7,8,9,32,512}, the
    affine 4-bit quantiser and a turbo_quant_h matvec.  Reported beside the headline; not part of `value`."""
    out = {}
    W, X, Y, ACT = 20, 21, 22, 23
    shapes = [(17408, 5120), (17408, 5120), (5120, 17408), (5120, 5120), (5120, 5120), (1024, 5120), (1024, 5120)]
    for name, wdtype, fmt in (("binary1", cc.BINARY1, fx.BINARY1), ("ternary2", cc.TERNARY2, fx.TERNARY2),
                              ("trit5", cc.TRIT5, fx.TRIT5)):
        c = rt.Context(act_dtype=rt.ACT_BF16)
        lay = cc.Layout()
        copies = 6  # rotate layer copies so launches stream from HBM rather than the Infinity Cache
        ents = [[lay.signed(r, k, wdtype) for (r, k) in shapes] for _ in range(copies)]
        image = np.zeros(lay.total_bytes, np.uint8)
        rng = fx.rng_for(2, 0)
        layer_bytes = 0
        for ti, e0 in enumerate(ents[0]):
            if fmt == fx.BINARY1:
                packed = rng.integers(0, 256, size=(e0.rows, e0.packed_row_stride), dtype=np.uint8)
            else:
                u = rng.random(size=(e0.rows, e0.cols), dtype=np.float32)
                codes = (u >= 0.3).astype(np.uint8) + (u >= 0.7).astype(np.uint8)  # P(-1,0,+1) = .3,.4,.3
                del u
                packed = fx.pack_signed_np(codes, fmt, e0.packed_row_stride)
                del codes
            scales = fx.f16_bits(np.abs(rng.normal(0, 0.02, size=(e0.rows, e0.cols // 128))).astype(np.float32))
            for layer in ents:  # every rotating copy holds the same seeded tensor
                cc.write_signed(image, layer[ti], packed, scales)
            layer_bytes += e0.size_bytes + e0.scales_size_bytes
        em = cc.Emitter(rt.ACT_BF16, cus)
        for layer in ents:
            for e in layer:
                em.matvec(W, e, cc.bind(X), cc.bind(Y))
        em.install(c)
        c.upload_weights(W, image)
        del image
        c.put(X, fx.bf16_bits(fx.rng_for(2, 1).normal(0, 1, 17408).astype(np.float32)))
        c.alloc(Y, 17408 * 2)
        table = em.records()
        g, n = c.capture_decode(table)
        c.graph_time(g, 3)
        reps = 20
        us = c.graph_time(g, reps) / (reps * copies)
        per_kernel = {}
        recs = list(table)
        for (r, k), rec in zip(shapes[:3:2] + shapes[3:4] + shapes[5:6], [recs[0], recs[2], recs[3], recs[5]]):
            t = c.benchmark_record(rec, warmup=5, iters=50)
            e = [x for x in ents[0] if (x.rows, x.cols) == (r, k)][0]
            b = e.size_bytes + e.scales_size_bytes
            per_kernel[f"{r}x{k}"] = {"us_warm_median": round(float(np.median(t)), 2), "weight_bytes": int(b)}
        c.graph_destroy(g)
        views = None
        if fmt in (fx.BINARY1, fx.TERNARY2):
            # the same layer through signed activation views (i5): one view per distinct input
            # (q/k/v share one, gate/up share one), every projection an integer popcount matvec
            VP, VS = 24, 25
            c.alloc(VP, 17408 // 128 * 5 * 16)
            c.alloc(VS, 17408 // 128 * 2)
            em2 = cc.Emitter(rt.ACT_BF16, cus)
            for layer in ents:
                for i, e in enumerate(layer):
                    if i in (0, 2, 3, 5):   # gate (up shares it), down, q (k/v share it), o: a new input
                        em2.activation_view(5, cc.bind(X), cc.bind(VP), cc.bind(VS), e.cols)
                    em2.view_matvec(W, e, 5, cc.bind(VP), cc.bind(VS), cc.bind(Y))
            remap = {i: c.pipeline(nm) for i, nm in enumerate(em2.pipelines)}
            recs2 = list(em2.records())
            for r in recs2:
                r.pipeline = remap[r.pipeline]
            g2, n2 = c.capture_decode(c.table(recs2))
            c.graph_time(g2, 3)
            us2 = c.graph_time(g2, reps) / (reps * copies)
            c.graph_destroy(g2)
            views = {"us_per_layer": round(us2, 2), "launches": n2 // copies, "planes": 5,
                     "GBps": round(layer_bytes / us2 / 1e3, 1)}
        out[f"bonsai27b_layer_{name}"] = {
            "us_per_layer": round(us, 2), "weight_bytes": int(layer_bytes),
            "GBps": round(layer_bytes / us / 1e3, 1), "pct_of_hbm_peak": round(100 * layer_bytes / us / 1e3 / HBM_PEAK_GBS, 2),
            "launches": len(shapes), "kernels": per_kernel, "activation_views_i5": views}
        c.close()
    # qmm: Qwen3.5-4B FFN (gate/up 2560->9216, down 9216->2560), affine u4 g64
    c = rt.Context(act_dtype=rt.ACT_BF16)
    lay = cc.Layout()
    copies = 4
    ents = [[lay.affine(9216, 2560, 64), lay.affine(9216, 2560, 64), lay.affine(2560, 9216, 64)] for _ in range(copies)]
    image = np.zeros(lay.total_bytes, np.uint8)
    rng = fx.rng_for(4, 0)
    for layer in ents:
        for e in layer:
            cc.write_affine(image, e, *synth_affine(rng, e.rows, e.cols, 64, fx.bf16_bits))
    c.upload_weights(W, image)
    del image
    xs = fx.rng_for(4, 1).normal(0, 1, (512, 9216)).astype(np.float32)
    xs[:, fx.rng_for(4, 2).choice(9216, 92, replace=False)] *= 10.0
    c.put(X, fx.bf16_bits(xs))
    c.alloc(Y, 512 * 9216 * 2)
    layer_bytes = sum(e.size_bytes + e.scales_size_bytes + e.biases_size_bytes for e in ents[0])
    qmm = {}
    pipes_installed = 0
    for M in (7, 8, 9, 32, 512):
        em = cc.Emitter(rt.ACT_BF16, cus)
        for layer in ents:
            for e in layer:
                em.matvec(W, e, cc.bind(X), cc.bind(Y), batch=M)
        names = em.pipelines
        remap = {i: c.pipeline(nm) for i, nm in enumerate(names)}
        recs = list(em.records())
        for r in recs:
            r.pipeline = remap[r.pipeline]
        table = c.table(recs)
        g, n = c.capture_prefill(table, seq_len=M)
        c.graph_time(g, 2)
        reps = 10 if M < 512 else 3
        us = c.graph_time(g, reps) / (reps * copies)
        c.graph_destroy(g)
        flops = 2.0 * M * sum(e.rows * e.cols for e in ents[0])
        qmm[f"M={M}"] = {"us_per_ffn": round(us, 2), "TFLOPs": round(flops / us / 1e6, 2),
                         "weight_GBps": round(layer_bytes / us / 1e3, 1)}
        pipes_installed += len(names)
    out["qwen35_4b_ffn_qmm"] = qmm
    c.close()
    # weight import: affine 4-bit quantiser over a 9216 x 2560 tensor resident in HBM
    # (algorithmic bytes = source read + packed codes, scales and biases written)
    c = rt.Context(act_dtype=rt.ACT_BF16)
    rows, cols, group = 9216, 2560, 64
    gpr = cols // group
    quant = {}
    for src_name, src_dtype, esize in (("f32", 0, 4), ("bf16", 2, 2)):
        w = fx.rng_for(5, src_dtype).normal(0, 0.05, (rows, cols)).astype(np.float32)
        c.put(1, w if esize == 4 else fx.bf16_bits(w))
        c.alloc(2, rows * cols // 2)
        c.alloc(3, rows * gpr * 2)
        c.alloc(4, rows * gpr * 2)
        pipe = c.pipeline(f"affine_quantize_u4:{cols}:{group}")
        moved = rows * cols * esize + rows * cols // 2 + 2 * rows * gpr * 2
        for clip_name, clip in (("min_max", 0), ("mse_optimal", 1)):
            rec = rt.make_record(pipe, [(1, 0, 0), (2, 1, 0), (3, 2, 0), (4, 3, 0)],
                                 [(5, rows), (6, src_dtype), (7, clip)], (cus * 16, 1, 1), (128, 1, 1))
            g, n = c.capture_decode(c.table([rec] * 4))
            c.graph_time(g, 1)
            us = c.graph_time(g, 3) / (3 * n)
            c.graph_destroy(g)
            quant[f"{src_name}_{clip_name}"] = {"us": round(us, 1), "GBps": round(moved / us / 1e3, 1),
                                               "Gweights_per_s": round(rows * cols / us / 1e3, 2)}
    out["affine_quantize_u4_9216x2560_g64"] = quant
    c.close()
    # turbo_quant_h matvec (2-bit codes, four-entry codebook per 128 columns) over a 65536 x 2560 matrix
    c = rt.Context(act_dtype=rt.ACT_F16)
    rows, cols = 65536, 2560
    groups = cols // 128
    rng = fx.rng_for(6, 0)
    copies = 4
    image = bytearray()
    offs = []
    for _ in range(copies):
        codes = rng.integers(0, 256, (rows, groups * 32), dtype=np.uint8)
        book = fx.f16_bits(np.sort(rng.normal(0, 0.1, (groups, 4)).astype(np.float32), axis=1))
        offs.append((len(image), len(image) + codes.nbytes))
        image += codes.tobytes() + book.tobytes() + bytes(-(codes.nbytes + book.nbytes) % 256)
    c.upload_weights(W, np.frombuffer(bytes(image), np.uint8))
    del image
    c.put(X, fx.f16_bits(rng.normal(0, 1, cols).astype(np.float32)))
    c.alloc(ACT, groups * 128 * 4)
    c.alloc(Y, rows * 2)
    prep = rt.make_record(c.pipeline("tqh_matvec_prepare_input"), [(X, 0, 0), (ACT, 1, 0)], [(2, cols)],
                          (groups * 128, 1, 1), (128, 1, 1), style=rt.STYLE_THREADS)
    c.interpret_decode(c.table([prep]))
    c.wait()
    mv = c.pipeline("tqh_matvec")
    recs = [rt.make_record(mv, [(W, 0, a), (W, 1, b), (ACT, 2, 0), (Y, 3, 0)],
                           [(4, rows), (5, cols), (6, groups * 32)], (cus * 8, 1, 1), (256, 1, 1)) for a, b in offs]
    g, n = c.capture_decode(c.table(recs * 4))
    c.graph_time(g, 2)
    us = c.graph_time(g, 5) / (5 * n)
    c.graph_destroy(g)
    code_bytes = rows * groups * 32
    out["tqh_matvec_65536x2560"] = {"us": round(us, 2), "code_GBps": round(code_bytes / us / 1e3, 1),
                                    "pct_of_hbm_peak": round(100 * code_bytes / us / 1e3 / HBM_PEAK_GBS, 2)}
    c.close()
    return out


def cpu_baseline(fx, per_layer, lm_head, group) -> dict:
    """Scalar restatement of the reference's CPU dequant-matvec (the oracle), row-parallel over
    the host cores with OpenMP, on a bounded sample of the same workload: the first layer's seven
    matrices plus the first 16384 lm_head rows (about 25 MB of weights per pass)."""
    from oracle import oracle as so
    sample = [(e.rows, e.cols) for e in per_layer[0].values()] + [(16384, lm_head.cols)]
    rng = fx.rng_for(1, 777)
    tensors = [synth_affine(rng, r, k, group, fx.bf16_bits) for r, k in sample]
    xs = {k: rng.normal(0, 1, (1, k)).astype(np.float32) for k in {k for _, k in sample}}
    nbytes = sum(t[0].nbytes + t[1].nbytes + t[2].nbytes for t in tensors)
    cores = len(os.sched_getaffinity(0))
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))

    def one_pass():
        for (r, k), t in zip(sample, tensors):
            so.affine_matvec(*t, xs[k], r, k, group, so.BF16, threads=True)

    one_pass()
    t0 = time.perf_counter()
    passes = 0
    while True:
        one_pass()
        passes += 1
        dt = time.perf_counter() - t0
        if dt > 10.0:
            break
    gbs = nbytes * passes / dt / 1e9
    return {"value": round(gbs, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"{passes} passes over layer 0 (7 matrices) + 16384 lm_head rows = {nbytes} weight bytes/pass, "
                      f"{dt:.1f} s, scalar C restatement of the reference dequant-matvec, OpenMP over rows"}


if __name__ == "__main__":
    sys.exit(main())
