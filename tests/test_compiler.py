"""Host-side mirror of the reference's build-time pieces: dtype gateway, weights.bin layout,
shape routes, record emitters and pipeline-name resolution (no GPU needed)."""
import ctypes as C

import pytest

from smelt_amd import compiler as cc
from smelt_amd import runtime as rt


def test_dtype_names_round_trip_the_manifest_spelling():
    l = cc.lib()
    # SmeltManifest.swift:1613-1625 raw values
    for i, name in enumerate(cc.DTYPES):
        assert l.smelt_dtype_name(i).decode() == name
        assert l.smelt_dtype_from_name(name.encode()) == i
    assert l.smelt_dtype_from_name(b"q8_0") == -1
    assert l.smelt_dtype_name(99) is None


def test_gateway_has_no_holes_and_never_defaults():
    """MatvecKernelTableTests.swift:47-55: every meaningful cell resolves; :110-164 family per
    cell; :166-211 rejections."""
    cells = cc.meaningful_cells()
    assert len(cells) > 40
    for c in cells:
        rc, fam = cc.select(c.activation, c.weight, c.shape, c.fusion, c.output, c.slot)
        assert rc == cc.SELECT_OK
        if c.weight in (cc.FP16, cc.BF16, cc.FP32):
            assert fam == cc.FAMILY_DENSE + c.weight
    fam_of = {cc.AFFINE_U4: cc.FAMILY_AFFINE_U4, cc.BINARY1: cc.FAMILY_BINARY1, cc.TERNARY2: cc.FAMILY_TERNARY2,
              cc.U4_LUT: cc.FAMILY_LUT_U4, cc.TURBO_QUANT_H: cc.FAMILY_TQH, cc.TRIT5: cc.FAMILY_TRIT5}
    for w, f in fam_of.items():
        assert cc.select(cc.ACT_FP16, w) == (cc.SELECT_OK, f)
    # no consumer: variable-slot tqh, int32/raw weights, fused dual on a dense weight, fp32-act ternary
    assert cc.select(cc.ACT_FP16, cc.TURBO_QUANT_H, slot=cc.SLOT_VARIABLE)[0] == cc.SELECT_NOT_MEANINGFUL
    assert cc.select(cc.ACT_FP16, cc.INT32)[0] == cc.SELECT_NOT_MEANINGFUL
    assert cc.select(cc.ACT_FP16, cc.RAW)[0] == cc.SELECT_NOT_MEANINGFUL
    assert cc.select(cc.ACT_FP16, cc.FP16, fusion=cc.FUSION_DUAL)[0] == cc.SELECT_NOT_MEANINGFUL
    assert cc.select(cc.ACT_FP32, cc.TERNARY2, output=cc.OUT_FP32)[0] == cc.SELECT_NOT_MEANINGFUL
    # the HIP backend registers the quantized families only: anything else is a loud hole
    assert cc.select(cc.ACT_FP16, cc.AFFINE_U4, hip_backend=True)[0] == cc.SELECT_OK
    assert cc.select(cc.ACT_FP16, cc.BINARY1, cc.GEMM, hip_backend=True)[0] == cc.SELECT_OK
    assert cc.select(cc.ACT_FP16, cc.FP16, hip_backend=True)[0] == cc.SELECT_MISSING
    assert cc.select(cc.ACT_FP16, cc.U4_LUT, hip_backend=True)[0] == cc.SELECT_OK
    assert cc.select(cc.ACT_FP16, cc.U4_LUT, cc.GEMM, hip_backend=True)[0] == cc.SELECT_OK            # fused_lut_matmul, one token per grid row
    assert cc.select(cc.ACT_FP16, cc.TURBO_QUANT_H, hip_backend=True)[0] == cc.SELECT_OK
    assert cc.select(cc.ACT_FP16, cc.AFFINE_U4, fusion=cc.FUSION_GATE_UP_GEGLU, hip_backend=True)[0] == cc.SELECT_OK
    assert cc.select(cc.ACT_FP16, cc.AFFINE_U4, cc.GEMM, fusion=cc.FUSION_GATE_UP_GEGLU, hip_backend=True)[0] == cc.SELECT_OK
    assert cc.select(cc.ACT_FP16, cc.BINARY1, fusion=cc.FUSION_GATE_UP_GEGLU, hip_backend=True)[0] == cc.SELECT_NOT_MEANINGFUL
    assert cc.select(cc.ACT_FP16, cc.AFFINE_U4, cc.GEMM, fusion=cc.FUSION_DUAL, hip_backend=True)[0] == cc.SELECT_OK


def test_weight_layout_alignment_sizes_and_no_overlap():
    """WeightPackerTests.swift:43-97, 386-456: 16-byte dense / 128-byte quantized alignment,
    no overlap, sizes from the formulas at SmeltWeightPacker.swift:788-862."""
    lay = cc.Layout()
    d = lay.dense(3, 5, cc.FP16)
    a = lay.affine(3584, 1024, 64)
    b = lay.signed(17408, 5120, cc.BINARY1)
    t = lay.signed(5120, 17408, cc.TERNARY2)
    t5 = lay.signed(5120, 17408, cc.TRIT5)
    odd = lay.signed(7, 200, cc.TERNARY2)          # cols padded to whole groups
    assert d.offset % 16 == 0 and d.size_bytes == 30
    assert (a.size_bytes, a.scales_size_bytes, a.biases_size_bytes) == (1835008, 114688, 114688)
    assert a.packed_row_stride == 512 and a.padded_cols == 1024
    for e in (a, b, t, t5, odd):
        assert e.offset % 128 == 0 and e.scales_offset % 128 == 0
    assert a.biases_offset % 128 == 0
    assert (b.size_bytes, b.scales_size_bytes, b.packed_row_stride) == (11141120, 1392640, 640)
    assert (t.size_bytes, t.packed_row_stride) == (5120 * 4352, 4352)
    assert (t5.packed_row_stride, t5.size_bytes) == (3488, 5120 * 3488)
    assert (odd.padded_cols, odd.packed_row_stride, odd.scales_size_bytes) == (256, 64, 7 * 2 * 2)
    spans = []
    for e in lay.entries:
        spans.append((e.offset, e.offset + e.size_bytes))
        if e.scales_size_bytes:
            spans.append((e.scales_offset, e.scales_offset + e.scales_size_bytes))
        if e.biases_size_bytes:
            spans.append((e.biases_offset, e.biases_offset + e.biases_size_bytes))
    spans.sort()
    for (s0, e0), (s1, _) in zip(spans, spans[1:]):
        assert e0 <= s1
    assert lay.total_bytes == spans[-1][1]
    # config-0 weight bytes: 2 064 384 counted once
    assert a.size_bytes + a.scales_size_bytes + a.biases_size_bytes == 2064384


def test_shape_routes():
    """KernelShapeRegistryTests.swift:8-150 (decode shapes -> tuned kernels, unknown shape ->
    generic function-constant entry) and :152-290 (prefill / QMM routes)."""
    r = cc.route_decode_affine(3584, 1024, 64)
    assert r.pipeline == b"affine_matvec_c1024_r3584_g64" and r.specialized == 1 and r.threads == 256
    assert r.rows_per_group == 8 and r.grid_w == 448           # small matrix: one row per wave slot, two slots per wave
    r = cc.route_decode_affine(3584, 1024, 64, compute_units=32)
    assert r.rows_per_group == 16 and r.grid_w == 128          # enough workgroups per CU: two rows per slot
    r = cc.route_decode_affine(151936, 1024, 64)
    assert r.grid_w == 1024                                     # capped at four workgroups per compute unit
    r = cc.route_decode_affine(777, 1056, 32)
    assert r.pipeline == b"affine_matvec:1056:32" and r.specialized == 0
    r = cc.route_decode_affine(3584, 1024, 64, fusion=cc.FUSION_GATE_UP_SWIGLU)
    assert r.pipeline == b"fused_affine_gate_up_swiglu_c1024_r3584_g64"
    r = cc.route_decode_affine(6144, 1536, 128, fusion=cc.FUSION_GATE_UP_GEGLU)
    assert r.pipeline == b"fused_affine_gate_up_geglu:1536:128"
    with pytest.raises(ValueError):
        cc.route_decode_affine(64, 1000, 64)                    # cols not a multiple of 32
    r = cc.route_prefill_affine(9216, 2560, 64, max_batch=8)     # 5..32 tokens, g64: split-K skinny MFMA kernel
    assert r.pipeline == b"affine_matvec_c2560_r9216_g64_batched_skinny" and (r.batch_tile, r.grid_w) == (32, 288)
    r = cc.route_prefill_affine(2560, 9216, 64, max_batch=32)
    assert r.pipeline == b"affine_matvec_c9216_r2560_g64_batched_skinny" and r.grid_w % 80 == 0 and r.grid_w >= 240
    r = cc.route_prefill_affine(9216, 2560, 128, max_batch=8)    # other group sizes keep the slab kernel
    assert r.pipeline == b"affine_matvec_c2560_r9216_g128_batched_full" and (r.batch_tile, r.grid_w) == (16, 144)
    r = cc.route_prefill_affine(9216, 2560, 64, max_batch=512)
    assert r.pipeline == b"affine_matvec_c2560_r9216_g64_batched_full_b64" and r.batch_tile == 64
    r = cc.route_prefill_affine(9216, 2560, 64, max_batch=3)
    assert r.pipeline == b"affine_matvec_c2560_r9216_g64_batched_tile4" and r.batch_tile == 4


def test_pipeline_names_resolve_to_kernels_with_the_reference_binding_counts():
    """Buffer / constant counts of SmeltKernelCatalog signatures (:2953-2972 and the affine
    macros) must equal the leading P / U counts the HIP kernels take."""
    cases = {
        "affine_matvec:1024:64": ("smelt_affine_matvec_f16", 5, 1),
        "affine_matvec_c2048_r151936_g64_rows8": ("smelt_affine_matvec_f16", 5, 0),
        "fused_affine_matvec_add_c3584_r1024_g64_rows4": ("smelt_affine_matvec_add_f16", 6, 0),
        "fused_affine_gate_up_swiglu_c1024_r3584_g64_rows4": ("smelt_affine_gate_up_swiglu_f16", 8, 0),
        "fused_dual_affine_matvec:1024:64": ("smelt_affine_dual_matvec_f16", 9, 1),
        "affine_matvec_c2560_r9216_g64_batched_full": ("smelt_affine_qmm_mt1_f16", 5, 1),
        "fused_affine_matvec_add_c2048_r1024_g64_batched_full_b8": ("smelt_affine_qmm_add_mt1_f16", 7, 1),
        "signed_binary_matvec_g128_rows8": ("smelt_signed_binary_matvec_f16", 4, 2),
        "signed_binary_matvec_add_g128_rows8": ("smelt_signed_binary_matvec_add_f16", 5, 2),
        "signed_binary_gate_up_swiglu_g128_rows8": ("smelt_signed_binary_gate_up_swiglu_f16", 6, 2),
        "signed_binary_matvec_g128_rows8_batched_b4": ("smelt_signed_binary_matvec_b4_f16", 4, 3),
        "signed_ternary_matvec_g128_rows8": ("smelt_signed_ternary_matvec_f16", 4, 2),
        "signed_ternary_affine_matvec_g128_rows8": ("smelt_teraff_matvec_f16", 5, 2),
        "signed_ternary_affine_qmm_g128_bm32_bn32_bk32": ("smelt_ternary_qmm_mt2_f16", 5, 3),
        "signed_ternary_affine_bank4_matvec_g128_rows8": ("smelt_teraff_bank4_matvec_f16", 8, 5),
        "signed_binary_embedding_gather_g128": ("smelt_signed_binary_embedding_gather_f16", 4, 1),
        "affine_matvec_argmax_c2560_r262144_g128_batched": ("smelt_affine_matvec_argmax_f16", 5, 2),
        # layer ops between the matvecs (SmeltKernelCatalog.swift:630, 700-707, 964, 1312, 1966, 3004-3014)
        "rms_norm_1pw": ("smelt_rms_norm_1pw_f16", 3, 2),
        "rms_norm_1pw_batched": ("smelt_rms_norm_1pw_f16", 3, 2),
        "rms_norm_1pw_d1024": ("smelt_rms_norm_1pw_f16", 3, 0),
        "rms_norm_1pw_d1536_add_batched": ("smelt_rms_norm_1pw_add_f16", 4, 0),
        "rms_norm_scale_only_precise": ("smelt_rms_norm_scale_only_f16", 2, 2),
        "rms_norm_scale_only_d2048_eps1e5_batched": ("smelt_rms_norm_scale_only_f16", 2, 0),
        "residual_add_rms_norm_scale_only_precise": ("smelt_residual_add_rms_norm_scale_only_f16", 4, 2),
        "swiglu_fused": ("smelt_swiglu_fused_f16", 3, 1),
        "elementwise_add": ("smelt_elementwise_add_f16", 3, 1),
    }
    for entry, (symbol, nbuf, nconst) in cases.items():
        rc, sym, kinds = cc.resolve_pipeline_name(entry)
        assert rc == 0 and sym == symbol, (entry, rc, sym)
        own = kinds[:nbuf + nconst]
        assert own.count("P") == nbuf and len(own) - own.count("P") == nconst, (entry, kinds)
    assert cc.resolve_pipeline_name("affine_matvec:1024:64@bf16")[1] == "smelt_affine_matvec_bf16"
    assert cc.resolve_pipeline_name("affine_matvec:1024:64", rt.ACT_BF16)[1] == "smelt_affine_matvec_bf16"
    assert cc.resolve_pipeline_name("affine_matvec:1024")[0] == -3        # malformed entry
    assert cc.resolve_pipeline_name("affine_matvec:10:64")[0] == -3       # cols not a multiple of 32
    assert cc.resolve_pipeline_name("fused_lut_matvec:1024:16")[1:] == ("smelt_lut_matvec_f16", "PPPPUUU")
    assert cc.resolve_pipeline_name("fused_gate_up_swiglu:1024:16")[1] == "smelt_lut_gate_up_swiglu_f16"
    assert cc.resolve_pipeline_name("fused_lut_matvec:1024:4")[0] == -3    # fewer than 8 rows per table
    assert cc.resolve_pipeline_name("tqh_matvec_batched")[1:] == ("smelt_tqh_matvec_f16", "PPPPUUU")
    assert cc.resolve_pipeline_name("u4_lut_qmm")[0] == -4
    # the compiler's generated variants (SmeltGeneratedKernelVariants.swift:17-35, 66-68)
    assert cc.resolve_pipeline_name("affine_matvec_c2560_r9216_g64_batched_verify_b4")[1:] == ("smelt_affine_matvec_batched_mb4_f16", "PPPPPUUUUU")
    assert cc.resolve_pipeline_name("fused_affine_gate_up_swiglu_c2560_r9216_g64_batched_verify_b4")[1:] == \
        ("smelt_affine_gate_up_swiglu_batched_mb4_f16", "PPPPPPPPUUUUU")
    assert cc.resolve_pipeline_name("fused_dual_affine_matvec_c2048_r16_g64_batched_verify_b4@bf16")[1:] == \
        ("smelt_affine_dual_matvec_batched_mb4_bf16", "PPPPPPPPPUUUUU")
    assert cc.resolve_pipeline_name("fused_dual_affine_matvec_add_c2048_r256_g64_rows4")[1:] == \
        ("smelt_affine_dual_matvec_add_f16", "PPPPPPPPPPPUUU")
    assert cc.resolve_pipeline_name("fused_dual_affine_matvec_add_c2048_r256_g64_batched")[0] == -4
    assert cc.resolve_pipeline_name("fused_dual_affine_matvec_c2048_r16_g64_batched_full")[0] == -4
    assert cc.resolve_pipeline_name("rms_norm_1pw_from_fp32")[1:] == ("smelt_rms_norm_1pw_from_fp32_f16", "PPPUF")
    assert cc.resolve_pipeline_name("rms_norm_gated_d128")[1] == "smelt_rms_norm_gated_f16"
    assert cc.resolve_pipeline_name("rms_norm_head_f32")[0] == -4          # fp32 trunk kernels are out of scope
    assert cc.resolve_pipeline_name("rope_apply")[0] == -4


def test_emitters_bind_what_the_reference_emitters_bind():
    lay = cc.Layout()
    wa = lay.affine(3584, 1024, 64)
    wb = lay.signed(1024, 5120, cc.BINARY1)
    wt = lay.signed(1024, 5120, cc.TERNARY2)
    em = cc.Emitter()
    em.matvec(0, wa, cc.bind(rt.SLOT_CUR), cc.bind(rt.SLOT_ALT))
    em.swap()
    em.matvec(0, wb, cc.bind(3), cc.bind(4))
    em.matvec(0, wt, cc.bind(3), cc.bind(4), batch=1, dynamic=True)
    em.matvec(0, wa, cc.bind(3), cc.bind(4), batch=1, dynamic=True)
    recs = em.records()
    assert len(recs) == 6 and C.sizeof(recs) == 6 * 360
    names = em.pipelines
    # affine decode (SmeltCodeEmitter.swift:2535-2549): 0 W, 1 S, 2 B, 3 x, 4 y
    r = recs[0]
    assert names[r.pipeline] == "affine_matvec_c1024_r3584_g64" and r.buffer_count == 5 and r.constant_count == 0
    assert [r.buffers[i].binding_index for i in range(5)] == [0, 1, 2, 3, 4]
    assert [r.buffers[i].offset for i in range(3)] == [wa.offset, wa.scales_offset, wa.biases_offset]
    assert (r.buffers[3].slot, r.buffers[4].slot) == (rt.SLOT_CUR, rt.SLOT_ALT)
    assert recs[1].op_kind == 1
    # binary decode (:1224-1262): 0 codes, 1 scales, 2 x, 3 y, const 4 rows, 5 cols
    r = recs[2]
    assert names[r.pipeline] == "signed_binary_matvec_g128_rows8"
    assert [(r.constants[i].binding_index, r.constants[i].value) for i in range(2)] == [(4, 1024), (5, 5120)]
    # ternary prefill pair (:1120-1182): QMV guarded to seqLen < 6, QMM with minSeqLen 6
    qmv, qmm = recs[3], recs[4]
    assert names[qmv.pipeline] == "signed_ternary_affine_matvec_g128_rows8"
    assert names[qmm.pipeline] == "signed_ternary_affine_qmm_g128_bm32_bn32_bk32"
    assert qmv.buffers[1].offset == qmv.buffers[2].offset == wt.scales_offset
    guard = qmv.constants[2]
    assert (guard.kind, guard.binding_index, guard.value) == (13, 0xFF, 6)
    assert qmm.min_seq_len == 6 and (qmm.style >> 4) & 3 == rt.GRID_SEQ_LEN_CEIL_DIV and qmm.grid_h == 32
    assert (qmm.constants[2].binding_index, qmm.constants[2].kind) == (7, rt.CONST_SEQ_LEN)
    # affine prefill (PrefillEmitter.swift:1184-1216): const 5 = seqLen, grid.y = ceil(seqLen / tile)
    r = recs[5]
    assert names[r.pipeline].startswith("affine_matvec_c1024_r3584_g64_batched")
    assert (r.constants[0].binding_index, r.constants[0].kind) == (5, rt.CONST_SEQ_LEN)
    # guards: signed kernels need exact g128 geometry (:1105-1115)
    bad = lay.signed(8, 200, cc.BINARY1)
    with pytest.raises(cc.EmitError) as e:
        em.matvec(0, bad, cc.bind(3), cc.bind(4))
    assert e.value.code == -7 and "g128" in e.value.message
    dense = lay.dense(8, 64, cc.FP16)
    with pytest.raises(cc.EmitError) as e:
        em.matvec(0, dense, cc.bind(3), cc.bind(4))
    assert e.value.code == cc.SELECT_MISSING
    # bf16 packages tag their pipeline entries
    em16 = cc.Emitter(rt.ACT_BF16)
    em16.matvec(0, wa, cc.bind(1), cc.bind(2))
    assert em16.pipelines == ["affine_matvec_c1024_r3584_g64@bf16"]
