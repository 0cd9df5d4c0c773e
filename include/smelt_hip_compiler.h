/*
 * smelt_hip_compiler.h — build-time half of the HIP backend: the pieces of SmeltCompiler that
 * decide which kernel a weight gets, where its bytes live in weights.bin, and which dispatch
 * records drive it.  Pure host code (no GPU needed); exported from the same libsmelt_hip.so.
 *
 * Each group cites the reference code it mirrors (paths relative to the Smelt repository).
 */
#ifndef SMELT_HIP_COMPILER_H
#define SMELT_HIP_COMPILER_H

#include <stddef.h>
#include <stdint.h>

#include "smelt_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- SmeltDType: Sources/SmeltSchema/SmeltManifest.swift:1613-1645 ------------------------ */
enum {
    SMELT_DTYPE_FP16 = 0,
    SMELT_DTYPE_FP32 = 1,
    SMELT_DTYPE_BF16 = 2,
    SMELT_DTYPE_INT32 = 3,
    SMELT_DTYPE_U4_LUT = 4,
    SMELT_DTYPE_AFFINE_U4 = 5,
    SMELT_DTYPE_BINARY1 = 6,
    SMELT_DTYPE_TERNARY2 = 7,
    SMELT_DTYPE_TURBO_QUANT_H = 8,
    SMELT_DTYPE_RAW = 9,
    SMELT_DTYPE_TRIT5 = 10, /* not in the reference: five base-3 digits per byte */
    SMELT_DTYPE_COUNT
};
/* manifest spelling ("affine_u4", "binary1", ...); NULL for an unknown value */
const char *smelt_dtype_name(int dtype);
int smelt_dtype_from_name(const char *name); /* -1 if unknown */

/* ---- MatvecKernelTable: Sources/SmeltCompiler/MatvecKernelTable.swift:51-284 --------------- */
enum { SMELT_ACT_FP16 = 0, SMELT_ACT_BF16 = 1, SMELT_ACT_FP32 = 2 };
enum { SMELT_SHAPE_GEMV = 0, SMELT_SHAPE_GEMM = 1, SMELT_SHAPE_GEMM_TN = 2 };
enum { SMELT_FUSION_NONE = 0, SMELT_FUSION_DUAL_MATVEC = 1, SMELT_FUSION_GATE_UP_SWIGLU = 2, SMELT_FUSION_GATE_UP_GEGLU = 3 };
enum { SMELT_OUT_FP16 = 0, SMELT_OUT_BF16 = 1, SMELT_OUT_FP32 = 2 };
enum { SMELT_SLOT_FIXED = 0, SMELT_SLOT_VARIABLE = 1 };

typedef struct SmeltMatvecCell {
    int activation, weight /* SMELT_DTYPE_* */, shape, fusion, output, slot;
} SmeltMatvecCell;

/* Family: dense families are SMELT_FAMILY_DENSE + weight dtype */
enum {
    SMELT_FAMILY_DENSE = 0,
    SMELT_FAMILY_AFFINE_U4 = 100,
    SMELT_FAMILY_BINARY1 = 101,
    SMELT_FAMILY_TERNARY2 = 102,
    SMELT_FAMILY_LUT_U4 = 103,
    SMELT_FAMILY_TQH = 104,
    SMELT_FAMILY_TRIT5 = 105,
};
enum {
    SMELT_SELECT_OK = 0,
    SMELT_SELECT_MISSING = -20,        /* meaningful cell, no kernel registered in this backend */
    SMELT_SELECT_NOT_MEANINGFUL = -21, /* no consumer needs this combination */
};
/* select(): total over the cell space, never defaults (MatvecKernelTable.swift:258-270).
 * `hip_backend` != 0 additionally reports SMELT_SELECT_MISSING for families this backend has no
 * kernel for (dense, u4_lut, tqh), so an emitter fails loudly instead of falling back. */
int smelt_kernel_table_select(const SmeltMatvecCell *cell, int hip_backend, int *out_family);
/* meaningfulCells (:155-237): returns the count, writes up to `cap` cells */
int smelt_kernel_table_meaningful_cells(SmeltMatvecCell *out, int cap);

/* ---- weights.bin layout: Sources/SmeltCompiler/SmeltWeightPacker.swift:740-872 -------------- */
typedef struct SmeltWeightEntryC {
    uint64_t offset, size_bytes; /* packed codes (or dense elements) */
    int32_t rows, cols;
    int32_t dtype, group_size;
    int32_t packed_row_stride, padded_cols;
    uint64_t scales_offset, scales_size_bytes;
    uint64_t biases_offset, biases_size_bytes;
} SmeltWeightEntryC;

/* makeAffineEntry (:788-826): [packed][scales][biases], each region 128-byte aligned */
int smelt_layout_make_affine_entry(int rows, int cols, int group_size, uint64_t *offset_io,
                                   SmeltWeightEntryC *out);
/* makeSignedEntry (:831-862): [codes][scales], 128-byte aligned, cols padded to whole groups.
 * dtype is binary1, ternary2, or trit5 (16-byte-aligned rows of ceil(cols/5) bytes). */
int smelt_layout_make_signed_entry(int rows, int cols, int dtype, int group_size,
                                   uint64_t *offset_io, SmeltWeightEntryC *out);
/* Projection bank (SmeltWeightLayoutPlanner.swift:404-572): 2-4 same-input members are re-offset
 * so their packed rows form one contiguous slab, followed by one 128-byte-aligned scale slab
 * (and, for affine, one bias slab).  Byte counts are unchanged and every member keeps its own
 * entry; a bank kernel then walks the members as one virtual row space. */
int smelt_layout_make_affine_bank(const int *member_rows, int members, int cols, int group_size,
                                  uint64_t *offset_io, SmeltWeightEntryC *out_members);
/* The same bank for signed members (binary1, ternary2, trit5): one contiguous code slab, then one
 * 128-byte-aligned scale slab. */
int smelt_layout_make_signed_bank(const int *member_rows, int members, int cols, int dtype, int group_size,
                                  uint64_t *offset_io, SmeltWeightEntryC *out_members);
/* dense fp16/bf16/fp32/int32 entry, 16-byte aligned (:700-737) */
int smelt_layout_make_dense_entry(int rows, int cols, int dtype, uint64_t *offset_io,
                                  SmeltWeightEntryC *out);

/* ---- shape routing: SmeltKernelShapeRegistry.swift + SmeltFusionPlanner.swift:71-152 --------- */
typedef struct SmeltRoute {
    char pipeline[128]; /* manifest pipeline entry */
    int32_t specialized; /* 1 fixed-shape name, 0 generic "name:cols:group" entry */
    int32_t rows_per_group; /* output rows one workgroup walks per step */
    int32_t batch_tile;     /* tokens per grid.y step (1 for batch-1 kernels) */
    int32_t threads;        /* workgroup size */
    int32_t grid_w;         /* workgroups along rows */
} SmeltRoute;

/* decodeAffineMatvec (SmeltFusionPlanner.swift:71-82), fused variants (:100-152) */
int smelt_route_decode_affine(int rows, int cols, int group, int fusion, int compute_units,
                              SmeltRoute *out);
/* prefillAffineFull / prefillAffineBatched (:96-152): max_batch chooses matvec vs MFMA tiles */
int smelt_route_prefill_affine(int rows, int cols, int group, int fusion, int max_batch,
                               int compute_units, SmeltRoute *out);

/* ---- record emitters: SmeltCodeEmitter.swift:1092-1263, 2380-2576; PrefillEmitter.swift:1123-1417 */
typedef struct smelt_emitter smelt_emitter;

typedef struct SmeltBinding {
    int32_t slot; /* >= 0, or SMELT_SLOT_CUR / SMELT_SLOT_ALT */
    uint64_t offset;
    uint8_t offset_kind;
} SmeltBinding;

int smelt_emitter_create(int act_dtype /* SMELT_HIP_ACT_* */, int compute_units, smelt_emitter **out);
void smelt_emitter_destroy(smelt_emitter *e);
const char *smelt_emitter_last_error(const smelt_emitter *e);

/* emitAffineMatvec / emitSignedMatvec through the dtype gateway (emitMatvecImpl, :3997-4082).
 * batch_size > 1 or dynamic != 0 lowers to the batched / qmm families with seqLen-driven grids. */
int smelt_emit_matvec(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *w,
                      SmeltBinding input, SmeltBinding output, int batch_size, int dynamic);
/* fused_*_matvec_add: output = round(matvec) + residual */
int smelt_emit_matvec_add(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *w,
                          SmeltBinding input, SmeltBinding output, SmeltBinding residual);
/* fused gate+up+SwiGLU (emitFusedAffineGateUpSwiglu :2380-2425; signed :1926-2030) */
int smelt_emit_gate_up_swiglu(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *gate,
                              const SmeltWeightEntryC *up, SmeltBinding input, SmeltBinding output,
                              int batch_size, int dynamic);
/* rms_norm_scale_only (norms.metal:944-1008): writes one fp32 scale per row; the first dispatch of the
 * scale-only + norm-scale pair (emitNormScaleAffineMatvecIfPossible, SmeltCodeEmitter.swift:2680-2754). */
int smelt_emit_rms_norm_scale_only(smelt_emitter *e, SmeltBinding input, SmeltBinding scale_output,
                                   int dim, float eps, int batch_size);
/* norm_scale_affine_matvec (lut_matvec.metal:1294-1469; fixed shapes :2743-3170): the kernel reads a
 * precomputed RMS scale and multiplies x_norm = half((x * scale) * (1 + norm_weight)); the normalised
 * row is also stored to norm_output.  affine_u4 weights, one token. */
int smelt_emit_norm_scale_matvec(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *w,
                                 SmeltBinding norm_scale, SmeltBinding input, SmeltBinding norm_weight,
                                 SmeltBinding norm_output, SmeltBinding output);
/* norm_scale_affine_gate_up_swiglu / _geglu (lut_matvec.metal:1471-1700): same prologue in front of
 * the fused gate+up projection; geglu != 0 selects the GeGLU product (:2235-2243). */
int smelt_emit_norm_scale_gate_up(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *gate,
                                  const SmeltWeightEntryC *up, int geglu, SmeltBinding norm_scale,
                                  SmeltBinding input, SmeltBinding norm_weight, SmeltBinding output);
/* AtomicNormFusionPass (SmeltDispatchOptimizer.swift:918-1046; kernels fused_norm_matvec.metal:19-297):
 * rms_norm_1pw and its affine consumer in one dispatch.  up == NULL: matvec, the normalised row is also
 * stored (norm_output required).  up != NULL: gate+up+SwiGLU, norm_output ignored.  scratch holds two
 * 32-bit words {scale, ready flag}. */
int smelt_emit_fused_norm_matvec(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *w,
                                 const SmeltWeightEntryC *up, SmeltBinding input, SmeltBinding norm_weight,
                                 const SmeltBinding *norm_output, SmeltBinding output, SmeltBinding scratch,
                                 float eps);
/* fused_dual_affine_matvec: two weights, one input, two outputs */
int smelt_emit_dual_matvec(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *w1,
                           const SmeltWeightEntryC *w2, SmeltBinding input, SmeltBinding output1,
                           SmeltBinding output2);
/* Common-input projection bank (emitSignedPackedProjectionBankIfPossible,
 * SmeltCodeEmitter.swift:1264-1340): one dispatch for 2-4 members whose slabs are contiguous.
 * Returns 1 (nothing emitted) when the members do not form a bank, so callers keep
 * independent matvecs. */
int smelt_emit_bank_matvec(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *members,
                           int count, SmeltBinding input, const SmeltBinding *outputs);
/* lm_head: affine_matvec_argmax + lm_head_argmax_reduce (TopLevelEmitter.swift:907) */
int smelt_emit_lm_head_argmax(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *w,
                              SmeltBinding input, SmeltBinding partial_keys, SmeltBinding token_out,
                              int batch_size, float logit_cap);
/* emitRMSNorm1PW (SmeltCodeEmitter.swift:2837-2872) and its batched / residual forms: one
 * threadgroup per token.  eps == 1e-6 selects the fixed-dimension pipeline
 * "rms_norm_1pw_d{dim}[_add][_batched]" (no constants); any other eps the generic
 * "rms_norm_1pw[_batched]" with dim and eps as constants 3 and 4 (no residual form exists for it).
 * `weight` is [dim] 16-bit values (a delta from 1); residual may be NULL. */
int smelt_emit_rms_norm_1pw(smelt_emitter *e, SmeltBinding input, SmeltBinding weight,
                            SmeltBinding output, const SmeltBinding *residual, int dim, float eps,
                            int batch_size);
/* emitElementwiseAdd (SmeltCodeEmitter.swift:2944-2966) / elementwise_mul: dispatchThreads over count */
int smelt_emit_elementwise(smelt_emitter *e, int multiply, SmeltBinding a, SmeltBinding b,
                           SmeltBinding output, int count);
/* staged swiglu_fused over `count` gate / up values (DenseTrunkEmitter.swift:209) */
int smelt_emit_swiglu_fused(smelt_emitter *e, SmeltBinding gate, SmeltBinding up,
                            SmeltBinding output, int count);
/* Signed activation views (emitSignedActivationBitplanes / emitSignedBitplane*IfPossible,
 * SmeltCodeEmitter.swift; kernels signed_quant.metal:746-2260).  A view is `planes` bit planes
 * (2..6) of [cols / 128] groups plus one 16-bit scale per group, built once per projection-bank
 * input and consumed by every binary1 / ternary2 member of the bank.
 *   smelt_emit_activation_view     signed_activation_bitplanes_i{N}_g128[_batched]
 *   smelt_emit_view_matvec         signed_{binary,ternary}_bitplane_i{N}_matvec[_add]_g128_rows8
 *   smelt_emit_view_gate_up_swiglu signed_{binary,ternary}_bitplane_i{N}_gate_up_swiglu_g128_rows8 */
int smelt_emit_activation_view(smelt_emitter *e, int planes, SmeltBinding input,
                               SmeltBinding view_planes, SmeltBinding view_scales, int cols,
                               int batch_size);
int smelt_emit_view_matvec(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *w, int planes,
                           SmeltBinding view_planes, SmeltBinding view_scales, SmeltBinding output,
                           const SmeltBinding *residual, int batch_size);
int smelt_emit_view_gate_up_swiglu(smelt_emitter *e, int weights_slot, const SmeltWeightEntryC *gate,
                                   const SmeltWeightEntryC *up, int planes, SmeltBinding view_planes,
                                   SmeltBinding view_scales, SmeltBinding output, int batch_size);
/* swap cur/alt (SmeltDispatchRecord.swap) */
int smelt_emit_swap(smelt_emitter *e);

size_t smelt_emitter_record_count(const smelt_emitter *e);
const SmeltDispatchRecord *smelt_emitter_records(const smelt_emitter *e); /* dispatches.bin bytes */
size_t smelt_emitter_pipeline_count(const smelt_emitter *e);
const char *smelt_emitter_pipeline_name(const smelt_emitter *e, size_t index);
/* bytes a partial-key buffer must hold for the argmax records emitted so far */
size_t smelt_emitter_argmax_partial_bytes(const smelt_emitter *e);

/* Resolve a pipeline entry without a device: writes the kernel symbol and argument kinds.
 * Returns 0, SMELT_HIP_ERR_UNKNOWN_PIPELINE or SMELT_HIP_ERR_INVALID_PACKAGE. */
int smelt_hip_resolve_pipeline_name(const char *entry, int default_act, char *symbol,
                                    size_t symbol_cap, char *kinds, size_t kinds_cap);

/* Launch plans of the kernels a record is re-routed to, without a device (no counterpart in the
 * reference: one kernel per pipeline name there; for tests and for integrators who want to know
 * what a record will run).  Each writes its answer as unsigned 32-bit fields and returns 1 when
 * the shape takes the kernel, 0 when it keeps the kernel its pipeline names, negative on error.
 *
 * smelt_hip_plan_qmm: an affine qmm record (groups of 64, 128 or 32 columns; plain, +add: nmat 1;
 * gate+up: nmat 2) of `batch` tokens.  (The plans of the other re-routed forms are not exposed here: the per-token
 * small-batch names of small matrices, which take the single-token kernel with a grid row per token, the norm-scale
 * qmm names, which run as normalised rows plus this plan, the ternary qmm and the binary / ternary records over
 * several tokens.)  out[0] = 1 streaming kernel, 2 token-tile kernel; out[1] row tiles per wave;
 * out[2] waves along K (streaming: waves of the workgroup); out[3] = 1 when the two matrices go to
 * separate waves; out[4] workgroups that share a tile along K; out[5..7] grid; out[8] threads;
 * out[9] LDS bytes; out[10] workspace bytes of the K split (low 32 bits).
 *
 * smelt_hip_plan_matvec: a single-token matvec of code layout 0 affine u4, 1 binary1, 2 ternary2,
 * 3 trit5.  out[0] 128-byte segments per wave; out[1] waves per workgroup; out[2] workgroups;
 * out[3] threads; out[4] LDS bytes. */
int smelt_hip_plan_qmm(uint32_t rows, uint32_t cols, uint32_t group, uint32_t nmat, uint32_t batch,
                       uint32_t compute_units, size_t lds_limit, size_t workspace_bytes,
                       uint32_t out[11]);
int smelt_hip_plan_matvec(int code_layout, uint32_t rows, uint32_t cols, uint32_t group,
                          uint32_t nmat, size_t lds_limit, int force, uint32_t out[5]);

#ifdef __cplusplus
}
#endif
#endif /* SMELT_HIP_COMPILER_H */
