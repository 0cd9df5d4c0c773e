/*
 * smelt_hip.h — C ABI of the MI355X (gfx950) backend for Smelt's quantized matvec / qmm path.
 *
 * The reference runtime is hard-wired to Metal: SmeltRuntime owns an MTLDevice, an MTLLibrary
 * built from model.metallib, one MTLComputePipelineState per manifest pipeline name, one
 * MTLBuffer per slot, and walks a table of fixed-width dispatch records every token.  This
 * header declares the HIP replacement for exactly those call sites; each entry point cites the
 * reference code it stands in for (paths relative to the Smelt repository root).
 *
 * Conventions (after Sources/CLLGuidance/include/llguidance.h): opaque handles, create/destroy
 * pairs, int status (0 = ok, negative = error, never aborts), and a per-context error string.
 * One context is used from one thread at a time; smelt_hip_pipeline_create may be called
 * concurrently with itself (pipeline compilation runs concurrently at startup in the
 * reference, SmeltRuntime.swift:482-494).
 */
#ifndef SMELT_HIP_H
#define SMELT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- dispatch record ABI: Sources/SmeltSchema/SmeltDispatchTable.swift:21-165 ----------- */

#define SMELT_MAX_BUFFERS_PER_DISPATCH 16 /* agentMaxBuffersPerDispatch, :15 */
#define SMELT_MAX_CONSTANTS_PER_DISPATCH 8 /* agentMaxConstantsPerDispatch, :18 */

typedef struct SmeltBufferRecord {
    int16_t slot;          /* >= 0 literal slot, -1 = cur, -2 = alt (:25-43) */
    uint8_t binding_index; /* kernel argument position */
    uint8_t offset_kind;   /* 0 literal, 1 position*stride, 2 startPos*lo32+hi32,
                              3 (seqLen-1)*offset, 4 floor(seqLen/hi32)*lo32 (:30-36) */
    uint32_t _pad;
    uint64_t offset;
} SmeltBufferRecord; /* 16 bytes */

typedef struct SmeltConstantRecord {
    uint8_t kind;          /* SMELT_CONST_* (:64-87) */
    uint8_t binding_index; /* 0xFF = evaluated only for its skip effect */
    uint16_t pad;
    uint32_t value;
} SmeltConstantRecord; /* 8 bytes */

typedef struct SmeltDispatchRecord {
    uint8_t op_kind; /* 0 dispatch, 1 swap cur/alt */
    uint8_t _pad0;
    uint16_t pipeline; /* index into the manifest pipeline list */
    uint8_t style;     /* bits 0-1 style (0 threadgroups, 1 threads); bits 2-3/4-5/6-7 grid W/H/D kind */
    uint8_t buffer_count;
    uint8_t constant_count;
    uint8_t _pad1;
    uint16_t min_seq_len; /* prefill guard, 0 = always */
    uint16_t _pad2;
    uint32_t grid_w, grid_h, grid_d;
    uint32_t tg_w, tg_h, tg_d;
    uint32_t _pad3;
    SmeltBufferRecord buffers[SMELT_MAX_BUFFERS_PER_DISPATCH];
    SmeltConstantRecord constants[SMELT_MAX_CONSTANTS_PER_DISPATCH];
} SmeltDispatchRecord; /* 360 bytes; strides pinned by DispatchTableTests.swift:12-31 */

enum {
    SMELT_OP_DISPATCH = 0,
    SMELT_OP_SWAP = 1,
    SMELT_STYLE_THREADGROUPS = 0,
    SMELT_STYLE_THREADS = 1,
    SMELT_GRID_LITERAL = 0,
    SMELT_GRID_SEQ_LEN = 1,
    SMELT_GRID_SEQ_LEN_MUL_LITERAL = 2,
    SMELT_GRID_SEQ_LEN_CEIL_DIV_LITERAL = 3, /* high bit of the literal set = floor */
    SMELT_SLOT_CUR = -1,
    SMELT_SLOT_ALT = -2,
};

enum {
    SMELT_CONST_LITERAL_U32 = 0,
    SMELT_CONST_LITERAL_F32 = 1,
    SMELT_CONST_POSITION = 2,
    SMELT_CONST_POSITION_PLUS1 = 3,
    SMELT_CONST_SEQ_LEN = 4,
    SMELT_CONST_START_POS = 5,
    SMELT_CONST_START_POS_PLUS_LITERAL = 6,
    SMELT_CONST_SEQ_LEN_MUL_LITERAL = 7,
    SMELT_CONST_SEQ_LEN_MOD_LITERAL = 8,
    SMELT_CONST_SEQ_LEN_MOD_LITERAL_SKIP_IF_ZERO = 9,
    SMELT_CONST_POSITION_PLUS1_LT_LITERAL_SKIP_IF_FALSE = 10,
    SMELT_CONST_POSITION_PLUS1_GE_LITERAL_SKIP_IF_FALSE = 11,
    SMELT_CONST_CACHE_SEQ_CAPACITY = 12,
    SMELT_CONST_SEQ_LEN_LT_LITERAL_SKIP_IF_FALSE = 13,
};

/* ---- status codes ------------------------------------------------------------------------- */
enum {
    SMELT_HIP_OK = 0,
    SMELT_HIP_ERR_INVALID_ARGUMENT = -1,
    SMELT_HIP_ERR_HIP = -2,              /* a HIP call failed; see smelt_hip_last_error */
    SMELT_HIP_ERR_INVALID_PACKAGE = -3,  /* SmeltRuntimeError.invalidPackage (SmeltRuntime.swift:7062) */
    SMELT_HIP_ERR_UNKNOWN_PIPELINE = -4, /* name is not a kernel this backend implements */
    SMELT_HIP_ERR_BINDING_MISMATCH = -5, /* record bindings do not match the kernel's arguments */
    SMELT_HIP_ERR_OUT_OF_RANGE = -6,     /* a binding would read or write outside its slot */
    SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY = -7,
    SMELT_HIP_ERR_NO_DEVICE = -8,
};

enum { SMELT_HIP_ACT_F16 = 0, SMELT_HIP_ACT_BF16 = 1 };

typedef struct smelt_hip_context smelt_hip_context;
typedef struct smelt_hip_graph smelt_hip_graph;

/* Device + queue creation: SmeltRuntime.swift:695-712 (MTLCreateSystemDefaultDevice, makeCommandQueue). */
int smelt_hip_context_create(int device_index, smelt_hip_context **out);
void smelt_hip_context_destroy(smelt_hip_context *ctx);

/* Error string of the last failed call on this context (NULL ctx: last context-less failure);
 * the analogue of the thrown SmeltRuntimeError description / llg_get_error. */
const char *smelt_hip_last_error(const smelt_hip_context *ctx);

/* Element type the package's activations, outputs and affine scales use unless a pipeline
 * entry overrides it with an "@f16" / "@bf16" suffix.  Default fp16, the reference's type for
 * every quantized matvec (MatvecKernelTable.swift:158-181). */
int smelt_hip_set_activation_dtype(smelt_hip_context *ctx, int act_dtype);

/* Which kernel a single-token quantized matvec record runs.  AUTO (the default): every shape the
 * single-pass matrix-core kernel of the same pipeline can express takes it, the rest the vector-ALU
 * kernel (the two add up a row in different orders: results agree to the output tolerance, not bit
 * for bit); MATRIX_CORE asks for the same explicitly (kept from when AUTO had size thresholds);
 * VECTOR keeps every record on the vector-ALU kernels.  The ternary qmm record takes a streaming kernel up to
 * 128 tokens (same dequantised fp16 weights, rows of a multiple of 256 columns).  Binary and ternary records over several tokens
 * (the "_batched_b4" forms, per-token records with several grid rows) take the same kernel two tokens per
 * pass, each token's row bit for bit the one-token launch's; from eight tokens on a streaming kernel (the
 * weights pass once per sixteen tokens; bf16 rows converted to fp16; one output step from those rows at most).  The same switch
 * covers the qmm records (groups of 64, 128 and 32 columns; rows of a multiple of 256, 512 and 256 columns) and, from
 * two tokens on, the per-token small-batch ("_batched", "_batched_verify_b4")
 * forms of the affine matvec and gate+up+SwiGLU, whose arguments are the skinny qmm's (while
 * tokens x weights stay below about 20M they run the single-token kernel with a grid row per token, bit for
 * bit the rows of a one-token record; beyond, the streaming kernel), and the
 * lm_head matvec+argmax over two tokens and more without a logit cap (logits of all tokens through the
 * streaming kernel into the context workspace, partial keys from a second launch: the record then counts as
 * two launches), the norm-scale prologue qmm records from two tokens on (the normalised rows from a launch of
 * their own, then the kernel of the plain record: two launches, the bits of the staged pair), and the lm_head record at one token where the rows' 16-byte pieces leave the fused kernel's last
 * pass over a row less than nine tenths full (1536, 2560, 3072, 3584, 5120 columns: the single-pass kernel
 * with the argmax as its epilogue, tiles that share a partial key meeting in the context workspace): AUTO and
 * MATRIX_CORE run the streaming kernel of the pipeline below 128
 * tokens (K split inside a workgroup, no workspace) and the token-tile kernel from 128 tokens on (from 96
 * for matrices of 20M weights and 2560 rows, from 33 for 40M weights and 3584 rows)
 * (matrices with few tiles and long rows split K across workgroups: partial sums in the
 * workspace, added in a fixed order), VECTOR the split-K or token-slab kernel the record's geometry
 * describes (split-K: partial sums in the workspace).  Results of the alternatives differ in
 * summation order only.  Consequence under AUTO: the records of one model run on two summation
 * orders, e.g. a matvec at one token (single-pass kernel) and its batched-verify form (streaming
 * kernel) agree to one step of the output type but not bit for bit; a caller that compares such
 * rows bit for bit pins one engine.  On one engine a fused kernel and the staged pair it
 * replaces are bit-identical.  No counterpart in the reference (one kernel per pipeline name there);
 * meant for A/B measurement and for tests. */
enum { SMELT_HIP_MATVEC_AUTO = 0, SMELT_HIP_MATVEC_MATRIX_CORE = 1, SMELT_HIP_MATVEC_VECTOR = 2 };
int smelt_hip_set_matvec_engine(smelt_hip_context *ctx, int engine);

/* dev.makeLibrary(URL: model.metallib): SmeltRuntime.swift:833-835.  A code object is a gfx950
 * image produced by hipcc --genco, loaded with hipModuleLoadData.  The kernels ship as several
 * code objects (smelt_kernels*.hsaco); load every one of them before creating pipelines. */
int smelt_hip_module_load(smelt_hip_context *ctx, const void *code_object, size_t bytes);
/* `path` names one code object, or a directory: then the code objects its smelt_kernels.manifest
 * lists (one file name per line, written by the build) are loaded, or, without a manifest, every
 * smelt_kernels*.hsaco in it. */
int smelt_hip_module_load_file(smelt_hip_context *ctx, const char *path);

/* pipelineFunction(for:library:) + makePipelineState: SmeltRuntime.swift:6229-6306.
 * `entry` is a manifest pipeline string: "fn", or "fn:cols:groupSize" for the function-constant
 * kernels (:6215-6223, :6233-6251).  Pipelines are appended in call order so that
 * *out_index equals SmeltDispatchRecord.pipeline.  An entry this backend does not implement
 * occupies its index as a "fallback to previous" slot (:453-456, :6305-6306) when
 * allow_missing != 0, otherwise the call fails with SMELT_HIP_ERR_UNKNOWN_PIPELINE.
 * A malformed "name:cols:group" entry fails with SMELT_HIP_ERR_INVALID_PACKAGE (:6236-6243). */
int smelt_hip_pipeline_create(smelt_hip_context *ctx, const char *entry, int allow_missing,
                              uint32_t *out_index);
int smelt_hip_pipeline_count(const smelt_hip_context *ctx);
/* 1 = launchable, 0 = fallback slot, negative = bad index */
int smelt_hip_pipeline_is_ready(const smelt_hip_context *ctx, uint32_t index);

/* Slot buffers: makeBuffer(length:) zero-filled, SmeltRuntime.swift:922-979. */
int smelt_hip_buffer_alloc(smelt_hip_context *ctx, int slot, size_t bytes);
int smelt_hip_buffer_write(smelt_hip_context *ctx, int slot, size_t offset, const void *src,
                           size_t bytes);
int smelt_hip_buffer_read(smelt_hip_context *ctx, int slot, size_t offset, void *dst,
                          size_t bytes);
int smelt_hip_buffer_size(const smelt_hip_context *ctx, int slot, size_t *bytes);

/* weights.bin mapping: SmeltMetalWeightStorage.swift:220-319 maps the file into page-aligned
 * MTLBuffers and resolves logical offsets (SmeltRuntime.swift:3153-3169).  HBM is not unified
 * with host memory, so the bytes are copied once into one device allocation that becomes the
 * read-only weights slot; logical offsets are byte offsets into it. */
int smelt_hip_weights_upload(smelt_hip_context *ctx, int weights_slot, const void *bytes,
                             size_t size);

/* cacheSeqCapacityValue used by constant kind 12 (SmeltRuntime.swift:1208, :1245). */
int smelt_hip_set_cache_seq_capacity(smelt_hip_context *ctx, uint32_t capacity);

/* loadDispatchTable size check: SmeltRuntime.swift:6322-6350 (size % 360 == 0). */
int smelt_hip_dispatch_table_count(size_t table_bytes, size_t *out_count);

/* emitDecodeDispatchRecord: SmeltRuntime.swift:3187-3247.  Returns 1 if a kernel was
 * launched, 0 if the record was a swap / skipped, negative on error. */
int smelt_hip_encode_decode_record(smelt_hip_context *ctx, const SmeltDispatchRecord *rec,
                                   int cur, int alt, int32_t position);
/* emitDispatchRecord: SmeltRuntime.swift:5990-6054 (minSeqLen guard, offset kinds 0-4, dynamic
 * grids :6186-6207, skip constants). */
int smelt_hip_encode_prefill_record(smelt_hip_context *ctx, const SmeltDispatchRecord *rec,
                                    int cur, int alt, int32_t seq_len, int32_t start_pos);
/* No counterpart in the reference.  For callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the same as
 * smelt_hip_encode_prefill_record, except that kernels which split K across workgroups (the
 * "_batched_skinny" qmm pipelines under the VECTOR engine, the token-tile qmm otherwise) keep their
 * partial sums and arrival counters in a file-scope device array of the library instead of the
 * workspace a context allocates, and the call itself allocates and frees nothing.  A
 * "_batched_skinny" record whose partials need more than SMELT_HIP_STATIC_SCRATCH_BYTES (4 KB per
 * workgroup and matrix) or more than 16384 row tiles is rejected with
 * SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY; the token-tile kernel does not split K when its partials do
 * not fit.  Each GPU holds one copy of the array for the
 * life of the process, shared by every context on it: calls that overlap on one GPU (two streams)
 * race; calls on one stream are ordered. */
#define SMELT_HIP_STATIC_SCRATCH_BYTES ((size_t)16 << 20)
int smelt_hip_encode_prefill_record_static_scratch(smelt_hip_context *ctx,
                                                   const SmeltDispatchRecord *rec, int cur, int alt,
                                                   int32_t seq_len, int32_t start_pos);
/* interpretDispatchTable: SmeltRuntime.swift:3251-3275 / interpretPrefillDispatchTable
 * :6059-6084 — walks the records, flipping cur/alt (initially cur = cur0, alt = alt0) on
 * swap records.  Returns the number of kernels launched or a negative status. */
int smelt_hip_interpret_decode_table(smelt_hip_context *ctx, const SmeltDispatchRecord *table,
                                     size_t count, int cur0, int alt0, int32_t position);
int smelt_hip_interpret_prefill_table(smelt_hip_context *ctx, const SmeltDispatchRecord *table,
                                      size_t count, int cur0, int alt0, int32_t seq_len,
                                      int32_t start_pos);

/* cmdBuf.commit() / waitUntilCompleted() / cmdBuf.error: SmeltRuntime.swift:1607-1621. */
int smelt_hip_submit(smelt_hip_context *ctx);
int smelt_hip_wait(smelt_hip_context *ctx);
/* gpuEndTime - gpuStartTime of the last submitted batch: SmeltRuntime.swift:3574,
 * KernelLab.swift:2965 (HIP events on the context's stream). */
int smelt_hip_last_gpu_ns(smelt_hip_context *ctx, uint64_t *out_ns);

/* benchmarkDecodeDispatch: SmeltRuntime.swift:3531-3608 — replays one record `iters` times
 * after `warmup` untimed launches and writes the per-launch GPU time in microseconds
 * (one HIP event pair per launch) to out_us[iters].  prefill != 0 resolves the record with
 * (a = seq_len, b = start_pos), otherwise with a = position. */
int smelt_hip_benchmark_record(smelt_hip_context *ctx, const SmeltDispatchRecord *rec, int cur,
                               int alt, int prefill, int32_t a, int32_t b, int warmup, int iters,
                               float *out_us);

/* Launch-bound tables (about a thousand records per token, SmeltRuntime.swift:3251-3275) are
 * captured once into a HIP graph and replayed; the analogue of the reference's indirect
 * command buffer replay.  A graph holds what the capture resolved: device addresses of the
 * slots (cur / alt included), byte offsets and constants derived from `position` (decode) or
 * `seq_len` / `start_pos` (prefill), grids derived from seq_len.  It therefore stays valid only
 * while no slot it binds is re-allocated or re-uploaded, and replays the position it was
 * captured with: a table whose records carry position-dependent offsets or constants needs one
 * capture per position (a table of matvec / qmm records carries none).  Destroy a graph before
 * freeing the slots it names. */
int smelt_hip_graph_capture_decode(smelt_hip_context *ctx, const SmeltDispatchRecord *table,
                                   size_t count, int cur0, int alt0, int32_t position,
                                   smelt_hip_graph **out);
int smelt_hip_graph_capture_prefill(smelt_hip_context *ctx, const SmeltDispatchRecord *table,
                                    size_t count, int cur0, int alt0, int32_t seq_len,
                                    int32_t start_pos, smelt_hip_graph **out);
int smelt_hip_graph_launch(smelt_hip_context *ctx, smelt_hip_graph *graph);
void smelt_hip_graph_destroy(smelt_hip_context *ctx, smelt_hip_graph *graph);

/* Timing helper for benchmarks: GPU time of `iters` back-to-back replays of a graph (or of a
 * table interpreted eagerly when graph is NULL is not supported), bracketed by one event pair. */
int smelt_hip_graph_time(smelt_hip_context *ctx, smelt_hip_graph *graph, int iters,
                         float *out_total_us);

/* Device facts for reports: name, compute units, LDS per workgroup, HBM bytes. */
int smelt_hip_device_info(smelt_hip_context *ctx, char *name, size_t name_cap, int *compute_units,
                          size_t *lds_per_block, size_t *hbm_bytes);

/* Free and total device memory as the runtime reports them (hipMemGetInfo).  No counterpart in the reference;
 * for callers and tests that must see that an entry point allocated nothing. */
int smelt_hip_memory_info(smelt_hip_context *ctx, size_t *free_bytes, size_t *total_bytes);

#ifdef __cplusplus
}
#endif
#endif /* SMELT_HIP_H */
