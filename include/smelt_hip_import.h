/*
 * smelt_hip_import.h — C ABI of the GPU weight-import producers: the build-time functions of
 * SmeltCompiler that turn checkpoint tensors into the packed layouts the matvec kernels read.
 *
 * The reference runs these on the CPU while it builds a package; each entry point below cites the
 * function it stands in for and returns bit-identical bytes.  Buffers are host memory (the
 * reference works on the mmap of the checkpoint and of weights.bin); the importer stages them
 * through device memory it owns.  Device-resident callers use the same kernels through the
 * pipelines "affine_quantize_u4[_weighted]:cols:group", "signed_validate_codes" and
 * "signed_normalize_mlx_scales" of smelt_hip.h.
 *
 * Conventions as in smelt_hip.h: opaque handle, int status (0 = ok, negative = error), error
 * string per handle.  One importer is used from one thread at a time.
 */
#ifndef SMELT_HIP_IMPORT_H
#define SMELT_HIP_IMPORT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct smelt_hip_importer smelt_hip_importer;

/* Source element types of SmeltAffineQuantizer.quantizeTensorAffine ("F32", "F16", "BF16";
 * SmeltAffineQuantizer.swift:417-431). */
enum { SMELT_IMPORT_SRC_F32 = 0, SMELT_IMPORT_SRC_F16 = 1, SMELT_IMPORT_SRC_BF16 = 2 };
/* SmeltAffineU4.ClipMode (SmeltAffineU4.swift:47-55). */
enum { SMELT_IMPORT_CLIP_MIN_MAX = 0, SMELT_IMPORT_CLIP_MSE_OPTIMAL = 1 };
/* SmeltSignedQuantFormat plus this backend's five-trits-per-byte format. */
enum { SMELT_IMPORT_FORMAT_BINARY1 = 0, SMELT_IMPORT_FORMAT_TERNARY2 = 1, SMELT_IMPORT_FORMAT_TRIT5 = 2 };

/* Status values beyond SMELT_HIP_ERR_* (smelt_hip.h), mirroring SmeltSignedQuantError
 * (Sources/SmeltRuntime/SmeltSignedQuantCodec.swift:38-49). */
enum {
    SMELT_IMPORT_ERR_INVALID_CODE = -20, /* .invalidCode: ternary code 3 / trit5 byte > 242 */
    SMELT_IMPORT_ERR_MLX_SCALE = -21,    /* .invalidMLXScale: scale not finite or negative */
    SMELT_IMPORT_ERR_MLX_BIAS = -22,     /* .invalidMLXBias: bias is not the negated canonical scale */
    SMELT_IMPORT_ERR_BUFFER_TOO_SMALL = -23 /* .bufferTooSmall */
};

/* Creates an importer on one GPU with the kernels under `code_object_path` (the directory that
 * holds the build's smelt_kernels*.hsaco files, or one code object). */
int smelt_hip_importer_create(int device_index, const char *code_object_path, smelt_hip_importer **out);
void smelt_hip_importer_destroy(smelt_hip_importer *imp);
const char *smelt_hip_importer_last_error(const smelt_hip_importer *imp);

/* SmeltAffineQuantizer.quantizeTensorAffine (SmeltAffineQuantizer.swift:399-513) over
 * SmeltAffineU4.quantizeRow (SmeltAffineU4.swift:94-136): group-wise affine 4-bit quantisation of
 * a row-major [rows, cols] tensor.  Writes rows * ceil(cols / 2) packed bytes (low nibble = even
 * column) and rows * ceil(cols / group) scale and bias bit patterns of `scale_dtype`
 * (SMELT_HIP_ACT_F16, the reference's, or SMELT_HIP_ACT_BF16).  `importance` (cols floats, may be
 * NULL) weights the endpoint search of SMELT_IMPORT_CLIP_MSE_OPTIMAL.  group is 32, 64 or 128. */
int smelt_hip_import_quantize_affine_u4(smelt_hip_importer *imp, const void *src, int src_dtype,
                                        int rows, int cols, int group, int clip,
                                        const float *importance, int scale_dtype, uint8_t *packed,
                                        uint16_t *scales, uint16_t *biases);

/* SmeltSignedQuantCodec.validateCodes (SmeltSignedQuantCodec.swift:128-145): byte_count must cover
 * logical_count codes; a ternary code 3 (or trit5 byte above 242) fails with
 * SMELT_IMPORT_ERR_INVALID_CODE and *bad_index (may be NULL) = index of the first offending code. */
int smelt_hip_import_validate_signed_codes(smelt_hip_importer *imp, const uint8_t *bytes,
                                           size_t byte_count, uint64_t logical_count, int format,
                                           int64_t *bad_index);

/* SmeltSignedQuantCodec.normalizeMLXScales (SmeltSignedQuantCodec.swift:154-215): MLX (scale,
 * bias) fp16 pairs -> canonical signed fp16 scale bits.  Fails with SMELT_IMPORT_ERR_MLX_SCALE /
 * _MLX_BIAS for the first group that is not a signed group, *bad_group (may be NULL) = its index;
 * `out` is then unspecified. */
int smelt_hip_import_normalize_mlx_scales(smelt_hip_importer *imp, int format, const uint16_t *scales,
                                          const uint16_t *biases, size_t group_count, uint16_t *out,
                                          int64_t *bad_group);

#ifdef __cplusplus
}
#endif
#endif /* SMELT_HIP_IMPORT_H */
