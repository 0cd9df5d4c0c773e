// GPU weight-import producers behind include/smelt_hip_import.h.  Built entirely on the runtime's
// own C ABI: an importer is a private context whose slots stage the host buffers, and each call
// is one dispatch record of an import pipeline.
#include "../../include/smelt_hip_import.h"

#include <string.h>

#include <algorithm>
#include <map>
#include <string>

#include "../../include/smelt_hip.h"

struct smelt_hip_importer {
    smelt_hip_context* ctx = nullptr;
    int compute_units = 256;
    std::map<std::string, uint32_t> pipelines;  // entry -> index in the private context
    std::string error;
};

namespace {

thread_local std::string g_error;

// staging slots of the private context
enum { kSrc = 0, kPacked = 1, kScales = 2, kBiases = 3, kImportance = 4, kStatus = 5, kOut = 6 };

int fail(smelt_hip_importer* imp, int code, const std::string& msg) {
    if (imp) imp->error = msg;
    else g_error = msg;
    return code;
}

int pass(smelt_hip_importer* imp, int rc) {
    if (rc != SMELT_HIP_OK) imp->error = smelt_hip_last_error(imp->ctx);
    return rc;
}

#define IMP_TRY(call)                               \
    do {                                            \
        int _rc = pass(imp, (call));                \
        if (_rc != SMELT_HIP_OK) return _rc;        \
    } while (0)

int stage(smelt_hip_importer* imp, int slot, const void* src, size_t bytes) {
    IMP_TRY(smelt_hip_buffer_alloc(imp->ctx, slot, bytes));
    if (src) IMP_TRY(smelt_hip_buffer_write(imp->ctx, slot, 0, src, bytes));
    return SMELT_HIP_OK;
}

void bind(SmeltDispatchRecord& r, int slot, int index) {
    SmeltBufferRecord& b = r.buffers[r.buffer_count++];
    b.slot = (int16_t)slot;
    b.binding_index = (uint8_t)index;
    b.offset_kind = 0;
    b.offset = 0;
}

void constant(SmeltDispatchRecord& r, int index, uint32_t value) {
    SmeltConstantRecord& c = r.constants[r.constant_count++];
    c.kind = 0;
    c.binding_index = (uint8_t)index;
    c.value = value;
}

int run(smelt_hip_importer* imp, const std::string& entry, SmeltDispatchRecord& r, uint32_t grid, uint32_t threads) {
    uint32_t index = 0;
    auto known = imp->pipelines.find(entry);
    if (known != imp->pipelines.end()) {
        index = known->second;
    } else {
        IMP_TRY(smelt_hip_pipeline_create(imp->ctx, entry.c_str(), 0, &index));
        imp->pipelines[entry] = index;
    }
    r.op_kind = 0;
    r.pipeline = (uint16_t)index;
    r.style = 0;
    r.grid_w = grid; r.grid_h = 1; r.grid_d = 1;
    r.tg_w = threads; r.tg_h = 1; r.tg_d = 1;
    const int rc = smelt_hip_encode_decode_record(imp->ctx, &r, 0, 0, 0);
    if (rc < 0) return pass(imp, rc);
    IMP_TRY(smelt_hip_wait(imp->ctx));
    return SMELT_HIP_OK;
}

}  // namespace

extern "C" {

int smelt_hip_importer_create(int device_index, const char* code_object_path, smelt_hip_importer** out) {
    if (!out || !code_object_path) return fail(nullptr, SMELT_HIP_ERR_INVALID_ARGUMENT, "null argument");
    smelt_hip_importer* imp = new smelt_hip_importer();
    int rc = smelt_hip_context_create(device_index, &imp->ctx);
    if (rc != SMELT_HIP_OK) {
        g_error = smelt_hip_last_error(nullptr);
        delete imp;
        return rc;
    }
    rc = smelt_hip_module_load_file(imp->ctx, code_object_path);
    if (rc == SMELT_HIP_OK) {
        char name[64];
        size_t lds = 0, hbm = 0;
        rc = smelt_hip_device_info(imp->ctx, name, sizeof(name), &imp->compute_units, &lds, &hbm);
    }
    if (rc != SMELT_HIP_OK) {
        g_error = smelt_hip_last_error(imp->ctx);
        smelt_hip_context_destroy(imp->ctx);
        delete imp;
        return rc;
    }
    *out = imp;
    return SMELT_HIP_OK;
}

void smelt_hip_importer_destroy(smelt_hip_importer* imp) {
    if (!imp) return;
    smelt_hip_context_destroy(imp->ctx);
    delete imp;
}

const char* smelt_hip_importer_last_error(const smelt_hip_importer* imp) {
    return imp ? imp->error.c_str() : g_error.c_str();
}

int smelt_hip_import_quantize_affine_u4(smelt_hip_importer* imp, const void* src, int src_dtype, int rows,
                                        int cols, int group, int clip, const float* importance,
                                        int scale_dtype, uint8_t* packed, uint16_t* scales, uint16_t* biases) {
    if (!imp || !src || !packed || !scales || !biases) return fail(imp, SMELT_HIP_ERR_INVALID_ARGUMENT, "null argument");
    if (rows <= 0 || cols <= 0) return fail(imp, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "rows and cols must be positive");
    if (src_dtype < 0 || src_dtype > 2) return fail(imp, SMELT_HIP_ERR_INVALID_ARGUMENT, "unsupported source dtype");
    if (scale_dtype != SMELT_HIP_ACT_F16 && scale_dtype != SMELT_HIP_ACT_BF16) return fail(imp, SMELT_HIP_ERR_INVALID_ARGUMENT, "scale dtype must be fp16 or bf16");
    if (group != 32 && group != 64 && group != 128) return fail(imp, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "group must be 32, 64 or 128");
    const size_t n = (size_t)rows * (size_t)cols;
    const size_t gpr = ((size_t)cols + (size_t)group - 1) / (size_t)group;
    const size_t cells = (size_t)rows * gpr;
    const size_t packed_bytes = (size_t)rows * (((size_t)cols + 1) / 2);
    if (int rc = stage(imp, kSrc, src, n * (src_dtype == SMELT_IMPORT_SRC_F32 ? 4 : 2))) return rc;
    if (int rc = stage(imp, kPacked, nullptr, packed_bytes)) return rc;
    if (int rc = stage(imp, kScales, nullptr, cells * 2)) return rc;
    if (int rc = stage(imp, kBiases, nullptr, cells * 2)) return rc;
    if (importance)
        if (int rc = stage(imp, kImportance, importance, (size_t)cols * 4)) return rc;
    SmeltDispatchRecord r;
    memset(&r, 0, sizeof(r));
    bind(r, kSrc, 0); bind(r, kPacked, 1); bind(r, kScales, 2); bind(r, kBiases, 3);
    if (importance) bind(r, kImportance, 4);
    constant(r, 5, (uint32_t)rows);
    constant(r, 6, (uint32_t)src_dtype);
    constant(r, 7, (uint32_t)clip);
    const uint32_t threads = (uint32_t)(128 / group) * 64;
    const size_t per_block = threads;  // cells one workgroup covers per round
    const uint32_t grid = (uint32_t)std::max<size_t>(1, std::min<size_t>((cells + per_block - 1) / per_block, (size_t)imp->compute_units * 16));
    const std::string entry = std::string(importance ? "affine_quantize_u4_weighted:" : "affine_quantize_u4:") +
                              std::to_string(cols) + ":" + std::to_string(group) +
                              (scale_dtype == SMELT_HIP_ACT_BF16 ? "@bf16" : "@f16");
    if (int rc = run(imp, entry, r, grid, threads)) return rc;
    IMP_TRY(smelt_hip_buffer_read(imp->ctx, kPacked, 0, packed, packed_bytes));
    IMP_TRY(smelt_hip_buffer_read(imp->ctx, kScales, 0, scales, cells * 2));
    IMP_TRY(smelt_hip_buffer_read(imp->ctx, kBiases, 0, biases, cells * 2));
    return SMELT_HIP_OK;
}

int smelt_hip_import_validate_signed_codes(smelt_hip_importer* imp, const uint8_t* bytes, size_t byte_count,
                                           uint64_t logical_count, int format, int64_t* bad_index) {
    if (!imp || (!bytes && byte_count)) return fail(imp, SMELT_HIP_ERR_INVALID_ARGUMENT, "null argument");
    if (format < SMELT_IMPORT_FORMAT_BINARY1 || format > SMELT_IMPORT_FORMAT_TRIT5) return fail(imp, SMELT_HIP_ERR_INVALID_ARGUMENT, "unknown signed format");
    const uint64_t need = format == SMELT_IMPORT_FORMAT_TRIT5 ? (logical_count + 4) / 5
                        : format == SMELT_IMPORT_FORMAT_BINARY1 ? (logical_count + 7) / 8
                                                                : (logical_count * 2 + 7) / 8;
    if (byte_count < need)
        return fail(imp, SMELT_IMPORT_ERR_BUFFER_TOO_SMALL, "signed-quant codes buffer needs " + std::to_string(need) + " bytes, got " + std::to_string(byte_count));
    if (format == SMELT_IMPORT_FORMAT_BINARY1 || logical_count == 0) return SMELT_HIP_OK;  // every bit pattern is a code
    if (int rc = stage(imp, kSrc, bytes, (size_t)need)) return rc;
    const uint64_t ones = ~0ull;
    if (int rc = stage(imp, kStatus, &ones, 8)) return rc;
    SmeltDispatchRecord r;
    memset(&r, 0, sizeof(r));
    bind(r, kSrc, 0); bind(r, kStatus, 1);
    constant(r, 2, (uint32_t)(logical_count & 0xFFFFFFFFu));
    constant(r, 3, (uint32_t)(logical_count >> 32));
    constant(r, 4, (uint32_t)format);
    const size_t units = ((size_t)need + 15) / 16;
    const uint32_t grid = (uint32_t)std::max<size_t>(1, std::min<size_t>((units + 255) / 256, (size_t)imp->compute_units * 8));
    if (int rc = run(imp, "signed_validate_codes", r, grid, 256)) return rc;
    uint64_t status = 0;
    IMP_TRY(smelt_hip_buffer_read(imp->ctx, kStatus, 0, &status, 8));
    if (status == ones) return SMELT_HIP_OK;
    if (bad_index) *bad_index = (int64_t)status;
    return fail(imp, SMELT_IMPORT_ERR_INVALID_CODE, "invalid code at logical index " + std::to_string(status));
}

int smelt_hip_import_normalize_mlx_scales(smelt_hip_importer* imp, int format, const uint16_t* scales,
                                          const uint16_t* biases, size_t group_count, uint16_t* out, int64_t* bad_group) {
    if (!imp || ((!scales || !biases || !out) && group_count)) return fail(imp, SMELT_HIP_ERR_INVALID_ARGUMENT, "null argument");
    if (format != SMELT_IMPORT_FORMAT_BINARY1 && format != SMELT_IMPORT_FORMAT_TERNARY2) return fail(imp, SMELT_HIP_ERR_INVALID_ARGUMENT, "MLX scale pairs exist for binary1 and ternary2");
    if (group_count == 0) return SMELT_HIP_OK;
    if (group_count >= ((size_t)1 << 31)) return fail(imp, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "more than 2^31 groups");
    if (int rc = stage(imp, kScales, scales, group_count * 2)) return rc;
    if (int rc = stage(imp, kBiases, biases, group_count * 2)) return rc;
    if (int rc = stage(imp, kOut, nullptr, group_count * 2)) return rc;
    const uint64_t ones = ~0ull;
    if (int rc = stage(imp, kStatus, &ones, 8)) return rc;
    SmeltDispatchRecord r;
    memset(&r, 0, sizeof(r));
    bind(r, kScales, 0); bind(r, kBiases, 1); bind(r, kOut, 2); bind(r, kStatus, 3);
    constant(r, 4, (uint32_t)group_count);
    constant(r, 5, (uint32_t)format);
    const uint32_t grid = (uint32_t)std::max<size_t>(1, std::min<size_t>((group_count + 255) / 256, (size_t)imp->compute_units * 8));
    if (int rc = run(imp, "signed_normalize_mlx_scales", r, grid, 256)) return rc;
    uint64_t status = 0;
    IMP_TRY(smelt_hip_buffer_read(imp->ctx, kStatus, 0, &status, 8));
    if (status != ones) {
        if (bad_group) *bad_group = (int64_t)(status >> 8);
        const bool scale = (status & 0xFF) == 1;
        return fail(imp, scale ? SMELT_IMPORT_ERR_MLX_SCALE : SMELT_IMPORT_ERR_MLX_BIAS,
                    std::string(scale ? "invalid MLX scale" : "invalid MLX bias") + " at group " + std::to_string(status >> 8));
    }
    IMP_TRY(smelt_hip_buffer_read(imp->ctx, kOut, 0, out, group_count * 2));
    return SMELT_HIP_OK;
}

}  // extern "C"
