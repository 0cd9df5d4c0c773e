// Build-time half of the HIP backend: dtype -> kernel family gateway, weights.bin layout,
// shape routing and dispatch-record emitters.  Mirrors the cited parts of SmeltCompiler; the
// launch geometry is this backend's own (256-thread workgroups, grid-stride rows).
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/smelt_hip_compiler.h"
#include "pipeline_table.hpp"

using namespace smelt_host;

namespace {

const char* kDTypeNames[SMELT_DTYPE_COUNT] = {"fp16", "fp32", "bf16", "int32", "u4_lut", "affine_u4",
                                              "binary1", "ternary2", "turbo_quant_h", "raw", "trit5"};

uint64_t align_to(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

bool cell_eq(const SmeltMatvecCell& a, const SmeltMatvecCell& b) {
    return a.activation == b.activation && a.weight == b.weight && a.shape == b.shape &&
           a.fusion == b.fusion && a.output == b.output && a.slot == b.slot;
}

// MatvecKernelTable.meaningfulCells (MatvecKernelTable.swift:155-237), plus the trit5 cells this
// backend adds beside ternary2.
const std::vector<SmeltMatvecCell>& meaningful_cells() {
    static const std::vector<SmeltMatvecCell> cells = [] {
        std::vector<SmeltMatvecCell> c;
        auto add = [&](int act, int w, int shape, int fusion, int out, int slot) {
            SmeltMatvecCell cell{act, w, shape, fusion, out, slot};
            for (const auto& e : c)
                if (cell_eq(e, cell)) return;
            c.push_back(cell);
        };
        const int gemv_weights[] = {SMELT_DTYPE_FP16, SMELT_DTYPE_BF16, SMELT_DTYPE_FP32, SMELT_DTYPE_AFFINE_U4,
                                    SMELT_DTYPE_BINARY1, SMELT_DTYPE_TERNARY2, SMELT_DTYPE_U4_LUT, SMELT_DTYPE_TRIT5};
        for (int slot : {SMELT_SLOT_FIXED, SMELT_SLOT_VARIABLE})
            for (int w : gemv_weights) add(SMELT_ACT_FP16, w, SMELT_SHAPE_GEMV, SMELT_FUSION_NONE, SMELT_OUT_FP16, slot);
        add(SMELT_ACT_FP16, SMELT_DTYPE_TURBO_QUANT_H, SMELT_SHAPE_GEMV, SMELT_FUSION_NONE, SMELT_OUT_FP16, SMELT_SLOT_FIXED);
        const int gemm_weights[] = {SMELT_DTYPE_FP16, SMELT_DTYPE_BF16, SMELT_DTYPE_FP32, SMELT_DTYPE_AFFINE_U4,
                                    SMELT_DTYPE_BINARY1, SMELT_DTYPE_TERNARY2, SMELT_DTYPE_U4_LUT,
                                    SMELT_DTYPE_TURBO_QUANT_H, SMELT_DTYPE_TRIT5};
        for (int w : gemm_weights) add(SMELT_ACT_FP16, w, SMELT_SHAPE_GEMM, SMELT_FUSION_NONE, SMELT_OUT_FP16, SMELT_SLOT_FIXED);
        for (int w : {SMELT_DTYPE_U4_LUT, SMELT_DTYPE_AFFINE_U4})
            add(SMELT_ACT_FP16, w, SMELT_SHAPE_GEMV, SMELT_FUSION_DUAL_MATVEC, SMELT_OUT_FP16, SMELT_SLOT_FIXED);
        for (int w : {SMELT_DTYPE_U4_LUT, SMELT_DTYPE_AFFINE_U4, SMELT_DTYPE_BINARY1, SMELT_DTYPE_TERNARY2, SMELT_DTYPE_TRIT5})
            add(SMELT_ACT_FP16, w, SMELT_SHAPE_GEMV, SMELT_FUSION_GATE_UP_SWIGLU, SMELT_OUT_FP16, SMELT_SLOT_FIXED);
        add(SMELT_ACT_FP16, SMELT_DTYPE_AFFINE_U4, SMELT_SHAPE_GEMV, SMELT_FUSION_GATE_UP_GEGLU, SMELT_OUT_FP16, SMELT_SLOT_FIXED);
        add(SMELT_ACT_FP16, SMELT_DTYPE_AFFINE_U4, SMELT_SHAPE_GEMM, SMELT_FUSION_GATE_UP_SWIGLU, SMELT_OUT_FP16, SMELT_SLOT_FIXED);
        add(SMELT_ACT_FP16, SMELT_DTYPE_BINARY1, SMELT_SHAPE_GEMM, SMELT_FUSION_GATE_UP_SWIGLU, SMELT_OUT_FP16, SMELT_SLOT_FIXED);
        add(SMELT_ACT_FP16, SMELT_DTYPE_AFFINE_U4, SMELT_SHAPE_GEMM, SMELT_FUSION_GATE_UP_GEGLU, SMELT_OUT_FP16, SMELT_SLOT_FIXED);
        add(SMELT_ACT_FP16, SMELT_DTYPE_AFFINE_U4, SMELT_SHAPE_GEMM, SMELT_FUSION_DUAL_MATVEC, SMELT_OUT_FP16, SMELT_SLOT_FIXED);
        for (int shape : {SMELT_SHAPE_GEMV, SMELT_SHAPE_GEMM, SMELT_SHAPE_GEMM_TN})
            for (int w : {SMELT_DTYPE_FP32, SMELT_DTYPE_FP16, SMELT_DTYPE_BF16})
                add(SMELT_ACT_FP32, w, shape, SMELT_FUSION_NONE, SMELT_OUT_FP32, SMELT_SLOT_FIXED);
        for (int shape : {SMELT_SHAPE_GEMV, SMELT_SHAPE_GEMM})
            add(SMELT_ACT_FP32, SMELT_DTYPE_AFFINE_U4, shape, SMELT_FUSION_NONE, SMELT_OUT_FP32, SMELT_SLOT_FIXED);
        for (int shape : {SMELT_SHAPE_GEMV, SMELT_SHAPE_GEMM})
            add(SMELT_ACT_BF16, SMELT_DTYPE_BF16, shape, SMELT_FUSION_NONE, SMELT_OUT_BF16, SMELT_SLOT_FIXED);
        // The reference registers quantized weights for fp16 activations only; this backend also
        // carries every quantized family with bf16 activations and outputs.
        for (int w : {SMELT_DTYPE_AFFINE_U4, SMELT_DTYPE_BINARY1, SMELT_DTYPE_TERNARY2, SMELT_DTYPE_TRIT5}) {
            for (int shape : {SMELT_SHAPE_GEMV, SMELT_SHAPE_GEMM})
                add(SMELT_ACT_BF16, w, shape, SMELT_FUSION_NONE, SMELT_OUT_BF16, SMELT_SLOT_FIXED);
            add(SMELT_ACT_BF16, w, SMELT_SHAPE_GEMV, SMELT_FUSION_GATE_UP_SWIGLU, SMELT_OUT_BF16, SMELT_SLOT_FIXED);
        }
        add(SMELT_ACT_BF16, SMELT_DTYPE_AFFINE_U4, SMELT_SHAPE_GEMV, SMELT_FUSION_GATE_UP_GEGLU, SMELT_OUT_BF16, SMELT_SLOT_FIXED);
        return c;
    }();
    return cells;
}

// family(for:) — exhaustive, no default (MatvecKernelTable.swift:272-284)
bool family_for(int weight, int* family) {
    switch (weight) {
        case SMELT_DTYPE_FP16: case SMELT_DTYPE_BF16: case SMELT_DTYPE_FP32: *family = SMELT_FAMILY_DENSE + weight; return true;
        case SMELT_DTYPE_AFFINE_U4: *family = SMELT_FAMILY_AFFINE_U4; return true;
        case SMELT_DTYPE_BINARY1: *family = SMELT_FAMILY_BINARY1; return true;
        case SMELT_DTYPE_TERNARY2: *family = SMELT_FAMILY_TERNARY2; return true;
        case SMELT_DTYPE_U4_LUT: *family = SMELT_FAMILY_LUT_U4; return true;
        case SMELT_DTYPE_TURBO_QUANT_H: *family = SMELT_FAMILY_TQH; return true;
        case SMELT_DTYPE_TRIT5: *family = SMELT_FAMILY_TRIT5; return true;
        case SMELT_DTYPE_INT32: case SMELT_DTYPE_RAW: return false;
        default: return false;
    }
}

bool hip_has_kernel(const SmeltMatvecCell& c, int family) {
    const bool quant = family == SMELT_FAMILY_AFFINE_U4 || family == SMELT_FAMILY_BINARY1 ||
                       family == SMELT_FAMILY_TERNARY2 || family == SMELT_FAMILY_TRIT5;
    // u4_lut: single-token matvec, dual and gate+up+SwiGLU kernels; prompt rows run the per-token matmul
    if (family == SMELT_FAMILY_LUT_U4)
        return c.activation != SMELT_ACT_FP32 && c.fusion != SMELT_FUSION_GATE_UP_GEGLU &&
               (c.shape == SMELT_SHAPE_GEMV || (c.shape == SMELT_SHAPE_GEMM && c.fusion == SMELT_FUSION_NONE));
    // turbo_quant_h: prepare + matvec pair (the batched names cover prefill rows), no fused forms
    if (family == SMELT_FAMILY_TQH) return c.activation != SMELT_ACT_FP32 && c.fusion == SMELT_FUSION_NONE;
    if (!quant) return false;
    if (c.activation == SMELT_ACT_FP32) return false;
    // GeGLU: affine only (single-token kernel and the MFMA slab kernel)
    if (c.fusion == SMELT_FUSION_GATE_UP_GEGLU) return family == SMELT_FAMILY_AFFINE_U4;
    // prompt rows of the dual matvec: the per-token "_batched" form and the token tiles of "_batched_verify_b4"
    if (c.shape == SMELT_SHAPE_GEMM && c.fusion == SMELT_FUSION_DUAL_MATVEC) return family == SMELT_FAMILY_AFFINE_U4;
    if (c.shape == SMELT_SHAPE_GEMM && c.fusion == SMELT_FUSION_GATE_UP_SWIGLU && family == SMELT_FAMILY_TERNARY2) return false;
    return true;
}

// Shapes that get a fixed-shape pipeline name (the tuned-route half of
// SmeltKernelShapeRegistry.decodeAffineDecodePipeline); every other shape takes the generic
// function-constant entry "name:cols:group".
bool is_specialized_shape(int rows, int cols, int group) {
    if (group != 64) return false;
    static const int k[][2] = {
        {2048, 1024}, {3584, 1024}, {4096, 1024}, {512, 1024}, {6144, 1024}, {1024, 1024}, {1024, 2048},
        {1024, 3584}, {151936, 1024}, {248320, 1024}, {2048, 2048}, {6144, 2048}, {4096, 2048},
        {512, 2048}, {2048, 6144}, {151936, 2048}, {248320, 2048}, {8192, 2560}, {9216, 2560},
        {4096, 2560}, {1024, 2560}, {2560, 4096}, {2560, 9216}, {248320, 2560}, {3072, 3072},
        {1024, 3072}, {8192, 3072}, {3072, 8192}};
    for (const auto& s : k)
        if (s[0] == rows && s[1] == cols) return true;
    return false;
}

struct MatvecGeometry {
    int rows_per_group;
    int grid_w;
};

// Rows one 256-thread workgroup walks per step and the workgroup count: four waves, each owning
// R rows per 64/L row groups (L = lanes a row's 16-byte units occupy), capped at 4 workgroups
// per compute unit (rows beyond that are covered by the kernels' grid-stride loop).  A matrix too
// small to give every compute unit two such workgroups is launched one row per wave slot instead:
// the kernels switch to single-row work items when the grid holds more waves than R-row tiles.
MatvecGeometry matvec_geometry(uint32_t row_stride, int rows, int rows_per_wave, int compute_units) {
    const int U = (int)(row_stride / 16);
    const int L = U > 32 ? 64 : (U > 16 ? 32 : 16);
    const int cus = std::max(1, compute_units);
    int tile = (64 / L) * rows_per_wave;
    if ((rows + tile * 4 - 1) / (tile * 4) < 2 * cus) tile = 64 / L;
    MatvecGeometry g;
    g.rows_per_group = tile * 4;
    const int want = (rows + g.rows_per_group - 1) / g.rows_per_group;
    g.grid_w = std::max(1, std::min(want, cus * 4));
    return g;
}

void set_route(SmeltRoute* r, const std::string& name, bool specialized, int rpg, int bt, int threads, int grid_w) {
    memset(r, 0, sizeof(*r));
    snprintf(r->pipeline, sizeof(r->pipeline), "%s", name.c_str());
    r->specialized = specialized;
    r->rows_per_group = rpg;
    r->batch_tile = bt;
    r->threads = threads;
    r->grid_w = grid_w;
}

std::string shape_tag(int rows, int cols, int group) {
    return "_c" + std::to_string(cols) + "_r" + std::to_string(rows) + "_g" + std::to_string(group);
}

}  // namespace

struct smelt_emitter {
    int act = SMELT_HIP_ACT_F16;
    int compute_units = 256;
    std::vector<SmeltDispatchRecord> records;
    std::vector<std::string> pipelines;
    size_t argmax_partial_bytes = 0;
    std::string error;

    std::string tagged(const std::string& name) const { return act == SMELT_HIP_ACT_BF16 ? name + "@bf16" : name; }

    uint16_t pipeline_index(const std::string& name) {
        const std::string n = tagged(name);
        for (size_t i = 0; i < pipelines.size(); ++i)
            if (pipelines[i] == n) return (uint16_t)i;
        pipelines.push_back(n);
        return (uint16_t)(pipelines.size() - 1);
    }
};

namespace {

int efail(smelt_emitter* e, int code, const std::string& msg) {
    if (e) e->error = msg;
    return code;
}

struct RecordBuilder {
    SmeltDispatchRecord r;
    RecordBuilder() { memset(&r, 0, sizeof(r)); }
    void buffer(uint8_t index, int slot, uint64_t offset, uint8_t kind = 0) {
        SmeltBufferRecord& b = r.buffers[r.buffer_count++];
        b.slot = (int16_t)slot;
        b.binding_index = index;
        b.offset_kind = kind;
        b.offset = offset;
    }
    void buffer(uint8_t index, const SmeltBinding& bind) { buffer(index, bind.slot, bind.offset, bind.offset_kind); }
    void constant(uint8_t index, uint32_t value, uint8_t kind = SMELT_CONST_LITERAL_U32) {
        SmeltConstantRecord& c = r.constants[r.constant_count++];
        c.kind = kind;
        c.binding_index = index;
        c.value = value;
    }
    void constant_f32(uint8_t index, float v) {
        uint32_t bits;
        memcpy(&bits, &v, 4);
        constant(index, bits, SMELT_CONST_LITERAL_F32);
    }
    void grid(uint32_t w, uint32_t h, uint32_t d, uint32_t tg) {
        r.grid_w = w; r.grid_h = h; r.grid_d = d;
        r.tg_w = tg; r.tg_h = 1; r.tg_d = 1;
    }
    void grid_h_kind(uint8_t kind) { r.style = (uint8_t)((r.style & ~(3u << 4)) | ((kind & 3u) << 4)); }
};

bool affine_entry_ok(const SmeltWeightEntryC* w) {
    return w && w->dtype == SMELT_DTYPE_AFFINE_U4 && w->rows > 0 && w->cols > 0 && w->group_size >= 32 &&
           (w->group_size & (w->group_size - 1)) == 0 && w->cols % 32 == 0 && w->scales_size_bytes && w->biases_size_bytes;
}

bool signed_dtype(int d) { return d == SMELT_DTYPE_BINARY1 || d == SMELT_DTYPE_TERNARY2 || d == SMELT_DTYPE_TRIT5; }

SignedFormat to_format(int d) {
    return d == SMELT_DTYPE_BINARY1 ? kFmtBinary1 : (d == SMELT_DTYPE_TERNARY2 ? kFmtTernary2 : kFmtTrit5);
}

const char* signed_stem(int d) {
    return d == SMELT_DTYPE_BINARY1 ? "binary" : (d == SMELT_DTYPE_TERNARY2 ? "ternary" : "trit5");
}

// emitSignedMatvec's geometry guard (SmeltCodeEmitter.swift:1105-1115)
int check_signed_entry(smelt_emitter* e, const SmeltWeightEntryC* w) {
    if (!w || !signed_dtype(w->dtype)) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "signed matvec received a non-signed weight");
    if (!w->scales_size_bytes || w->group_size != 128 || w->padded_cols != w->cols || w->cols % 128 != 0 || w->rows <= 0)
        return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "signed matvec requires exact rank-2 g128 geometry");
    return 0;
}

int gateway(smelt_emitter* e, const SmeltWeightEntryC* w, int shape, int fusion, int* family) {
    SmeltMatvecCell cell{e->act == SMELT_HIP_ACT_BF16 ? SMELT_ACT_BF16 : SMELT_ACT_FP16, w ? w->dtype : -1, shape, fusion,
                         e->act == SMELT_HIP_ACT_BF16 ? SMELT_OUT_BF16 : SMELT_OUT_FP16, SMELT_SLOT_FIXED};
    const int rc = smelt_kernel_table_select(&cell, 1, family);
    if (rc == SMELT_SELECT_MISSING) return efail(e, rc, std::string("MatvecKernelTable: no registered HIP kernel for ") + (smelt_dtype_name(cell.weight) ? smelt_dtype_name(cell.weight) : "?") + " weights in this cell");
    if (rc == SMELT_SELECT_NOT_MEANINGFUL) return efail(e, rc, "MatvecKernelTable: not a meaningful matvec cell");
    return rc;
}

}  // namespace

extern "C" {

const char* smelt_dtype_name(int dtype) {
    return dtype >= 0 && dtype < SMELT_DTYPE_COUNT ? kDTypeNames[dtype] : nullptr;
}

int smelt_dtype_from_name(const char* name) {
    if (!name) return -1;
    for (int i = 0; i < SMELT_DTYPE_COUNT; ++i)
        if (strcmp(name, kDTypeNames[i]) == 0) return i;
    return -1;
}

int smelt_kernel_table_select(const SmeltMatvecCell* cell, int hip_backend, int* out_family) {
    if (!cell || !out_family) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    bool found = false;
    for (const auto& c : meaningful_cells())
        if (cell_eq(c, *cell)) { found = true; break; }
    if (!found) return SMELT_SELECT_NOT_MEANINGFUL;
    int family = 0;
    if (!family_for(cell->weight, &family)) return SMELT_SELECT_NOT_MEANINGFUL;
    *out_family = family;
    if (hip_backend && !hip_has_kernel(*cell, family)) return SMELT_SELECT_MISSING;
    return SMELT_SELECT_OK;
}

int smelt_kernel_table_meaningful_cells(SmeltMatvecCell* out, int cap) {
    const auto& cells = meaningful_cells();
    for (int i = 0; out && i < cap && i < (int)cells.size(); ++i) out[i] = cells[(size_t)i];
    return (int)cells.size();
}

int smelt_layout_make_affine_entry(int rows, int cols, int group_size, uint64_t* offset_io, SmeltWeightEntryC* out) {
    if (!offset_io || !out || rows <= 0 || cols <= 0 || group_size <= 0) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    memset(out, 0, sizeof(*out));
    const uint64_t packed_size = (uint64_t)rows * (uint64_t)((cols + 1) / 2);
    const uint64_t groups = (uint64_t)((cols + group_size - 1) / group_size);
    const uint64_t sb = (uint64_t)rows * groups * 2;
    out->offset = align_to(*offset_io, 128);
    out->scales_offset = align_to(out->offset + packed_size, 128);
    out->biases_offset = align_to(out->scales_offset + sb, 128);
    *offset_io = out->biases_offset + sb;
    out->size_bytes = packed_size;
    out->rows = rows; out->cols = cols;
    out->dtype = SMELT_DTYPE_AFFINE_U4;
    out->group_size = group_size;
    out->packed_row_stride = (cols + 1) / 2;
    out->padded_cols = cols;
    out->scales_size_bytes = sb;
    out->biases_size_bytes = sb;
    return SMELT_HIP_OK;
}

int smelt_layout_make_signed_entry(int rows, int cols, int dtype, int group_size, uint64_t* offset_io, SmeltWeightEntryC* out) {
    if (!offset_io || !out || rows <= 0 || cols <= 0 || group_size <= 0 || !signed_dtype(dtype)) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    memset(out, 0, sizeof(*out));
    const int padded = (cols + group_size - 1) / group_size * group_size;
    int stride;
    if (dtype == SMELT_DTYPE_TRIT5) stride = (((cols + 4) / 5) + 15) & ~15;
    else stride = (padded * (dtype == SMELT_DTYPE_BINARY1 ? 1 : 2) + 7) / 8;
    const uint64_t packed_size = (uint64_t)rows * (uint64_t)stride;
    const uint64_t scales = (uint64_t)rows * (uint64_t)(padded / group_size) * 2;
    out->offset = align_to(*offset_io, 128);
    out->scales_offset = align_to(out->offset + packed_size, 128);
    *offset_io = out->scales_offset + scales;
    out->size_bytes = packed_size;
    out->rows = rows; out->cols = cols;
    out->dtype = dtype;
    out->group_size = group_size;
    out->packed_row_stride = stride;
    out->padded_cols = padded;
    out->scales_size_bytes = scales;
    return SMELT_HIP_OK;
}

int smelt_layout_make_affine_bank(const int* member_rows, int members, int cols, int group_size, uint64_t* offset_io, SmeltWeightEntryC* out) {
    if (!member_rows || !offset_io || !out || members < 2 || members > 4 || cols <= 0 || group_size <= 0) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    const uint64_t stride = (uint64_t)((cols + 1) / 2);
    const uint64_t groups = (uint64_t)((cols + group_size - 1) / group_size);
    uint64_t total_rows = 0;
    for (int m = 0; m < members; ++m) {
        if (member_rows[m] <= 0) return SMELT_HIP_ERR_INVALID_ARGUMENT;
        total_rows += (uint64_t)member_rows[m];
    }
    const uint64_t packed0 = align_to(*offset_io, 128);
    const uint64_t scales0 = align_to(packed0 + total_rows * stride, 128);
    const uint64_t biases0 = align_to(scales0 + total_rows * groups * 2, 128);
    *offset_io = biases0 + total_rows * groups * 2;
    uint64_t before = 0;
    for (int m = 0; m < members; ++m) {
        SmeltWeightEntryC& e = out[m];
        memset(&e, 0, sizeof(e));
        e.rows = member_rows[m]; e.cols = cols;
        e.dtype = SMELT_DTYPE_AFFINE_U4;
        e.group_size = group_size;
        e.packed_row_stride = (int32_t)stride;
        e.padded_cols = cols;
        e.offset = packed0 + before * stride;
        e.size_bytes = (uint64_t)e.rows * stride;
        e.scales_offset = scales0 + before * groups * 2;
        e.biases_offset = biases0 + before * groups * 2;
        e.scales_size_bytes = e.biases_size_bytes = (uint64_t)e.rows * groups * 2;
        before += (uint64_t)e.rows;
    }
    return SMELT_HIP_OK;
}

int smelt_layout_make_signed_bank(const int* member_rows, int members, int cols, int dtype, int group_size, uint64_t* offset_io, SmeltWeightEntryC* out) {
    if (!member_rows || !offset_io || !out || members < 2 || members > 4 || cols <= 0 || group_size <= 0 || !signed_dtype(dtype)) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    const int padded = (cols + group_size - 1) / group_size * group_size;
    uint64_t stride;
    if (dtype == SMELT_DTYPE_TRIT5) stride = (uint64_t)((((cols + 4) / 5) + 15) & ~15);
    else stride = (uint64_t)((padded * (dtype == SMELT_DTYPE_BINARY1 ? 1 : 2) + 7) / 8);
    const uint64_t groups = (uint64_t)(padded / group_size);
    uint64_t total_rows = 0;
    for (int m = 0; m < members; ++m) {
        if (member_rows[m] <= 0) return SMELT_HIP_ERR_INVALID_ARGUMENT;
        total_rows += (uint64_t)member_rows[m];
    }
    const uint64_t packed0 = align_to(*offset_io, 128);
    const uint64_t scales0 = align_to(packed0 + total_rows * stride, 128);
    *offset_io = scales0 + total_rows * groups * 2;
    uint64_t before = 0;
    for (int m = 0; m < members; ++m) {
        SmeltWeightEntryC& e = out[m];
        memset(&e, 0, sizeof(e));
        e.rows = member_rows[m]; e.cols = cols;
        e.dtype = dtype;
        e.group_size = group_size;
        e.packed_row_stride = (int32_t)stride;
        e.padded_cols = padded;
        e.offset = packed0 + before * stride;
        e.size_bytes = (uint64_t)e.rows * stride;
        e.scales_offset = scales0 + before * groups * 2;
        e.scales_size_bytes = (uint64_t)e.rows * groups * 2;
        before += (uint64_t)e.rows;
    }
    return SMELT_HIP_OK;
}

int smelt_layout_make_dense_entry(int rows, int cols, int dtype, uint64_t* offset_io, SmeltWeightEntryC* out) {
    if (!offset_io || !out || rows <= 0 || cols <= 0) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    int bpe = 0;
    switch (dtype) {
        case SMELT_DTYPE_FP16: case SMELT_DTYPE_BF16: bpe = 2; break;
        case SMELT_DTYPE_FP32: case SMELT_DTYPE_INT32: bpe = 4; break;
        default: return SMELT_HIP_ERR_INVALID_ARGUMENT;
    }
    memset(out, 0, sizeof(*out));
    out->offset = align_to(*offset_io, 16);
    out->size_bytes = (uint64_t)rows * (uint64_t)cols * (uint64_t)bpe;
    *offset_io = out->offset + out->size_bytes;
    out->rows = rows; out->cols = cols;
    out->dtype = dtype;
    return SMELT_HIP_OK;
}

int smelt_route_decode_affine(int rows, int cols, int group, int fusion, int compute_units, SmeltRoute* out) {
    if (!out || rows <= 0 || cols <= 0 || cols % 32 != 0 || group < 32 || (group & (group - 1))) return SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY;
    const char* stem;
    const int rows_per_wave = 2;  // the R of the single-token affine kernels
    switch (fusion) {
        case SMELT_FUSION_NONE: stem = "affine_matvec"; break;
        case SMELT_FUSION_GATE_UP_SWIGLU: stem = "fused_affine_gate_up_swiglu"; break;
        case SMELT_FUSION_DUAL_MATVEC: stem = "fused_dual_affine_matvec"; break;
        case SMELT_FUSION_GATE_UP_GEGLU: stem = "fused_affine_gate_up_geglu"; break;
        default: return SMELT_SELECT_MISSING;
    }
    const bool spec = is_specialized_shape(rows, cols, group);
    const MatvecGeometry g = matvec_geometry((uint32_t)cols / 2, rows, rows_per_wave, compute_units);
    const std::string name = spec ? std::string(stem) + shape_tag(rows, cols, group)
                                  : std::string(stem) + ":" + std::to_string(cols) + ":" + std::to_string(group);
    set_route(out, name, spec, g.rows_per_group, 1, 256, g.grid_w);
    return SMELT_HIP_OK;
}

int smelt_route_prefill_affine(int rows, int cols, int group, int fusion, int max_batch, int compute_units, SmeltRoute* out) {
    if (!out || rows <= 0 || cols <= 0 || cols % 32 != 0 || group < 32 || (group & (group - 1)) || max_batch <= 0) return SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY;
    const char* stem;
    switch (fusion) {
        case SMELT_FUSION_NONE: stem = "affine_matvec"; break;
        case SMELT_FUSION_GATE_UP_SWIGLU: stem = "fused_affine_gate_up_swiglu"; break;
        case SMELT_FUSION_GATE_UP_GEGLU: stem = "fused_affine_gate_up_geglu"; break;
        default: return SMELT_SELECT_MISSING;
    }
    const std::string base = std::string(stem) + shape_tag(rows, cols, group);
    if (fusion == SMELT_FUSION_GATE_UP_GEGLU) {
        // GeGLU has the MFMA slab kernel only
        const int bt = max_batch > 32 ? 64 : 16;
        set_route(out, base + (bt == 16 ? "_batched_full" : "_batched_full_b64"), true, 64, bt, 256, (rows + 63) / 64);
        return SMELT_HIP_OK;
    }
    if (max_batch <= 4) {
        // weights stream once per four tokens through the matvec kernel
        const int rpw = fusion == SMELT_FUSION_NONE ? 4 : 2;
        const MatvecGeometry g = matvec_geometry((uint32_t)cols / 2, rows, rpw, compute_units);
        set_route(out, base + "_batched_tile4", true, g.rows_per_group, 4, 256, g.grid_w);
        return SMELT_HIP_OK;
    }
    if (max_batch <= 32 && group == 64 && cols % 512 == 0) {
        // skinny MFMA qmm: 32-row tiles.  K is split over as few workgroups as keep the staged
        // activations of a chunk within ~96 KB of LDS and give every CU a workgroup; each extra
        // split costs a round trip through the split-K workspace.
        const int nwin = cols / 64, tiles = (rows + 31) / 32;
        int tpad = 1;
        while (tpad < max_batch) tpad *= 2;
        const int nmat = fusion == SMELT_FUSION_GATE_UP_SWIGLU ? 2 : 1;
        auto lds = [&](int ks) { return qmm_skinny_lds_bytes((uint32_t)cols, (uint32_t)ks, (uint32_t)nmat, (uint32_t)tpad, 4); };
        int ksplit = 1;
        while (ksplit < nwin && lds(ksplit) > (size_t)96 * 1024) ++ksplit;
        const int want = (std::max(1, compute_units) + tiles / 2) / tiles;
        while (ksplit < want && (nwin + ksplit) / (ksplit + 1) >= 8) ++ksplit;
        set_route(out, base + "_batched_skinny", true, 32, 32, 256, tiles * ksplit);
        return SMELT_HIP_OK;
    }
    // MFMA qmm: 64-row slabs; 16-token tiles up to 32 tokens, 64-token tiles beyond
    const int bt = max_batch > 32 ? 64 : 16;
    const std::string suffix = bt == 16 ? "_batched_full" : "_batched_full_b64";
    set_route(out, base + suffix, true, 64, bt, 256, (rows + 63) / 64);
    return SMELT_HIP_OK;
}

int smelt_emitter_create(int act_dtype, int compute_units, smelt_emitter** out) {
    if (!out || (act_dtype != SMELT_HIP_ACT_F16 && act_dtype != SMELT_HIP_ACT_BF16)) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    smelt_emitter* e = new smelt_emitter();
    e->act = act_dtype;
    e->compute_units = compute_units > 0 ? compute_units : 256;
    *out = e;
    return SMELT_HIP_OK;
}

void smelt_emitter_destroy(smelt_emitter* e) { delete e; }

const char* smelt_emitter_last_error(const smelt_emitter* e) { return e ? e->error.c_str() : ""; }

int smelt_emit_rms_norm_1pw(smelt_emitter* e, SmeltBinding input, SmeltBinding weight, SmeltBinding output,
                            const SmeltBinding* residual, int dim, float eps, int batch_size) {
    if (!e) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    if (dim <= 0 || batch_size <= 0) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "rms norm needs positive dim and batch");
    const bool fixed = eps == 1e-6f;
    if (residual && !fixed) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "the residual form of rms_norm_1pw exists for eps 1e-6 only");
    RecordBuilder rb;
    rb.buffer(0, input);
    rb.buffer(1, weight);
    std::string name = "rms_norm_1pw";
    if (fixed) name += "_d" + std::to_string(dim);
    if (residual) {
        rb.buffer(2, *residual);
        rb.buffer(3, output);
        name += "_add";
    } else {
        rb.buffer(2, output);
    }
    if (batch_size > 1) name += "_batched";
    if (!fixed) {
        rb.constant(3, (uint32_t)dim);
        rb.constant_f32(4, eps);
    }
    // whole waves, eight elements per thread, at most 1024 threads
    const int threads = std::min(1024, std::max(64, ((dim + 7) / 8 + 63) / 64 * 64));
    rb.grid((uint32_t)batch_size, 1, 1, (uint32_t)threads);
    rb.r.pipeline = e->pipeline_index(name);
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

// rms_norm_scale_only (norms.metal:944-1008): one fp32 scale 1 / sqrt(mean(x^2) + eps) per row, the
// first half of the scale-only + norm-scale pair (emitNormScaleAffineMatvecIfPossible,
// SmeltCodeEmitter.swift:2680-2754).
int smelt_emit_rms_norm_scale_only(smelt_emitter* e, SmeltBinding input, SmeltBinding scale_output, int dim, float eps, int batch_size) {
    if (!e) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    if (dim <= 0 || batch_size <= 0) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "rms norm needs positive dim and batch");
    RecordBuilder rb;
    rb.buffer(0, input);
    rb.buffer(1, scale_output);
    rb.constant(2, (uint32_t)dim);
    rb.constant_f32(3, eps);
    const int threads = std::min(1024, std::max(64, ((dim + 7) / 8 + 63) / 64 * 64));
    rb.grid((uint32_t)batch_size, 1, 1, (uint32_t)threads);
    rb.r.pipeline = e->pipeline_index(batch_size > 1 ? "rms_norm_scale_only_batched" : "rms_norm_scale_only");
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

static int emit_pointwise(smelt_emitter* e, const char* name, SmeltBinding a, SmeltBinding b, SmeltBinding output, int count) {
    if (!e) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    if (count <= 0) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "element count must be positive");
    RecordBuilder rb;
    rb.buffer(0, a);
    rb.buffer(1, b);
    rb.buffer(2, output);
    rb.constant(3, (uint32_t)count);
    rb.r.style = SMELT_STYLE_THREADS;   // the grid counts threads (dispatchThreads)
    rb.grid((uint32_t)count, 1, 1, (uint32_t)std::min(count, 1024));
    rb.r.pipeline = e->pipeline_index(name);
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

int smelt_emit_elementwise(smelt_emitter* e, int multiply, SmeltBinding a, SmeltBinding b, SmeltBinding output, int count) {
    return emit_pointwise(e, multiply ? "elementwise_mul" : "elementwise_add", a, b, output, count);
}

int smelt_emit_swiglu_fused(smelt_emitter* e, SmeltBinding gate, SmeltBinding up, SmeltBinding output, int count) {
    return emit_pointwise(e, "swiglu_fused", gate, up, output, count);
}

static int check_view(smelt_emitter* e, int planes, int cols, int batch_size) {
    if (planes < 2 || planes > 6) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "activation views hold 2 to 6 planes");
    if (cols <= 0 || cols % 128 != 0 || batch_size <= 0) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "activation views need cols % 128 == 0 and a positive batch");
    return 0;
}

int smelt_emit_activation_view(smelt_emitter* e, int planes, SmeltBinding input, SmeltBinding view_planes,
                               SmeltBinding view_scales, int cols, int batch_size) {
    if (!e) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    if (int rc = check_view(e, planes, cols, batch_size)) return rc;
    RecordBuilder rb;
    rb.buffer(0, input);
    rb.buffer(1, view_planes);
    rb.buffer(2, view_scales);
    rb.constant(3, (uint32_t)cols);
    // one wave per group, four groups per workgroup
    rb.grid((uint32_t)((cols / 128 + 3) / 4), (uint32_t)batch_size, 1, 256);
    rb.r.pipeline = e->pipeline_index("signed_activation_bitplanes_i" + std::to_string(planes) + "_g128" + (batch_size > 1 ? "_batched" : ""));
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

static const char* view_weight_stem(smelt_emitter* e, const SmeltWeightEntryC* w) {
    if (!w || (w->dtype != SMELT_DTYPE_BINARY1 && w->dtype != SMELT_DTYPE_TERNARY2)) {
        efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "activation views are consumed by binary1 and ternary2 weights");
        return nullptr;
    }
    if (check_signed_entry(e, w)) return nullptr;
    return w->dtype == SMELT_DTYPE_BINARY1 ? "signed_binary_bitplane_i" : "signed_ternary_bitplane_i";
}

int smelt_emit_view_matvec(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* w, int planes, SmeltBinding view_planes,
                           SmeltBinding view_scales, SmeltBinding output, const SmeltBinding* residual, int batch_size) {
    if (!e) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    const char* stem = view_weight_stem(e, w);
    if (!stem) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    if (int rc = check_view(e, planes, w->cols, batch_size)) return rc;
    const MatvecGeometry g = matvec_geometry(signed_row_stride(to_format(w->dtype), (uint32_t)w->cols), w->rows, 4, e->compute_units);
    RecordBuilder rb;
    rb.buffer(0, weights_slot, w->offset);
    rb.buffer(1, weights_slot, w->scales_offset);
    rb.buffer(2, view_planes);
    rb.buffer(3, view_scales);
    rb.buffer(4, output);
    uint8_t next = 5;
    if (residual) rb.buffer(next++, *residual);
    rb.constant(next, (uint32_t)w->rows);
    rb.constant((uint8_t)(next + 1), (uint32_t)w->cols);
    rb.grid((uint32_t)g.grid_w, (uint32_t)batch_size, 1, 256);
    rb.r.pipeline = e->pipeline_index(std::string(stem) + std::to_string(planes) + (residual ? "_matvec_add_g128_rows8" : "_matvec_g128_rows8"));
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

int smelt_emit_view_gate_up_swiglu(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* gate, const SmeltWeightEntryC* up,
                                   int planes, SmeltBinding view_planes, SmeltBinding view_scales, SmeltBinding output, int batch_size) {
    if (!e) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    const char* stem = view_weight_stem(e, gate);
    if (!stem || !view_weight_stem(e, up)) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    if (gate->dtype != up->dtype || gate->rows != up->rows || gate->cols != up->cols)
        return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "gate and up must share format and shape");
    if (int rc = check_view(e, planes, gate->cols, batch_size)) return rc;
    const MatvecGeometry g = matvec_geometry(signed_row_stride(to_format(gate->dtype), (uint32_t)gate->cols), gate->rows, 2, e->compute_units);
    RecordBuilder rb;
    rb.buffer(0, weights_slot, gate->offset);
    rb.buffer(1, weights_slot, gate->scales_offset);
    rb.buffer(2, weights_slot, up->offset);
    rb.buffer(3, weights_slot, up->scales_offset);
    rb.buffer(4, view_planes);
    rb.buffer(5, view_scales);
    rb.buffer(6, output);
    rb.constant(7, (uint32_t)gate->rows);
    rb.constant(8, (uint32_t)gate->cols);
    rb.grid((uint32_t)g.grid_w, (uint32_t)batch_size, 1, 256);
    rb.r.pipeline = e->pipeline_index(std::string(stem) + std::to_string(planes) + "_gate_up_swiglu_g128_rows8");
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

int smelt_emit_swap(smelt_emitter* e) {
    if (!e) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    RecordBuilder rb;
    rb.r.op_kind = SMELT_OP_SWAP;
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

static void bind_affine(RecordBuilder& rb, uint8_t first, int weights_slot, const SmeltWeightEntryC* w) {
    rb.buffer(first, weights_slot, w->offset);
    rb.buffer(first + 1, weights_slot, w->scales_offset);
    rb.buffer(first + 2, weights_slot, w->biases_offset);
}

static void batch_constant_and_grid(RecordBuilder& rb, uint8_t index, int grid_w, int batch_size, int bt, int dynamic, int threads) {
    if (dynamic) {
        rb.constant(index, 0, SMELT_CONST_SEQ_LEN);
        rb.grid((uint32_t)grid_w, (uint32_t)bt, 1, (uint32_t)threads);
        rb.grid_h_kind(bt == 1 ? SMELT_GRID_SEQ_LEN : SMELT_GRID_SEQ_LEN_CEIL_DIV_LITERAL);
    } else {
        rb.constant(index, (uint32_t)batch_size);
        rb.grid((uint32_t)grid_w, (uint32_t)((batch_size + bt - 1) / bt), 1, (uint32_t)threads);
    }
}

int smelt_emit_matvec(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* w, SmeltBinding input, SmeltBinding output, int batch_size, int dynamic) {
    if (!e || !w || batch_size <= 0) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "null emitter or weight, or empty batch");
    const bool batched = batch_size > 1 || dynamic;
    int family = 0;
    if (int rc = gateway(e, w, batched ? SMELT_SHAPE_GEMM : SMELT_SHAPE_GEMV, SMELT_FUSION_NONE, &family)) return rc;
    if (family == SMELT_FAMILY_AFFINE_U4) {
        if (!affine_entry_ok(w)) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "affine matvec needs cols % 32 == 0 and a power-of-two group >= 32 with scale and bias planes");
        SmeltRoute route;
        RecordBuilder rb;
        bind_affine(rb, 0, weights_slot, w);
        rb.buffer(3, input);
        rb.buffer(4, output);
        if (!batched) {
            if (int rc = smelt_route_decode_affine(w->rows, w->cols, w->group_size, SMELT_FUSION_NONE, e->compute_units, &route)) return efail(e, rc, "no decode route");
            if (!route.specialized) rb.constant(5, (uint32_t)w->rows);
            rb.grid((uint32_t)route.grid_w, 1, 1, (uint32_t)route.threads);
        } else {
            if (int rc = smelt_route_prefill_affine(w->rows, w->cols, w->group_size, SMELT_FUSION_NONE, batch_size, e->compute_units, &route)) return efail(e, rc, "no prefill route");
            batch_constant_and_grid(rb, 5, route.grid_w, batch_size, route.batch_tile, dynamic, route.threads);
        }
        rb.r.pipeline = e->pipeline_index(route.pipeline);
        e->records.push_back(rb.r);
        return SMELT_HIP_OK;
    }
    // signed families: emitSignedMatvec (SmeltCodeEmitter.swift:1092-1263)
    if (int rc = check_signed_entry(e, w)) return rc;
    const MatvecGeometry g = matvec_geometry(signed_row_stride(to_format(w->dtype), (uint32_t)w->cols), w->rows, 4, e->compute_units);
    if (w->dtype == SMELT_DTYPE_TERNARY2) {
        // production ternary route: affine-QMV pipeline below 6 tokens, QMM from 6 tokens on
        auto bind = [&](RecordBuilder& rb) {
            rb.buffer(0, weights_slot, w->offset);
            rb.buffer(1, weights_slot, w->scales_offset);
            rb.buffer(2, weights_slot, w->scales_offset);
            rb.buffer(3, input);
            rb.buffer(4, output);
            rb.constant(5, (uint32_t)w->rows);
            rb.constant(6, (uint32_t)w->cols);
        };
        const int qmm_min_batch = 6;
        if (!batched || dynamic || batch_size < qmm_min_batch) {
            RecordBuilder rb;
            bind(rb);
            rb.r.pipeline = e->pipeline_index("signed_ternary_affine_matvec_g128_rows8");
            if (dynamic) {
                rb.constant(0xFF, (uint32_t)qmm_min_batch, SMELT_CONST_SEQ_LEN_LT_LITERAL_SKIP_IF_FALSE);
                rb.grid((uint32_t)g.grid_w, 1, 1, 256);
                rb.grid_h_kind(SMELT_GRID_SEQ_LEN);
            } else {
                rb.grid((uint32_t)g.grid_w, (uint32_t)batch_size, 1, 256);
            }
            e->records.push_back(rb.r);
        }
        if (dynamic || batch_size >= qmm_min_batch) {
            RecordBuilder rb;
            bind(rb);
            rb.r.pipeline = e->pipeline_index("signed_ternary_affine_qmm_g128_bm32_bn32_bk32");
            if (dynamic) {
                rb.constant(7, 0, SMELT_CONST_SEQ_LEN);
                rb.grid((uint32_t)((w->rows + 63) / 64), 32, 1, 256);
                rb.grid_h_kind(SMELT_GRID_SEQ_LEN_CEIL_DIV_LITERAL);
                rb.r.min_seq_len = (uint16_t)qmm_min_batch;
            } else {
                rb.constant(7, (uint32_t)batch_size);
                rb.grid((uint32_t)((w->rows + 63) / 64), (uint32_t)((batch_size + 31) / 32), 1, 256);
            }
            e->records.push_back(rb.r);
        }
        return SMELT_HIP_OK;
    }
    RecordBuilder rb;
    rb.buffer(0, weights_slot, w->offset);
    rb.buffer(1, weights_slot, w->scales_offset);
    rb.buffer(2, input);
    rb.buffer(3, output);
    rb.constant(4, (uint32_t)w->rows);
    rb.constant(5, (uint32_t)w->cols);
    std::string name = std::string("signed_") + signed_stem(w->dtype) + "_matvec_g128_rows8";
    if (batched) {
        name += "_batched_b4";
        batch_constant_and_grid(rb, 6, g.grid_w, batch_size, 4, dynamic, 256);
    } else {
        rb.grid((uint32_t)g.grid_w, 1, 1, 256);
    }
    rb.r.pipeline = e->pipeline_index(name);
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

int smelt_emit_matvec_add(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* w, SmeltBinding input, SmeltBinding output, SmeltBinding residual) {
    if (!e || !w) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "null emitter or weight");
    int family = 0;
    if (int rc = gateway(e, w, SMELT_SHAPE_GEMV, SMELT_FUSION_NONE, &family)) return rc;
    RecordBuilder rb;
    if (family == SMELT_FAMILY_AFFINE_U4) {
        if (!affine_entry_ok(w)) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "unsupported affine geometry");
        SmeltRoute route;
        if (int rc = smelt_route_decode_affine(w->rows, w->cols, w->group_size, SMELT_FUSION_NONE, e->compute_units, &route)) return efail(e, rc, "no decode route");
        bind_affine(rb, 0, weights_slot, w);
        rb.buffer(3, input);
        rb.buffer(4, output);
        rb.buffer(5, residual);
        std::string name = route.specialized ? "fused_affine_matvec_add" + shape_tag(w->rows, w->cols, w->group_size)
                                             : "fused_affine_matvec_add:" + std::to_string(w->cols) + ":" + std::to_string(w->group_size);
        if (!route.specialized) rb.constant(6, (uint32_t)w->rows);
        rb.grid((uint32_t)route.grid_w, 1, 1, 256);
        rb.r.pipeline = e->pipeline_index(name);
        e->records.push_back(rb.r);
        return SMELT_HIP_OK;
    }
    if (int rc = check_signed_entry(e, w)) return rc;
    const MatvecGeometry g = matvec_geometry(signed_row_stride(to_format(w->dtype), (uint32_t)w->cols), w->rows, 4, e->compute_units);
    rb.buffer(0, weights_slot, w->offset);
    rb.buffer(1, weights_slot, w->scales_offset);
    if (w->dtype == SMELT_DTYPE_TERNARY2) {
        rb.buffer(2, weights_slot, w->scales_offset);
        rb.buffer(3, input);
        rb.buffer(4, output);
        rb.buffer(5, residual);
        rb.constant(6, (uint32_t)w->rows);
        rb.constant(7, (uint32_t)w->cols);
        rb.r.pipeline = e->pipeline_index("signed_ternary_affine_matvec_add_g128_rows8");
    } else {
        rb.buffer(2, input);
        rb.buffer(3, output);
        rb.buffer(4, residual);
        rb.constant(5, (uint32_t)w->rows);
        rb.constant(6, (uint32_t)w->cols);
        rb.r.pipeline = e->pipeline_index(std::string("signed_") + signed_stem(w->dtype) + "_matvec_add_g128_rows8");
    }
    rb.grid((uint32_t)g.grid_w, 1, 1, 256);
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

int smelt_emit_gate_up_swiglu(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* gate, const SmeltWeightEntryC* up,
                              SmeltBinding input, SmeltBinding output, int batch_size, int dynamic) {
    if (!e || !gate || !up || batch_size <= 0) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "null emitter or weight");
    if (gate->dtype != up->dtype || gate->rows != up->rows || gate->cols != up->cols || gate->group_size != up->group_size)
        return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "gate and up projections must share dtype, shape and group size");
    const bool batched = batch_size > 1 || dynamic;
    int family = 0;
    if (int rc = gateway(e, gate, batched ? SMELT_SHAPE_GEMM : SMELT_SHAPE_GEMV, SMELT_FUSION_GATE_UP_SWIGLU, &family)) return rc;
    RecordBuilder rb;
    if (family == SMELT_FAMILY_AFFINE_U4) {
        if (!affine_entry_ok(gate) || !affine_entry_ok(up)) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "unsupported affine geometry");
        bind_affine(rb, 0, weights_slot, gate);
        bind_affine(rb, 3, weights_slot, up);
        rb.buffer(6, input);
        rb.buffer(7, output);
        SmeltRoute route;
        if (!batched) {
            if (int rc = smelt_route_decode_affine(gate->rows, gate->cols, gate->group_size, SMELT_FUSION_GATE_UP_SWIGLU, e->compute_units, &route)) return efail(e, rc, "no decode route");
            if (!route.specialized) rb.constant(8, (uint32_t)gate->rows);
            rb.grid((uint32_t)route.grid_w, 1, 1, 256);
        } else {
            if (int rc = smelt_route_prefill_affine(gate->rows, gate->cols, gate->group_size, SMELT_FUSION_GATE_UP_SWIGLU, batch_size, e->compute_units, &route)) return efail(e, rc, "no prefill route");
            batch_constant_and_grid(rb, 8, route.grid_w, batch_size, route.batch_tile, dynamic, route.threads);
        }
        rb.r.pipeline = e->pipeline_index(route.pipeline);
        e->records.push_back(rb.r);
        return SMELT_HIP_OK;
    }
    if (int rc = check_signed_entry(e, gate)) return rc;
    if (int rc = check_signed_entry(e, up)) return rc;
    const MatvecGeometry g = matvec_geometry(signed_row_stride(to_format(gate->dtype), (uint32_t)gate->cols), gate->rows, 2, e->compute_units);
    if (gate->dtype == SMELT_DTYPE_TERNARY2) {
        if (batched) return efail(e, SMELT_SELECT_MISSING, "no batched ternary gate-up kernel; emit two matvecs and swiglu");
        rb.buffer(0, weights_slot, gate->offset);
        rb.buffer(1, weights_slot, gate->scales_offset);
        rb.buffer(2, weights_slot, gate->scales_offset);
        rb.buffer(3, weights_slot, up->offset);
        rb.buffer(4, weights_slot, up->scales_offset);
        rb.buffer(5, weights_slot, up->scales_offset);
        rb.buffer(6, input);
        rb.buffer(7, output);
        rb.constant(8, (uint32_t)gate->rows);
        rb.constant(9, (uint32_t)gate->cols);
        rb.grid((uint32_t)g.grid_w, 1, 1, 256);
        rb.r.pipeline = e->pipeline_index("signed_ternary_affine_gate_up_swiglu_g128_rows8");
    } else {
        rb.buffer(0, weights_slot, gate->offset);
        rb.buffer(1, weights_slot, gate->scales_offset);
        rb.buffer(2, weights_slot, up->offset);
        rb.buffer(3, weights_slot, up->scales_offset);
        rb.buffer(4, input);
        rb.buffer(5, output);
        rb.constant(6, (uint32_t)gate->rows);
        rb.constant(7, (uint32_t)gate->cols);
        std::string name = std::string("signed_") + signed_stem(gate->dtype) + "_gate_up_swiglu_g128_rows8";
        if (batched) {
            name += "_batched_b4";
            batch_constant_and_grid(rb, 8, g.grid_w, batch_size, 4, dynamic, 256);
        } else {
            rb.grid((uint32_t)g.grid_w, 1, 1, 256);
        }
        rb.r.pipeline = e->pipeline_index(name);
    }
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

// norm_scale_affine_matvec (lut_matvec.metal:1294-1469): bindings 0 scale, 1 input, 2 norm weight,
// 3 normalised row out, 4..6 W S B, 7 output, constant 8 rows (generic name only).
int smelt_emit_norm_scale_matvec(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* w, SmeltBinding norm_scale,
                                 SmeltBinding input, SmeltBinding norm_weight, SmeltBinding norm_output, SmeltBinding output) {
    if (!e || !w) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "null emitter or weight");
    int family = 0;
    if (int rc = gateway(e, w, SMELT_SHAPE_GEMV, SMELT_FUSION_NONE, &family)) return rc;
    if (family != SMELT_FAMILY_AFFINE_U4) return efail(e, SMELT_SELECT_MISSING, "the norm-scale prologue exists for affine_u4 weights only");
    if (!affine_entry_ok(w)) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "unsupported affine geometry");
    SmeltRoute route;
    if (int rc = smelt_route_decode_affine(w->rows, w->cols, w->group_size, SMELT_FUSION_NONE, e->compute_units, &route)) return efail(e, rc, "no decode route");
    RecordBuilder rb;
    rb.buffer(0, norm_scale);
    rb.buffer(1, input);
    rb.buffer(2, norm_weight);
    rb.buffer(3, norm_output);
    bind_affine(rb, 4, weights_slot, w);
    rb.buffer(7, output);
    if (!route.specialized) rb.constant(8, (uint32_t)w->rows);
    rb.grid((uint32_t)route.grid_w, 1, 1, (uint32_t)route.threads);
    rb.r.pipeline = e->pipeline_index(std::string("norm_scale_") + route.pipeline);
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

// norm_scale_affine_gate_up_swiglu / _geglu (lut_matvec.metal:1471-1700): bindings 0 scale, 1 input,
// 2 norm weight, 3..5 gate W S B, 6..8 up W S B, 9 output, constant 10 rows (generic name only).
int smelt_emit_norm_scale_gate_up(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* gate, const SmeltWeightEntryC* up,
                                  int geglu, SmeltBinding norm_scale, SmeltBinding input, SmeltBinding norm_weight, SmeltBinding output) {
    if (!e || !gate || !up) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "null emitter or weight");
    if (gate->dtype != up->dtype || gate->rows != up->rows || gate->cols != up->cols || gate->group_size != up->group_size)
        return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "gate and up projections must share dtype, shape and group size");
    const int fusion = geglu ? SMELT_FUSION_GATE_UP_GEGLU : SMELT_FUSION_GATE_UP_SWIGLU;
    int family = 0;
    if (int rc = gateway(e, gate, SMELT_SHAPE_GEMV, fusion, &family)) return rc;
    if (family != SMELT_FAMILY_AFFINE_U4) return efail(e, SMELT_SELECT_MISSING, "the norm-scale prologue exists for affine_u4 weights only");
    if (!affine_entry_ok(gate) || !affine_entry_ok(up)) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "unsupported affine geometry");
    SmeltRoute route;
    if (int rc = smelt_route_decode_affine(gate->rows, gate->cols, gate->group_size, fusion, e->compute_units, &route)) return efail(e, rc, "no decode route");
    RecordBuilder rb;
    rb.buffer(0, norm_scale);
    rb.buffer(1, input);
    rb.buffer(2, norm_weight);
    bind_affine(rb, 3, weights_slot, gate);
    bind_affine(rb, 6, weights_slot, up);
    rb.buffer(9, output);
    if (!route.specialized) rb.constant(10, (uint32_t)gate->rows);
    rb.grid((uint32_t)route.grid_w, 1, 1, 256);
    // "fused_affine_gate_up_*" -> "norm_scale_affine_gate_up_*"
    rb.r.pipeline = e->pipeline_index(std::string("norm_scale_") + (route.pipeline + 6));
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

// AtomicNormFusionPass (SmeltDispatchOptimizer.swift:918-1046): rms_norm_1pw followed by its consumer
// becomes one dispatch.  Matvec: 0 input, 1 norm weight, 2 normalised row out, 3..5 W S B, 6 output,
// 7 scratch {scale, flag}, constants 8 rows, 9 eps.  up != NULL emits the gate+up+SwiGLU form: 0 input,
// 1 norm weight, 2..7 weights, 8 output, 9 scratch, constants 10 rows, 11 eps (no normalised row out).
int smelt_emit_fused_norm_matvec(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* w, const SmeltWeightEntryC* up,
                                 SmeltBinding input, SmeltBinding norm_weight, const SmeltBinding* norm_output,
                                 SmeltBinding output, SmeltBinding scratch, float eps) {
    if (!e || !w) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "null emitter or weight");
    if (!up && !norm_output) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "the matvec form stores the normalised row: bind it");
    if (up && (w->dtype != up->dtype || w->rows != up->rows || w->cols != up->cols || w->group_size != up->group_size))
        return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "gate and up projections must share dtype, shape and group size");
    int family = 0;
    if (int rc = gateway(e, w, SMELT_SHAPE_GEMV, up ? SMELT_FUSION_GATE_UP_SWIGLU : SMELT_FUSION_NONE, &family)) return rc;
    if (family != SMELT_FAMILY_AFFINE_U4) return efail(e, SMELT_SELECT_MISSING, "the fused norm exists for affine_u4 weights only");
    if (!affine_entry_ok(w) || (up && !affine_entry_ok(up))) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "unsupported affine geometry");
    const MatvecGeometry g = matvec_geometry((uint32_t)w->cols / 2, w->rows, 2, e->compute_units);
    RecordBuilder rb;
    rb.buffer(0, input);
    rb.buffer(1, norm_weight);
    uint8_t next = 2;
    if (!up) rb.buffer(next++, *norm_output);
    bind_affine(rb, next, weights_slot, w);
    next += 3;
    if (up) { bind_affine(rb, next, weights_slot, up); next += 3; }
    rb.buffer(next++, output);
    rb.buffer(next++, scratch);
    rb.constant(next++, (uint32_t)w->rows);
    rb.constant_f32(next, eps);
    rb.grid((uint32_t)g.grid_w, 1, 1, 256);
    rb.r.pipeline = e->pipeline_index(std::string(up ? "atomic_norm_affine_gate_up_swiglu:" : "atomic_norm_affine_matvec:") +
                                      std::to_string(w->cols) + ":" + std::to_string(w->group_size));
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

int smelt_emit_dual_matvec(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* w1, const SmeltWeightEntryC* w2,
                           SmeltBinding input, SmeltBinding output1, SmeltBinding output2) {
    if (!e || !w1 || !w2) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "null emitter or weight");
    if (w1->dtype != w2->dtype || w1->rows != w2->rows || w1->cols != w2->cols || w1->group_size != w2->group_size)
        return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "dual projections must share dtype, shape and group size");
    int family = 0;
    if (int rc = gateway(e, w1, SMELT_SHAPE_GEMV, SMELT_FUSION_DUAL_MATVEC, &family)) return rc;
    if (!affine_entry_ok(w1) || !affine_entry_ok(w2)) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "unsupported affine geometry");
    SmeltRoute route;
    if (int rc = smelt_route_decode_affine(w1->rows, w1->cols, w1->group_size, SMELT_FUSION_DUAL_MATVEC, e->compute_units, &route)) return efail(e, rc, "no decode route");
    RecordBuilder rb;
    bind_affine(rb, 0, weights_slot, w1);
    bind_affine(rb, 3, weights_slot, w2);
    rb.buffer(6, input);
    rb.buffer(7, output1);
    rb.buffer(8, output2);
    if (!route.specialized) rb.constant(9, (uint32_t)w1->rows);
    rb.grid((uint32_t)route.grid_w, 1, 1, 256);
    rb.r.pipeline = e->pipeline_index(route.pipeline);
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

int smelt_emit_bank_matvec(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* members, int count, SmeltBinding input, const SmeltBinding* outputs) {
    if (!e || !members || !outputs || count < 2 || count > 4) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "a bank has 2 to 4 members");
    int family = 0;
    if (int rc = gateway(e, &members[0], SMELT_SHAPE_GEMV, SMELT_FUSION_NONE, &family)) return rc;
    const SmeltWeightEntryC& first = members[0];
    uint64_t rows = 0;
    for (int m = 0; m < count; ++m) {
        const SmeltWeightEntryC& w = members[m];
        if (w.dtype != first.dtype || w.cols != first.cols || w.group_size != first.group_size) return 1;
        if (m > 0) {
            const SmeltWeightEntryC& p = members[m - 1];
            if (w.offset != p.offset + p.size_bytes || w.scales_offset != p.scales_offset + p.scales_size_bytes) return 1;
            if (family == SMELT_FAMILY_AFFINE_U4 && w.biases_offset != p.biases_offset + p.biases_size_bytes) return 1;
        }
        rows += (uint64_t)w.rows;
    }
    RecordBuilder rb;
    if (family == SMELT_FAMILY_AFFINE_U4) {
        for (int m = 0; m < count; ++m)
            if (!affine_entry_ok(&members[m])) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "unsupported affine geometry");
        const MatvecGeometry g = matvec_geometry((uint32_t)first.cols / 2, (int)rows, 4, e->compute_units);
        bind_affine(rb, 0, weights_slot, &first);
        rb.buffer(3, input);
        for (int m = 0; m < 4; ++m) rb.buffer((uint8_t)(4 + m), outputs[m < count ? m : 0]);
        for (int m = 0; m < 4; ++m) rb.constant((uint8_t)(8 + m), m < count ? (uint32_t)members[m].rows : 0u);
        rb.grid((uint32_t)g.grid_w, 1, 1, 256);
        rb.r.pipeline = e->pipeline_index("affine_bank4_matvec:" + std::to_string(first.cols) + ":" + std::to_string(first.group_size));
        e->records.push_back(rb.r);
        return SMELT_HIP_OK;
    }
    if (family != SMELT_FAMILY_TERNARY2 && family != SMELT_FAMILY_BINARY1 && family != SMELT_FAMILY_TRIT5) return 1;  // banks exist for these
    for (int m = 0; m < count; ++m)
        if (int rc = check_signed_entry(e, &members[m])) return rc;
    if (family == SMELT_FAMILY_BINARY1 || family == SMELT_FAMILY_TRIT5) {
        // binary packed bank (C S x y0..y3 rows0..rows3 cols); five-digit-byte rows take the same bindings
        const bool trit5 = family == SMELT_FAMILY_TRIT5;
        const MatvecGeometry g = matvec_geometry(signed_row_stride(trit5 ? kFmtTrit5 : kFmtBinary1, (uint32_t)first.cols), (int)rows, 4, e->compute_units);
        rb.buffer(0, weights_slot, first.offset);
        rb.buffer(1, weights_slot, first.scales_offset);
        rb.buffer(2, input);
        for (int m = 0; m < 4; ++m) rb.buffer((uint8_t)(3 + m), outputs[m < count ? m : 0]);
        for (int m = 0; m < 4; ++m) rb.constant((uint8_t)(7 + m), m < count ? (uint32_t)members[m].rows : 0u);
        rb.constant(11, (uint32_t)first.cols);
        rb.grid((uint32_t)g.grid_w, 1, 1, 256);
        rb.r.pipeline = e->pipeline_index(trit5 ? "signed_trit5_packed_bank4_matvec_g128_rows8" : "signed_binary_packed_bank4_matvec_g128_rows8");
        e->records.push_back(rb.r);
        return SMELT_HIP_OK;
    }
    const MatvecGeometry g = matvec_geometry(signed_row_stride(kFmtTernary2, (uint32_t)first.cols), (int)rows, 4, e->compute_units);
    rb.buffer(0, weights_slot, first.offset);
    rb.buffer(1, weights_slot, first.scales_offset);
    rb.buffer(2, weights_slot, first.scales_offset);
    rb.buffer(3, input);
    for (int m = 0; m < 4; ++m) rb.buffer((uint8_t)(4 + m), outputs[m < count ? m : 0]);
    for (int m = 0; m < 4; ++m) rb.constant((uint8_t)(8 + m), m < count ? (uint32_t)members[m].rows : 0u);
    rb.constant(12, (uint32_t)first.cols);
    rb.grid((uint32_t)g.grid_w, 1, 1, 256);
    rb.r.pipeline = e->pipeline_index("signed_ternary_affine_bank4_matvec_g128_rows8");
    e->records.push_back(rb.r);
    return SMELT_HIP_OK;
}

int smelt_emit_lm_head_argmax(smelt_emitter* e, int weights_slot, const SmeltWeightEntryC* w, SmeltBinding input,
                              SmeltBinding partial_keys, SmeltBinding token_out, int batch_size, float logit_cap) {
    if (!e || !w || batch_size <= 0) return efail(e, SMELT_HIP_ERR_INVALID_ARGUMENT, "null emitter or weight");
    if (!affine_entry_ok(w)) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "fused lm_head argmax exists for affine_u4 weights");
    if (w->rows > (1 << 18)) return efail(e, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "argmax keys hold 18 index bits");
    const MatvecGeometry g = matvec_geometry((uint32_t)w->cols / 2, w->rows, 2, e->compute_units);
    const int bt = 8;
    RecordBuilder r1;
    bind_affine(r1, 0, weights_slot, w);
    r1.buffer(3, input);
    r1.buffer(4, partial_keys);
    r1.constant(5, (uint32_t)batch_size);
    r1.constant_f32(6, logit_cap);
    r1.grid((uint32_t)g.grid_w, (uint32_t)((batch_size + bt - 1) / bt), 1, 256);
    r1.r.pipeline = e->pipeline_index("affine_matvec_argmax" + shape_tag(w->rows, w->cols, w->group_size) + "_batched");
    e->records.push_back(r1.r);
    RecordBuilder r2;
    r2.buffer(0, partial_keys);
    r2.buffer(1, token_out);
    r2.constant(2, (uint32_t)batch_size);
    r2.constant(3, (uint32_t)g.grid_w);
    r2.grid((uint32_t)batch_size, 1, 1, 256);
    r2.r.pipeline = e->pipeline_index("lm_head_argmax_reduce_r" + std::to_string(w->rows));
    e->records.push_back(r2.r);
    e->argmax_partial_bytes = std::max(e->argmax_partial_bytes, (size_t)batch_size * (size_t)g.grid_w * 8);
    return SMELT_HIP_OK;
}

size_t smelt_emitter_record_count(const smelt_emitter* e) { return e ? e->records.size() : 0; }
const SmeltDispatchRecord* smelt_emitter_records(const smelt_emitter* e) { return e && !e->records.empty() ? e->records.data() : nullptr; }
size_t smelt_emitter_pipeline_count(const smelt_emitter* e) { return e ? e->pipelines.size() : 0; }
const char* smelt_emitter_pipeline_name(const smelt_emitter* e, size_t index) {
    return e && index < e->pipelines.size() ? e->pipelines[index].c_str() : nullptr;
}
size_t smelt_emitter_argmax_partial_bytes(const smelt_emitter* e) { return e ? e->argmax_partial_bytes : 0; }

int smelt_hip_plan_qmm(uint32_t rows, uint32_t cols, uint32_t group, uint32_t nmat, uint32_t batch, uint32_t compute_units,
                       size_t lds_limit, size_t workspace_bytes, uint32_t out[11]) {
    if (!out || nmat < 1 || nmat > 2) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    memset(out, 0, 11 * sizeof(uint32_t));
    smelt_host::QmtPlan t;
    if (smelt_host::qmt_plan(rows, cols, group, nmat, batch, compute_units, lds_limit, &t)) {
        const uint32_t ksplit = t.partial_bytes <= workspace_bytes ? t.ksplit : 1;
        out[0] = 2; out[1] = t.rt; out[2] = t.kw; out[3] = t.per_wave ? 1u : 0u; out[4] = ksplit;
        out[5] = (rows + t.bn - 1) / t.bn; out[6] = (batch + t.bm - 1) / t.bm; out[7] = ksplit;
        out[8] = 256 * t.kw; out[9] = (uint32_t)t.lds; out[10] = ksplit > 1 ? (uint32_t)t.partial_bytes : 0u;
        return 1;
    }
    smelt_host::QmsPlan q;
    if (batch > 0 && smelt_host::qms_plan(rows, cols, group, nmat, batch, compute_units, lds_limit, &q)) {
        out[0] = 1; out[1] = q.rt; out[2] = q.kc; out[4] = 1;
        out[5] = (rows + 16 * q.rt - 1) / (16 * q.rt); out[6] = (batch + 15) / 16; out[7] = 1;
        out[8] = 64 * q.kc; out[9] = (uint32_t)q.lds;
        return 1;
    }
    return 0;
}

int smelt_hip_plan_matvec(int code_layout, uint32_t rows, uint32_t cols, uint32_t group, uint32_t nmat, size_t lds_limit,
                          int force, uint32_t out[5]) {
    if (!out || code_layout < 0 || code_layout > 3 || nmat < 1 || nmat > 2) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    memset(out, 0, 5 * sizeof(uint32_t));
    smelt_host::Mm1Plan p;
    if (!smelt_host::mm1_plan((smelt_host::CodeLayout)code_layout, rows, cols, group, nmat, lds_limit, force != 0, &p)) return 0;
    out[0] = p.nl; out[1] = p.kc; out[2] = (rows + 7) / 8; out[3] = 64 * p.kc; out[4] = (uint32_t)p.lds;
    return 1;
}

int smelt_hip_resolve_pipeline_name(const char* entry, int default_act, char* symbol, size_t symbol_cap, char* kinds, size_t kinds_cap) {
    if (!entry) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    ResolvedPipeline r;
    std::string why;
    const ResolveStatus st = resolve_pipeline(entry, default_act == SMELT_HIP_ACT_BF16 ? kActBF16 : kActF16, 163840, &r, &why);
    if (st == kResolveMalformed) return SMELT_HIP_ERR_INVALID_PACKAGE;
    if (st == kResolveUnknown) return SMELT_HIP_ERR_UNKNOWN_PIPELINE;
    if (symbol && symbol_cap) snprintf(symbol, symbol_cap, "%s", r.symbol.c_str());
    if (kinds && kinds_cap) snprintf(kinds, kinds_cap, "%s", r.kinds.c_str());
    return SMELT_HIP_OK;
}

}  // extern "C"
