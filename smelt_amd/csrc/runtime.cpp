// libsmelt_hip runtime: the HIP side of Smelt's dispatch-record interpreter.
// Mirrors what SmeltRuntime does with MTLDevice / MTLLibrary / MTLComputePipelineState /
// MTLBuffer / MTLComputeCommandEncoder (SmeltRuntime.swift:668-998, 3150-3275, 5990-6207).
#include <hip/hip_runtime.h>

#include <dirent.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/smelt_hip.h"
#include "pipeline_table.hpp"
#include "runtime_internal.hpp"

using namespace smelt_host;

static_assert(sizeof(SmeltBufferRecord) == 16, "SmeltBufferRecord stride");
static_assert(sizeof(SmeltConstantRecord) == 8, "SmeltConstantRecord stride");
static_assert(sizeof(SmeltDispatchRecord) == 360, "SmeltDispatchRecord stride");
static_assert(offsetof(SmeltDispatchRecord, pipeline) == 2, "pipeline offset");
static_assert(offsetof(SmeltDispatchRecord, min_seq_len) == 8, "minSeqLen offset");
static_assert(offsetof(SmeltDispatchRecord, grid_w) == 12, "gridW offset");
static_assert(offsetof(SmeltDispatchRecord, buffers) == 40, "buffers offset");
static_assert(offsetof(SmeltDispatchRecord, constants) == 296, "constants offset");

namespace {

constexpr int kMaxSlots = 4096;

struct SlotBuffer {
    void* ptr = nullptr;
    size_t bytes = 0;
    bool read_only = false;
};

struct Pipeline {
    std::string entry;
    bool ready = false;
    hipFunction_t fn = nullptr;
    hipFunction_t fn_single = nullptr;  // used when the record's batch argument is 1
    hipFunction_t fn_mm1[kMm1MaxSegments + 1] = {};               // single-pass matrix-core matvec, by segments per wave
    hipFunction_t fn_mm1_t2[kMm1MaxSegments + 1] = {};            // ... two tokens per pass (binary and ternary codes)
    hipFunction_t fn_qmt[5][5][3] = {};                           // token-tile qmm, by row tiles and token blocks per wave and waves along K
    hipFunction_t fn_qmt_per_wave[5][5][3] = {};                  // ... with one matrix per wave along the rows (gate and up)
    hipFunction_t fn_qms[kQmsMaxRowTiles + 1][2] = {};            // streaming skinny qmm, by row tiles per wave and 8 / 16 staged token rows
    hipFunction_t fn_qms_g32[2] = {};                             // ... for groups of 32 columns
    hipFunction_t fn_qss[2] = {};                                 // binary / ternary per-token records over many tokens
    hipFunction_t fn_tqs[2] = {};                                 // streaming ternary qmm, eight / sixteen staged token rows
    hipFunction_t fn_norm_rows = nullptr;                         // norm-scale qmm: the normalised rows, written once
    hipFunction_t fn_logits_keys = nullptr;                       // lm_head over several tokens: partial argmax keys from stored logits
    ResolvedPipeline res;
};

thread_local std::string g_global_error;

}  // namespace

struct smelt_hip_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    int launches = 0;
};

struct smelt_hip_context {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_end = nullptr;
    bool batch_open = false;
    bool timing_valid = false;
    std::vector<hipModule_t> modules;   // every code object loaded so far; kernels are looked up in load order
    int matvec_engine = SMELT_HIP_MATVEC_AUTO;
    std::vector<Pipeline> pipelines;
    std::mutex pipeline_mutex;
    std::vector<SlotBuffer> slots;
    int weights_slot = -1;
    ActDType default_act = kActF16;
    uint32_t cache_seq_capacity = 0;
    // split-K workspace shared by every launch on the stream: partial sums and arrival counters
    // (counters are zero between launches; the last workgroup of each tile resets its own)
    void* ws_partial = nullptr;
    void* ws_counters = nullptr;
    size_t ws_partial_bytes = 0, ws_counter_bytes = 0;
    size_t lds_limit = 65536;
    hipDeviceProp_t props;
    mutable std::string error;
};

namespace {

int fail(const smelt_hip_context* ctx, int code, const std::string& msg) {
    if (ctx) ctx->error = msg;
    else g_global_error = msg;
    return code;
}

int hip_fail(const smelt_hip_context* ctx, hipError_t e, const char* what) {
    return fail(ctx, SMELT_HIP_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
}

#define HIP_TRY(ctx, call)                                      \
    do {                                                        \
        hipError_t _e = (call);                                 \
        if (_e != hipSuccess) return hip_fail(ctx, _e, #call);  \
    } while (0)

struct Arg {
    char kind = 0;  // 'P', 'U', 'F' or 0 (unset)
    uint32_t value = 0;
    char* ptr = nullptr;
    size_t avail = 0;  // bytes from ptr to the end of its slot
    size_t need = 0;   // bytes the pipeline's own kernel touches (set by validate_launch)
    bool writable = false;
};

// Argument list of one launch; fixed capacity, so encoding a record touches no heap.
constexpr size_t kMaxLaunchArgs = 40;
struct ArgList {
    Arg items[kMaxLaunchArgs];
    size_t count = 0;
    size_t size() const { return count; }
    void resize(size_t n) { count = n; }
    void push_back(const Arg& a) { items[count++] = a; }
    Arg& operator[](size_t i) { return items[i]; }
    const Arg& operator[](size_t i) const { return items[i]; }
    const Arg* begin() const { return items; }
    const Arg* end() const { return items + count; }
};

struct Launch {
    ArgList args;
    uint32_t grid[3];
    uint32_t block[3];
    size_t lds = 0;
    // split-K workspace the pipeline's own kernel needs; checked once the kernel that actually runs is
    // known (the streaming kernel a skinny record is re-routed to needs none)
    size_t ws_partial_need = 0, ws_counter_need = 0;
};

size_t cdiv(size_t a, size_t b) { return (a + b - 1) / b; }

// Checks operand extents against what the kernel will touch, and computes its LDS need.
// Every hand-written kernel is only launched after this passes.
int validate_launch(smelt_hip_context* ctx, const Pipeline& p, Launch& L, const SplitKWorkspace& /* checked after routing */) {
    const ResolvedPipeline& r = p.res;
    auto U = [&](size_t i) -> size_t { return L.args[i].value; };
    size_t need[kMaxLaunchArgs] = {};
    bool written[kMaxLaunchArgs] = {};
    size_t align[kMaxLaunchArgs];
    for (size_t i = 0; i < kMaxLaunchArgs; ++i) align[i] = 2;
    const size_t gy = L.grid[1];
    auto bad_geom = [&](const std::string& m) {
        return fail(ctx, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "pipeline '" + p.entry + "': " + m);
    };
    const bool lut_matvec = r.family == kFamLutMatvec || r.family == kFamLutAdd || r.family == kFamLutDual || r.family == kFamLutGateUp ||
                            r.family == kFamLutMatmul;
    const bool plane_matvec = r.family == kFamPlaneMatvec || r.family == kFamPlaneAdd || r.family == kFamPlaneGateUp ||
                              r.family == kFamPlaneBank4 || r.family == kFamPlaneBatched || r.family == kFamBinaryPackedBank || r.family == kFamBinaryPackedBank4 ||
                              r.family == kFamBinaryTwoMatrix;
    const bool norm_scale_matvec = r.family == kFamNormScaleAffineMatvec || r.family == kFamNormScaleAffineGateUp || r.family == kFamNormScaleAffineBatched ||
                                   r.family == kFamNormScaleAffineQmm || r.family == kFamNormScaleAffineQmmGateUp ||
                                   r.family == kFamNormAddScaleAffineMatvec || r.family == kFamNormScaleAffineDual ||
                                   r.family == kFamFusedNormAffineMatvec || r.family == kFamFusedNormAffineGateUp;
    const bool matvec_like = r.family <= kFamAffineBank4 || plane_matvec || lut_matvec || norm_scale_matvec ||
                             r.family == kFamAffineDualAdd || r.family == kFamAffineDualBatched;
    const bool skinny = r.lds_variant == kSkinnyVariant &&
                        (r.family == kFamAffineQmm || r.family == kFamAffineQmmAdd || r.family == kFamAffineQmmGateUp);
    if (matvec_like) {
        if (L.block[0] % 64 != 0 || L.block[0] == 0 || (L.block[0] > 256 && !skinny) || L.block[1] != 1 || L.block[2] != 1)
            return bad_geom("threadgroup must be 64..256 threads in whole wavefronts, got " +
                            std::to_string(L.block[0]) + "x" + std::to_string(L.block[1]) + "x" + std::to_string(L.block[2]));
        if (L.grid[2] != 1) return bad_geom("grid depth must be 1");
    }
    auto affine = [&](size_t w, size_t s, size_t b, size_t rows, size_t cols, size_t group) {
        need[w] = rows * (cols / 2);
        align[w] = 16;
        const size_t gpr = cdiv(cols, group);
        need[s] = need[b] = rows * gpr * 2;
    };
    auto signed_w = [&](size_t c, size_t s, size_t rows, size_t cols) {
        need[c] = rows * (size_t)signed_row_stride(r.format, (uint32_t)cols);
        align[c] = 16;
        need[s] = rows * cdiv(cols, 128) * 2;
    };
    auto check_affine_shape = [&](size_t rows, size_t cols, size_t group) -> int {
        if (rows == 0 || cols == 0 || cols % 32 != 0 || group < 32 || (group & (group - 1)))
            return bad_geom("affine kernels need rows > 0, cols % 32 == 0 and a power-of-two group >= 32");
        return 0;
    };
    auto check_signed_shape = [&](size_t rows, size_t cols) -> int {
        if (rows == 0 || cols == 0 || cols % 128 != 0)
            return bad_geom("signed g128 kernels need rows > 0 and cols % 128 == 0");
        return 0;
    };
    const CodeLayout layout = code_layout(r.format);
    auto signed_lds = [&](size_t cols, uint32_t mb) { return matvec_lds_bytes(layout, signed_row_stride(r.format, (uint32_t)cols), mb); };
    auto plane_lds = [&](size_t cols, uint32_t mb) { return plane_matvec_lds_bytes(signed_row_stride(r.format, (uint32_t)cols), mb); };
    auto need_256 = [&]() -> int {
        if (L.block[0] != 256) return bad_geom("MFMA qmm kernels run with 256-thread workgroups, got " + std::to_string(L.block[0]));
        return 0;
    };
    switch (r.family) {
        case kFamAffineMatvec:
        case kFamAffineAdd: {
            const size_t o = r.family == kFamAffineAdd ? 6 : 5;
            const size_t rows = U(o), cols = U(o + 1), group = U(o + 2);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            affine(0, 1, 2, rows, cols, group);
            need[3] = gy * cols * 2; align[3] = 16;
            need[4] = gy * rows * 2; written[4] = true;
            if (r.family == kFamAffineAdd) need[5] = gy * rows * 2;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamAffineGateUp:
        case kFamAffineDualAdd:
        case kFamAffineDual: {
            const size_t o = r.family == kFamAffineDualAdd ? 11 : (r.family == kFamAffineDual ? 9 : 8);
            const size_t rows = U(o), cols = U(o + 1), group = U(o + 2);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            affine(0, 1, 2, rows, cols, group);
            affine(3, 4, 5, rows, cols, group);
            need[6] = gy * cols * 2; align[6] = 16;
            need[7] = gy * rows * 2; written[7] = true;
            if (r.family != kFamAffineGateUp) { need[8] = gy * rows * 2; written[8] = true; }
            if (r.family == kFamAffineDualAdd) need[9] = need[10] = gy * rows * 2;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamNormScaleAffineMatvec: {
            const size_t rows = U(8), cols = U(9), group = U(10);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            affine(4, 5, 6, rows, cols, group);
            need[0] = gy * 4; align[0] = 4;
            need[1] = gy * cols * 2; align[1] = 16;
            need[2] = cols * 2;
            need[3] = gy * cols * 2; written[3] = true;
            need[7] = gy * rows * 2; written[7] = true;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamFusedNormAffineMatvec: {
            const size_t rows = U(8), cols = U(10), group = U(11);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            if (gy != 1) return bad_geom("the fused-norm kernels take one token");
            affine(3, 4, 5, rows, cols, group);
            need[0] = cols * 2; align[0] = 16;
            need[1] = cols * 2;
            need[2] = cols * 2; written[2] = true;
            need[6] = rows * 2; written[6] = true;
            need[7] = 8; align[7] = 4; written[7] = true;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamFusedNormAffineGateUp: {
            const size_t rows = U(10), cols = U(12), group = U(13);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            if (gy != 1) return bad_geom("the fused-norm kernels take one token");
            affine(2, 3, 4, rows, cols, group);
            affine(5, 6, 7, rows, cols, group);
            need[0] = cols * 2; align[0] = 16;
            need[1] = cols * 2;
            need[8] = rows * 2; written[8] = true;
            need[9] = 8; align[9] = 4; written[9] = true;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamNormAddScaleAffineMatvec: {
            const size_t rows = U(9), cols = U(10), group = U(11);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            affine(5, 6, 7, rows, cols, group);
            need[0] = gy * 4; align[0] = 4;
            need[1] = gy * cols * 2; align[1] = 16;
            need[2] = cols * 2;
            need[3] = gy * cols * 2;
            need[4] = gy * cols * 2; written[4] = true;
            need[8] = gy * rows * 2; written[8] = true;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamNormScaleAffineDual: {
            const size_t rows = U(11), cols = U(12), group = U(13);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            affine(3, 4, 5, rows, cols, group);
            affine(6, 7, 8, rows, cols, group);
            need[0] = gy * 4; align[0] = 4;
            need[1] = gy * cols * 2; align[1] = 16;
            need[2] = cols * 2;
            need[9] = gy * rows * 2; written[9] = true;
            need[10] = gy * rows * 2; written[10] = true;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamNormScaleAffineGateUp: {
            const size_t rows = U(10), cols = U(11), group = U(12);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            affine(3, 4, 5, rows, cols, group);
            affine(6, 7, 8, rows, cols, group);
            need[0] = gy * 4; align[0] = 4;
            need[1] = gy * cols * 2; align[1] = 16;
            need[2] = cols * 2;
            need[9] = gy * rows * 2; written[9] = true;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamNormScaleAffineBatched: {
            const size_t batch = U(8), rows = U(9), cols = U(10), group = U(11), bt = U(12);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            if (bt == 0 || gy * bt < batch) return bad_geom("grid height * batch tile does not cover the batch");
            affine(4, 5, 6, rows, cols, group);
            need[0] = batch * 4; align[0] = 4;
            need[1] = batch * cols * 2; align[1] = 16;
            need[2] = cols * 2;
            need[3] = batch * cols * 2; written[3] = true;
            need[7] = batch * rows * 2; written[7] = true;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), r.lds_variant);
            break;
        }
        case kFamNormScaleAffineQmm:
        case kFamNormScaleAffineQmmGateUp: {
            if (int e = need_256()) return e;
            const bool gate_up = r.family == kFamNormScaleAffineQmmGateUp;
            const size_t o = gate_up ? 10 : 8;
            const size_t batch = U(o), rows = U(o + 1), cols = U(o + 2), group = U(o + 3), bt = U(o + 4);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            if (bt == 0 || gy * bt < batch) return bad_geom("grid height * batch tile does not cover the batch");
            need[0] = batch * 4; align[0] = 4;
            need[1] = batch * cols * 2; align[1] = 16;
            need[2] = cols * 2; align[2] = 16;
            if (gate_up) {
                affine(3, 4, 5, rows, cols, group);
                affine(6, 7, 8, rows, cols, group);
                need[9] = batch * rows * 2; written[9] = true;
            } else {
                need[3] = batch * cols * 2; align[3] = 16; written[3] = true;
                affine(4, 5, 6, rows, cols, group);
                need[7] = batch * rows * 2; written[7] = true;
            }
            L.lds = qmm_affine_lds_bytes(gate_up ? 2 : 1, r.lds_variant);
            break;
        }
        case kFamAffineBatched:
        case kFamAffineDualBatched:
        case kFamAffineGateUpBatched: {
            const size_t o = r.family == kFamAffineDualBatched ? 9 : (r.family == kFamAffineGateUpBatched ? 8 : 5);
            const size_t batch = U(o), rows = U(o + 1), cols = U(o + 2), group = U(o + 3), bt = U(o + 4);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            if (bt == 0 || gy * bt < batch) return bad_geom("grid height * batch tile does not cover the batch");
            affine(0, 1, 2, rows, cols, group);
            size_t xi = 3, yi = 4;
            if (r.family != kFamAffineBatched) { affine(3, 4, 5, rows, cols, group); xi = 6; yi = 7; }
            need[xi] = batch * cols * 2; align[xi] = 16;
            need[yi] = batch * rows * 2; written[yi] = true;
            if (r.family == kFamAffineDualBatched) { need[8] = batch * rows * 2; written[8] = true; }
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), r.lds_variant);
            break;
        }
        case kFamSignedMatvec:
        case kFamSignedAdd: {
            const size_t o = r.family == kFamSignedAdd ? 5 : 4;
            const size_t rows = U(o), cols = U(o + 1);
            if (int e = check_signed_shape(rows, cols)) return e;
            signed_w(0, 1, rows, cols);
            need[2] = gy * cols * 2; align[2] = 16;
            need[3] = gy * rows * 2; written[3] = true;
            if (r.family == kFamSignedAdd) need[4] = gy * rows * 2;
            L.lds = signed_lds(cols, 1);
            break;
        }
        case kFamSignedGateUp: {
            const size_t rows = U(6), cols = U(7);
            if (int e = check_signed_shape(rows, cols)) return e;
            signed_w(0, 1, rows, cols);
            signed_w(2, 3, rows, cols);
            need[4] = gy * cols * 2; align[4] = 16;
            need[5] = gy * rows * 2; written[5] = true;
            L.lds = signed_lds(cols, 1);
            break;
        }
        case kFamSignedB4:
        case kFamSignedGateUpB4: {
            const size_t o = r.family == kFamSignedGateUpB4 ? 6 : 4;
            const size_t rows = U(o), cols = U(o + 1), batch = U(o + 2);
            if (int e = check_signed_shape(rows, cols)) return e;
            if (gy * 4 < batch) return bad_geom("grid height * 4 does not cover the batch");
            signed_w(0, 1, rows, cols);
            size_t xi = 2, yi = 3;
            if (r.family == kFamSignedGateUpB4) { signed_w(2, 3, rows, cols); xi = 4; yi = 5; }
            need[xi] = batch * cols * 2; align[xi] = 16;
            need[yi] = batch * rows * 2; written[yi] = true;
            L.lds = signed_lds(cols, 2);
            break;
        }
        case kFamAffineArgmax: {
            const size_t batch = U(5), rows = U(7), cols = U(8), group = U(9), bt = U(10);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            if (bt == 0 || gy * bt < batch) return bad_geom("grid height * batch tile does not cover the batch");
            if (rows > (1u << 18)) return bad_geom("argmax keys hold 18 index bits");
            affine(0, 1, 2, rows, cols, group);
            need[3] = batch * cols * 2; align[3] = 16;
            need[4] = batch * (size_t)L.grid[0] * 8; align[4] = 8; written[4] = true;
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamLmHeadReduce: {
            const size_t batch = U(2), parts = U(3);
            if ((size_t)L.grid[0] < batch) return bad_geom("one workgroup per batch row is required");
            need[0] = batch * parts * 8; align[0] = 8;
            need[1] = batch * 4; align[1] = 4; written[1] = true;
            break;
        }
        case kFamAffineQmm:
        case kFamAffineQmmAdd:
        case kFamAffineQmmGateUp: {
            if (skinny) {
                const uint32_t max_threads = 512;
                if (L.block[0] < 256 || L.block[0] % 64 != 0 || L.block[0] > max_threads || L.block[1] != 1 || L.block[2] != 1)
                    return bad_geom("skinny qmm runs with 256.." + std::to_string(max_threads) + " threads in whole waves, got " + std::to_string(L.block[0]));
            } else if (int e = need_256()) {
                return e;
            }
            const size_t o = r.family == kFamAffineQmm ? 5 : (r.family == kFamAffineQmmAdd ? 7 : 8);
            const size_t batch = U(o), rows = U(o + 1), cols = U(o + 2), group = U(o + 3), bt = U(o + 4);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            if (bt == 0 || gy * bt < batch) return bad_geom("grid height * batch tile does not cover the batch");
            affine(0, 1, 2, rows, cols, group);
            if (r.family == kFamAffineQmmGateUp) {
                affine(3, 4, 5, rows, cols, group);
                need[6] = batch * cols * 2; align[6] = 16;
                need[7] = batch * rows * 2; written[7] = true;
            } else {
                need[3] = batch * cols * 2; align[3] = 16;
                need[4] = batch * rows * 2; written[4] = true;
                if (r.family == kFamAffineQmmAdd) { need[5] = batch * rows * 2; need[6] = batch * rows * 2; written[6] = true; }
            }
            const uint32_t nmat = r.family == kFamAffineQmmGateUp ? 2 : 1;
            if (r.lds_variant == kSkinnyVariant) {
                const size_t tiles = (rows + 31) / 32;
                if (bt > 32) return bad_geom("skinny qmm handles at most 32 tokens per pass");
                if (L.grid[0] < tiles || L.grid[0] % tiles != 0)
                    return bad_geom("skinny qmm needs grid width = row tiles (" + std::to_string(tiles) + ") * k-splits");
                const uint32_t ksplit = (uint32_t)(L.grid[0] / tiles);
                L.lds = qmm_skinny_lds_bytes((uint32_t)cols, ksplit, nmat, (uint32_t)std::min(batch, bt), L.block[0] / 64);
                if (ksplit > 1) {
                    L.ws_partial_need = (size_t)L.grid[0] * gy * nmat * 4096;
                    L.ws_counter_need = tiles * gy * 4;
                }
                break;
            }
            L.lds = qmm_affine_lds_bytes(nmat, r.lds_variant);
            break;
        }
        case kFamTerAffMatvec:
        case kFamTerAffAdd: {
            const size_t o = r.family == kFamTerAffAdd ? 6 : 5;
            const size_t rows = U(o), cols = U(o + 1);
            if (int e = check_signed_shape(rows, cols)) return e;
            signed_w(0, 1, rows, cols);
            need[2] = need[1];
            need[3] = gy * cols * 2; align[3] = 16;
            need[4] = gy * rows * 2; written[4] = true;
            if (r.family == kFamTerAffAdd) need[5] = gy * rows * 2;
            L.lds = signed_lds(cols, 1);
            break;
        }
        case kFamTerAffGateUp: {
            const size_t rows = U(8), cols = U(9);
            if (int e = check_signed_shape(rows, cols)) return e;
            signed_w(0, 1, rows, cols); need[2] = need[1];
            signed_w(3, 4, rows, cols); need[5] = need[4];
            need[6] = gy * cols * 2; align[6] = 16;
            need[7] = gy * rows * 2; written[7] = true;
            L.lds = signed_lds(cols, 1);
            break;
        }
        case kFamTerAffBank4: {
            const size_t rows = U(8) + U(9) + U(10) + U(11), cols = U(12);
            if (int e = check_signed_shape(rows, cols)) return e;
            if (gy != 1) return bad_geom("projection banks are batch-1 kernels");
            signed_w(0, 1, rows, cols); need[2] = need[1];
            need[3] = cols * 2; align[3] = 16;
            for (size_t m = 0; m < 4; ++m) { need[4 + m] = U(8 + m) * 2; written[4 + m] = U(8 + m) > 0; }
            L.lds = signed_lds(cols, 1);
            break;
        }
        case kFamAffineBank4: {
            const size_t rows = U(8) + U(9) + U(10) + U(11), cols = U(12), group = U(13);
            if (int e = check_affine_shape(rows, cols, group)) return e;
            if (gy != 1) return bad_geom("projection banks are batch-1 kernels");
            affine(0, 1, 2, rows, cols, group);
            need[3] = cols * 2; align[3] = 16;
            for (size_t m = 0; m < 4; ++m) { need[4 + m] = U(8 + m) * 2; written[4 + m] = U(8 + m) > 0; }
            L.lds = matvec_lds_bytes(kCodesU4, (uint32_t)(cols / 2), 1);
            break;
        }
        case kFamTerAffQmm: {
            if (int e = need_256()) return e;
            const size_t rows = U(5), cols = U(6), batch = U(7);
            if (int e = check_signed_shape(rows, cols)) return e;
            if (gy * 32 < batch) return bad_geom("grid height * 32 does not cover the batch");
            signed_w(0, 1, rows, cols); need[2] = need[1];
            need[3] = batch * cols * 2; align[3] = 16;
            need[4] = batch * rows * 2; written[4] = true;
            L.lds = qmm_lds_bytes(1, 2);
            break;
        }
        case kFamAffineGather:
        case kFamAffineGatherBatched: {
            const bool batched = r.family == kFamAffineGatherBatched;
            const size_t cols = U(5), batch = batched ? U(6) : 1, group = batched ? U(7) : U(6);
            if (cols == 0 || cols % 2 != 0 || group == 0 || cols % group != 0)
                return bad_geom("gather needs even cols divisible by the group size");
            need[3] = batch * 4; align[3] = 4;
            need[4] = batch * cols * 2; written[4] = true;
            if (L.grid[0] * (size_t)L.block[0] < cols / 2 || (batched && gy < batch))
                return bad_geom("grid does not cover the gather");
            break;
        }
        case kFamSignedGather: {
            const size_t hidden = U(4);
            if (hidden == 0 || hidden % 128 != 0) return bad_geom("signed gather needs hidden % 128 == 0");
            need[2] = gy * 4; align[2] = 4;
            need[3] = gy * hidden * 2; written[3] = true;
            if (L.grid[0] * (size_t)L.block[0] < hidden) return bad_geom("grid does not cover the gather");
            break;
        }
        case kFamArgmaxPartials: {
            const size_t vocab = U(2), chunk = U(3);
            if (chunk == 0 || (size_t)L.grid[0] * chunk < vocab) return bad_geom("chunks do not cover the vocabulary");
            if (vocab > (1u << 18)) return bad_geom("argmax keys hold 18 index bits");
            need[0] = vocab * 2;
            need[1] = (size_t)L.grid[0] * 8; align[1] = 8; written[1] = true;
            break;
        }
        case kFamArgmaxReduce: {
            need[0] = (size_t)L.grid[0] * U(2) * 8; align[0] = 8;
            need[1] = (size_t)L.grid[0] * 4; align[1] = 4; written[1] = true;
            break;
        }
        case kFamCopy: {
            need[0] = U(2) * 16; align[0] = 16;
            need[1] = U(2) * 16; align[1] = 16; written[1] = true;
            break;
        }
        case kFamRmsNorm:
        case kFamRmsNormAdd:
        case kFamRmsScale:
        case kFamResidualAddRmsScale: {
            // one workgroup per token row; the row is staged in LDS
            const bool norm = r.family == kFamRmsNorm || r.family == kFamRmsNormAdd;
            const size_t first_u = r.family == kFamRmsNorm ? 3 : (r.family == kFamRmsScale ? 2 : 4);
            const size_t dim = U(first_u), tokens = L.grid[0];
            if (dim == 0) return bad_geom("dim must be positive");
            if (L.block[0] % 64 != 0 || L.block[1] != 1 || L.block[2] != 1 || L.grid[1] != 1 || L.grid[2] != 1)
                return bad_geom("norm kernels run whole waves in a 1-D launch, one workgroup per token");
            const size_t row = tokens * dim * 2;
            if (norm) {
                need[0] = row; need[1] = dim * 2;
                if (r.family == kFamRmsNormAdd) { need[2] = row; need[3] = row; written[3] = true; }
                else { need[2] = row; written[2] = true; }
            } else if (r.family == kFamRmsScale) {
                need[0] = row; need[1] = tokens * 4; align[1] = 4; written[1] = true;
            } else {
                need[0] = row; need[1] = row; need[2] = row; written[2] = true;
                need[3] = tokens * 4; align[3] = 4; written[3] = true;
            }
            L.lds = 64 + dim * 2;
            break;
        }
        case kFamRmsNormGated:
        case kFamRmsNormGatedBatched:
        case kFamRmsNormGatedPlanes: {
            // one workgroup (32 threads or whole waves) per head
            const bool batched = r.family == kFamRmsNormGatedBatched, view = r.family == kFamRmsNormGatedPlanes;
            const size_t dim = U(batched ? 5 : (view ? 5 : 4));
            if (dim == 0) return bad_geom("head_dim must be positive");
            if ((L.block[0] != 32 && L.block[0] % 64 != 0) || L.block[1] != 1 || L.block[2] != 1 || L.grid[2] != 1)
                return bad_geom("gated norm kernels run 32 threads or whole waves per workgroup");
            if (!batched && L.grid[1] != 1) return bad_geom("one token per launch");
            if (batched && U(4) != L.grid[0]) return bad_geom("grid width must equal the heads per token");
            const size_t heads = (size_t)L.grid[0] * L.grid[1];
            need[0] = heads * dim * 2; need[1] = heads * dim * 2; need[2] = dim * 2;
            if (view) {
                if (dim != 128) return bad_geom("the gated-norm view producer takes heads of 128 values");
                need[3] = heads * 6 * 16; align[3] = 16; written[3] = true;
                need[4] = heads * 2; written[4] = true;
            } else {
                need[3] = heads * dim * 2; written[3] = true;
            }
            break;
        }
        case kFamRmsNormAddScalar:
        case kFamRmsNormFromFp32: {
            const size_t first_u = r.family == kFamRmsNormAddScalar ? 5 : 3;
            const size_t dim = U(first_u), tokens = L.grid[0];
            if (dim == 0) return bad_geom("dim must be positive");
            if (L.block[0] % 64 != 0 || L.block[1] != 1 || L.block[2] != 1 || L.grid[1] != 1 || L.grid[2] != 1)
                return bad_geom("norm kernels run whole waves in a 1-D launch, one workgroup per row");
            const size_t row = tokens * dim * 2;
            if (r.family == kFamRmsNormAddScalar) {
                need[0] = row; need[1] = dim * 2; need[2] = row; need[3] = 2; need[4] = row; written[4] = true;
            } else {
                need[0] = tokens * dim * 4; align[0] = 4; need[1] = dim * 2; need[2] = row; written[2] = true;
            }
            L.lds = 64 + dim * 2;
            break;
        }
        case kFamUnary:
        case kFamScalarMul:
        case kFamScalarMulWeight: {
            const size_t count = U(r.family == kFamUnary ? 2 : 3);
            if (L.block[1] != 1 || L.block[2] != 1 || L.grid[1] != 1 || L.grid[2] != 1) return bad_geom("1-D launch expected");
            if ((size_t)L.grid[0] * L.block[0] < count) return bad_geom("grid covers " + std::to_string((size_t)L.grid[0] * L.block[0]) + " of " + std::to_string(count) + " elements");
            need[0] = count * 2;
            if (r.family == kFamScalarMulWeight) { need[1] = 2; need[2] = count * 2; written[2] = true; }
            else { need[1] = count * 2; written[1] = true; }
            break;
        }
        case kFamGegluStridedBatched:
        case kFamBiasAddBatched: {
            const bool geglu = r.family == kFamGegluStridedBatched;
            const size_t count = U(3), stride = geglu ? U(4) : 0;
            if (L.block[1] != 1 || L.block[2] != 1 || L.grid[2] != 1) return bad_geom("threads x tokens launch expected");
            if (count == 0 || gy == 0) return bad_geom("count and token rows must be positive");
            if ((size_t)L.grid[0] * L.block[0] < count) return bad_geom("grid covers " + std::to_string((size_t)L.grid[0] * L.block[0]) + " of " + std::to_string(count) + " elements");
            need[0] = gy * count * 2;
            need[1] = geglu ? ((gy - 1) * stride + count) * 2 : count * 2;
            need[2] = gy * count * 2; written[2] = true;
            break;
        }
        case kFamElementwise:
        case kFamCopy16: {
            const size_t ci = r.family == kFamCopy16 ? 2 : 3;
            const size_t count = U(ci);
            if (L.block[1] != 1 || L.block[2] != 1 || L.grid[1] != 1 || L.grid[2] != 1) return bad_geom("1-D launch expected");
            if ((size_t)L.grid[0] * L.block[0] < count) return bad_geom("grid covers " + std::to_string((size_t)L.grid[0] * L.block[0]) + " of " + std::to_string(count) + " elements");
            for (size_t i = 0; i < ci; ++i) need[i] = count * 2;
            written[ci - 1] = true;
            break;
        }
        case kFamLutMatvec:
        case kFamLutAdd:
        case kFamLutDual:
        case kFamLutGateUp: {
            // [W lut]+ x y [y2 | res] rows cols group
            const size_t nmat = (r.family == kFamLutDual || r.family == kFamLutGateUp) ? 2 : 1;
            const size_t xi = 2 * nmat;
            const size_t ri = r.family == kFamLutMatvec ? 4 : (r.family == kFamLutAdd ? 5 : (r.family == kFamLutDual ? 7 : 6));
            const size_t rows = U(ri), cols = U(ri + 1), group = U(ri + 2);
            if (rows == 0 || cols == 0 || cols % 32 != 0 || group < 8) return bad_geom("u4_lut kernels need rows > 0, cols % 32 == 0 and at least 8 rows per table");
            if (gy != 1) return bad_geom("u4_lut kernels take one token");
            for (size_t m = 0; m < nmat; ++m) {
                need[2 * m] = rows * (cols / 2); align[2 * m] = 16;
                need[2 * m + 1] = cdiv(rows, group) * 32;
            }
            need[xi] = cols * 2; align[xi] = 16;
            need[xi + 1] = rows * 2; written[xi + 1] = true;
            if (r.family == kFamLutDual) { need[xi + 2] = rows * 2; written[xi + 2] = true; }
            if (r.family == kFamLutAdd) need[xi + 2] = rows * 2;
            L.lds = cols * 2 + (L.block[0] / 64) * nmat * 4 * 1024;
            break;
        }
        case kFamLutMatmul: {
            const size_t cols = U(4), group = U(5), rows = U(6);
            if (rows == 0 || cols == 0 || cols % 32 != 0 || group < 8) return bad_geom("u4_lut kernels need rows > 0, cols % 32 == 0 and at least 8 rows per table");
            need[0] = rows * (cols / 2); align[0] = 16;
            need[1] = cdiv(rows, group) * 32;
            need[2] = gy * cols * 2; align[2] = 16;
            need[3] = gy * rows * 2; written[3] = true;
            L.lds = cols * 2 + (L.block[0] / 64) * 4 * 1024;
            break;
        }
        case kFamLutGather: {
            // W lut token out cols group
            const size_t cols = U(4), group = U(5);
            if (cols == 0 || cols % 2 != 0 || group == 0) return bad_geom("gather needs an even hidden size and a positive group");
            if ((size_t)L.grid[0] * L.block[0] < cols / 2) return bad_geom("grid does not cover hidden / 2 threads");
            if (L.grid[1] != 1 || L.grid[2] != 1 || L.block[1] != 1 || L.block[2] != 1) return bad_geom("1-D launch expected");
            need[2] = 4; align[2] = 4;
            need[3] = cols * 2; written[3] = true;
            // rows are data (the token id): the table must at least hold one row and one table
            need[0] = cols / 2; need[1] = 32;
            break;
        }
        case kFamTqhPrepare: {
            // x xhat cols; dispatchThreads over groups * 128, grid.y = token
            const size_t cols = U(2), groups = cdiv(cols, 128);
            if (cols == 0) return bad_geom("cols must be positive");
            if ((size_t)L.grid[0] * L.block[0] < groups * 128) return bad_geom("grid does not cover groups * 128 threads");
            if (L.grid[2] != 1 || L.block[1] != 1 || L.block[2] != 1) return bad_geom("1-D workgroups expected");
            need[0] = gy * cols * 2;
            need[1] = gy * groups * 128 * 4; align[1] = 16; written[1] = true;
            break;
        }
        case kFamTqhMatvec: {
            // codes codebook xhat y rows cols codes_per_row; grid.y = token
            const size_t rows = U(4), cols = U(5), cpr = U(6), groups = cdiv(cols, 128);
            if (rows == 0 || cols == 0) return bad_geom("rows and cols must be positive");
            if (cpr != groups * 32) return bad_geom("codes_per_row must be 32 bytes per 128-column group");
            if (L.block[0] % 64 != 0 || L.block[0] > 256 || L.block[1] != 1 || L.block[2] != 1 || L.grid[2] != 1)
                return bad_geom("tqh_matvec runs 64..256 threads in whole waves");
            need[0] = rows * cpr; align[0] = 16;
            need[1] = groups * 8; align[1] = 8;
            need[2] = gy * groups * 128 * 4; align[2] = 16;
            need[3] = gy * rows * 2; written[3] = true;
            {
                // rotated activations at 272 bytes per 64-value unit (bank padding), then per wave one
                // float4 of partial sums per (row quad, unit) item; the quad bound follows the kernel's
                // own rule (tqh_max_quads_per_tile in tqh_kernels.hpp)
                const size_t units = groups * 2, waves = L.block[0] / 64;
                size_t low = units & (0 - units);
                if (low > 64) low = 64;
                size_t q = 64 / low;
                if (q > 8) q = 8;
                while (q > 1 && q * units * 16 * waves > 32768) q >>= 1;
                L.lds = units * 17 * 16 + waves * q * units * 16;
            }
            break;
        }
        case kFamTqhGather: {
            // codes codebook token out codes_per_row cols
            const size_t cpr = U(4), cols = U(5), groups = cdiv(cols, 128);
            if (cols == 0 || cpr != groups * 32) return bad_geom("codes_per_row must be 32 bytes per 128-column group");
            if ((size_t)L.grid[0] * L.block[0] < cols) return bad_geom("grid does not cover the row");
            if (L.grid[1] != 1 || L.grid[2] != 1 || L.block[1] != 1 || L.block[2] != 1) return bad_geom("1-D launch expected");
            need[0] = cpr; need[1] = groups * 8;
            need[2] = 4; align[2] = 4;
            need[3] = cols * 2; written[3] = true;
            break;
        }
        case kFamPlaneBatched: {
            // C S planes ascales Y rows cols batch nplanes tile
            const size_t rows = U(5), cols = U(6), batch = U(7), nplanes = U(8), tile = U(9);
            if (int e = check_signed_shape(rows, cols)) return e;
            if (nplanes < 2 || nplanes > 6) return bad_geom("activation views hold 2 to 6 planes");
            if (batch == 0 || gy * tile < batch) return bad_geom("grid height * token tile does not cover the batch");
            signed_w(0, 1, rows, cols);
            need[2] = batch * (cols / 128) * nplanes * 16; align[2] = 16;
            need[3] = batch * (cols / 128) * 2;
            need[4] = batch * rows * 2; written[4] = true;
            L.lds = plane_lds(cols, 4);
            break;
        }
        case kFamPlaneBank4:
        case kFamBinaryPackedBank:
        case kFamBinaryPackedBank4: {
            // C S (planes ascales | x) y0 .. y{n-1} rows0 .. rows{n-1} cols [nplanes]; one token
            const bool view = r.family == kFamPlaneBank4;
            const size_t nout = r.family == kFamBinaryPackedBank ? 2 : 4;
            const size_t y0 = view ? 4 : 3, r0 = y0 + nout, ci = r0 + nout;
            const size_t cols = U(ci);
            size_t rows = 0;
            for (size_t m = 0; m < nout; ++m) rows += U(r0 + m);
            if (int e = check_signed_shape(rows, cols)) return e;
            if (gy != 1) return bad_geom("projection-bank kernels take one token");
            signed_w(0, 1, rows, cols);
            if (view) {
                const size_t nplanes = U(ci + 1);
                if (nplanes < 2 || nplanes > 6) return bad_geom("activation views hold 2 to 6 planes");
                need[2] = (cols / 128) * nplanes * 16; align[2] = 16;
                need[3] = (cols / 128) * 2;
            } else {
                need[2] = cols * 2; align[2] = 16;
            }
            for (size_t m = 0; m < nout; ++m) {
                need[y0 + m] = U(r0 + m) * 2;
                written[y0 + m] = true;
            }
            L.lds = view ? plane_lds(cols, 1) : signed_lds(cols, 1);
            break;
        }
        case kFamBinaryTwoMatrix: {
            // C1 S1 C2 S2 x y1 y2 rows1 rows2 cols
            const size_t rows1 = U(7), rows2 = U(8), cols = U(9);
            if (int e = check_signed_shape(rows1 + rows2, cols)) return e;
            if (gy != 1) return bad_geom("projection-bank kernels take one token");
            signed_w(0, 1, rows1, cols);
            signed_w(2, 3, rows2, cols);
            need[4] = cols * 2; align[4] = 16;
            need[5] = rows1 * 2; written[5] = true;
            need[6] = rows2 * 2; written[6] = true;
            L.lds = signed_lds(cols, 1);
            break;
        }
        case kFamPlaneMatvec:
        case kFamPlaneAdd:
        case kFamPlaneGateUp: {
            // C S [uC uS] planes ascales Y [res] rows cols nplanes
            const size_t pi = r.family == kFamPlaneGateUp ? 4 : 2;               // planes argument
            const size_t ri = r.family == kFamPlaneMatvec ? 5 : (r.family == kFamPlaneAdd ? 6 : 7);
            const size_t rows = U(ri), cols = U(ri + 1), nplanes = U(ri + 2);
            if (int e = check_signed_shape(rows, cols)) return e;
            if (nplanes < 2 || nplanes > 6) return bad_geom("activation views hold 2 to 6 planes");
            signed_w(0, 1, rows, cols);
            if (r.family == kFamPlaneGateUp) signed_w(2, 3, rows, cols);
            const size_t groups = cols / 128;
            need[pi] = gy * groups * nplanes * 16; align[pi] = 16;
            need[pi + 1] = gy * groups * 2;
            need[pi + 2] = gy * rows * 2; written[pi + 2] = true;
            if (r.family == kFamPlaneAdd) need[pi + 3] = gy * rows * 2;
            L.lds = plane_lds(cols, 1);
            break;
        }
        case kFamActivationPlanes:
        case kFamSwigluPlanes:
        case kFamNormScalePlanes: {
            // [norm_scale] a [b] planes scales cols nplanes; one wave per 128-value group, grid.y = token
            const size_t ai = r.family == kFamNormScalePlanes ? 1 : 0;
            const size_t pl = r.family == kFamActivationPlanes ? 1 : (r.family == kFamSwigluPlanes ? 2 : 3);
            const size_t cols = U(pl + 2), nplanes = U(pl + 3), tokens = gy;
            if (cols == 0 || cols % 128 != 0) return bad_geom("activation views need cols % 128 == 0");
            if (nplanes < 2 || nplanes > 6) return bad_geom("activation views hold 2 to 6 planes");
            if ((L.block[0] != 32 && L.block[0] % 64 != 0) || L.block[1] != 1 || L.block[2] != 1 || L.grid[2] != 1)
                return bad_geom("activation-view producers run 32 threads or whole waves per workgroup");
            if (r.family == kFamNormScalePlanes) {
                if (tokens != 1) return bad_geom("the norm-scale producer takes one token");
                need[0] = 4; align[0] = 4;
                need[2] = cols * 2;
            }
            need[ai] = tokens * cols * 2;
            if (r.family == kFamSwigluPlanes) need[1] = tokens * cols * 2;
            need[pl] = tokens * (cols / 128) * nplanes * 16; align[pl] = 16; written[pl] = true;
            need[pl + 1] = tokens * (cols / 128) * 2; written[pl + 1] = true;
            break;
        }
        case kFamAffineQuantize: {
            // src packed scales biases importance rows src_dtype clip cols group
            const size_t rows = U(5), dt = U(6), clip = U(7), cols = U(8), group = U(9);
            if (dt > 2) return bad_geom("source dtype must be 0 (fp32), 1 (fp16) or 2 (bf16)");
            if (clip > 1) return bad_geom("clip mode must be 0 (min/max) or 1 (least reconstruction error)");
            if (rows == 0) return bad_geom("rows must be positive");
            const size_t gpr = cdiv(cols, group);
            if (rows * gpr >= ((size_t)1 << 31)) return bad_geom("more than 2^31 groups in one tensor");
            const size_t waves = 128 / group;  // about 34 KB of staging per workgroup
            if (L.block[0] != waves * 64 || L.block[1] != 1 || L.block[2] != 1 || L.grid[1] != 1 || L.grid[2] != 1)
                return bad_geom("group " + std::to_string(group) + " quantiser runs with " + std::to_string(waves * 64) + "-thread workgroups in a 1-D grid");
            need[0] = rows * cols * (dt == 0 ? 4 : 2); align[0] = dt == 0 ? 4 : 2;
            need[1] = rows * cdiv(cols, 2); align[1] = 1; written[1] = true;
            need[2] = rows * gpr * 2; written[2] = true;
            need[3] = rows * gpr * 2; written[3] = true;
            if (L.args[4].kind == 'P') { need[4] = cols * 4; align[4] = 4; }
            L.lds = waves * (64 * (group + 1) + 128) * 4;
            break;
        }
        case kFamSignedValidate: {
            // codes status count_lo count_hi format
            const size_t count = ((size_t)U(3) << 32) | U(2);
            if (U(4) != 1 && U(4) != 2) return bad_geom("format must be 1 (ternary2) or 2 (trit5)");
            need[0] = U(4) == 2 ? cdiv(count, 5) : cdiv(count * 2, 8); align[0] = 1;
            need[1] = 8; align[1] = 8; written[1] = true;
            if (L.grid[1] != 1 || L.grid[2] != 1 || L.block[1] != 1 || L.block[2] != 1) return bad_geom("1-D launch expected");
            break;
        }
        case kFamSignedMlxScales: {
            // scales biases out status groups format
            if (U(5) > 1) return bad_geom("format must be 0 (binary1) or 1 (ternary2)");
            need[0] = U(4) * 2; need[1] = U(4) * 2;
            need[2] = U(4) * 2; written[2] = true;
            need[3] = 8; align[3] = 8; written[3] = true;
            if (L.grid[1] != 1 || L.grid[2] != 1 || L.block[1] != 1 || L.block[2] != 1) return bad_geom("1-D launch expected");
            break;
        }
        default:
            return fail(ctx, SMELT_HIP_ERR_UNKNOWN_PIPELINE, "pipeline '" + p.entry + "' has no launch validator");
    }
    if (L.lds > ctx->lds_limit)
        return bad_geom("needs " + std::to_string(L.lds) + " bytes of LDS, device allows " + std::to_string(ctx->lds_limit));
    for (size_t i = 0; i < L.args.size(); ++i) {
        if (L.args[i].kind != 'P') continue;
        L.args[i].need = need[i];
        if (need[i] > L.args[i].avail)
            return fail(ctx, SMELT_HIP_ERR_OUT_OF_RANGE,
                        "pipeline '" + p.entry + "': argument " + std::to_string(i) + " needs " +
                            std::to_string(need[i]) + " bytes, slot has " + std::to_string(L.args[i].avail) + " from its offset");
        if (((uintptr_t)L.args[i].ptr) % align[i] != 0)
            return fail(ctx, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY,
                        "pipeline '" + p.entry + "': argument " + std::to_string(i) + " must be " + std::to_string(align[i]) + "-byte aligned");
        if (written[i] && !L.args[i].writable)
            return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT,
                        "pipeline '" + p.entry + "': output argument " + std::to_string(i) + " is bound to the read-only weights slot");
    }
    return 0;
}

struct Dyn {
    bool prefill;
    int32_t position;  // decode
    int32_t seq_len, start_pos;
};

// resolveDispatchBufferOffset: SmeltRuntime.swift:6158-6184; decode form :3207-3209
int resolve_offset(smelt_hip_context* ctx, const SmeltBufferRecord& b, const Dyn& d, size_t* out) {
    if (!d.prefill) {
        *out = b.offset_kind == 0 ? (size_t)b.offset : (size_t)((int64_t)d.position * (int64_t)b.offset);
        return 0;
    }
    switch (b.offset_kind) {
        case 0: *out = (size_t)b.offset; return 0;
        case 1: *out = (size_t)((int64_t)d.start_pos * (int64_t)b.offset); return 0;
        case 2: *out = (size_t)((int64_t)d.start_pos * (int64_t)(b.offset & 0xFFFFFFFFu) + (int64_t)(b.offset >> 32)); return 0;
        case 3: *out = (size_t)((int64_t)(d.seq_len - 1) * (int64_t)b.offset); return 0;
        case 4: {
            const int64_t stride = (int64_t)(b.offset & 0xFFFFFFFFu);
            const int64_t divisor = std::max<int64_t>((int64_t)(b.offset >> 32), 1);
            *out = (size_t)(((int64_t)d.seq_len / divisor) * stride);
            return 0;
        }
        default:
            return fail(ctx, SMELT_HIP_ERR_INVALID_PACKAGE,
                        "unknown dispatch offsetKind " + std::to_string(b.offset_kind) + " - emitter/runtime mismatch");
    }
}

// resolveDecodeConstant / resolvePrefillConstant: SmeltRuntime.swift:1189-1252
uint32_t resolve_constant(const smelt_hip_context* ctx, const SmeltConstantRecord& c, const Dyn& d, bool* skip) {
    if (!d.prefill) {
        switch (c.kind) {
            case SMELT_CONST_POSITION: return (uint32_t)d.position;
            case SMELT_CONST_POSITION_PLUS1: return (uint32_t)(d.position + 1);
            case SMELT_CONST_POSITION_PLUS1_LT_LITERAL_SKIP_IF_FALSE: {
                const uint32_t v = (uint32_t)(d.position + 1) < c.value ? 1 : 0;
                if (!v) *skip = true;
                return v;
            }
            case SMELT_CONST_POSITION_PLUS1_GE_LITERAL_SKIP_IF_FALSE: {
                const uint32_t v = (uint32_t)(d.position + 1) >= c.value ? 1 : 0;
                if (!v) *skip = true;
                return v;
            }
            case SMELT_CONST_CACHE_SEQ_CAPACITY: return ctx->cache_seq_capacity;
            default: return c.value;
        }
    }
    const uint32_t s = (uint32_t)d.seq_len, p = (uint32_t)d.start_pos;
    switch (c.kind) {
        case SMELT_CONST_POSITION: return p;
        case SMELT_CONST_POSITION_PLUS1: return p + 1;
        case SMELT_CONST_SEQ_LEN: return s;
        case SMELT_CONST_SEQ_LEN_MUL_LITERAL: return s * c.value;
        case SMELT_CONST_SEQ_LEN_MOD_LITERAL: return c.value == 0 ? 0 : s % c.value;
        case SMELT_CONST_SEQ_LEN_MOD_LITERAL_SKIP_IF_ZERO: {
            const uint32_t v = c.value == 0 ? 0 : s % c.value;
            if (!v) *skip = true;
            return v;
        }
        case SMELT_CONST_SEQ_LEN_LT_LITERAL_SKIP_IF_FALSE: {
            const uint32_t v = s < c.value ? 1 : 0;
            if (!v) *skip = true;
            return v;
        }
        case SMELT_CONST_START_POS: return p;
        case SMELT_CONST_START_POS_PLUS_LITERAL: return p + c.value;
        case SMELT_CONST_CACHE_SEQ_CAPACITY: return ctx->cache_seq_capacity;
        default: return c.value;
    }
}

// resolvePrefillGrid: SmeltRuntime.swift:6186-6207
uint32_t resolve_grid(uint32_t literal, uint8_t kind, int32_t seq_len) {
    const int64_t s = std::max<int64_t>(seq_len, 0);
    switch (kind) {
        case SMELT_GRID_SEQ_LEN: return (uint32_t)s;
        case SMELT_GRID_SEQ_LEN_MUL_LITERAL: return (uint32_t)(s * (int64_t)literal);
        case SMELT_GRID_SEQ_LEN_CEIL_DIV_LITERAL: {
            const int64_t divisor = std::max<int64_t>(literal & 0x7FFFFFFFu, 1);
            if (literal & 0x80000000u) return (uint32_t)(s / divisor);
            return (uint32_t)((s + divisor - 1) / divisor);
        }
        default: return literal;
    }
}

const Pipeline* pipeline_for(smelt_hip_context* ctx, uint32_t index) {
    // "fallback to previous": SmeltRuntime.swift:453-456, 6305-6306
    std::lock_guard<std::mutex> lock(ctx->pipeline_mutex);
    if (index >= ctx->pipelines.size()) return nullptr;
    for (int64_t i = index; i >= 0; --i)
        if (ctx->pipelines[(size_t)i].ready) return &ctx->pipelines[(size_t)i];
    return nullptr;
}

// Returns 1 launched, 0 skipped, <0 error.
int encode_record(smelt_hip_context* ctx, const SmeltDispatchRecord* rec, int cur, int alt, const Dyn& d,
                  const SplitKWorkspace* ws_override = nullptr) {
    if (!ctx || !rec) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context or record");
    SplitKWorkspace ws;
    if (ws_override) ws = *ws_override;
    else { ws.partial = ctx->ws_partial; ws.counters = ctx->ws_counters; ws.partial_bytes = ctx->ws_partial_bytes; ws.counter_bytes = ctx->ws_counter_bytes; }
    if (rec->op_kind != SMELT_OP_DISPATCH) return 0;
    if (d.prefill && rec->min_seq_len > 0 && (uint32_t)d.seq_len < (uint32_t)rec->min_seq_len) return 0;
    if (rec->buffer_count > SMELT_MAX_BUFFERS_PER_DISPATCH || rec->constant_count > SMELT_MAX_CONSTANTS_PER_DISPATCH)
        return fail(ctx, SMELT_HIP_ERR_INVALID_PACKAGE, "record binding counts exceed the table format");
    const Pipeline* p = pipeline_for(ctx, rec->pipeline);
    if (!p) return fail(ctx, SMELT_HIP_ERR_UNKNOWN_PIPELINE, "record names pipeline index " + std::to_string(rec->pipeline) + " which has no launchable kernel");

    const std::string& kinds = p->res.kinds;
    if (kinds.size() + 1 > kMaxLaunchArgs)
        return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "pipeline '" + p->entry + "' has too many arguments");
    Launch L;
    L.args.resize(kinds.size());
    const size_t own = kinds.size() - p->res.appended.size();
    for (int i = 0; i < rec->buffer_count; ++i) {
        const SmeltBufferRecord& b = rec->buffers[i];
        int slot = b.slot >= 0 ? b.slot : (b.slot == SMELT_SLOT_CUR ? cur : alt);
        if (slot < 0 || (size_t)slot >= ctx->slots.size() || !ctx->slots[(size_t)slot].ptr)
            return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "record binds slot " + std::to_string(slot) + " which has no buffer");
        size_t off = 0;
        if (int e = resolve_offset(ctx, b, d, &off)) return e;
        const SlotBuffer& sb = ctx->slots[(size_t)slot];
        if (off > sb.bytes)
            return fail(ctx, SMELT_HIP_ERR_OUT_OF_RANGE, slot == ctx->weights_slot
                            ? "weight offset " + std::to_string(off) + " is outside the mapped weight segments"
                            : "offset " + std::to_string(off) + " is outside slot " + std::to_string(slot));
        if (b.binding_index >= own || kinds[b.binding_index] != 'P')
            return fail(ctx, SMELT_HIP_ERR_BINDING_MISMATCH, "pipeline '" + p->entry + "' takes no buffer at index " + std::to_string(b.binding_index));
        Arg& a = L.args[b.binding_index];
        a.kind = 'P';
        a.ptr = (char*)sb.ptr + off;
        a.avail = sb.bytes - off;
        a.writable = !sb.read_only;
    }
    bool skip = false;
    for (int i = 0; i < rec->constant_count; ++i) {
        const SmeltConstantRecord& c = rec->constants[i];
        const uint32_t v = resolve_constant(ctx, c, d, &skip);
        if (c.binding_index == 0xFF) continue;
        if (c.binding_index >= own || kinds[c.binding_index] == 'P')
            return fail(ctx, SMELT_HIP_ERR_BINDING_MISMATCH, "pipeline '" + p->entry + "' takes no constant at index " + std::to_string(c.binding_index));
        Arg& a = L.args[c.binding_index];
        a.kind = kinds[c.binding_index];
        a.value = v;
    }
    if (skip) return 0;
    for (size_t i = 0; i < p->res.appended.size(); ++i) {
        Arg& a = L.args[own + i];
        a.kind = 'U';
        a.value = p->res.appended[i];
    }
    for (size_t i = 0; i < L.args.size(); ++i)
        if (L.args[i].kind == 0 && kinds[i] == 'Z') L.args[i].kind = 'Z';  // optional pointer: null
    for (size_t i = 0; i < L.args.size(); ++i)
        if (L.args[i].kind == 0)
            return fail(ctx, SMELT_HIP_ERR_BINDING_MISMATCH, "pipeline '" + p->entry + "': argument " + std::to_string(i) + " is not bound by the record");

    uint32_t gw = rec->grid_w, gh = rec->grid_h, gd = rec->grid_d;
    if (d.prefill) {
        gw = resolve_grid(rec->grid_w, (rec->style >> 2) & 3, d.seq_len);
        gh = resolve_grid(rec->grid_h, (rec->style >> 4) & 3, d.seq_len);
        gd = resolve_grid(rec->grid_d, (rec->style >> 6) & 3, d.seq_len);
    }
    if (gw == 0 || gh == 0 || gd == 0) return 0;
    if (rec->tg_w == 0 || rec->tg_h == 0 || rec->tg_d == 0)
        return fail(ctx, SMELT_HIP_ERR_INVALID_PACKAGE, "record has an empty threadgroup");
    L.block[0] = rec->tg_w; L.block[1] = rec->tg_h; L.block[2] = rec->tg_d;
    if ((rec->style & 3) == SMELT_STYLE_THREADGROUPS) {
        L.grid[0] = gw; L.grid[1] = gh; L.grid[2] = gd;
    } else {  // dispatchThreads: grid counts threads; kernels bounds-check the ragged edge
        L.grid[0] = (uint32_t)cdiv(gw, rec->tg_w);
        L.grid[1] = (uint32_t)cdiv(gh, rec->tg_h);
        L.grid[2] = (uint32_t)cdiv(gd, rec->tg_d);
    }
    if ((size_t)L.block[0] * L.block[1] * L.block[2] > 1024)
        return fail(ctx, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY, "threadgroup exceeds 1024 threads");
    if (int e = validate_launch(ctx, *p, L, ws)) return e;
    hipFunction_t fn = p->fn;
    bool routed = false, qms_routed = false;
    // the re-routed kernels fetch codes, scales, biases and activations 16 bytes at a time: the
    // first `n` arguments (the read-only operands) have to sit on 16-byte boundaries, as the layouts
    // the library writes do; a record that binds them elsewhere keeps the kernel its name describes
    auto aligned16 = [&](size_t n, size_t first = 0) {
        for (size_t i = first; i < n && i < L.args.size(); ++i)
            if (L.args[i].kind == 'P' && (reinterpret_cast<uintptr_t>(L.args[i].ptr) & 15u)) return false;
        return true;
    };
    // ... and in whole 16-byte pieces: a plane whose validated extent ends inside a piece (rows * groups * 2
    // not a multiple of 16) must have the rest of that piece inside its slot as well
    auto whole_pieces = [&](size_t n, size_t first = 0) {
        for (size_t i = first; i < n && i < L.args.size(); ++i)
            if (L.args[i].kind == 'P' && ((L.args[i].need + 15) & ~(size_t)15) > L.args[i].avail) return false;
        return true;
    };
    const bool mm1_b4 = p->res.family == kFamSignedB4 || p->res.family == kFamSignedGateUpB4;
    // (the single-token families of the binary and ternary codes: with several grid rows, two tokens per pass)
    const bool mm1_per_row = p->res.family == kFamSignedMatvec || p->res.family == kFamSignedAdd || p->res.family == kFamSignedGateUp ||
                             p->res.family == kFamTerAffMatvec || p->res.family == kFamTerAffAdd || p->res.family == kFamTerAffGateUp;
    // the per-token small-batch forms of the affine matvec and gate+up (W S B X Y batch | rows cols group tile): a few
    // tokens of a small matrix are launch-bound, and the single-token kernel with a grid row per token is the shorter
    // launch while tokens x weights stay below about 20M (cold, streaming kernel against a grid row per token:
    // 1024 x 1024 at 2 / 4 / 8 / 16 tokens 4.4 / 4.5 / 4.5 / 4.7 us against 2.5 / 2.8 / 3.2 / 4.0; 2048 x 2048 at 2 / 4 / 6
    // 4.8 / 4.9 / 4.9 against 3.3 / 4.0 / 5.1; 6144 x 1024 at 3 / 4 4.9 / 4.9 against 4.5 / 5.2; 4096 x 4096 at 2 5.5 against 5.7)
    // (not the skinny and token-slab qmm names: their fused-add sibling writes two outputs, has no such form and
    // would no longer match the plain record bit for bit)
    const bool mm1_pair_batch = p->res.family == kFamAffineGateUpBatched;
    const bool mm1_batch_family = p->res.family == kFamAffineBatched || mm1_pair_batch;
    bool mm1_small_batch = false;
    if (mm1_batch_family && p->res.mm1_layout >= 0) {
        const size_t o = mm1_pair_batch ? 8 : 5;
        const uint64_t batch = L.args[o].value, weights = (uint64_t)L.args[o + 1].value * L.args[o + 2].value * (mm1_pair_batch ? 2 : 1);
        mm1_small_batch = batch >= 1 && batch <= 16 && weights * batch <= ((uint64_t)20 << 20);
    }
    if (p->res.mm1_layout >= 0 && ctx->matvec_engine != SMELT_HIP_MATVEC_VECTOR && p->res.family != kFamAffineArgmax &&
        (!mm1_batch_family || mm1_small_batch)) {
        // single-token matvecs: the single-pass matrix-core kernel of the same pipeline, same
        // arguments, its own launch geometry (one workgroup per eight rows)
        // (every single-token kernel takes its token from the grid row: a record with several rows is one launch per token
        // of the same kernel, each row the one-token launch's bits)
        uint32_t rows = 0, cols = 0, group = 128, tokens = L.grid[1];
        size_t ro = 0;   // leading read-only operands (codes, scales[, biases], ..., x)
        size_t lead = 0; // ... behind this many leading arguments that are not fetched 16 bytes at a time
        auto U = [&](size_t i) { return L.args[i].value; };
        switch (p->res.family) {
            case kFamAffineDual: rows = U(9); cols = U(10); group = U(11); ro = 7; break;
            case kFamAffineDualAdd: rows = U(11); cols = U(12); group = U(13); ro = 7; break;
            // norm-scale prologue: the fp32 scale comes first; x, the norm weight, [the residual,] the
            // normalised row (stored 16 bytes at a time by workgroup 0) and the planes follow
            case kFamNormScaleAffineMatvec: rows = U(8); cols = U(9); group = U(10); lead = 1; ro = 6; break;
            case kFamNormAddScaleAffineMatvec: rows = U(9); cols = U(10); group = U(11); lead = 1; ro = 7; break;
            case kFamNormScaleAffineDual: rows = U(11); cols = U(12); group = U(13); lead = 1; ro = 8; break;
            case kFamNormScaleAffineGateUp: rows = U(10); cols = U(11); group = U(12); lead = 1; ro = 8; break;
            case kFamAffineMatvec: rows = U(5); cols = U(6); group = U(7); ro = 4; break;
            case kFamAffineAdd: rows = U(6); cols = U(7); group = U(8); ro = 4; break;
            case kFamAffineGateUp: rows = U(8); cols = U(9); group = U(10); ro = 7; break;
            case kFamAffineBank4: rows = U(8) + U(9) + U(10) + U(11); cols = U(12); group = U(13); ro = 4; break;
            case kFamSignedMatvec: rows = U(4); cols = U(5); ro = 3; break;
            case kFamSignedAdd: rows = U(5); cols = U(6); ro = 3; break;
            case kFamSignedGateUp: rows = U(6); cols = U(7); ro = 5; break;
            // four tokens per grid row in the record: one grid row per token here (the kernel takes its token from
            // blockIdx.y; the trailing batch argument is dropped from the argument block)
            case kFamSignedB4: rows = U(4); cols = U(5); tokens = U(6); ro = 3; break;
            case kFamSignedGateUpB4: rows = U(6); cols = U(7); tokens = U(8); ro = 5; break;
            case kFamAffineBatched: tokens = U(5); rows = U(6); cols = U(7); group = U(8); ro = 4; break;
            case kFamAffineGateUpBatched: tokens = U(8); rows = U(9); cols = U(10); group = U(11); ro = 7; break;
            case kFamBinaryPackedBank: rows = U(5) + U(6); cols = U(7); ro = 3; break;
            case kFamBinaryPackedBank4: rows = U(7) + U(8) + U(9) + U(10); cols = U(11); ro = 3; break;
            case kFamTerAffMatvec: rows = U(5); cols = U(6); ro = 4; break;
            case kFamTerAffAdd: rows = U(6); cols = U(7); ro = 4; break;
            case kFamTerAffGateUp: rows = U(8); cols = U(9); ro = 7; break;
            case kFamTerAffBank4: rows = U(8) + U(9) + U(10) + U(11); cols = U(12); ro = 4; break;
            default: break;
        }
        Mm1Plan plan;
        if (rows > 0 && aligned16(lead + ro, lead) && whole_pieces(lead + ro, lead) && mm1_plan((CodeLayout)p->res.mm1_layout, rows, cols, group, p->res.mm1_nmat, ctx->lds_limit,
                                 ctx->matvec_engine == SMELT_HIP_MATVEC_MATRIX_CORE, &plan) &&
            p->fn_mm1[plan.nl]) {
            fn = p->fn_mm1[plan.nl];
            L.grid[0] = (rows + 7) / 8; L.grid[1] = tokens; L.grid[2] = 1;
            // binary and ternary codes from two tokens on: two tokens per pass (the weights are unpacked and multiplied
            // once for both; the token count is the kernels' last argument: the four-token forms bring it along)
            // ... and from eight tokens on (rows of a multiple of 256 columns; bf16 rows converted to fp16) the streaming kernel
            // of the format: the weights pass once per sixteen tokens
            // (cold, binary gate+up 2 x 17408 x 5120 at 8 / 16 / 32 / 64 tokens: 20 / 23 / 36 / 67 us against 47 / 89 / 173 / 325
            // two tokens per pass; binary 5120 x 5120 7.5 / 9.6 / 12 / 20 against 11 / 19 / 33 / 62; 2048 x 2048 at eight 4.3 against 4.0)
            QmsPlan splan;
            if ((mm1_per_row || mm1_b4) && tokens >= 8u && p->fn_qss[tokens > 8] &&
                qss_plan(p->res.mm1_layout == (int)kCodesBinary1 ? 1 : 2, p->res.mm1_nmat, rows, cols, tokens, ctx->lds_limit, &splan)) {
                fn = p->fn_qss[tokens > 8];
                L.grid[0] = (rows + 15) / 16; L.grid[1] = (tokens + 15) / 16; L.grid[2] = 1;
                L.block[0] = 64 * splan.kc; L.block[1] = 1; L.block[2] = 1;
                L.lds = splan.lds;
                if (!mm1_b4) { Arg a; a.kind = 'U'; a.value = tokens; L.args.push_back(a); }   // (the four-token forms bring the count along)
                routed = true;
            }
            const bool streamed = routed;
            Mm1Plan plan2;
            const bool two = !streamed && tokens >= 2 && (mm1_b4 || mm1_per_row) &&
                             mm1_plan((CodeLayout)p->res.mm1_layout, rows, cols, group, p->res.mm1_nmat, ctx->lds_limit,
                                      ctx->matvec_engine == SMELT_HIP_MATVEC_MATRIX_CORE, &plan2, 2) && p->fn_mm1_t2[plan2.nl];
            if (two) {
                plan = plan2;
                fn = p->fn_mm1_t2[plan.nl];
                L.grid[1] = (tokens + 1) / 2;
                if (!mm1_b4) { Arg a; a.kind = 'U'; a.value = tokens; L.args.push_back(a); }
            } else if (mm1_b4 && !streamed) L.args.count -= 1;
            if (mm1_small_batch) {
                // W S B X Y batch rows cols group tile -> W S B X Y rows cols group
                const size_t o = mm1_pair_batch ? 8 : 5;
                for (size_t i = o; i + 1 < L.args.count; ++i) L.args[i] = L.args[i + 1];
                L.args.count -= 2;
            }
            if (!streamed) {
                L.block[0] = 64 * plan.kc; L.block[1] = 1; L.block[2] = 1;
                L.lds = plan.lds;
            }
            routed = true;
        }
    }
    const bool qms_pair = p->res.family == kFamAffineQmmGateUp || p->res.family == kFamAffineGateUpBatched;
    const bool qms_small_batch = p->res.family == kFamAffineBatched || p->res.family == kFamAffineGateUpBatched;
    if (p->res.family == kFamAffineArgmax) {
        // lm_head over two tokens and more (W S B X keys batch logit_cap | rows cols group batch_tile): the fused
        // kernel walks the weights once per token tile; instead the streaming qmm leaves the rounded logits of all
        // tokens in the workspace and a second launch forms the same partial keys from them (151936 x 1024 at four
        // tokens: 26 + 3 us against 67).  Not with a logit cap (the fused kernel caps before it rounds), and not
        // when the workspace is too small for the logits.
        const uint32_t batch = L.args[5].value, rows = L.args[7].value, cols = L.args[8].value, group = L.args[9].value;
        // At one token: the single-pass kernel with the argmax as its epilogue, where the fused vector kernel leaves
        // lanes idle.  That kernel covers a row in whole passes of 64 (32, 16) 16-byte pieces; with the last pass partly
        // empty it loses (cold, per launch: 151936 x 2560 52 against 43-46 us, x 1536 30 against 27, x 5120 87 against
        // 80-82, 32000 x 2560 16.0 against 12.9-13.7, x 5120 24.3 against 20.3-20.8), with full passes it wins or ties
        // (151936 x 1024 19.6 against 21.3, x 2048 33.5 against 34.4, x 4096 64 against 73-75, 32000 x 8192 32.3 against 32).
        // The record's consumer reads grid-width keys per token, any partition of the rows: the eight-row tiles
        // t, t + width, ... meet in partial t through the workspace (a key per tile, a counter per partial), so
        // the route needs at least one tile per partial, at most a wave's worth, and room in the workspace.
        const uint32_t tiles = (rows + 7) / 8, parts = L.grid[0];
        const uint32_t units = cols / 32, pass = units > 32 ? 64 : (units > 16 ? 32 : 16);
        const bool idle_lanes = (uint64_t)units * 10 < (uint64_t)((units + pass - 1) / pass * pass) * 9;
        Mm1Plan mplan;
        hipFunction_t fn_argmax = nullptr;
        if (batch == 1 && idle_lanes && ctx->matvec_engine != SMELT_HIP_MATVEC_VECTOR && p->res.mm1_layout >= 0 && parts > 0 &&
            aligned16(4) && whole_pieces(4) &&
            mm1_plan((CodeLayout)p->res.mm1_layout, rows, cols, group, 1, ctx->lds_limit,
                     ctx->matvec_engine == SMELT_HIP_MATVEC_MATRIX_CORE, &mplan) && p->fn_mm1[mplan.nl]) {
            fn_argmax = p->fn_mm1[mplan.nl];
        }
        if (fn_argmax && tiles >= parts && tiles <= 64u * (uint64_t)parts && ws.partial && ws.counters &&
            (size_t)tiles * 8 <= ws.partial_bytes && (size_t)parts * 4 <= ws.counter_bytes) {
            alignas(16) unsigned char ka[128];
            size_t at = 0;
            auto put_ptr = [&](const void* v) { at = (at + 7) & ~(size_t)7; memcpy(ka + at, &v, 8); at += 8; };
            auto put_u32 = [&](uint32_t v) { memcpy(ka + at, &v, 4); at += 4; };
            for (int i = 0; i < 5; ++i) put_ptr(L.args[(size_t)i].ptr);   // W S B X keys
            put_ptr(ws.partial); put_ptr(ws.counters);
            put_u32(rows); put_u32(cols); put_u32(group); put_u32(parts); put_u32(L.args[6].value);   // (the cap's float bits)
            size_t ka_size = at;
            void* cfg[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, ka, HIP_LAUNCH_PARAM_BUFFER_SIZE, &ka_size, HIP_LAUNCH_PARAM_END};
            if (!ctx->batch_open) {
                HIP_TRY(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
                ctx->batch_open = true;
                ctx->timing_valid = false;
            }
            HIP_TRY(ctx, hipModuleLaunchKernel(fn_argmax, tiles, 1, 1, 64 * mplan.kc, 1, 1, (unsigned)mplan.lds, ctx->stream, nullptr, cfg));
            return 1;
        }
        QmsPlan plan;
        if (batch >= 2 && ctx->matvec_engine != SMELT_HIP_MATVEC_VECTOR && L.args[6].value == 0u && p->fn_logits_keys &&
            aligned16(4) && whole_pieces(4) && (size_t)batch * rows * 2 <= ws.partial_bytes && ws.partial &&
            qms_plan(rows, cols, group, 1, batch, (uint32_t)ctx->props.multiProcessorCount, ctx->lds_limit, &plan) &&
            (group == 32 ? p->fn_qms_g32[batch > 8] : p->fn_qms[plan.rt][batch > 8])) {
            alignas(16) unsigned char ka[128];
            size_t at = 0;
            auto put_ptr = [&](const void* v) { at = (at + 7) & ~(size_t)7; memcpy(ka + at, &v, 8); at += 8; };
            auto put_u32 = [&](uint32_t v) { memcpy(ka + at, &v, 4); at += 4; };
            for (int i = 0; i < 4; ++i) put_ptr(L.args[(size_t)i].ptr);
            put_ptr(ws.partial);                       // logits [batch][rows] in the activation type
            put_u32(batch); put_u32(rows); put_u32(cols); put_u32(group); put_u32(0u);
            put_ptr(ws.partial); put_ptr(ws.counters);  // the skinny kernels' workspace arguments: unused
            size_t ka_size = at;
            void* cfg_a[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, ka, HIP_LAUNCH_PARAM_BUFFER_SIZE, &ka_size, HIP_LAUNCH_PARAM_END};
            if (!ctx->batch_open) {
                HIP_TRY(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
                ctx->batch_open = true;
                ctx->timing_valid = false;
            }
            HIP_TRY(ctx, hipModuleLaunchKernel(group == 32 ? p->fn_qms_g32[batch > 8] : p->fn_qms[plan.rt][batch > 8], (rows + 16 * plan.rt - 1) / (16 * plan.rt), (batch + 15) / 16, 1,
                                               64 * plan.kc, 1, 1, (unsigned)plan.lds, ctx->stream, nullptr, cfg_a));
            alignas(16) unsigned char kb[64];
            at = 0;
            auto put_ptr_b = [&](const void* v) { at = (at + 7) & ~(size_t)7; memcpy(kb + at, &v, 8); at += 8; };
            put_ptr_b(ws.partial); put_ptr_b(L.args[4].ptr);
            const uint32_t tail[3] = {batch, rows, (uint32_t)L.grid[0]};
            memcpy(kb + at, tail, sizeof tail); at += sizeof tail;
            size_t kb_size = at;
            void* cfg_b[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, kb, HIP_LAUNCH_PARAM_BUFFER_SIZE, &kb_size, HIP_LAUNCH_PARAM_END};
            HIP_TRY(ctx, hipModuleLaunchKernel(p->fn_logits_keys, L.grid[0], batch, 1, 64, 1, 1, 0, ctx->stream, nullptr, cfg_b));
            return 2;
        }
    } else if (p->res.family == kFamNormScaleAffineQmm || p->res.family == kFamNormScaleAffineQmmGateUp || p->res.family == kFamNormScaleAffineBatched) {
        // Norm-scale prologue in front of a qmm (rs X nw XN W S B Y batch | rows cols group tile; gate+up: rs X nw gW gS gB
        // uW uS uB Y batch | ...): the fused kernels are the token-slab and vector ones; instead one launch writes the
        // normalised rows (into the record's XN, or into the end of the workspace where the record has none) and the
        // streaming or token-tile kernel of the plain form multiplies them: the bits of the staged pair.  From two tokens on.
        const bool pair = p->res.family == kFamNormScaleAffineQmmGateUp;
        const size_t o = pair ? 10 : 8;
        const uint32_t batch = L.args[o].value, rows = L.args[o + 1].value, cols = L.args[o + 2].value, group = L.args[o + 3].value;
        const size_t xn_bytes = ((size_t)batch * cols * 2 + 255) & ~(size_t)255;
        char* xn = !pair && L.args[3].ptr ? L.args[3].ptr : nullptr;
        const bool scratch = xn == nullptr;
        if (scratch && ws.partial && xn_bytes <= ws.partial_bytes) xn = (char*)ws.partial + (ws.partial_bytes - xn_bytes);
        const size_t ws_left = scratch ? ws.partial_bytes - (xn ? xn_bytes : 0) : ws.partial_bytes;
        const size_t wfirst = pair ? 3 : 4, wcount = pair ? 6 : 3;
        hipFunction_t fn2 = nullptr;
        uint32_t g2[3] = {0, 0, 0}, block2 = 0;
        size_t lds2 = 0;
        QmtPlan tplan;
        QmsPlan plan;
        if (batch >= 2 && xn && (reinterpret_cast<uintptr_t>(xn) & 15u) == 0 && p->fn_norm_rows && ctx->matvec_engine != SMELT_HIP_MATVEC_VECTOR && cols % 8 == 0 &&
            aligned16(wfirst + wcount, wfirst) && whole_pieces(wfirst + wcount, wfirst) && aligned16(3, 1)) {
            if (qmt_plan(rows, cols, group, p->res.qms_nmat, batch, (uint32_t)ctx->props.multiProcessorCount, ctx->lds_limit, &tplan) &&
                (tplan.per_wave ? p->fn_qmt_per_wave : p->fn_qmt)[tplan.rt][tplan.tb][tplan.kw]) {
                fn2 = (tplan.per_wave ? p->fn_qmt_per_wave : p->fn_qmt)[tplan.rt][tplan.tb][tplan.kw];
                const uint32_t ksplit = tplan.partial_bytes <= ws_left && tplan.counter_bytes <= ws.counter_bytes ? tplan.ksplit : 1;
                g2[0] = (rows + tplan.bn - 1) / tplan.bn; g2[1] = (batch + tplan.bm - 1) / tplan.bm; g2[2] = ksplit;
                block2 = 256 * tplan.kw; lds2 = tplan.lds;
            } else if (qms_plan(rows, cols, group, p->res.qms_nmat, batch, (uint32_t)ctx->props.multiProcessorCount, ctx->lds_limit, &plan) &&
                       (group == 32 ? p->fn_qms_g32[batch > 8] : p->fn_qms[plan.rt][batch > 8])) {
                fn2 = group == 32 ? p->fn_qms_g32[batch > 8] : p->fn_qms[plan.rt][batch > 8];
                g2[0] = (rows + 16 * plan.rt - 1) / (16 * plan.rt); g2[1] = (batch + 15) / 16; g2[2] = 1;
                block2 = 64 * plan.kc; lds2 = plan.lds;
            }
        }
        if (fn2) {
            alignas(16) unsigned char ka[64], kb[160];
            size_t at = 0;
            auto put = [&](unsigned char* buf, const void* v, size_t n, size_t align) { at = (at + align - 1) & ~(align - 1); memcpy(buf + at, v, n); at += n; };
            const void* rs = L.args[0].ptr; const void* xin = L.args[1].ptr; const void* nw = L.args[2].ptr;
            put(ka, &rs, 8, 8); put(ka, &xin, 8, 8); put(ka, &nw, 8, 8); put(ka, &xn, 8, 8); put(ka, &batch, 4, 4); put(ka, &cols, 4, 4);
            size_t ka_size = at;
            void* cfg_a[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, ka, HIP_LAUNCH_PARAM_BUFFER_SIZE, &ka_size, HIP_LAUNCH_PARAM_END};
            if (!ctx->batch_open) {
                HIP_TRY(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
                ctx->batch_open = true;
                ctx->timing_valid = false;
            }
            HIP_TRY(ctx, hipModuleLaunchKernel(p->fn_norm_rows, (cols / 8 + 255) / 256, batch, 1, 256, 1, 1, 0, ctx->stream, nullptr, cfg_a));
            at = 0;
            for (size_t i = 0; i < wcount; ++i) { const void* w = L.args[wfirst + i].ptr; put(kb, &w, 8, 8); }
            put(kb, &xn, 8, 8);
            const void* y = L.args[pair ? 9 : 7].ptr;
            put(kb, &y, 8, 8);
            const uint32_t tail[5] = {batch, rows, cols, group, L.args[o + 4].value};
            put(kb, tail, sizeof tail, 4);
            const void* wsp = ws.partial; const void* wsc = ws.counters;
            put(kb, &wsp, 8, 8); put(kb, &wsc, 8, 8);
            size_t kb_size = at;
            void* cfg_b[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, kb, HIP_LAUNCH_PARAM_BUFFER_SIZE, &kb_size, HIP_LAUNCH_PARAM_END};
            HIP_TRY(ctx, hipModuleLaunchKernel(fn2, g2[0], g2[1], g2[2], block2, 1, 1, (unsigned)lds2, ctx->stream, nullptr, cfg_b));
            return 2;
        }
    } else if (!routed && !p->res.qms_tail.empty() && ctx->matvec_engine != SMELT_HIP_MATVEC_VECTOR &&
        aligned16(qms_pair ? 7 : 4) && whole_pieces(qms_pair ? 7 : 4)) {
        // skinny qmm (and, from two tokens on, the per-token small-batch forms, whose arguments are the
        // same): the streaming kernel of the same pipeline, same arguments, its own launch
        // geometry (16 * rt rows per workgroup, 16 tokens per grid row); it uses no workspace
        const size_t o = qms_pair ? 8 : (p->res.family == kFamAffineQmmAdd ? 7 : 5);
        const uint32_t batch = L.args[o].value, rows = L.args[o + 1].value, cols = L.args[o + 2].value, group = L.args[o + 3].value;
        QmtPlan tplan;
        if (qms_small_batch && batch < 2) {
            // one token: the kernel the record names
        } else if (qmt_plan(rows, cols, group, p->res.qms_nmat, batch, (uint32_t)ctx->props.multiProcessorCount, ctx->lds_limit, &tplan) && (tplan.per_wave ? p->fn_qmt_per_wave : p->fn_qmt)[tplan.rt][tplan.tb][tplan.kw]) {
            fn = (tplan.per_wave ? p->fn_qmt_per_wave : p->fn_qmt)[tplan.rt][tplan.tb][tplan.kw];
            // a split that the workspace of this call cannot hold is not taken
            const uint32_t ksplit = tplan.partial_bytes <= ws.partial_bytes && tplan.counter_bytes <= ws.counter_bytes ? tplan.ksplit : 1;
            L.grid[0] = (rows + tplan.bn - 1) / tplan.bn; L.grid[1] = (batch + tplan.bm - 1) / tplan.bm; L.grid[2] = ksplit;
            L.block[0] = 256 * tplan.kw; L.block[1] = 1; L.block[2] = 1;
            L.lds = tplan.lds;
            routed = true;
            qms_routed = true;
        }
        QmsPlan plan;
        if (!routed && batch > (qms_small_batch ? 1u : 0u) && qms_plan(rows, cols, group, p->res.qms_nmat, batch, (uint32_t)ctx->props.multiProcessorCount, ctx->lds_limit, &plan) &&
            (group == 32 ? p->fn_qms_g32[batch > 8] : p->fn_qms[plan.rt][batch > 8])) {
            fn = group == 32 ? p->fn_qms_g32[batch > 8] : p->fn_qms[plan.rt][batch > 8];
            L.grid[0] = (rows + 16 * plan.rt - 1) / (16 * plan.rt); L.grid[1] = (batch + 15) / 16; L.grid[2] = 1;
            L.block[0] = 64 * plan.kc; L.block[1] = 1; L.block[2] = 1;
            L.lds = plan.lds;
            routed = true;
            qms_routed = true;
        }
    }
    if (p->res.family == kFamTerAffQmm && ctx->matvec_engine != SMELT_HIP_MATVEC_VECTOR && aligned16(4) && whole_pieces(4)) {
        // ternary qmm (C S S2 X Y rows cols batch): the streaming kernel, same arguments, its own geometry, up to 128
        // tokens (256 for matrices of fewer than 8192 rows, which leave the token-slab kernel short of slabs).  Cold,
        // streaming against token slabs at 8 / 32 / 128 / 256 / 512 tokens: 17408 x 5120 15 / 33 / 101 / 183 / 341 us against
        // 57 / 62 / 104 / 168 / 291; 5120 x 17408 20 / 35 / 107 / 194 / 367 against 156 / 203 / 208 / 253 / 328; 4096 x 4096
        // 5.2 / 9.0 / 23 / 40 / 76 against 37 / 41 / 41 / 48 / 73.
        const uint32_t rows = L.args[5].value, cols = L.args[6].value, batch = L.args[7].value;
        QmsPlan plan;
        if (batch <= (rows < 8192 ? 256u : 128u) && qts_plan(rows, cols, batch, ctx->lds_limit, &plan) && p->fn_tqs[batch > 8]) {
            fn = p->fn_tqs[batch > 8];
            L.grid[0] = (rows + 15) / 16; L.grid[1] = (batch + 15) / 16; L.grid[2] = 1;
            L.block[0] = 64 * plan.kc; L.block[1] = 1; L.block[2] = 1;
            L.lds = plan.lds;
            routed = true;
        }
    }
    if (!qms_routed && (L.ws_partial_need > ws.partial_bytes || L.ws_counter_need > ws.counter_bytes))
        return fail(ctx, SMELT_HIP_ERR_UNSUPPORTED_GEOMETRY,
                    "pipeline '" + p->entry + "': split-K partials (" + std::to_string(L.ws_partial_need) + " bytes, " +
                        std::to_string(L.ws_counter_need / 4) + " counters) exceed the workspace (" + std::to_string(ws.partial_bytes) +
                        " bytes, " + std::to_string(ws.counter_bytes / 4) + " counters)");
    // kernarg block: natural alignment in argument order
    alignas(16) unsigned char kernarg[512];
    size_t pos = 0;
    for (const Arg& a : L.args) {
        if (a.kind == 'P' || a.kind == 'Z') {
            pos = (pos + 7) & ~(size_t)7;
            void* ptr = a.ptr;
            memcpy(kernarg + pos, &ptr, 8);
            pos += 8;
        } else {
            memcpy(kernarg + pos, &a.value, 4);
            pos += 4;
        }
    }
    if (p->res.workspace || qms_routed) {
        // (the streaming qmm declares the two workspace pointers of the skinny kernels and ignores them)
        pos = (pos + 7) & ~(size_t)7;
        memcpy(kernarg + pos, &ws.partial, 8);
        memcpy(kernarg + pos + 8, &ws.counters, 8);
        pos += 16;
    }
    size_t kernarg_size = pos;
    void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, kernarg, HIP_LAUNCH_PARAM_BUFFER_SIZE, &kernarg_size, HIP_LAUNCH_PARAM_END};
    if (!ctx->batch_open) {
        HIP_TRY(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
        ctx->batch_open = true;
        ctx->timing_valid = false;
    }
    if (!routed && p->fn_single && p->res.single_arg >= 0 && L.args[(size_t)p->res.single_arg].value == 1 && L.grid[1] == 1) fn = p->fn_single;
    HIP_TRY(ctx, hipModuleLaunchKernel(fn, L.grid[0], L.grid[1], L.grid[2], L.block[0], L.block[1], L.block[2],
                                       (unsigned)L.lds, ctx->stream, nullptr, config));
    return 1;
}

int interpret(smelt_hip_context* ctx, const SmeltDispatchRecord* table, size_t count, int cur, int alt, const Dyn& d) {
    if (!ctx || (!table && count)) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context or table");
    int launched = 0;
    for (size_t i = 0; i < count; ++i) {
        if (table[i].op_kind == SMELT_OP_SWAP) { std::swap(cur, alt); continue; }
        const int rc = encode_record(ctx, &table[i], cur, alt, d);
        if (rc < 0) {
            ctx->error = "record " + std::to_string(i) + ": " + ctx->error;
            return rc;
        }
        launched += rc;
    }
    return launched;
}

}  // namespace

namespace smelt_host {

int encode_prefill_with_workspace(smelt_hip_context* ctx, const SmeltDispatchRecord* rec, int cur, int alt,
                                  int32_t seq_len, int32_t start_pos, const SplitKWorkspace& ws) {
    Dyn d{true, 0, seq_len, start_pos};
    return encode_record(ctx, rec, cur, alt, d, &ws);
}

int context_device(const smelt_hip_context* ctx) { return ctx->device; }
hipStream_t context_stream(const smelt_hip_context* ctx) { return ctx->stream; }
int context_fail(const smelt_hip_context* ctx, int code, const std::string& message) { return fail(ctx, code, message); }

}  // namespace smelt_host

extern "C" {

int smelt_hip_context_create(int device_index, smelt_hip_context** out) {
    if (!out) return fail(nullptr, SMELT_HIP_ERR_INVALID_ARGUMENT, "out is null");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return fail(nullptr, SMELT_HIP_ERR_NO_DEVICE, std::string("no HIP device: ") + (e != hipSuccess ? hipGetErrorString(e) : "device count is 0"));
    if (device_index < 0 || device_index >= count)
        return fail(nullptr, SMELT_HIP_ERR_INVALID_ARGUMENT, "device index out of range");
    smelt_hip_context* ctx = new smelt_hip_context();
    ctx->device = device_index;
    ctx->slots.resize(64);
    auto release = [&]() {
        if (ctx->ws_partial) (void)hipFree(ctx->ws_partial);
        if (ctx->ws_counters) (void)hipFree(ctx->ws_counters);
        if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
        if (ctx->ev_end) (void)hipEventDestroy(ctx->ev_end);
        if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
        delete ctx;
    };
    auto bail = [&](hipError_t err, const char* what) {
        int rc = hip_fail(nullptr, err, what);
        release();
        return rc;
    };
    if ((e = hipSetDevice(device_index)) != hipSuccess) return bail(e, "hipSetDevice");
    if ((e = hipGetDeviceProperties(&ctx->props, device_index)) != hipSuccess) return bail(e, "hipGetDeviceProperties");
    if ((e = hipStreamCreate(&ctx->stream)) != hipSuccess) return bail(e, "hipStreamCreate");
    if ((e = hipEventCreate(&ctx->ev_start)) != hipSuccess) return bail(e, "hipEventCreate");
    if ((e = hipEventCreate(&ctx->ev_end)) != hipSuccess) return bail(e, "hipEventCreate");
    ctx->lds_limit = ctx->props.sharedMemPerBlock ? ctx->props.sharedMemPerBlock : 65536;
    ctx->ws_partial_bytes = (size_t)64 << 20;
    ctx->ws_counter_bytes = (size_t)256 << 10;
    if ((e = hipMalloc(&ctx->ws_partial, ctx->ws_partial_bytes)) != hipSuccess) return bail(e, "hipMalloc(workspace)");
    if ((e = hipMalloc(&ctx->ws_counters, ctx->ws_counter_bytes)) != hipSuccess) return bail(e, "hipMalloc(workspace counters)");
    if ((e = hipMemset(ctx->ws_counters, 0, ctx->ws_counter_bytes)) != hipSuccess) return bail(e, "hipMemset(workspace counters)");
    // the library's static scratch on this device (used by smelt_hip_encode_prefill_record_static_scratch)
    std::string why;
    if (int rc = static_scratch_prepare(device_index, ctx->stream, &why)) {
        release();
        return fail(nullptr, rc, why);
    }
    *out = ctx;
    return SMELT_HIP_OK;
}

void smelt_hip_context_destroy(smelt_hip_context* ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    for (SlotBuffer& s : ctx->slots)
        if (s.ptr) (void)hipFree(s.ptr);
    if (ctx->ws_partial) (void)hipFree(ctx->ws_partial);
    if (ctx->ws_counters) (void)hipFree(ctx->ws_counters);
    for (hipModule_t m : ctx->modules) (void)hipModuleUnload(m);
    if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
    if (ctx->ev_end) (void)hipEventDestroy(ctx->ev_end);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

const char* smelt_hip_last_error(const smelt_hip_context* ctx) {
    return ctx ? ctx->error.c_str() : g_global_error.c_str();
}

int smelt_hip_set_activation_dtype(smelt_hip_context* ctx, int act_dtype) {
    if (!ctx || (act_dtype != SMELT_HIP_ACT_F16 && act_dtype != SMELT_HIP_ACT_BF16))
        return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "activation dtype must be SMELT_HIP_ACT_F16 or SMELT_HIP_ACT_BF16");
    ctx->default_act = act_dtype == SMELT_HIP_ACT_BF16 ? kActBF16 : kActF16;
    return SMELT_HIP_OK;
}

int smelt_hip_set_matvec_engine(smelt_hip_context* ctx, int engine) {
    if (!ctx || engine < SMELT_HIP_MATVEC_AUTO || engine > SMELT_HIP_MATVEC_VECTOR)
        return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "matvec engine must be SMELT_HIP_MATVEC_AUTO, _MATRIX_CORE or _VECTOR");
    ctx->matvec_engine = engine;
    return SMELT_HIP_OK;
}

int smelt_hip_module_load(smelt_hip_context* ctx, const void* code_object, size_t bytes) {
    if (!ctx || !code_object || bytes == 0) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context or empty code object");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    hipModule_t module = nullptr;
    HIP_TRY(ctx, hipModuleLoadData(&module, code_object));
    std::lock_guard<std::mutex> lock(ctx->pipeline_mutex);
    ctx->modules.push_back(module);
    return SMELT_HIP_OK;
}

int smelt_hip_module_load_file(smelt_hip_context* ctx, const char* path) {
    if (!ctx || !path) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context or path");
    if (DIR* dir = opendir(path)) {
        // a directory: every code object of the build in it, in name order
        std::vector<std::string> names;
        closedir(dir);
        // the build writes the list of its code objects next to them: load exactly those, so that a code
        // object left behind by an older build is never picked up (and never wins a duplicate symbol)
        {
            std::ifstream manifest(std::string(path) + "/smelt_kernels.manifest");
            std::string line;
            while (manifest && std::getline(manifest, line)) {
                while (!line.empty() && (line.back() == '\r' || line.back() == ' ')) line.pop_back();
                if (!line.empty() && line[0] != '#') names.push_back(line);
            }
        }
        if (names.empty()) {   // no manifest: every smelt_kernels*.hsaco of the directory
            dir = opendir(path);
            while (const dirent* e = dir ? readdir(dir) : nullptr) {
                const std::string n = e->d_name;
                if (n.size() > 6 && n.compare(n.size() - 6, 6, ".hsaco") == 0 && n.compare(0, 13, "smelt_kernels") == 0) names.push_back(n);
            }
            if (dir) closedir(dir);
        }
        if (names.empty()) return fail(ctx, SMELT_HIP_ERR_INVALID_PACKAGE, std::string("no smelt_kernels*.hsaco under '") + path + "'");
        std::sort(names.begin(), names.end());
        for (const std::string& n : names)
            if (int rc = smelt_hip_module_load_file(ctx, (std::string(path) + "/" + n).c_str())) return rc;
        return SMELT_HIP_OK;
    }
    std::ifstream f(path, std::ios::binary);
    if (!f) return fail(ctx, SMELT_HIP_ERR_INVALID_PACKAGE, std::string("cannot open code object '") + path + "'");
    std::vector<char> data((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    if (data.empty()) return fail(ctx, SMELT_HIP_ERR_INVALID_PACKAGE, std::string("code object '") + path + "' is empty");
    return smelt_hip_module_load(ctx, data.data(), data.size());
}

int smelt_hip_pipeline_create(smelt_hip_context* ctx, const char* entry, int allow_missing, uint32_t* out_index) {
    if (!ctx || !entry) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context or entry");
    if (ctx->modules.empty()) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "load a code object before creating pipelines");
    // a kernel lives in exactly one of the loaded code objects
    std::vector<hipModule_t> modules;
    {
        std::lock_guard<std::mutex> lock(ctx->pipeline_mutex);   // smelt_hip_module_load appends under this lock
        modules = ctx->modules;
    }
    auto find = [&](hipFunction_t* fn, const std::string& symbol) {
        hipError_t last = hipErrorNotFound;
        for (hipModule_t m : modules) {
            last = hipModuleGetFunction(fn, m, symbol.c_str());
            if (last == hipSuccess) break;
        }
        (void)hipGetLastError();   // a miss in one code object is not an error of the context
        if (last != hipSuccess) *fn = nullptr;
        return last;
    };
    Pipeline p;
    p.entry = entry;
    std::string why;
    const ResolveStatus st = resolve_pipeline(p.entry, ctx->default_act, ctx->lds_limit, &p.res, &why);
    if (st == kResolveMalformed) return fail(ctx, SMELT_HIP_ERR_INVALID_PACKAGE, why);
    if (st == kResolveUnknown && !allow_missing) return fail(ctx, SMELT_HIP_ERR_UNKNOWN_PIPELINE, why);
    if (st == kResolveOk) {
        hipError_t e = find(&p.fn, p.res.symbol);
        if (e != hipSuccess) {
            if (!allow_missing)
                return fail(ctx, SMELT_HIP_ERR_UNKNOWN_PIPELINE, "code object has no kernel '" + p.res.symbol + "' for pipeline '" + p.entry + "': " + hipGetErrorString(e));
        } else {
            p.ready = true;
            if (!p.res.symbol_single.empty() && find(&p.fn_single, p.res.symbol_single) != hipSuccess) p.fn_single = nullptr;
            if (!p.res.mm1_prefix.empty())
                for (uint32_t nl = 1; nl <= kMm1MaxSegments; ++nl)
                    (void)find(&p.fn_mm1[nl], p.res.mm1_prefix + "nl" + std::to_string(nl) + "_" + p.res.mm1_tail);
            if (!p.res.mm1_prefix.empty() && (p.res.mm1_layout == (int)kCodesBinary1 || p.res.mm1_layout == (int)kCodesTernary2))
                for (uint32_t nl = 1; nl <= kMm1MaxSegments; ++nl)
                    (void)find(&p.fn_mm1_t2[nl], p.res.mm1_prefix + "nl" + std::to_string(nl) + "_t2_" + p.res.mm1_tail);
            if (!p.res.qms_tail.empty()) {
                // the variants qmt_plan can return: (row tiles, token blocks, waves along K), one matrix per wave or not
                static const struct { uint32_t rt, tb, kw; bool per_wave; } kQmtVariants[] = {
                    {2, 2, 2, false}, {3, 2, 2, false}, {2, 2, 1, false}, {3, 2, 2, true}};
                for (const auto& v : kQmtVariants) {
                    const std::string rest = std::to_string(v.rt) + "_t" + std::to_string(v.tb) + "_k" + std::to_string(v.kw) + "_" + p.res.qms_tail;
                    if (v.per_wave) (void)find(&p.fn_qmt_per_wave[v.rt][v.tb][v.kw], "smelt_affine_qmt_w" + rest);
                    else (void)find(&p.fn_qmt[v.rt][v.tb][v.kw], "smelt_affine_qmt_r" + rest);
                }
            }
            if (p.res.family == kFamAffineArgmax) (void)find(&p.fn_logits_keys, "smelt_logits_argmax_partials");
            if (!p.res.mm1_prefix.empty() && p.res.mm1_prefix.size() > 4 &&
                (p.res.mm1_layout == (int)kCodesBinary1 || p.res.mm1_layout == (int)kCodesTernary2))
                for (uint32_t wide = 0; wide < 2; ++wide)
                    (void)find(&p.fn_qss[wide], p.res.mm1_prefix.substr(0, p.res.mm1_prefix.size() - 4) + (wide ? "qss_x4_" : "qss_x2_") + p.res.mm1_tail);
            if (p.res.family == kFamTerAffQmm)
                for (uint32_t wide = 0; wide < 2; ++wide)
                    (void)find(&p.fn_tqs[wide], std::string("smelt_ternary_qms_") + (wide ? "x4_" : "x2_") + (p.res.act == kActBF16 ? "bf16" : "f16"));
            if (p.res.family == kFamNormScaleAffineQmm || p.res.family == kFamNormScaleAffineQmmGateUp || p.res.family == kFamNormScaleAffineBatched)
                (void)find(&p.fn_norm_rows, std::string("smelt_norm_scale_rows_") + (p.res.act == kActBF16 ? "bf16" : "f16"));
            if (!p.res.qms_tail.empty())
                for (uint32_t rt = 1; rt <= kQmsMaxRowTiles; ++rt)
                    for (uint32_t wide = 0; wide < 2; ++wide)
                        (void)find(&p.fn_qms[rt][wide], "smelt_affine_qms_r" + std::to_string(rt) + (wide ? "_x4_" : "_x2_") + p.res.qms_tail);
            if (!p.res.qms_tail.empty())
                for (uint32_t wide = 0; wide < 2; ++wide)
                    (void)find(&p.fn_qms_g32[wide], std::string("smelt_affine_qms_g32") + (wide ? "_x4_" : "_x2_") + p.res.qms_tail);
        }
    }
    std::lock_guard<std::mutex> lock(ctx->pipeline_mutex);
    if (ctx->pipelines.size() >= 65536) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "pipeline index is 16 bits");
    ctx->pipelines.push_back(std::move(p));
    if (out_index) *out_index = (uint32_t)(ctx->pipelines.size() - 1);
    return SMELT_HIP_OK;
}

int smelt_hip_pipeline_count(const smelt_hip_context* ctx) {
    return ctx ? (int)ctx->pipelines.size() : SMELT_HIP_ERR_INVALID_ARGUMENT;
}

int smelt_hip_pipeline_is_ready(const smelt_hip_context* ctx, uint32_t index) {
    if (!ctx || index >= ctx->pipelines.size()) return SMELT_HIP_ERR_INVALID_ARGUMENT;
    return ctx->pipelines[index].ready ? 1 : 0;
}

static int alloc_slot(smelt_hip_context* ctx, int slot, size_t bytes, bool read_only) {
    if (!ctx || slot < 0 || slot >= kMaxSlots) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "slot index out of range");
    if (bytes == 0) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "zero-length buffer");
    if ((size_t)slot >= ctx->slots.size()) ctx->slots.resize((size_t)slot + 1);
    SlotBuffer& s = ctx->slots[(size_t)slot];
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    if (s.ptr) {
        HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
        HIP_TRY(ctx, hipFree(s.ptr));
        s = SlotBuffer();
    }
    // 256 bytes of slack keep whole-vector loads of a ragged tail inside the allocation
    HIP_TRY(ctx, hipMalloc(&s.ptr, bytes + 256));
    HIP_TRY(ctx, hipMemset(s.ptr, 0, bytes + 256));
    s.bytes = bytes;
    s.read_only = read_only;
    return SMELT_HIP_OK;
}

int smelt_hip_buffer_alloc(smelt_hip_context* ctx, int slot, size_t bytes) {
    return alloc_slot(ctx, slot, bytes, false);
}

int smelt_hip_weights_upload(smelt_hip_context* ctx, int weights_slot, const void* bytes, size_t size) {
    if (!bytes) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null weights");
    if (int e = alloc_slot(ctx, weights_slot, size, true)) return e;
    HIP_TRY(ctx, hipMemcpy(ctx->slots[(size_t)weights_slot].ptr, bytes, size, hipMemcpyHostToDevice));
    ctx->weights_slot = weights_slot;
    return SMELT_HIP_OK;
}

int smelt_hip_buffer_write(smelt_hip_context* ctx, int slot, size_t offset, const void* src, size_t bytes) {
    if (!ctx || !src || slot < 0 || (size_t)slot >= ctx->slots.size() || !ctx->slots[(size_t)slot].ptr)
        return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "bad slot or null source");
    SlotBuffer& s = ctx->slots[(size_t)slot];
    if (offset > s.bytes || bytes > s.bytes - offset) return fail(ctx, SMELT_HIP_ERR_OUT_OF_RANGE, "write past the end of the slot");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    HIP_TRY(ctx, hipMemcpy((char*)s.ptr + offset, src, bytes, hipMemcpyHostToDevice));
    return SMELT_HIP_OK;
}

int smelt_hip_buffer_read(smelt_hip_context* ctx, int slot, size_t offset, void* dst, size_t bytes) {
    if (!ctx || !dst || slot < 0 || (size_t)slot >= ctx->slots.size() || !ctx->slots[(size_t)slot].ptr)
        return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "bad slot or null destination");
    SlotBuffer& s = ctx->slots[(size_t)slot];
    if (offset > s.bytes || bytes > s.bytes - offset) return fail(ctx, SMELT_HIP_ERR_OUT_OF_RANGE, "read past the end of the slot");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    HIP_TRY(ctx, hipMemcpy(dst, (char*)s.ptr + offset, bytes, hipMemcpyDeviceToHost));
    return SMELT_HIP_OK;
}

int smelt_hip_buffer_size(const smelt_hip_context* ctx, int slot, size_t* bytes) {
    if (!ctx || !bytes || slot < 0 || (size_t)slot >= ctx->slots.size() || !ctx->slots[(size_t)slot].ptr)
        return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "bad slot");
    *bytes = ctx->slots[(size_t)slot].bytes;
    return SMELT_HIP_OK;
}

int smelt_hip_set_cache_seq_capacity(smelt_hip_context* ctx, uint32_t capacity) {
    if (!ctx) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context");
    ctx->cache_seq_capacity = capacity;
    return SMELT_HIP_OK;
}

int smelt_hip_dispatch_table_count(size_t table_bytes, size_t* out_count) {
    if (!out_count) return fail(nullptr, SMELT_HIP_ERR_INVALID_ARGUMENT, "out_count is null");
    if (table_bytes % sizeof(SmeltDispatchRecord) != 0)
        return fail(nullptr, SMELT_HIP_ERR_INVALID_PACKAGE,
                    "dispatch table size " + std::to_string(table_bytes) + " is not a multiple of dispatch stride " + std::to_string(sizeof(SmeltDispatchRecord)));
    *out_count = table_bytes / sizeof(SmeltDispatchRecord);
    return SMELT_HIP_OK;
}

int smelt_hip_encode_decode_record(smelt_hip_context* ctx, const SmeltDispatchRecord* rec, int cur, int alt, int32_t position) {
    Dyn d{false, position, 0, 0};
    return encode_record(ctx, rec, cur, alt, d);
}

int smelt_hip_encode_prefill_record(smelt_hip_context* ctx, const SmeltDispatchRecord* rec, int cur, int alt, int32_t seq_len, int32_t start_pos) {
    Dyn d{true, 0, seq_len, start_pos};
    return encode_record(ctx, rec, cur, alt, d);
}

int smelt_hip_interpret_decode_table(smelt_hip_context* ctx, const SmeltDispatchRecord* table, size_t count, int cur0, int alt0, int32_t position) {
    Dyn d{false, position, 0, 0};
    return interpret(ctx, table, count, cur0, alt0, d);
}

int smelt_hip_interpret_prefill_table(smelt_hip_context* ctx, const SmeltDispatchRecord* table, size_t count, int cur0, int alt0, int32_t seq_len, int32_t start_pos) {
    Dyn d{true, 0, seq_len, start_pos};
    return interpret(ctx, table, count, cur0, alt0, d);
}

int smelt_hip_submit(smelt_hip_context* ctx) {
    if (!ctx) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context");
    if (ctx->batch_open) {
        HIP_TRY(ctx, hipEventRecord(ctx->ev_end, ctx->stream));
        ctx->batch_open = false;
        ctx->timing_valid = true;
    }
    return SMELT_HIP_OK;
}

int smelt_hip_wait(smelt_hip_context* ctx) {
    if (!ctx) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context");
    if (ctx->batch_open) {
        if (int e = smelt_hip_submit(ctx)) return e;
    }
    HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return SMELT_HIP_OK;
}

int smelt_hip_last_gpu_ns(smelt_hip_context* ctx, uint64_t* out_ns) {
    if (!ctx || !out_ns) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null argument");
    if (!ctx->timing_valid) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "no submitted batch to time");
    HIP_TRY(ctx, hipEventSynchronize(ctx->ev_end));
    float ms = 0;
    HIP_TRY(ctx, hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_end));
    *out_ns = (uint64_t)((double)ms * 1e6);
    return SMELT_HIP_OK;
}

int smelt_hip_benchmark_record(smelt_hip_context* ctx, const SmeltDispatchRecord* rec, int cur, int alt, int prefill,
                               int32_t a, int32_t b, int warmup, int iters, float* out_us) {
    if (!ctx || !rec || !out_us || iters <= 0 || warmup < 0) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "bad benchmark arguments");
    Dyn d{prefill != 0, prefill ? 0 : a, prefill ? a : 0, prefill ? b : 0};
    if (int e = smelt_hip_wait(ctx)) return e;
    for (int i = 0; i < warmup; ++i) {
        const int rc = encode_record(ctx, rec, cur, alt, d);
        if (rc < 0) return rc;
        if (rc == 0) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "record does not dispatch for these arguments");
    }
    if (int e = smelt_hip_wait(ctx)) return e;
    std::vector<hipEvent_t> ev((size_t)iters * 2, nullptr);
    for (hipEvent_t& e : ev) {
        const hipError_t err = hipEventCreate(&e);
        if (err != hipSuccess) {
            for (hipEvent_t& made : ev)
                if (made) (void)hipEventDestroy(made);
            return hip_fail(ctx, err, "hipEventCreate");
        }
    }
    int status = SMELT_HIP_OK;
    ctx->batch_open = true;  // keep encode_record from re-recording the batch start event
    for (int i = 0; i < iters && status == SMELT_HIP_OK; ++i) {
        if (hipEventRecord(ev[(size_t)2 * i], ctx->stream) != hipSuccess) { status = fail(ctx, SMELT_HIP_ERR_HIP, "hipEventRecord"); break; }
        const int rc = encode_record(ctx, rec, cur, alt, d);
        if (rc < 0) { status = rc; break; }
        if (hipEventRecord(ev[(size_t)2 * i + 1], ctx->stream) != hipSuccess) { status = fail(ctx, SMELT_HIP_ERR_HIP, "hipEventRecord"); break; }
    }
    ctx->batch_open = false;
    ctx->timing_valid = false;
    if (hipStreamSynchronize(ctx->stream) != hipSuccess && status == SMELT_HIP_OK) status = fail(ctx, SMELT_HIP_ERR_HIP, "hipStreamSynchronize");
    if (status == SMELT_HIP_OK) {
        for (int i = 0; i < iters; ++i) {
            float ms = 0;
            if (hipEventElapsedTime(&ms, ev[(size_t)2 * i], ev[(size_t)2 * i + 1]) != hipSuccess) { status = fail(ctx, SMELT_HIP_ERR_HIP, "hipEventElapsedTime"); break; }
            out_us[i] = ms * 1000.0f;
        }
    }
    for (hipEvent_t& e : ev) (void)hipEventDestroy(e);
    return status;
}

static int capture(smelt_hip_context* ctx, const SmeltDispatchRecord* table, size_t count, int cur0, int alt0, const Dyn& d, smelt_hip_graph** out) {
    if (!ctx || !out) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null argument");
    *out = nullptr;
    if (int e = smelt_hip_wait(ctx)) return e;
    HIP_TRY(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->batch_open = true;  // no event records inside the capture
    const int launched = interpret(ctx, table, count, cur0, alt0, d);
    ctx->batch_open = false;
    ctx->timing_valid = false;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    if (launched < 0) {
        if (graph) (void)hipGraphDestroy(graph);
        return launched;
    }
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamEndCapture");
    smelt_hip_graph* g = new smelt_hip_graph();
    g->graph = graph;
    g->launches = launched;
    e = hipGraphInstantiate(&g->exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        delete g;
        return hip_fail(ctx, e, "hipGraphInstantiate");
    }
    *out = g;
    return launched;
}

int smelt_hip_graph_capture_decode(smelt_hip_context* ctx, const SmeltDispatchRecord* table, size_t count, int cur0, int alt0, int32_t position, smelt_hip_graph** out) {
    Dyn d{false, position, 0, 0};
    return capture(ctx, table, count, cur0, alt0, d, out);
}

int smelt_hip_graph_capture_prefill(smelt_hip_context* ctx, const SmeltDispatchRecord* table, size_t count, int cur0, int alt0, int32_t seq_len, int32_t start_pos, smelt_hip_graph** out) {
    Dyn d{true, 0, seq_len, start_pos};
    return capture(ctx, table, count, cur0, alt0, d, out);
}

int smelt_hip_graph_launch(smelt_hip_context* ctx, smelt_hip_graph* graph) {
    if (!ctx || !graph) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null argument");
    if (!ctx->batch_open) {
        HIP_TRY(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
        ctx->batch_open = true;
        ctx->timing_valid = false;
    }
    HIP_TRY(ctx, hipGraphLaunch(graph->exec, ctx->stream));
    return graph->launches;
}

void smelt_hip_graph_destroy(smelt_hip_context* ctx, smelt_hip_graph* graph) {
    if (!graph) return;
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    delete graph;
}

int smelt_hip_graph_time(smelt_hip_context* ctx, smelt_hip_graph* graph, int iters, float* out_total_us) {
    if (!ctx || !graph || !out_total_us || iters <= 0) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "bad arguments");
    if (int e = smelt_hip_wait(ctx)) return e;
    HIP_TRY(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
    for (int i = 0; i < iters; ++i) HIP_TRY(ctx, hipGraphLaunch(graph->exec, ctx->stream));
    HIP_TRY(ctx, hipEventRecord(ctx->ev_end, ctx->stream));
    HIP_TRY(ctx, hipEventSynchronize(ctx->ev_end));
    float ms = 0;
    HIP_TRY(ctx, hipEventElapsedTime(&ms, ctx->ev_start, ctx->ev_end));
    *out_total_us = ms * 1000.0f;
    ctx->timing_valid = true;
    return SMELT_HIP_OK;
}

int smelt_hip_device_info(smelt_hip_context* ctx, char* name, size_t name_cap, int* compute_units, size_t* lds_per_block, size_t* hbm_bytes) {
    if (!ctx) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context");
    if (name && name_cap) {
        std::string n = std::string(ctx->props.name) + " (" + ctx->props.gcnArchName + ")";
        snprintf(name, name_cap, "%s", n.c_str());
    }
    if (compute_units) *compute_units = ctx->props.multiProcessorCount;
    if (lds_per_block) *lds_per_block = ctx->lds_limit;
    if (hbm_bytes) *hbm_bytes = ctx->props.totalGlobalMem;
    return SMELT_HIP_OK;
}

int smelt_hip_memory_info(smelt_hip_context* ctx, size_t* free_bytes, size_t* total_bytes) {
    if (!ctx) return fail(ctx, SMELT_HIP_ERR_INVALID_ARGUMENT, "null context");
    HIP_TRY(ctx, hipSetDevice(ctx->device));
    size_t f = 0, t = 0;
    HIP_TRY(ctx, hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return SMELT_HIP_OK;
}

}  // extern "C"
