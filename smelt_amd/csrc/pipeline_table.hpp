// Pipeline-name resolution: manifest pipeline strings -> (code-object symbol, argument
// signature, appended shape arguments, validator).  Host-only; shared by the runtime (to
// launch) and the record emitters (to know what a family binds).
#pragma once
#include <stdint.h>

#include <string>
#include <vector>

namespace smelt_host {

enum ActDType { kActF16 = 0, kActBF16 = 1 };

enum FamilyId {
    kFamAffineMatvec = 0,     // W S B x y | rows cols group
    kFamAffineAdd,            // W S B x y res | rows cols group
    kFamAffineGateUp,         // gW gS gB uW uS uB x y | rows cols group
    kFamAffineDual,           // W1 S1 B1 W2 S2 B2 x y1 y2 | rows cols group
    kFamAffineBatched,        // W S B X Y batch | rows cols group batch_tile
    kFamAffineGateUpBatched,  // gW gS gB uW uS uB X Y batch | rows cols group batch_tile
    kFamAffineQmm,            // W S B X Y batch | rows cols group batch_tile
    kFamAffineQmmAdd,         // W S B X mv res out batch | rows cols group batch_tile
    kFamAffineQmmGateUp,      // gW gS gB uW uS uB X Y batch | rows cols group batch_tile
    kFamAffineArgmax,         // W S B X keys batch logit_cap | rows cols group batch_tile rows_per_block
    kFamLmHeadReduce,         // keys out batch | num_partials(const from record or appended)
    kFamSignedMatvec,         // C S X Y rows cols                      (batch = grid.y)
    kFamSignedAdd,            // C S X Y res rows cols
    kFamSignedGateUp,         // gC gS uC uS X Y rows cols
    kFamSignedB4,             // C S X Y rows cols batch                (4 batch rows per grid.y)
    kFamSignedGateUpB4,       // gC gS uC uS X Y rows cols batch
    kFamTerAffMatvec,         // C S S2 X Y rows cols                   (batch = grid.y)
    kFamTerAffAdd,            // C S S2 X Y res rows cols
    kFamTerAffGateUp,         // gC gS gS2 uC uS uS2 X Y rows cols
    kFamTerAffBank4,          // C S S2 x y0 y1 y2 y3 rows0 rows1 rows2 rows3 cols
    kFamTerAffQmm,            // C S S2 X Y rows cols batch
    kFamAffineBank4,          // W S B x y0 y1 y2 y3 rows0 rows1 rows2 rows3 | cols group
    kFamAffineGather,         // W S B id out cols group
    kFamAffineGatherBatched,  // W S B ids out cols batch group
    kFamSignedGather,         // C S ids out hidden
    kFamArgmaxPartials,       // logits partials vocab chunk
    kFamArgmaxReduce,         // partials out num_partials
    kFamCopy,                 // src dst n16
    kFamAffineQuantize,       // src packed scales biases [importance] rows src_dtype clip | cols group
    kFamSignedValidate,       // codes status count_lo count_hi format
    kFamSignedMlxScales,      // scales biases out status groups format
    kFamRmsNorm,              // x w y | dim eps two_step            (grid.x = token row)
    kFamRmsNormAdd,           // x w res y | dim eps two_step
    kFamRmsScale,             // x scale | dim eps
    kFamResidualAddRmsScale,  // a b out scale dim eps
    kFamElementwise,          // a b out count
    kFamLutMatvec,            // W lut x y rows | cols group                 (group = rows per table)
    kFamLutAdd,               // W lut x y res rows | cols group
    kFamLutDual,              // W1 lut1 W2 lut2 x y1 y2 rows | cols group
    kFamLutGateUp,            // gW glut uW ulut x y rows | cols group
    kFamLutGather,            // W lut token out cols group
    kFamTqhPrepare,           // x xhat cols                                 (grid.y = token)
    kFamTqhMatvec,            // codes codebook xhat y rows cols codes_per_row (grid.y = token)
    kFamTqhGather,            // codes codebook token out codes_per_row cols
    kFamActivationPlanes,     // x planes scales cols | nplanes             (grid.y = token)
    kFamSwigluPlanes,         // gate up planes scales cols | nplanes
    kFamNormScalePlanes,      // norm_scale x w planes scales cols | nplanes
    kFamPlaneMatvec,          // C S planes ascales Y rows cols | nplanes   (grid.y = token)
    kFamPlaneAdd,             // C S planes ascales Y res rows cols | nplanes
    kFamPlaneGateUp,          // gC gS uC uS planes ascales Y rows cols | nplanes
    kFamPlaneBatched,         // C S planes ascales Y rows cols batch | nplanes tile   (grid.y = token tile)
    kFamPlaneBank4,           // C S planes ascales y0 y1 y2 y3 rows0 rows1 rows2 rows3 cols | nplanes
    kFamBinaryPackedBank,     // C S x y0 y1 rows0 rows1 cols
    kFamBinaryPackedBank4,    // C S x y0 y1 y2 y3 rows0 rows1 rows2 rows3 cols
    kFamBinaryTwoMatrix,      // C1 S1 C2 S2 x y1 y2 rows1 rows2 cols
    kFamCopy16,               // src dst count
    kFamNormScaleAffineMatvec,   // rs x nw xn W S B y | rows cols group           (grid.y = token)
    kFamNormScaleAffineGateUp,   // rs x nw gW gS gB uW uS uB y | rows cols group
    kFamNormScaleAffineBatched,  // rs X nw XN W S B Y batch | rows cols group batch_tile
    kFamNormAddScaleAffineMatvec,// rs x nw res xn W S B y | rows cols group           (grid.y = token)
    kFamNormScaleAffineDual,     // rs x nw W1 S1 B1 W2 S2 B2 y1 y2 | rows cols group (grid.y = token)
    kFamFusedNormAffineMatvec,   // x nw xn W S B y scratch rows eps | cols group
    kFamFusedNormAffineGateUp,   // x nw gW gS gB uW uS uB y scratch rows eps | cols group
    kFamRmsNormAddScalar,        // x w res scalar y | dim eps mode             (grid.x = token row)
    kFamRmsNormFromFp32,         // x(fp32) w y dim eps
    kFamRmsNormGated,            // x gate w y head_dim eps | precise            (grid.x = head)
    kFamRmsNormGatedBatched,     // x gate w y heads_per_token | head_dim eps precise (grid = heads x tokens)
    kFamRmsNormGatedPlanes,      // x gate w planes scales head_dim eps          (grid.x = head = 128-value group)
    kFamUnary,                   // in out count [param] | ... op                 (threads grid)
    kFamScalarMul,               // in out scalar count
    kFamScalarMulWeight,         // in scalar out count
    kFamLutMatmul,               // W lut X Y cols group rows                    (grid.y = token)
    kFamGegluStridedBatched,     // gate up out count up_stride                  (threads grid, grid.y = token)
    kFamBiasAddBatched,          // in bias out rows                             (threads grid, grid.y = token)
    kFamNormScaleAffineQmm,      // rs X nw XN W S B Y batch | rows cols group batch_tile          (MFMA slabs)
    kFamNormScaleAffineQmmGateUp,// rs X nw gW gS gB uW uS uB Y batch | rows cols group batch_tile
    kFamAffineDualAdd,           // W1 S1 B1 W2 S2 B2 x y1 y2 res1 res2 | rows cols group          (grid.y = token)
    kFamAffineDualBatched,       // W1 S1 B1 W2 S2 B2 X Y1 Y2 batch | rows cols group batch_tile
    kFamCount
};

enum SignedFormat { kFmtNone = -1, kFmtBinary1 = 0, kFmtTernary2 = 1, kFmtTrit5 = 2 };

struct ResolvedPipeline {
    FamilyId family = kFamCount;     // kFamCount: not resolved (a pipeline created with allow_missing keeps it)
    std::string symbol;              // kernel symbol in the code object
    std::string kinds;               // final argument kinds: 'P' pointer, 'U' u32, 'F' f32,
                                     // 'Z' pointer the record does not bind (passed as null)
    std::vector<uint32_t> appended;  // values appended after the record's own bindings
    ActDType act = kActF16;
    SignedFormat format = kFmtNone;
    uint32_t lds_variant = 0;        // batched matvec: activation rows resident per pass (1, 2, 4);
                                     // qmm: 16-token blocks per workgroup tile (1, 2, 4),
                                     // or kSkinnyVariant for the split-K skinny kernels
    std::string symbol_single;       // optional kernel for launches whose batch argument is 1
    int single_arg = -1;             // index of that batch argument
    // Single-pass matrix-core matvec of the same pipeline, picked per launch by shape: the kernel is
    // mm1_prefix + "nl<N>_" + mm1_tail for N segments per wave (empty prefix: the pipeline has none).
    std::string mm1_prefix, mm1_tail;
    int mm1_layout = -1;             // CodeLayout of its weights
    uint32_t mm1_nmat = 1;
    bool workspace = false;          // kernel takes the context's (partials, counters) pointers last
    // Streaming form of a skinny qmm pipeline, picked per launch by shape: the kernel is
    // "smelt_affine_qms_r<R>_x<X>_" + qms_tail for R row tiles per wave and 4 X staged token rows.
    std::string qms_tail;
    uint32_t qms_nmat = 1;
};

constexpr uint32_t kSkinnyVariant = 32;
// LDS bytes of the skinny qmm kernels for a K split into `ksplit` chunks.
size_t qmm_skinny_lds_bytes(uint32_t cols, uint32_t ksplit, uint32_t nmat, uint32_t live_tokens, uint32_t waves);

enum ResolveStatus { kResolveOk = 0, kResolveUnknown = 1, kResolveMalformed = 2 };

// entry: "fn", "fn:cols:group", optionally followed by "@f16" / "@bf16".
ResolveStatus resolve_pipeline(const std::string& entry, ActDType default_act, size_t lds_limit,
                               ResolvedPipeline* out, std::string* why);

// Packed-code layouts the matvec kernels consume.
enum CodeLayout { kCodesU4 = 0, kCodesBinary1 = 1, kCodesTernary2 = 2, kCodesTrit5 = 3 };
CodeLayout code_layout(SignedFormat f);

// LDS bytes the matvec kernels need for one packed row stride with `mb` resident activation rows.
size_t matvec_lds_bytes(CodeLayout layout, uint32_t row_stride_bytes, uint32_t mb);
// LDS bytes of the activation-view consumers: eight 16-byte plane slots and four floats per token and unit.
size_t plane_matvec_lds_bytes(uint32_t row_stride_bytes, uint32_t mb);
// LDS bytes of the MFMA qmm kernels: nmat weight tiles of 64 x 128 fp16 plus 16*mt token rows.
size_t qmm_lds_bytes(uint32_t nmat, uint32_t mt);
// LDS bytes of the affine qmm kernels: packed code tiles, fp32 scale/bias tiles, token rows and sums.
size_t qmm_affine_lds_bytes(uint32_t nmat, uint32_t mt);

uint32_t signed_row_stride(SignedFormat f, uint32_t cols);

// Launch plan of the single-pass matrix-core matvec: one workgroup of `kc` waves per eight rows,
// `nl` 128-byte row segments per wave.  False when the shape stays on the vector-ALU kernels
// (`force` drops the size threshold, not the geometry limits).
constexpr uint32_t kMm1MaxSegments = 8;
struct Mm1Plan {
    uint32_t kc = 0, nl = 0;
    size_t lds = 0;
};
// (`tokens_per_pass` 2: the kernels that multiply two tokens per pass stage two sets of activation fragments)
bool mm1_plan(CodeLayout layout, uint32_t rows, uint32_t cols, uint32_t group, uint32_t nmat, size_t lds_limit,
              bool force, Mm1Plan* out, uint32_t tokens_per_pass = 1);

// Launch plan of the streaming skinny qmm: workgroups of `kc` waves over 16 * rt rows each, 16 tokens
// per grid row; wave c takes the pairs of scale groups c, c + kc, ...  False when the shape has no
// such kernel.
constexpr uint32_t kQmsMaxRowTiles = 2;   // what qms_plan returns: one or two
struct QmsPlan {
    uint32_t rt = 0, kc = 0;
    size_t lds = 0;
};
bool qms_plan(uint32_t rows, uint32_t cols, uint32_t group, uint32_t nmat, uint32_t batch, uint32_t compute_units,
              size_t lds_limit, QmsPlan* out);
// Launch plan of the streaming ternary qmm (two-bit codes, groups of 128 columns): workgroups of `kc` waves over
// sixteen rows, sixteen tokens per grid row, wave c takes the 128-column steps c, c + kc, ...
bool qts_plan(uint32_t rows, uint32_t cols, uint32_t batch, size_t lds_limit, QmsPlan* out);
// ... and of the streaming kernels of the binary (bits = 1) and ternary (2) per-token records over many tokens.
bool qss_plan(uint32_t bits, uint32_t nmat, uint32_t rows, uint32_t cols, uint32_t batch, size_t lds_limit, QmsPlan* out);


// Launch plan of the token-tile qmm: workgroups of 4 * kw waves over 32 * rt rows (per matrix) and
// 32 * tb tokens.  False when the shape has no such kernel or too few tokens to pay for the tiles.
struct QmtPlan {
    uint32_t rt = 0, tb = 0, kw = 1;           // row tiles and token blocks per wave, waves along K
    bool per_wave = false;                     // two matrices: one per wave along the rows (16 * rt rows of each per workgroup)
    uint32_t bn = 0, bm = 0;                   // rows (per matrix) and tokens of a workgroup tile
    uint32_t ksplit = 1;                       // workgroups that share a tile (grid z); above 1 they meet in the workspace
    size_t partial_bytes = 0, counter_bytes = 0;   // workspace the split needs
    size_t lds = 0;
};
bool qmt_plan(uint32_t rows, uint32_t cols, uint32_t group, uint32_t nmat, uint32_t batch, uint32_t compute_units,
              size_t lds_limit, QmtPlan* out);

}  // namespace smelt_host
