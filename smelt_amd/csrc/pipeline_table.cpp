// Pipeline-name resolution.  The reference resolves a manifest pipeline string to a Metal
// function by exact name, or by "name:cols:groupSize" function constants
// (SmeltRuntime.swift:6229-6263); its catalog carries one Metal function per tuned shape
// (SmeltKernelCatalog.swift).  The HIP kernels take the shape as arguments, so every name of
// an in-scope family maps onto a handful of symbols plus appended shape values.
#include "pipeline_table.hpp"

#include <cstring>

namespace smelt_host {

namespace {

bool starts_with(const std::string& s, const char* p) { return s.compare(0, strlen(p), p) == 0; }

bool parse_uint(const std::string& s, uint32_t* out) {
    if (s.empty() || s.size() > 9) return false;
    uint32_t v = 0;
    for (char c : s) {
        if (c < '0' || c > '9') return false;
        v = v * 10 + (uint32_t)(c - '0');
    }
    *out = v;
    return true;
}

// "_c1024_r2048_g64<suffix>" -> cols, rows, group, suffix
bool parse_fixed_shape(const std::string& rest, uint32_t* cols, uint32_t* rows, uint32_t* group,
                       std::string* suffix) {
    if (!starts_with(rest, "_c")) return false;
    size_t p = 2, q = rest.find("_r", p);
    if (q == std::string::npos || !parse_uint(rest.substr(p, q - p), cols)) return false;
    p = q + 2;
    q = rest.find("_g", p);
    if (q == std::string::npos || !parse_uint(rest.substr(p, q - p), rows)) return false;
    p = q + 2;
    q = p;
    while (q < rest.size() && rest[q] >= '0' && rest[q] <= '9') ++q;
    if (!parse_uint(rest.substr(p, q - p), group)) return false;
    *suffix = rest.substr(q);
    return true;
}

bool is_pow2(uint32_t v) { return v && !(v & (v - 1)); }

const char* act_suffix(ActDType a) { return a == kActBF16 ? "bf16" : "f16"; }

// resident activation rows per pass for the batched matvec kernels, bounded by LDS
uint32_t pick_mb(CodeLayout layout, uint32_t row_stride, uint32_t want, size_t lds_limit) {
    for (uint32_t mb = want; mb > 1; mb >>= 1)
        if (matvec_lds_bytes(layout, row_stride, mb) <= lds_limit) return mb;
    return 1;
}

struct AffineName {
    const char* prefix;
    FamilyId m1;
};

}  // namespace

CodeLayout code_layout(SignedFormat f) {
    switch (f) {
        case kFmtBinary1: return kCodesBinary1;
        case kFmtTernary2: return kCodesTernary2;
        case kFmtTrit5: return kCodesTrit5;
        default: return kCodesU4;
    }
}

size_t matvec_lds_bytes(CodeLayout layout, uint32_t row_stride_bytes, uint32_t mb) {
    const size_t U = row_stride_bytes / 16;
    // 16-byte LDS chunks of fp16 pairs per unit, and floats of per-dword corrections per unit
    size_t chunks = 4, corr = 4, extra = 0;
    switch (layout) {
        case kCodesU4: chunks = 4; break;
        case kCodesTernary2: chunks = 8; break;
        case kCodesBinary1: chunks = 16; break;
        case kCodesTrit5: chunks = 10; corr = 8; extra = 512; break;  // + decode table
    }
    return (size_t)mb * U * (16 * chunks + 2 * 4 * corr) + extra;
}

size_t plane_matvec_lds_bytes(uint32_t row_stride_bytes, uint32_t mb) {
    const size_t U = row_stride_bytes / 16;
    return (size_t)mb * U * (16 * 8 + 2 * 4 * 4);
}

size_t qmm_lds_bytes(uint32_t nmat, uint32_t mt) {
    const size_t ld = 128 + 8;
    return ((size_t)nmat * 64 + (size_t)mt * 16) * ld * 2;
}

size_t qmm_affine_lds_bytes(uint32_t nmat, uint32_t mt) {
    return (size_t)nmat * (64 * 80 + 2 * 4 * 64 * 4) + (size_t)mt * (16 * (128 + 8) * 2 + 16 * 4 * 4);
}

size_t qmm_skinny_lds_bytes(uint32_t cols, uint32_t ksplit, uint32_t nmat, uint32_t live_tokens, uint32_t waves) {
    // staged activations: per 64-column window of a chunk, 8 operand rows of (tokens + 1) 16-byte
    // slots and 8 rows of (tokens + 1) run sums (live tokens rounded up to a power of two), plus
    // fp16 high/low activation sums in blocks of 16 groups; the wave reduction
    // (waves x nmat x 4 KB) reuses the same bytes
    uint32_t shift = 0;
    while ((1u << shift) < live_tokens) ++shift;
    const size_t nwin = cols / 64, cw = (nwin + ksplit - 1) / ksplit;
    const size_t stage = cw * 8 * ((1u << shift) + 1) * 20 + ((cw + 15) / 16 + 1) * 2048;
    const size_t reduce = (size_t)waves * nmat * 4096;
    return stage > reduce ? stage : reduce;
}

uint32_t signed_row_stride(SignedFormat f, uint32_t cols) {
    const uint32_t padded = (cols + 127u) / 128u * 128u;
    switch (f) {
        case kFmtBinary1: return padded / 8;
        case kFmtTernary2: return padded / 4;
        case kFmtTrit5: return (((cols + 4u) / 5u) + 15u) & ~15u;
        default: return 0;
    }
}

bool mm1_plan(CodeLayout layout, uint32_t rows, uint32_t cols, uint32_t group, uint32_t nmat, size_t lds_limit,
              bool force, Mm1Plan* out, uint32_t tokens_per_pass) {
    uint32_t row_stride, frags, nl_max, dw = 4;
    switch (layout) {
        case kCodesU4: row_stride = cols / 2; frags = 4; nl_max = 8; break;
        case kCodesTernary2: row_stride = (cols + 127u) / 128u * 32u; frags = 8; nl_max = 6; break;
        case kCodesBinary1: row_stride = (cols + 127u) / 128u * 16u; frags = 16; nl_max = 6; break;
        // five digits per byte: a 16-byte piece is five dwords of sixteen columns, a 128-byte segment five groups
        case kCodesTrit5: if (cols % 16 != 0) return false; row_stride = (((cols + 4u) / 5u) + 15u) & ~15u; frags = 10; nl_max = 3; dw = 5; break;
        default: return false;
    }
    if (rows == 0 || cols == 0 || row_stride % 16 != 0 || group < 32 || (group & (group - 1))) return false;
    if (tokens_per_pass != 1 && (tokens_per_pass != 2 || dw != 4)) return false;
    if (layout != kCodesU4 && group != 128) return false;
    // No size threshold: measured on MI355X (cold, per launch in a graph) the single-pass kernel is the faster one
    // at every size once small matrices walk one segment per wave: affine 4-bit 64 x 1024 to 1024 x 1024 2.1-2.7 us
    // against 2.5-4.0 on the vector-ALU kernel, binary / ternary / five-digit bytes 256 x 1024 to 2048 x 640
    // 2.1-2.6 / 2.1-2.5 / 2.7-3.0 against 3.2-3.3 / 2.8-3.0 / 3.5-4.0.  (`force` is kept for callers that ask.)
    (void)force;
    const uint32_t pieces = row_stride / 16, nseg = (pieces + 7) / 8, gpr = (cols + group - 1) / group;
    const uint32_t planes = layout == kCodesU4 ? 2 : 1;
    auto lds_of = [&](uint32_t kc, uint32_t nl) {
        // four-dword pieces are stored one fragment apart (LDS banks), except the four-fragment ones (swizzled instead)
        const size_t tok = tokens_per_pass;
        const size_t wave = tok * ((size_t)nl * 8 * (dw == 4 ? (frags == 4 ? 4 : frags + 1) : frags) * 16 + (dw == 4 ? (size_t)nl * 8 * 8 : (size_t)nl * 8 * dw * 4)) + (size_t)frags * 16;
        return kc * wave + (size_t)nmat * planes * 8 * gpr * 2 + (size_t)kc * nmat * tok * 32 + (dw == 4 ? 0 : 512);   // + decode table
    };
    Mm1Plan best;
    uint32_t best_waste = ~0u;
    const uint32_t tolerated = nseg / 10 > 1 ? nseg / 10 : 1;
    // Segments per wave, in order of preference.  Affine 4-bit rows are long (a 5120-column row is twenty
    // segments): as many segments per wave as the kernels have.  The signed formats measured best with two
    // (binary 27B layer 33.5 -> 31.5 us, five-digit bytes 50.2 -> 47.6 against three; one or four and more
    // were slower), then three where two would need more than sixteen waves.
    // (seven and eight only where nothing shorter covers the row: rows of more than 24576 columns)
    // (binary and ternary: four to six only for rows that three per wave on sixteen waves do not cover, ternary
    // beyond 24576 columns; the five-digit kernels exist for one to three: up to 30720 columns)
    static const uint32_t kLongRows[] = {6, 5, 4, 3, 2, 1, 7, 8}, kSigned[] = {2, 3, 1, 4, 5, 6, 7, 8};
    const uint32_t* order = layout == kCodesU4 ? kLongRows : kSigned;
    const uint32_t norder = 8;
    // Affine matrices below 8M weights (a 0.8B model's projections) are a launch and one memory round trip:
    // the more waves share a row the shorter that trip, so the fewest segments per wave that eight waves cover
    // (config-1 step 0.366 -> 0.346 ms against the vector kernels)
    static const uint32_t kShortWalk[] = {1, 2, 3, 4, 5, 6, 7, 8};
    const bool small_affine = layout == kCodesU4 && (uint64_t)rows * cols < (8u << 20);
    if (small_affine) order = kShortWalk;
    // Between 8M and 24M weights (a 4B model's projections: 13 MB, a few workgroups per compute unit) two
    // segments per wave, as long as twelve waves cover the row and all waves of the launch fit the machine about
    // at once; measured per launch, cold, against the long walk: 9216 x 2560 5.0 against 5.5 us, 2560 x 9216 (three
    // segments: twelve waves) 6.4 against 7.0, 4096 x 4096 4.2 against 4.5, 3072 x 3072 3.8 against 4.4.  From 24M
    // weights on (5120-column rows and longer) the long walk stays: 5120 x 5120 5.7 against 6.0, 17408 x 5120
    // gate+up 19.5 against 22.4.
    static const uint32_t kMidWalk[] = {2, 1, 3, 4, 5, 6, 7, 8};
    const bool mid_affine = layout == kCodesU4 && !small_affine && (uint64_t)rows * cols < (24u << 20);
    if (mid_affine) order = kMidWalk;
    // The signed formats below the 27B shapes: one segment per wave (binary 4096 x 4096 3.5 against 3.8 us,
    // 9216 x 2560 4.25 against 4.5; five-digit bytes 4.55 against 4.9 and 5.3 against 5.7; 2048 x 2048 in all three
    // 2.6 / 2.6 / 3.35 against 2.8 / 2.8 / 3.8); ternary from 8M weights keeps two (3.5 against 3.7, 4.3 against 4.4).
    static const uint32_t kSignedShort[] = {1, 2, 3, 4, 5, 6, 7, 8};
    if (layout != kCodesU4 && (uint64_t)rows * cols < (layout == kCodesTernary2 ? (8u << 20) : (24u << 20))) order = kSignedShort;
    const uint64_t tiles = ((uint64_t)rows + 7) / 8;
    // Affine matrices from 24M weights: a wave count that is a multiple of four (every SIMD of the compute unit
    // carries the same number of the workgroup's waves) with next to no idle segments, eight first, then twelve,
    // four, sixteen.  Measured per launch, cold, against the long walk below: 8192 x 8192 9.6 against 10.8 us
    // (four segments on eight waves), 28672 x 8192 27.2 against 31.1, 4096 x 8192 6.25 against 6.9, 14336 x 4096
    // 8.4 against 8.6 (two on eight), 4096 x 14336 9.7 against 10.5 (five on twelve); 5120- and 17408-column rows
    // come out as before (five on four, six on twelve).  Never one segment per wave here: a tall matrix of short
    // rows (an lm_head read as plain logits) has thousands of tiles and wants few, long waves (151936 x 1024: four
    // segments on one wave 18.4 us, one on four 27.3, the vector kernel 19-20; 151936 x 2048: 31.8-34.8 against 53).
    if (layout == kCodesU4 && !small_affine && !mid_affine && tiles >= 16384 && nseg <= 16) {
        // more tiles than twice the machine's wave slots: as few waves per tile as cover the row, one up to eight
        // segments, two up to sixteen (151936 x 2048: eight segments on one wave 31.8 us, two on four 34.8-43.3,
        // the vector kernel 38-39; cold, 151936 x 3072: six on two 51.0, three on four 58.5, vector 65; 151936 x 3584:
        // seven on two 61.6, five on three 66.3-68.6, vector 70; 151936 x 4096: two, four and eight waves 74-75)
        for (uint32_t nl = nl_max < nseg ? nl_max : nseg; nl >= 1; --nl) {
            const uint32_t kc = (nseg + nl - 1) / nl;
            const size_t lds = lds_of(kc, nl);
            if (kc > 16 || gpr > 64 * kc || kc * nl - nseg > tolerated || lds > lds_limit) continue;
            out->kc = kc; out->nl = nl; out->lds = lds;
            return true;
        }
    }
    if (layout == kCodesU4 && !small_affine && !mid_affine) {
        static const uint32_t kWaves[] = {8, 12, 4, 16};
        for (uint32_t longest : {6u, nl_max})   // seven and eight segments only where six cover no such split
        for (uint32_t kc : kWaves) {
            const uint32_t nl = (nseg + kc - 1) / kc;
            if (nl < 2 || nl > longest || (nseg + nl - 1) / nl != kc || gpr > 64 * kc) continue;
            const uint32_t waste = kc * nl - nseg;
            const size_t lds = lds_of(kc, nl);
            if (waste > tolerated || lds > lds_limit) continue;
            out->kc = kc; out->nl = nl; out->lds = lds;
            return true;
        }
    }
    // (a second pass without the size class's own limits: a short matrix of very long rows still has a plan)
    for (int pass = 0; pass < 2 && best.kc == 0; ++pass)
    for (uint32_t o = 0; o < norder; ++o) {
        const uint32_t nl = order[o];
        if (nl > nl_max || (nl > nseg && nl > 1)) continue;
        const uint32_t kc = (nseg + nl - 1) / nl;
        const uint32_t most = pass == 0 ? (small_affine ? 8u : (mid_affine ? 12u : 16u)) : 16u;
        if (kc > most || gpr > 64 * kc) continue;   // one workgroup; its threads carry one scale piece each
        if (pass == 0 && mid_affine && nl < 6 && tiles * kc > 11264) continue;   // 1.375 x the 8192 wave slots of the machine
        const size_t lds = lds_of(kc, nl);
        if (lds > lds_limit) continue;
        const uint32_t waste = kc * nl - nseg;
        if (waste <= tolerated) { best.kc = kc; best.nl = nl; best.lds = lds; best_waste = waste; break; }
        if (waste < best_waste) { best.kc = kc; best.nl = nl; best.lds = lds; best_waste = waste; }
    }
    if (best.kc == 0) return false;
    *out = best;
    return true;
}

namespace {

// The vector-ALU kernels that have a single-pass matrix-core form, by symbol stem.
void attach_mm1(ResolvedPipeline* r) {
    struct Form { const char* stem; const char* prefix; const char* tail; CodeLayout layout; uint32_t nmat; };
    static const Form kForms[] = {
        {"smelt_affine_matvec_", "smelt_affine_mm1_", "matvec_", kCodesU4, 1},
        {"smelt_affine_matvec_add_", "smelt_affine_mm1_", "matvec_add_", kCodesU4, 1},
        {"smelt_affine_gate_up_swiglu_", "smelt_affine_mm1_", "gate_up_swiglu_", kCodesU4, 2},
        {"smelt_affine_bank4_matvec_", "smelt_affine_mm1_", "bank4_matvec_", kCodesU4, 1},
        {"smelt_affine_dual_matvec_", "smelt_affine_mm1_", "dual_matvec_", kCodesU4, 2},
        {"smelt_affine_dual_matvec_add_", "smelt_affine_mm1_", "dual_matvec_add_", kCodesU4, 2},
        {"smelt_affine_gate_up_geglu_", "smelt_affine_mm1_", "gate_up_geglu_", kCodesU4, 2},
        {"smelt_norm_scale_affine_matvec_", "smelt_affine_mm1_", "norm_scale_matvec_", kCodesU4, 1},
        {"smelt_norm_add_scale_affine_matvec_", "smelt_affine_mm1_", "norm_add_scale_matvec_", kCodesU4, 1},
        {"smelt_norm_scale_affine_dual_matvec_", "smelt_affine_mm1_", "norm_scale_dual_matvec_", kCodesU4, 2},
        {"smelt_norm_scale_affine_gate_up_swiglu_", "smelt_affine_mm1_", "norm_scale_gate_up_swiglu_", kCodesU4, 2},
        {"smelt_norm_scale_affine_gate_up_geglu_", "smelt_affine_mm1_", "norm_scale_gate_up_geglu_", kCodesU4, 2},
        {"smelt_signed_binary_matvec_", "smelt_signed_binary_mm1_", "matvec_", kCodesBinary1, 1},
        {"smelt_signed_binary_matvec_add_", "smelt_signed_binary_mm1_", "matvec_add_", kCodesBinary1, 1},
        {"smelt_signed_binary_gate_up_swiglu_", "smelt_signed_binary_mm1_", "gate_up_swiglu_", kCodesBinary1, 2},
        {"smelt_signed_binary_packed_bank_matvec_", "smelt_signed_binary_mm1_", "packed_bank_matvec_", kCodesBinary1, 1},
        {"smelt_signed_binary_packed_bank4_matvec_", "smelt_signed_binary_mm1_", "packed_bank4_matvec_", kCodesBinary1, 1},
        {"smelt_signed_ternary_matvec_", "smelt_signed_ternary_mm1_", "matvec_", kCodesTernary2, 1},
        {"smelt_signed_ternary_matvec_add_", "smelt_signed_ternary_mm1_", "matvec_add_", kCodesTernary2, 1},
        {"smelt_signed_ternary_gate_up_swiglu_", "smelt_signed_ternary_mm1_", "gate_up_swiglu_", kCodesTernary2, 2},
        {"smelt_signed_trit5_matvec_", "smelt_signed_trit5_mm1_", "matvec_", kCodesTrit5, 1},
        {"smelt_signed_trit5_matvec_add_", "smelt_signed_trit5_mm1_", "matvec_add_", kCodesTrit5, 1},
        {"smelt_signed_trit5_gate_up_swiglu_", "smelt_signed_trit5_mm1_", "gate_up_swiglu_", kCodesTrit5, 2},
        {"smelt_signed_trit5_packed_bank4_matvec_", "smelt_signed_trit5_mm1_", "packed_bank4_matvec_", kCodesTrit5, 1},
        // the four-token forms: the single-token kernels with one grid row per token
        {"smelt_signed_binary_matvec_b4_", "smelt_signed_binary_mm1_", "matvec_", kCodesBinary1, 1},
        {"smelt_signed_binary_gate_up_swiglu_b4_", "smelt_signed_binary_mm1_", "gate_up_swiglu_", kCodesBinary1, 2},
        {"smelt_signed_ternary_matvec_b4_", "smelt_signed_ternary_mm1_", "matvec_", kCodesTernary2, 1},
        {"smelt_signed_ternary_gate_up_swiglu_b4_", "smelt_signed_ternary_mm1_", "gate_up_swiglu_", kCodesTernary2, 2},
        {"smelt_signed_trit5_matvec_b4_", "smelt_signed_trit5_mm1_", "matvec_", kCodesTrit5, 1},
        {"smelt_signed_trit5_gate_up_swiglu_b4_", "smelt_signed_trit5_mm1_", "gate_up_swiglu_", kCodesTrit5, 2},
        // the lm_head at one token (its own argument block: a key per tile and a counter per partial in the workspace)
        {"smelt_affine_matvec_argmax_", "smelt_affine_mm1_", "matvec_argmax_", kCodesU4, 1},
        {"smelt_teraff_matvec_", "smelt_teraff_mm1_", "matvec_", kCodesTernary2, 1},
        {"smelt_teraff_matvec_add_", "smelt_teraff_mm1_", "matvec_add_", kCodesTernary2, 1},
        {"smelt_teraff_gate_up_swiglu_", "smelt_teraff_mm1_", "gate_up_swiglu_", kCodesTernary2, 2},
        {"smelt_teraff_bank4_matvec_", "smelt_teraff_mm1_", "bank4_matvec_", kCodesTernary2, 1},
    };
    const std::string t = act_suffix(r->act);
    // the per-token small-batch forms of the plain matvec and of gate+up (SwiGLU, GeGLU): the single-token kernels with one
    // grid row per token (small matrices at a few tokens; the batch argument leaves the argument block)
    if (r->family == kFamAffineBatched || r->family == kFamAffineGateUpBatched) {
        const bool pair = r->family == kFamAffineGateUpBatched;
        r->mm1_prefix = "smelt_affine_mm1_";
        r->mm1_tail = std::string(!pair ? "matvec_" : (r->symbol.find("geglu") != std::string::npos ? "gate_up_geglu_" : "gate_up_swiglu_")) + t;
        r->mm1_layout = (int)kCodesU4;
        r->mm1_nmat = pair ? 2 : 1;
        return;
    }
    for (const Form& f : kForms) {
        if (r->symbol == std::string(f.stem) + t) {
            r->mm1_prefix = f.prefix;
            r->mm1_tail = std::string(f.tail) + t;
            r->mm1_layout = (int)f.layout;
            r->mm1_nmat = f.nmat;
            return;
        }
    }
}

// The skinny qmm kernels that have a streaming form.
void attach_qms(ResolvedPipeline* r) {
    const std::string t = act_suffix(r->act);
    // (the per-token small-batch forms of the plain matvec and of gate+up+SwiGLU take the same arguments as the
    // skinny qmm of their family: from two tokens on they stream too, 9216 x 2560 at four tokens 7.8 against 16.2 us)
    if (r->family == kFamAffineQmm || r->family == kFamAffineBatched) { r->qms_tail = "store_" + t; r->qms_nmat = 1; }
    else if (r->family == kFamAffineQmmAdd) { r->qms_tail = "add_" + t; r->qms_nmat = 1; }
    // (the lm_head over two tokens and more: logits through the streaming kernel, keys from a second launch)
    else if (r->family == kFamAffineArgmax) { r->qms_tail = "store_" + t; r->qms_nmat = 1; }
    else if ((r->family == kFamAffineQmmGateUp || r->family == kFamAffineGateUpBatched) && r->symbol.find("swiglu") != std::string::npos) { r->qms_tail = "gate_up_swiglu_" + t; r->qms_nmat = 2; }
    else if ((r->family == kFamAffineQmmGateUp || r->family == kFamAffineGateUpBatched) && r->symbol.find("geglu") != std::string::npos) { r->qms_tail = "gate_up_geglu_" + t; r->qms_nmat = 2; }
    // (the norm-scale prologue forms: the rows are normalised by a launch of their own, then the kernels of the plain forms)
    else if (r->family == kFamNormScaleAffineQmm || r->family == kFamNormScaleAffineBatched) { r->qms_tail = "store_" + t; r->qms_nmat = 1; }
    else if (r->family == kFamNormScaleAffineQmmGateUp) { r->qms_tail = std::string(r->symbol.find("geglu") != std::string::npos ? "gate_up_geglu_" : "gate_up_swiglu_") + t; r->qms_nmat = 2; }
}

ResolveStatus resolve_pipeline_entry(const std::string& entry_in, ActDType default_act, size_t lds_limit,
                                     ResolvedPipeline* out, std::string* why);

}  // namespace

bool qmt_plan(uint32_t rows, uint32_t cols, uint32_t group, uint32_t nmat, uint32_t batch, uint32_t compute_units,
              size_t lds_limit, QmtPlan* out) {
    // Measured on MI355X at the 4B FFN shapes: below about 96 tokens the streaming kernel's 16-token
    // passes are as fast or faster (the weights of the later passes come from cache); from there on the
    // shared activation tile wins (128 tokens: 22 against 27 us on 9216 x 2560, 29 against 38 on 2560 x 9216).
    if (group != 64 || cols == 0 || cols % 512 != 0 || rows == 0 || nmat == 0 || nmat > 2) return false;
    // The streaming kernel's time grows with its 16-token passes, this kernel's is flat over a 64-token block, and
    // the larger the matrix the sooner they cross (cold, streaming against token tiles at 33 / 64 / 96 tokens:
    // 5120 x 25600 76 / 100 / 140 us against 51 / 53 / 81; 4096 x 12288 29 / 42 / 57 against 26 / 26 / 36; 8192 x 8192
    // 33 / 41 / 60 against 29 / 28 / 43; 18944 x 3584 33 / 41 / 60 against 28 / 28 / 42; 5120 x 5120 21 / 25 / 33 against
    // 29 / 30 / 29; 9216 x 2560 14 / 18 / 22 against 17 / 17 / 21; 2560 x 9216 16 / 21 / 27 against 23 / 24 / 24; few rows
    // leave this kernel short of tiles: 2048 x 16384 22 / 25 / 34 against 28 / 28 / 38).
    const uint64_t weights = (uint64_t)rows * cols * nmat;
    // Small matrices the other way round: this kernel's walk along K is a latency chain whatever the matrix (9 us at 1024
    // columns, 19 at 3072) while a streaming pass over a small matrix is short (128 / 256 / 512 / 1024 tokens, streaming
    // against token tiles: 1024 x 1024 5.0 / 5.7 / 8.0 / 12.7 against 9.1 - 9.2; 1024 x 3072 7.6 / 11.5 / 20.1 / 36 against
    // 19 - 20; 3072 x 1024 7.3 / 11.0 / 18.0 / 33 against 9.2 / 9.2 / 11.2 / 16; 2048 x 2048 8.8 / 13.0 / 22.4 / 43 against
    // 14.2 / 14.2 / 14.3 / 26; from 6144 x 1024 on the tiles win at 128: 11.3 against 9.3).
    const uint32_t min_batch = weights < (2u << 20) ? 1024u : weights < (5u << 20) ? 384u
                               : weights >= (40u << 20) && rows >= 3584 ? 33u : (weights >= (20u << 20) && rows >= 2560 ? 96u : 128u);
    if (batch < min_batch) return false;
    // buffer loads address the activations and each weight matrix with 32-bit byte offsets
    if ((uint64_t)batch * cols * 2 >= (1ull << 31) || (uint64_t)rows * (cols / 2) >= (1ull << 31)) return false;
    // 96 rows x 64 tokens per workgroup and eight waves (two along K) measured best at 256 to 1024 tokens on
    // the 9216 x 2560 and 2560 x 9216 matrices (48 / 63 us at 512 tokens against 57 / 77 with 64-row and 57 / 83
    // with 128-row tiles of four waves); 64-row tiles when the 96-row ones would leave a quarter of the compute
    // units without a workgroup (2560 rows at 256 tokens: 51 against 62 us).
    const uint32_t token_blocks = (batch + 63) / 64;
    out->tb = 2;
    out->kw = 2;
    out->per_wave = false;
    if (nmat == 2) {
        // gate and up together (9216 x 2560 each): 64 rows of each matrix per workgroup of four waves once that
        // leaves three workgroups per compute unit (104 us at 512 tokens, 170 at 1024); below, the two waves along
        // the rows take one matrix each, 48 rows of it, eight waves: the loop of the one-matrix kernel (54 us at
        // 256 tokens against 61; 106 / 185 at 512 / 1024)
        if ((uint64_t)((rows + 63) / 64) * token_blocks >= 3ull * compute_units) { out->rt = 2; out->kw = 1; }
        else { out->per_wave = true; out->rt = 3; }
    } else {
        const uint64_t tiles3 = (uint64_t)((rows + 95) / 96) * token_blocks;
        out->rt = tiles3 * 4 >= (uint64_t)compute_units * 3 ? 3 : 2;
    }
    out->bn = (out->per_wave ? 16 : 32) * out->rt;
    out->bm = 32 * out->tb;
    const uint64_t tiles = (uint64_t)((rows + out->bn - 1) / out->bn) * token_blocks;
    // few tiles and long rows: workgroups share a tile along K so that every compute unit has about two, each
    // with at least six blocks of 512 columns (2560 x 9216: 58 against 64 us at 512 tokens with two, 34 against
    // 50 us at 256 tokens with three; splitting the 2560-column matrix only cost time)
    out->ksplit = (uint32_t)((2ull * compute_units + tiles / 2) / tiles);
    if (out->ksplit > cols / 512 / 6) out->ksplit = cols / 512 / 6;
    if (out->ksplit < 1) out->ksplit = 1;
    out->partial_bytes = out->ksplit > 1 ? (size_t)tiles * out->ksplit * (out->per_wave ? 1 : nmat) * out->rt * out->tb * 4 * 256 * sizeof(float) : 0;
    out->counter_bytes = out->ksplit > 1 ? (size_t)tiles * sizeof(uint32_t) : 0;
    // two buffers of: token rows, weight rows, scale pairs
    out->lds = 2 * ((size_t)out->bm * 272 + (size_t)nmat * out->bn * 72 + (size_t)nmat * out->bn * 16);
    return out->lds <= lds_limit;
}

bool qms_plan(uint32_t rows, uint32_t cols, uint32_t group, uint32_t nmat, uint32_t batch, uint32_t compute_units,
              size_t lds_limit, QmsPlan* out) {
    // groups of 64 columns (rows of a multiple of 256 columns), of 128 (512) or of 32 (256): scale rows are staged four or
    // eight groups at a time
    if ((group != 32 && group != 64 && group != 128) || cols == 0 || cols % (group == 32 ? 256 : 4 * group) != 0 || rows == 0 ||
        nmat == 0 || nmat > 2 || batch == 0) return false;
    // (groups of 32 take every 64-column half twice: beyond 256 tokens the token-slab kernel is as fast or faster,
    // 14336 x 4096 at 512 tokens 283 us against 356)
    if (group == 32 && batch > 256) return false;
    const uint32_t gt = cols / group, npairs = cols / 128;
    // Measured on MI355X at 2560- and 9216-column rows: about four steps per wave hide the memory
    // round trips best, up to twelve waves; two row tiles per wave (half the activation traffic per
    // weight byte) pay once a pass stages sixteen tokens and the matrix still fills the machine
    // with 32-row workgroups.
    const uint32_t rt = nmat == 1 && batch > 8 && rows >= 32 * 256 && group != 32 ? 2 : 1;   // (the 32-column kernels: one tile)
    uint32_t kc = (npairs + 3) / 4;
    if (kc < 2) kc = npairs < 2 ? 1 : 2;
    if (kc > 12) kc = 12;
    uint32_t steps = (npairs + kc - 1) / kc;
    kc = (npairs + steps - 1) / steps;   // same steps per wave, no idle wave
    // Matrices of many rows: fewer waves with longer walks, about 3500 waves in the launch's first pass, never
    // fewer than four, and only a count that leaves no wave idle (cold, 4 / 8 / 16 tokens: 17408 x 5120 four waves
    // 17.1 / 19.0 / 21.8 us against 19.3 / 20.9 / 24.1 with ten; 14336 x 4096 four 11.8 / 12.3 / 12.6 against 12.3 /
    // 12.8 / 13.4 with eight; 8192 x 8192 eight 12.5 / 13.0 / 13.6 against 13.2 / 14.0 / 15.0 with eleven; 9216 x 2560
    // and 4096 x 4096 keep five and eight: fewer were slower).
    if (nmat == 1) {
        const uint32_t tiles16 = (rows + 15) / 16;
        uint32_t want = (3500 + tiles16 / 2) / tiles16;
        if (want < 4) want = 4;
        for (uint32_t k = want; k < kc; ++k)
            if (npairs % k == 0) { kc = k; steps = npairs / k; break; }
    }
    const uint32_t tiles = nmat * rt;
    const uint32_t token_rows = batch > 8 ? 16 : 8;   // staged per pass
    auto lds_of = [&](uint32_t waves) {
        return (size_t)tiles * 16 * (gt + 1) * 8 + (size_t)waves * (token_rows * 272 + (size_t)tiles * 16 * 72);
    };
    // A launch of more workgroups than compute units runs two per unit only if two fit in LDS together, and a
    // long row's scale table takes a large share: fewer waves with more steps each then beat a second round
    // (2560 x 9216 at 32 tokens: 14.0 us with nine waves against 16.6 with twelve; 5120 x 17408: 37.6 against 41.4).
    const uint64_t workgroups = (uint64_t)((rows + 16 * rt - 1) / (16 * rt)) * ((batch + 15) / 16);
    if (workgroups > compute_units)
        while (kc > 2 && lds_of(kc) > lds_limit / 2 && lds_of(2) <= lds_limit / 2) {
            ++steps;
            kc = (npairs + steps - 1) / steps;
        }
    if (kc < rt) return false;
    out->rt = rt; out->kc = kc;
    out->lds = lds_of(kc);
    return out->lds <= lds_limit;
}

bool qts_plan(uint32_t rows, uint32_t cols, uint32_t batch, size_t lds_limit, QmsPlan* out) {
    // scale rows are staged two, four or eight groups at a time: rows of a multiple of 256 columns
    if (rows == 0 || cols == 0 || cols % 256 != 0 || batch == 0) return false;
    const uint32_t gt = cols / 128;
    uint32_t kc = (gt + 3) / 4;          // about four steps per wave, at most twelve waves, none idle
    if (kc < 1) kc = 1;
    if (kc > 12) kc = 12;
    uint32_t steps = (gt + kc - 1) / kc;
    kc = (gt + steps - 1) / steps;
    const uint32_t tiles16 = (rows + 15) / 16;
    uint32_t want = (3500 + tiles16 / 2) / tiles16;   // matrices of many rows: fewer waves, longer walks (as qms_plan)
    if (want < 4) want = 4;
    for (uint32_t k = want; k < kc; ++k)
        if (gt % k == 0) { kc = k; break; }
    const size_t token_rows = batch > 8 ? 16 : 8;
    size_t wave = token_rows * 272 + 16 * 40;
    if (wave < 1024) wave = 1024;
    out->rt = 1; out->kc = kc;
    out->lds = (size_t)16 * (gt + 1) * 4 + kc * wave;
    return out->lds <= lds_limit;
}

bool qss_plan(uint32_t bits, uint32_t nmat, uint32_t rows, uint32_t cols, uint32_t batch, size_t lds_limit, QmsPlan* out) {
    if ((bits != 1 && bits != 2) || nmat < 1 || nmat > 2 || !qts_plan(rows, cols, batch, lds_limit, out)) return false;
    const uint32_t gt = cols / 128;
    const size_t token_rows = batch > 8 ? 16 : 8;
    size_t wave = token_rows * 272 + (size_t)nmat * 16 * (16 * bits + 8);
    if (wave < (size_t)nmat * 1024) wave = (size_t)nmat * 1024;
    out->lds = (size_t)nmat * 16 * (gt + 1) * 4 + out->kc * wave;
    return out->lds <= lds_limit;
}

ResolveStatus resolve_pipeline(const std::string& entry_in, ActDType default_act,
                               size_t lds_limit, ResolvedPipeline* out, std::string* why) {
    const ResolveStatus st = resolve_pipeline_entry(entry_in, default_act, lds_limit, out, why);
    if (st == kResolveOk) { attach_mm1(out); attach_qms(out); }
    return st;
}

namespace {

ResolveStatus resolve_pipeline_entry(const std::string& entry_in, ActDType default_act,
                                     size_t lds_limit, ResolvedPipeline* out, std::string* why) {
    std::string entry = entry_in;
    ActDType act = default_act;
    size_t at = entry.find('@');
    if (at != std::string::npos) {
        const std::string tag = entry.substr(at + 1);
        if (tag == "bf16") act = kActBF16;
        else if (tag == "f16") act = kActF16;
        else { *why = "unknown dtype tag '" + tag + "'"; return kResolveMalformed; }
        entry = entry.substr(0, at);
    }
    out->act = act;
    out->appended.clear();
    out->format = kFmtNone;
    out->lds_variant = 0;
    const std::string t = act_suffix(act);

    // ---- function-constant entries: "name:cols:groupSize" --------------------------------
    size_t colon = entry.find(':');
    if (colon != std::string::npos) {
        const std::string name = entry.substr(0, colon);
        size_t colon2 = entry.find(':', colon + 1);
        uint32_t cols = 0, group = 0;
        if (colon2 == std::string::npos || entry.find(':', colon2 + 1) != std::string::npos ||
            !parse_uint(entry.substr(colon + 1, colon2 - colon - 1), &cols) ||
            !parse_uint(entry.substr(colon2 + 1), &group)) {
            *why = "Malformed specialized pipeline entry: '" + entry_in + "'";
            return kResolveMalformed;
        }
        if (name == "affine_quantize_u4" || name == "affine_quantize_u4_weighted") {
            // producer of the affine 4-bit layout: one kernel per group size, scales in the tagged type
            if (cols == 0 || (group != 32 && group != 64 && group != 128)) {
                *why = "affine quantiser kernels exist for groups of 32, 64 and 128 (got cols " +
                       std::to_string(cols) + ", group " + std::to_string(group) + ")";
                return kResolveMalformed;
            }
            out->family = kFamAffineQuantize;
            out->symbol = "smelt_affine_quantize_g" + std::to_string(group) + "_" + t;
            out->kinds = name == "affine_quantize_u4" ? "PPPPZUUU" : "PPPPPUUU";
            out->appended = {cols, group};
            out->kinds += "UU";
            return kResolveOk;
        }
        // u4_lut family (lut_matvec.metal:28-790): the second constant is the number of rows that share a table
        {
            const char* lut_symbol = nullptr;
            if (name == "fused_lut_matvec") { out->family = kFamLutMatvec; lut_symbol = "smelt_lut_matvec_"; out->kinds = "PPPPUUU"; }
            else if (name == "fused_lut_matvec_add") { out->family = kFamLutAdd; lut_symbol = "smelt_lut_matvec_add_"; out->kinds = "PPPPPUUU"; }
            else if (name == "fused_dual_lut_matvec") { out->family = kFamLutDual; lut_symbol = "smelt_dual_lut_matvec_"; out->kinds = "PPPPPPPUUU"; }
            else if (name == "fused_gate_up_swiglu") { out->family = kFamLutGateUp; lut_symbol = "smelt_lut_gate_up_swiglu_"; out->kinds = "PPPPPPUUU"; }
            if (lut_symbol) {
                if (cols == 0 || cols % 32 != 0 || group < 8) {
                    *why = "u4_lut kernels need cols % 32 == 0 and at least 8 rows per table (got cols " +
                           std::to_string(cols) + ", group " + std::to_string(group) + ")";
                    return kResolveMalformed;
                }
                out->symbol = lut_symbol + t;
                out->appended = {cols, group};
                return kResolveOk;
            }
        }
        if (name == "affine_matvec") { out->family = kFamAffineMatvec; out->symbol = "smelt_affine_matvec_" + t; out->kinds = "PPPPPUUU"; }
        else if (name == "fused_affine_matvec_add") { out->family = kFamAffineAdd; out->symbol = "smelt_affine_matvec_add_" + t; out->kinds = "PPPPPPUUU"; }
        else if (name == "fused_affine_gate_up_swiglu") { out->family = kFamAffineGateUp; out->symbol = "smelt_affine_gate_up_swiglu_" + t; out->kinds = "PPPPPPPPUUU"; }
        else if (name == "fused_dual_affine_matvec") { out->family = kFamAffineDual; out->symbol = "smelt_affine_dual_matvec_" + t; out->kinds = "PPPPPPPPPUUU"; }
        else if (name == "fused_affine_gate_up_geglu") { out->family = kFamAffineGateUp; out->symbol = "smelt_affine_gate_up_geglu_" + t; out->kinds = "PPPPPPPPUUU"; }
        else if (name == "norm_scale_affine_matvec") { out->family = kFamNormScaleAffineMatvec; out->symbol = "smelt_norm_scale_affine_matvec_" + t; out->kinds = "PPPPPPPPUUU"; }
        else if (name == "norm_scale_affine_gate_up_swiglu") { out->family = kFamNormScaleAffineGateUp; out->symbol = "smelt_norm_scale_affine_gate_up_swiglu_" + t; out->kinds = "PPPPPPPPPPUUU"; }
        else if (name == "norm_scale_affine_gate_up_geglu") { out->family = kFamNormScaleAffineGateUp; out->symbol = "smelt_norm_scale_affine_gate_up_geglu_" + t; out->kinds = "PPPPPPPPPPUUU"; }
        else if (name == "atomic_norm_affine_matvec") { out->family = kFamFusedNormAffineMatvec; out->symbol = "smelt_atomic_norm_affine_matvec_" + t; out->kinds = "PPPPPPPPUFUU"; }
        else if (name == "atomic_norm_affine_gate_up_swiglu") { out->family = kFamFusedNormAffineGateUp; out->symbol = "smelt_atomic_norm_affine_gate_up_swiglu_" + t; out->kinds = "PPPPPPPPPPUFUU"; }
        else if (name == "affine_bank4_matvec") { out->family = kFamAffineBank4; out->symbol = "smelt_affine_bank4_matvec_" + t; out->kinds = "PPPPPPPPUUUUUU"; }
        else { *why = "no HIP kernel for function-constant pipeline '" + name + "'"; return kResolveUnknown; }
        if (!is_pow2(group) || group < 32 || cols % 32 != 0 || cols == 0) {
            *why = "affine kernels need cols % 32 == 0 and a power-of-two group >= 32 (got cols " +
                   std::to_string(cols) + ", group " + std::to_string(group) + ")";
            return kResolveMalformed;
        }
        out->appended = {cols, group};
        return kResolveOk;
    }

    // ---- fixed-shape affine names -----------------------------------------------------------
    static const AffineName kAffine[] = {
        {"affine_matvec_argmax", kFamAffineArgmax},
        {"affine_matvec", kFamAffineMatvec},
        {"fused_affine_matvec_add", kFamAffineAdd},
        {"fused_affine_gate_up_swiglu", kFamAffineGateUp},
        {"fused_dual_affine_matvec", kFamAffineDual},
        {"fused_dual_affine_matvec_add", kFamAffineDualAdd},
        {"fused_affine_gate_up_geglu", kFamAffineGateUp},
        {"norm_scale_affine_matvec", kFamNormScaleAffineMatvec},
        {"norm_add_scale_affine_matvec", kFamNormAddScaleAffineMatvec},
        {"norm_scale_fused_dual_affine_matvec", kFamNormScaleAffineDual},
        {"norm_scale_affine_gate_up_swiglu", kFamNormScaleAffineGateUp},
        {"norm_scale_affine_gate_up_geglu", kFamNormScaleAffineGateUp},
    };
    for (const AffineName& a : kAffine) {
        const size_t n = strlen(a.prefix);
        if (entry.compare(0, n, a.prefix) != 0 || entry.size() <= n || entry[n] != '_' || entry[n + 1] != 'c') continue;
        uint32_t cols, rows, group;
        std::string suffix;
        if (!parse_fixed_shape(entry.substr(n), &cols, &rows, &group, &suffix)) continue;
        if (!is_pow2(group) || group < 32 || cols % 32 != 0 || cols == 0 || rows == 0) {
            *why = "unsupported affine geometry in '" + entry + "'";
            return kResolveMalformed;
        }
        const uint32_t row_stride = cols / 2;
        // A/B variants the reference keeps beside its tuned kernels compute the same thing
        for (const char* alias : {"_padded_reference", "_nocache_reference"}) {
            const size_t n_alias = strlen(alias);
            if (suffix.size() >= n_alias && suffix.compare(suffix.size() - n_alias, n_alias, alias) == 0) suffix.resize(suffix.size() - n_alias);
        }
        // ("_mfma" after the variant suffix once asked for a ring-buffered matrix-core matvec; that engine is gone,
        // the single-pass matrix-core kernels are picked per launch under the pipeline's own name)
        if (suffix.size() >= 5 && suffix.compare(suffix.size() - 5, 5, "_mfma") == 0) {
            *why = "no HIP kernel for '" + entry + "' (the '_mfma' opt-in names are withdrawn)";
            return kResolveUnknown;
        }
        // the norm-scale dual kernel's "_batched" form takes its token from grid.y, like the single-token kernels
        const bool m1 = suffix.empty() || suffix == "_rows4" || suffix == "_rows8" || suffix == "_rows4_sg1" ||
                        ((a.m1 == kFamNormScaleAffineDual || a.m1 == kFamAffineDual) && suffix == "_batched");
        uint32_t bt = 0;
        bool full = false, skinny = false;
        if (suffix == "_batched") bt = 8;
        else if (suffix == "_batched_skinny") { bt = 32; full = true; skinny = true; }
        else if (suffix == "_batched_tile3") bt = 3;
        // "_batched_verify_b4": the generated small-batch kernels (SmeltGeneratedKernelVariants.swift:17-35), token tiles of 4
        else if (suffix == "_batched_tile4" || suffix == "_batched_ext_b4" || suffix == "_batched_verify_b4") bt = 4;
        else if (suffix == "_batched_ext_b5" || suffix == "_batched_sg4_bt5") bt = 5;
        else if (suffix == "_batched_full") { bt = 16; full = true; }
        else if (starts_with(suffix, "_batched_full_b") && parse_uint(suffix.substr(15), &bt) && bt >= 1 && bt <= 4096) { full = true; }
        else if (suffix == "_batched_bt4_sg4" && strstr(a.prefix, "geglu")) bt = 4;
        else if (!m1) { *why = "unknown kernel variant '" + suffix + "' in '" + entry + "'"; return kResolveUnknown; }

        if (a.m1 == kFamAffineArgmax) {
            if (m1 || full) { *why = "affine_matvec_argmax exists only as '_batched'"; return kResolveUnknown; }
            out->family = kFamAffineArgmax;
            out->symbol = "smelt_affine_matvec_argmax_" + t;
            out->symbol_single = "smelt_affine_matvec_argmax_single_" + t;  // decode: one token, no token loop
            out->single_arg = 5;
            out->kinds = "PPPPPUFUUUU";
            out->appended = {rows, cols, group, bt};
            return kResolveOk;
        }
        if (m1) {
            out->family = a.m1;
            switch (a.m1) {
                case kFamAffineMatvec: out->symbol = "smelt_affine_matvec_" + t; out->kinds = "PPPPPUUU"; break;
                case kFamAffineAdd: out->symbol = "smelt_affine_matvec_add_" + t; out->kinds = "PPPPPPUUU"; break;
                case kFamAffineGateUp: out->symbol = "smelt_affine_gate_up_swiglu_" + t; out->kinds = "PPPPPPPPUUU"; break;
                case kFamAffineDual: out->symbol = "smelt_affine_dual_matvec_" + t; out->kinds = "PPPPPPPPPUUU"; break;
                case kFamAffineDualAdd: out->symbol = "smelt_affine_dual_matvec_add_" + t; out->kinds = "PPPPPPPPPPPUUU"; break;
                case kFamNormScaleAffineMatvec: out->symbol = "smelt_norm_scale_affine_matvec_" + t; out->kinds = "PPPPPPPPUUU"; break;
                case kFamNormScaleAffineGateUp: out->symbol = std::string("smelt_") + a.prefix + "_" + t; out->kinds = "PPPPPPPPPPUUU"; break;
                case kFamNormAddScaleAffineMatvec: out->symbol = "smelt_norm_add_scale_affine_matvec_" + t; out->kinds = "PPPPPPPPPUUU"; break;
                case kFamNormScaleAffineDual: out->symbol = "smelt_norm_scale_affine_dual_matvec_" + t; out->kinds = "PPPPPPPPPPPUUU"; break;
                default: break;
            }
            if (a.m1 == kFamAffineGateUp && strstr(a.prefix, "geglu")) out->symbol = "smelt_affine_gate_up_geglu_" + t;
            out->appended = {rows, cols, group};
            return kResolveOk;
        }
        const bool geglu = strstr(a.prefix, "geglu") != nullptr;
        if (a.m1 == kFamNormAddScaleAffineMatvec || a.m1 == kFamNormScaleAffineDual || a.m1 == kFamAffineDualAdd) {
            *why = "no batched HIP kernel for '" + entry + "'";
            return kResolveUnknown;
        }
        if (a.m1 == kFamAffineDual) {
            // token tiles of two same-shape projections (fused_dual_affine_matvec_fixed_ext, lut_matvec.metal:3816-3922)
            if (full || suffix != "_batched_verify_b4") { *why = "no batched HIP kernel for '" + entry + "'"; return kResolveUnknown; }
            const uint32_t mbv = pick_mb(kCodesU4, row_stride, 4, lds_limit);
            out->lds_variant = mbv;
            out->family = kFamAffineDualBatched;
            out->symbol = "smelt_affine_dual_matvec_batched_mb" + std::to_string(mbv) + "_" + t;
            out->kinds = "PPPPPPPPPUUUUU";
            out->appended = {rows, cols, group, bt};
            return kResolveOk;
        }
        if (a.m1 == kFamAffineGateUp && geglu && (suffix == "_batched" || suffix == "_batched_bt4_sg4")) {
            // small-batch GeGLU (lut_matvec.metal:8342-8364, 8752-8753): token tiles of 3 and 4
            bt = suffix == "_batched" ? 3 : 4;
            const uint32_t mbv = pick_mb(kCodesU4, row_stride, 4, lds_limit);
            out->lds_variant = mbv;
            out->family = kFamAffineGateUpBatched;
            out->symbol = "smelt_affine_gate_up_geglu_batched_mb" + std::to_string(mbv) + "_" + t;
            out->kinds = "PPPPPPPPUUUUU";
            out->appended = {rows, cols, group, bt};
            return kResolveOk;
        }
        if (a.m1 == kFamNormScaleAffineMatvec || a.m1 == kFamNormScaleAffineGateUp || geglu) {
            // prologue and GeGLU forms: the MFMA slab kernel for "_batched_full", the vector-ALU
            // token tile for the plain "_batched" matvec, nothing else
            if (skinny || (!full && a.m1 != kFamNormScaleAffineMatvec)) {
                *why = "no batched HIP kernel for '" + entry + "'";
                return kResolveUnknown;
            }
            if (full) {
                const uint32_t mt = bt >= 64 ? 4 : 1;
                out->lds_variant = mt;
                const std::string mts = "mt" + std::to_string(mt) + "_" + t;
                if (a.m1 == kFamNormScaleAffineMatvec) {
                    out->family = kFamNormScaleAffineQmm; out->symbol = "smelt_norm_scale_affine_qmm_" + mts; out->kinds = "PPPPPPPPUUUUU";
                } else if (a.m1 == kFamNormScaleAffineGateUp) {
                    out->family = kFamNormScaleAffineQmmGateUp;
                    out->symbol = std::string("smelt_norm_scale_affine_qmm_gate_up_") + (geglu ? "geglu_" : "swiglu_") + mts;
                    out->kinds = "PPPPPPPPPPUUUUU";
                } else {
                    out->family = kFamAffineQmmGateUp; out->symbol = "smelt_affine_qmm_gate_up_geglu_" + mts; out->kinds = "PPPPPPPPUUUUU";
                }
                out->appended = {rows, cols, group, bt};
                return kResolveOk;
            }
        }
        if (full && skinny) {
            if (group != 64 || cols % 512 != 0) { *why = "skinny qmm needs group 64 and cols % 512 == 0: '" + entry + "'"; return kResolveMalformed; }
            out->lds_variant = kSkinnyVariant;
            out->workspace = true;
            if (a.m1 == kFamAffineMatvec) { out->family = kFamAffineQmm; out->symbol = "smelt_affine_qmm_skinny_" + t; out->kinds = "PPPPPUUUUU"; }
            else if (a.m1 == kFamAffineAdd) { out->family = kFamAffineQmmAdd; out->symbol = "smelt_affine_qmm_add_skinny_" + t; out->kinds = "PPPPPPPUUUUU"; }
            else if (a.m1 == kFamAffineGateUp) { out->family = kFamAffineQmmGateUp; out->symbol = "smelt_affine_qmm_gate_up_swiglu_skinny_" + t; out->kinds = "PPPPPPPPUUUUU"; }
            else { *why = "no skinny qmm HIP kernel for '" + entry + "'"; return kResolveUnknown; }
            out->appended = {rows, cols, group, bt};
            return kResolveOk;
        }
        if (full) {
            const uint32_t mt = bt >= 64 ? 4 : 1;
            out->lds_variant = mt;
            const std::string mts = "mt" + std::to_string(mt) + "_" + t;
            if (a.m1 == kFamAffineMatvec) { out->family = kFamAffineQmm; out->symbol = "smelt_affine_qmm_" + mts; out->kinds = "PPPPPUUUUU"; }
            else if (a.m1 == kFamAffineAdd) { out->family = kFamAffineQmmAdd; out->symbol = "smelt_affine_qmm_add_" + mts; out->kinds = "PPPPPPPUUUUU"; }
            else if (a.m1 == kFamAffineGateUp) { out->family = kFamAffineQmmGateUp; out->symbol = "smelt_affine_qmm_gate_up_swiglu_" + mts; out->kinds = "PPPPPPPPUUUUU"; }
            else { *why = "no qmm HIP kernel for '" + entry + "'"; return kResolveUnknown; }
            out->appended = {rows, cols, group, bt};
            return kResolveOk;
        }
        const uint32_t mb = pick_mb(kCodesU4, row_stride, 4, lds_limit);
        out->lds_variant = mb;
        const std::string mbs = "mb" + std::to_string(mb) + "_" + t;
        if (a.m1 == kFamAffineMatvec) { out->family = kFamAffineBatched; out->symbol = "smelt_affine_matvec_batched_" + mbs; out->kinds = "PPPPPUUUUU"; }
        else if (a.m1 == kFamNormScaleAffineMatvec) { out->family = kFamNormScaleAffineBatched; out->symbol = "smelt_norm_scale_affine_matvec_batched_" + mbs; out->kinds = "PPPPPPPPUUUUU"; }
        else if (a.m1 == kFamAffineGateUp) { out->family = kFamAffineGateUpBatched; out->symbol = "smelt_affine_gate_up_swiglu_batched_" + mbs; out->kinds = "PPPPPPPPUUUUU"; }
        else { *why = "no batched HIP kernel for '" + entry + "'"; return kResolveUnknown; }
        out->appended = {rows, cols, group, bt};
        return kResolveOk;
    }

    // ---- signed g128 names ------------------------------------------------------------------
    struct SignedName { const char* name; FamilyId fam; SignedFormat fmt; const char* sym; const char* kinds; };
    static const SignedName kSigned[] = {
        {"signed_binary_matvec_g128_rows8", kFamSignedMatvec, kFmtBinary1, "smelt_signed_binary_matvec_", "PPPPUU"},
        {"signed_binary_matvec_add_g128_rows8", kFamSignedAdd, kFmtBinary1, "smelt_signed_binary_matvec_add_", "PPPPPUU"},
        {"signed_binary_gate_up_swiglu_g128_rows8", kFamSignedGateUp, kFmtBinary1, "smelt_signed_binary_gate_up_swiglu_", "PPPPPPUU"},
        {"signed_binary_matvec_g128_rows8_batched_b4", kFamSignedB4, kFmtBinary1, "smelt_signed_binary_matvec_b4_", "PPPPUUU"},
        {"signed_binary_gate_up_swiglu_g128_rows8_batched_b4", kFamSignedGateUpB4, kFmtBinary1, "smelt_signed_binary_gate_up_swiglu_b4_", "PPPPPPUUU"},
        {"signed_ternary_matvec_g128_rows8", kFamSignedMatvec, kFmtTernary2, "smelt_signed_ternary_matvec_", "PPPPUU"},
        {"signed_ternary_matvec_add_g128_rows8", kFamSignedAdd, kFmtTernary2, "smelt_signed_ternary_matvec_add_", "PPPPPUU"},
        {"signed_ternary_gate_up_swiglu_g128_rows8", kFamSignedGateUp, kFmtTernary2, "smelt_signed_ternary_gate_up_swiglu_", "PPPPPPUU"},
        {"signed_ternary_matvec_g128_rows8_batched_b4", kFamSignedB4, kFmtTernary2, "smelt_signed_ternary_matvec_b4_", "PPPPUUU"},
        {"signed_ternary_gate_up_swiglu_g128_rows8_batched_b4", kFamSignedGateUpB4, kFmtTernary2, "smelt_signed_ternary_gate_up_swiglu_b4_", "PPPPPPUUU"},
        {"signed_trit5_matvec_g128_rows8", kFamSignedMatvec, kFmtTrit5, "smelt_signed_trit5_matvec_", "PPPPUU"},
        {"signed_trit5_matvec_add_g128_rows8", kFamSignedAdd, kFmtTrit5, "smelt_signed_trit5_matvec_add_", "PPPPPUU"},
        {"signed_trit5_gate_up_swiglu_g128_rows8", kFamSignedGateUp, kFmtTrit5, "smelt_signed_trit5_gate_up_swiglu_", "PPPPPPUU"},
        {"signed_trit5_matvec_g128_rows8_batched_b4", kFamSignedB4, kFmtTrit5, "smelt_signed_trit5_matvec_b4_", "PPPPUUU"},
        {"signed_trit5_gate_up_swiglu_g128_rows8_batched_b4", kFamSignedGateUpB4, kFmtTrit5, "smelt_signed_trit5_gate_up_swiglu_b4_", "PPPPPPUUU"},
        {"signed_ternary_affine_matvec_g128_rows8", kFamTerAffMatvec, kFmtTernary2, "smelt_teraff_matvec_", "PPPPPUU"},
        {"signed_ternary_affine_matvec_add_g128_rows8", kFamTerAffAdd, kFmtTernary2, "smelt_teraff_matvec_add_", "PPPPPPUU"},
        {"signed_ternary_affine_gate_up_swiglu_g128_rows8", kFamTerAffGateUp, kFmtTernary2, "smelt_teraff_gate_up_swiglu_", "PPPPPPPPUU"},
        {"signed_ternary_affine_bank4_matvec_g128_rows8", kFamTerAffBank4, kFmtTernary2, "smelt_teraff_bank4_matvec_", "PPPPPPPPUUUUU"},
        {"signed_ternary_affine_qmm_g128_bm32_bn32_bk32", kFamTerAffQmm, kFmtTernary2, "smelt_ternary_qmm_mt2_", "PPPPPUUU"},
    };
    for (const SignedName& s : kSigned) {
        if (entry == s.name) {
            out->family = s.fam;
            out->format = s.fmt;
            out->symbol = std::string(s.sym) + t;
            out->kinds = s.kinds;
            return kResolveOk;
        }
    }

    // ---- gathers and argmax -----------------------------------------------------------------
    if (entry == "affine_embedding_gather") { out->family = kFamAffineGather; out->symbol = "smelt_affine_embedding_gather_" + t; out->kinds = "PPPPPUU"; return kResolveOk; }
    if (entry == "affine_embedding_gather_batched") { out->family = kFamAffineGatherBatched; out->symbol = "smelt_affine_embedding_gather_batched_" + t; out->kinds = "PPPPPUUU"; return kResolveOk; }
    if (entry == "signed_binary_embedding_gather_g128") { out->family = kFamSignedGather; out->format = kFmtBinary1; out->symbol = "smelt_signed_binary_embedding_gather_" + t; out->kinds = "PPPPU"; return kResolveOk; }
    if (entry == "signed_ternary_embedding_gather_g128") { out->family = kFamSignedGather; out->format = kFmtTernary2; out->symbol = "smelt_signed_ternary_embedding_gather_" + t; out->kinds = "PPPPU"; return kResolveOk; }
    if (entry == "signed_trit5_embedding_gather_g128") { out->family = kFamSignedGather; out->format = kFmtTrit5; out->symbol = "smelt_signed_trit5_embedding_gather_" + t; out->kinds = "PPPPU"; return kResolveOk; }
    if (entry == "argmax_fp16_partials") { out->family = kFamArgmaxPartials; out->symbol = "smelt_argmax16_partials"; out->kinds = "PPUU"; return kResolveOk; }
    if (starts_with(entry, "lm_head_argmax_reduce_r")) {
        uint32_t n = 0;
        if (!parse_uint(entry.substr(23), &n) || n == 0) { *why = "Malformed pipeline entry: '" + entry_in + "'"; return kResolveMalformed; }
        out->family = kFamLmHeadReduce; out->symbol = "smelt_lm_head_argmax_reduce"; out->kinds = "PPUU";
        return kResolveOk;
    }
    // ---- layer ops between the matvecs: norms.metal, activations_precise.metal, activations.metal ----
    {
        auto eps_bits = [](float e) { uint32_t b; memcpy(&b, &e, 4); return b; };
        auto strip = [](std::string& s, const char* suffix) {
            const size_t n = strlen(suffix);
            if (s.size() >= n && s.compare(s.size() - n, n, suffix) == 0) { s.resize(s.size() - n); return true; }
            return false;
        };
        if (entry == "rms_norm_1pw_d256_add_scalar_weight") {
            out->family = kFamRmsNormAddScalar; out->symbol = "smelt_rms_norm_1pw_add_scalar_" + t;
            out->kinds = "PPPPPUUU"; out->appended = {256u, eps_bits(1e-6f), 2u};
            return kResolveOk;
        }
        if (entry == "rms_norm_1pw_from_fp32" || entry == "rms_norm_1pw_from_fp32_batched") {
            out->family = kFamRmsNormFromFp32; out->symbol = "smelt_rms_norm_1pw_from_fp32_" + t; out->kinds = "PPPUF";
            return kResolveOk;
        }
        if (entry == "rms_norm_gated") {                      // head_dim, eps from the record
            out->family = kFamRmsNormGated; out->symbol = "smelt_rms_norm_gated_" + t; out->kinds = "PPPPUFU"; out->appended = {0u};
            return kResolveOk;
        }
        if (entry == "rms_norm_gated_d128") {                 // norms_gated_precise.metal:20-52
            out->family = kFamRmsNormGated; out->symbol = "smelt_rms_norm_gated_" + t; out->kinds = "PPPPUUU";
            out->appended = {128u, eps_bits(1e-6f), 1u};
            return kResolveOk;
        }
        if (entry == "rms_norm_gated_d128_batched") {         // heads per token from the record (:54-88)
            out->family = kFamRmsNormGatedBatched; out->symbol = "smelt_rms_norm_gated_batched_" + t; out->kinds = "PPPPUUUU";
            out->appended = {128u, eps_bits(1e-6f), 1u};
            return kResolveOk;
        }
        if (entry == "rms_norm_gated_d128_signed_activation_bitplanes_i6_g128") {   // signed_quant.metal:1149-1173
            out->family = kFamRmsNormGatedPlanes; out->symbol = "smelt_rms_norm_gated_signed_activation_bitplanes_" + t;
            out->kinds = "PPPPPUF";
            return kResolveOk;
        }
        if (starts_with(entry, "rms_norm_1pw")) {
            std::string rest = entry.substr(12);
            strip(rest, "_batched");            // batch rows are the grid width either way
            const bool add = strip(rest, "_add");
            uint32_t dim = 0;
            bool ok = rest.empty();
            if (!ok && starts_with(rest, "_d") && parse_uint(rest.substr(2), &dim) && dim > 0) ok = true;
            if (ok && !(add && dim == 0)) {
                out->family = add ? kFamRmsNormAdd : kFamRmsNorm;
                out->symbol = std::string(add ? "smelt_rms_norm_1pw_add_" : "smelt_rms_norm_1pw_") + t;
                if (dim == 0) { out->kinds = "PPPUFU"; out->appended = {1u}; }                  // dim, eps from the record
                else { out->kinds = add ? "PPPPUUU" : "PPPUUU"; out->appended = {dim, eps_bits(1e-6f), dim == 256 ? 2u : 0u}; }   // d256: products left to right
                return kResolveOk;
            }
        }
        if (starts_with(entry, "rms_norm_scale_only")) {
            std::string rest = entry.substr(19);
            strip(rest, "_batched");
            const bool eps5 = strip(rest, "_eps1e5");
            uint32_t dim = 0;
            if (rest.empty() || rest == "_precise") {
                out->family = kFamRmsScale; out->symbol = "smelt_rms_norm_scale_only_" + t; out->kinds = "PPUF";
                return kResolveOk;
            }
            if (starts_with(rest, "_d") && parse_uint(rest.substr(2), &dim) && dim > 0) {
                out->family = kFamRmsScale; out->symbol = "smelt_rms_norm_scale_only_" + t; out->kinds = "PPUU";
                out->appended = {dim, eps_bits(eps5 ? 1e-5f : 1e-6f)};
                return kResolveOk;
            }
        }
        if (entry == "residual_add_rms_norm_scale_only_precise") {
            out->family = kFamResidualAddRmsScale; out->symbol = "smelt_residual_add_rms_norm_scale_only_" + t; out->kinds = "PPPPUF";
            return kResolveOk;
        }
        if (entry == "swiglu_fused" || entry == "elementwise_add" || entry == "elementwise_mul") {
            out->family = kFamElementwise; out->symbol = "smelt_" + entry + "_" + t; out->kinds = "PPPU";
            return kResolveOk;
        }
        if (entry == "sigmoid_mul" || entry == "geglu_fused") {
            out->family = kFamElementwise; out->symbol = "smelt_" + entry + "_" + t; out->kinds = "PPPU";
            return kResolveOk;
        }
        if (entry == "geglu_fused_strided_batched") {
            out->family = kFamGegluStridedBatched; out->symbol = "smelt_geglu_fused_strided_batched_" + t; out->kinds = "PPPUU";
            return kResolveOk;
        }
        if (entry == "projection_bias_add_batched") {
            out->family = kFamBiasAddBatched; out->symbol = "smelt_projection_bias_add_batched_" + t; out->kinds = "PPPU";
            return kResolveOk;
        }
        if (entry == "silu" || entry == "sigmoid_kernel" || entry == "softplus") {
            out->family = kFamUnary; out->symbol = "smelt_unary_" + t; out->kinds = "PPUUU";
            out->appended = {0u, entry == "silu" ? 0u : (entry == "sigmoid_kernel" ? 1u : 2u)};
            return kResolveOk;
        }
        if (entry == "logit_cap") { out->family = kFamUnary; out->symbol = "smelt_unary_" + t; out->kinds = "PPUFU"; out->appended = {4u}; return kResolveOk; }
        if (entry == "scalar_mul") { out->family = kFamScalarMul; out->symbol = "smelt_scalar_mul_param_first_" + t; out->kinds = "PPFU"; return kResolveOk; }
        if (entry == "scalar_mul_weight") { out->family = kFamScalarMulWeight; out->symbol = "smelt_scalar_mul_weight_" + t; out->kinds = "PPPU"; return kResolveOk; }
        if (entry == "buffer_copy") { out->family = kFamCopy16; out->symbol = "smelt_buffer_copy16"; out->kinds = "PPU"; return kResolveOk; }
    }
    // ---- signed activation views (bit planes): signed_quant.metal:746-2260 ----------------------
    {
        // "..._i{N}_..." with N planes, 2 <= N <= 6
        auto planes_of = [](const std::string& s, size_t at, uint32_t* n, size_t* after) {
            if (at + 2 > s.size() || s[at] != 'i' || s[at + 1] < '2' || s[at + 1] > '6') return false;
            *n = (uint32_t)(s[at + 1] - '0');
            *after = at + 2;
            return true;
        };
        uint32_t n = 0;
        size_t after = 0;
        if (starts_with(entry, "signed_activation_bitplanes_") && planes_of(entry, 28, &n, &after) &&
            (entry.substr(after) == "_g128" || entry.substr(after) == "_g128_batched")) {
            out->family = kFamActivationPlanes; out->symbol = "smelt_signed_activation_bitplanes_" + t;
            out->kinds = "PPPUU"; out->appended = {n};
            return kResolveOk;
        }
        if (entry == "sigmoid_mul_signed_activation_bitplanes_i6_g128") {
            // same bindings as the SwiGLU producer: a b planes scales cols
            out->family = kFamSwigluPlanes; out->symbol = "smelt_sigmoid_mul_signed_activation_bitplanes_" + t;
            out->kinds = "PPPPUU"; out->appended = {6u};
            return kResolveOk;
        }
        if (entry == "swiglu_signed_activation_bitplanes_i5_g128") {
            out->family = kFamSwigluPlanes; out->symbol = "smelt_swiglu_signed_activation_bitplanes_" + t;
            out->kinds = "PPPPUU"; out->appended = {5u};
            return kResolveOk;
        }
        if (starts_with(entry, "norm_scale_signed_activation_bitplanes_") && planes_of(entry, 39, &n, &after) &&
            entry.substr(after) == "_g128") {
            out->family = kFamNormScalePlanes; out->symbol = "smelt_norm_scale_signed_activation_bitplanes_" + t;
            out->kinds = "PPPPPUU"; out->appended = {n};
            return kResolveOk;
        }
        for (const char* fmt : {"binary", "ternary"}) {
            const std::string head = std::string("signed_") + fmt + "_bitplane_";
            if (!starts_with(entry, head.c_str()) || !planes_of(entry, head.size(), &n, &after)) continue;
            const std::string tail = entry.substr(after);
            const std::string stem = std::string("smelt_signed_") + fmt + "_bitplane_";
            out->format = fmt[0] == 'b' ? kFmtBinary1 : kFmtTernary2;
            out->appended = {n};
            if (tail == "_matvec_g128_rows8" || tail == "_matvec_g128_rows2_wide") {
                out->family = kFamPlaneMatvec; out->symbol = stem + "matvec_" + t; out->kinds = "PPPPPUUU";
                return kResolveOk;
            }
            if (tail == "_matvec_add_g128_rows8") {
                out->family = kFamPlaneAdd; out->symbol = stem + "matvec_add_" + t; out->kinds = "PPPPPPUUU";
                return kResolveOk;
            }
            for (uint32_t tile : {4u, 8u, 16u}) {
                if (tail == "_matvec_g128_rows8_batched_b" + std::to_string(tile)) {
                    out->family = kFamPlaneBatched; out->symbol = stem + "matvec_batched_" + t; out->kinds = "PPPPPUUUUU";
                    out->appended = {n, tile};
                    out->lds_variant = 4;
                    return kResolveOk;
                }
            }
            if (tail == "_bank4_matvec_g128_rows8") {
                out->family = kFamPlaneBank4; out->symbol = stem + "bank4_matvec_" + t; out->kinds = "PPPPPPPPUUUUUU";
                return kResolveOk;
            }
            if (tail == "_gate_up_swiglu_g128_rows8") {
                out->family = kFamPlaneGateUp; out->symbol = stem + "gate_up_swiglu_" + t; out->kinds = "PPPPPPPUUU";
                return kResolveOk;
            }
        }
    }
    // turbo_quant_h (lut_matvec.metal:1045-1079, 9207-9486); the batched names differ only in the grid height
    if (entry == "tqh_matvec_prepare_input" || entry == "tqh_matvec_prepare_input_batched") {
        out->family = kFamTqhPrepare; out->symbol = "smelt_tqh_matvec_prepare_input_" + t; out->kinds = "PPU"; return kResolveOk;
    }
    if (entry == "tqh_matvec" || entry == "tqh_matvec_batched") {
        out->family = kFamTqhMatvec; out->symbol = "smelt_tqh_matvec_" + t; out->kinds = "PPPPUUU"; return kResolveOk;
    }
    if (entry == "tqh_embedding_gather") { out->family = kFamTqhGather; out->symbol = "smelt_tqh_embedding_gather_" + t; out->kinds = "PPPPUU"; return kResolveOk; }
    if (entry == "fused_lut_matmul") { out->family = kFamLutMatmul; out->symbol = "smelt_lut_matmul_" + t; out->kinds = "PPPPUUU"; return kResolveOk; }
    if (entry == "lut_embedding_gather") { out->family = kFamLutGather; out->symbol = "smelt_lut_embedding_gather"; out->kinds = "PPPPUU"; return kResolveOk; }
    // binary projection banks on the direct path (signed_quant.metal:2638-2935)
    if (entry == "signed_binary_packed_bank_matvec_g128_rows8") {
        out->family = kFamBinaryPackedBank; out->format = kFmtBinary1; out->symbol = "smelt_signed_binary_packed_bank_matvec_" + t; out->kinds = "PPPPPUUU"; return kResolveOk;
    }
    if (entry == "signed_binary_packed_bank4_matvec_g128_rows8") {
        out->family = kFamBinaryPackedBank4; out->format = kFmtBinary1; out->symbol = "smelt_signed_binary_packed_bank4_matvec_" + t; out->kinds = "PPPPPPPUUUUU"; return kResolveOk;
    }
    if (entry == "signed_trit5_packed_bank4_matvec_g128_rows8") {   // same bindings over five-digit-byte rows
        out->family = kFamBinaryPackedBank4; out->format = kFmtTrit5; out->symbol = "smelt_signed_trit5_packed_bank4_matvec_" + t; out->kinds = "PPPPPPPUUUUU"; return kResolveOk;
    }
    if (entry == "signed_binary_dual_matvec_g128_rows8" || entry == "signed_binary_virtual_bank_matvec_g128_rows8") {
        out->family = kFamBinaryTwoMatrix; out->format = kFmtBinary1; out->symbol = "smelt_signed_binary_two_matrix_matvec_" + t; out->kinds = "PPPPPPPUUU"; return kResolveOk;
    }
    if (entry == "signed_validate_codes") { out->family = kFamSignedValidate; out->symbol = "smelt_signed_validate_codes"; out->kinds = "PPUUU"; return kResolveOk; }
    if (entry == "signed_normalize_mlx_scales") { out->family = kFamSignedMlxScales; out->symbol = "smelt_signed_normalize_mlx_scales"; out->kinds = "PPPPUU"; return kResolveOk; }
    if (entry == "copy_u128") { out->family = kFamCopy; out->symbol = "smelt_copy_u128"; out->kinds = "PPU"; return kResolveOk; }
    if (entry == "read_u128") { out->family = kFamCopy; out->symbol = "smelt_read_u128"; out->kinds = "PPU"; return kResolveOk; }
    if (entry == "read_u128_nt4" || entry == "read_u128_nt8" || entry == "read_u128_nt16") {
        out->family = kFamCopy; out->symbol = "smelt_" + entry; out->kinds = "PPU"; return kResolveOk;
    }
    if (entry == "argmax_key_reduce") { out->family = kFamArgmaxReduce; out->symbol = "smelt_argmax_key_reduce"; out->kinds = "PPU"; return kResolveOk; }

    *why = "no HIP kernel named '" + entry + "'";
    return kResolveUnknown;
}

}  // namespace

}  // namespace smelt_host
