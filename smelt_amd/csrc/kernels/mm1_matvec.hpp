// Single-pass matrix-core matvec for gfx950: y[r] = sum_c w(r, c) * x[c] for one activation row,
// for matrices whose packed weights stream from HBM (batch-1 decode at large-model layer shapes).
//
// The kernel is built around the latency of one memory round trip.  Every wave owns one job, a
// tile of 16 weight rows times a run of up to NL 64-byte row segments, and issues every weight
// load of that job (one 16-byte load per lane and segment, plus the group scales) before it does
// anything else; nothing in the kernel waits on memory twice.  While the loads are in flight the
// wave stages the slice of the activation row its segments need, privately, in LDS.  K is split
// over the `kc` waves of a workgroup that share a row tile; their partial sums meet in LDS.
//
// Arithmetic: v_mfma_f32_16x16x32_{f16,bf16} with the weights as the B operand.
//   * MFMA lane (n = lane % 16, q = lane / 16) supplies eight weights of row n taken from the
//     16-byte piece q of the current 64-byte segment.  Packed codes become (base + code) operands
//     with one AND-OR per pair of weights: a code whose lowest bit sits at mantissa bit m of a
//     16-bit float with exponent 2^(M - m) (M = mantissa width) counts in units of one.
//   * The MFMA contracts over all four q, which would mix four 16-byte pieces (up to four scale
//     groups).  The A operand (the activations) separates them: token slot 4 q carries x only in
//     k-block q, every other slot is zero, so D[4 q][n] is the dot product of piece q of row n and
//     lands in accumulator register 0 of lane (n, q).  Only lanes 0, 20, 40 and 60 of the A
//     operand are ever non-zero; they alone read the staged activations.
//   * sum((base + offset) * x) per 16-byte piece is formed at staging time and subtracted before
//     the group scale is applied in fp32.
// Activations enter the MFMA in their own type (fp16 or bf16), unconverted.
#pragma once
#include "matvec_kernels.hpp"

namespace smelt {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

// 16-bit float geometry of the activation type
template <class ActT>
struct Elem16;
template <>
struct Elem16<F16> {
    static constexpr int kMant = 10, kExpBias = 15;
    static __device__ __forceinline__ float4_t mfma(const uint4_t& a, const uint4_t& b, const float4_t& c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    }
    // acc + lo(pair) * lo(k) + hi(pair) * hi(k), fp32 accumulate
    static __device__ __forceinline__ float dot2k(uint32_t pair, uint32_t k, float acc) {
        return __builtin_amdgcn_fdot2(as_half2(pair), as_half2(k), acc, false);
    }
};
template <>
struct Elem16<BF16> {
    static constexpr int kMant = 7, kExpBias = 127;
    static __device__ __forceinline__ float4_t mfma(const uint4_t& a, const uint4_t& b, const float4_t& c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2k(uint32_t pair, uint32_t k, float acc) {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pair), __builtin_bit_cast(bf16x2_t, k), acc, false);
    }
};

// Where the codes of a dword go.  A dword holds 32 / WIDTH codes, LSB first.  Pair j is codes
// (j, j + 16 / WIDTH): the two sit at the same bit of the low and the high half-word, so one
// 32-bit AND-OR forms both operands.  kPerPass pairs share one shifted copy of the dword; the
// code of pair j then sits at mantissa bit kMLo + WIDTH * (j % kPerPass).  A larger kMLo means
// smaller bases (less cancellation in sum (base + code) x - sum base x) and more shifts.
template <int WIDTH, class ActT>
struct M1Plan;
template <> struct M1Plan<1, BF16> { static constexpr int kPerPass = 7, kMLo = 0; };
template <> struct M1Plan<1, F16> { static constexpr int kPerPass = 7, kMLo = 3; };
template <> struct M1Plan<2, BF16> { static constexpr int kPerPass = 3, kMLo = 0; };
template <> struct M1Plan<2, F16> { static constexpr int kPerPass = 4, kMLo = 2; };
template <> struct M1Plan<4, BF16> { static constexpr int kPerPass = 1, kMLo = 0; };
template <> struct M1Plan<4, F16> { static constexpr int kPerPass = 2, kMLo = 2; };

template <int WIDTH, class ActT>
struct M1Codes {
    using E = Elem16<ActT>;
    using P = M1Plan<WIDTH, ActT>;
    static constexpr int kFields = 32 / WIDTH;          // columns per dword
    static constexpr int kPairs = kFields / 2;
    static constexpr int kFPD = kPairs / 4;             // MFMAs (operand fragments) per dword
    static constexpr int kDW = 4;                       // dwords of codes in one lane's 16 bytes
    static constexpr bool kDecode = false;              // the 16 bytes are the codes themselves
    static constexpr int kFPL = 4 * kFPD;               // per 16-byte piece
    static constexpr int kPieceCols = 4 * kFields;      // columns of one lane's 16 bytes
    // bytes of one packed row of a g128 format (rows are padded to whole groups)
    static __host__ __device__ constexpr int row_stride(int cols) { return (cols + 127) / 128 * 128 * 4 / kFields; }
    static constexpr int kPasses = (kPairs + P::kPerPass - 1) / P::kPerPass;
    static __device__ __forceinline__ constexpr int mant_pos(int j) { return P::kMLo + WIDTH * (j % P::kPerPass); }
    // right shift (left when negative) that brings the codes of a pass to their mantissa positions
    static __device__ __forceinline__ constexpr int pass_shift(int pass) { return WIDTH * P::kPerPass * pass - P::kMLo; }
    static __device__ __forceinline__ constexpr uint32_t both(uint32_t h) { return h | (h << 16); }
    static __device__ __forceinline__ constexpr uint32_t mask(int j) { return both(((1u << WIDTH) - 1u) << mant_pos(j)); }
    static __device__ __forceinline__ constexpr uint32_t base_half(int j) { return (uint32_t)(E::kExpBias + E::kMant - mant_pos(j)) << E::kMant; }
    // bits of (base, base) as a pair of 16-bit floats: what the AND-OR adds to the codes of pair j
    static __device__ __forceinline__ constexpr uint32_t base_pair(int j) { return both(base_half(j)); }
    // one packed dword -> the B operands of its kFPD MFMAs
    static __device__ __forceinline__ void operands(uint32_t c, uint4_t (&out)[kFPD]) {
        uint32_t src[kPasses];
#pragma unroll
        for (int p = 0; p < kPasses; ++p) {
            const int sh = pass_shift(p);
            src[p] = sh == 0 ? c : (sh > 0 ? c >> sh : c << -sh);
        }
        uint32_t r[kPairs];
#pragma unroll
        for (int j = 0; j < kPairs; ++j) r[j] = and_or(src[j / P::kPerPass], mask(j), base_pair(j));
#pragma unroll
        for (int t = 0; t < kFPD; ++t) out[t] = uint4_t{r[4 * t], r[4 * t + 1], r[4 * t + 2], r[4 * t + 3]};
    }
};

// semantic weight = kSemMul * (code - kOffset) * scale (+ bias for affine codes)
template <class ActT>
struct M1Bin : M1Codes<1, ActT> {
    static constexpr bool kHasBias = false;
    static constexpr float kSemMul = 2.0f, kOffset = 0.5f;
};
template <class ActT>
struct M1Ter2 : M1Codes<2, ActT> {
    static constexpr bool kHasBias = false;
    static constexpr float kSemMul = 1.0f, kOffset = 1.0f;
};
// The 243-entry decode table of the five-digit bytes (five 2-bit codes, digit i at bits 2i..2i+1; invalid
// bytes decode to five semantic zeros), built at compile time.
struct Trit5Lut {
    uint16_t e[256];
    constexpr Trit5Lut() : e() {
        for (unsigned b = 0; b < 256; ++b) {
            unsigned v = b, code = 0;
            for (int i = 0; i < 5; ++i) { code |= (v % 3u) << (2 * i); v /= 3u; }
            e[b] = b >= 243u ? 0x0155u : (uint16_t)code;
        }
    }
};
__device__ __constant__ constexpr Trit5Lut kTrit5Lut{};

// trit5: the 16 bytes of a lane hold 80 base-3 digits, decoded through the 243-entry table into five
// dwords of ternary2 codes.  A 128-byte row segment is 640 columns, five scale groups: a piece spans up
// to two of them, and the kernel keeps the two apart (see the job).
template <class ActT>
struct M1Trit5 : M1Codes<2, ActT> {
    using Base = M1Codes<2, ActT>;
    static constexpr bool kHasBias = false;
    static constexpr float kSemMul = 1.0f, kOffset = 1.0f;
    static constexpr int kDW = 5;
    static constexpr bool kDecode = true;
    static constexpr int kFPL = 5 * Base::kFPD;
    static constexpr int kPieceCols = 5 * Base::kFields;
    static __host__ __device__ constexpr int row_stride(int cols) { return (((cols + 4) / 5) + 15) & ~15; }
};
template <class ActT>
struct M1U4 : M1Codes<4, ActT> {
    static constexpr bool kHasBias = true;
    static constexpr float kSemMul = 1.0f, kOffset = 0.0f;
};

// LDS layout of a workgroup of `waves` waves with `nl` segments each:
//   per wave: operand fragments [nl * 8 pieces][frags per piece] x 16 B, then per piece the
//             folded-out constant and the plain sum of x (8 B), then one piece of zero fragments;
//   then the scale rows (and bias rows) of the workgroup's eight rows, one block per matrix and
//   plane; then the waves' partial sums [wave][matrix][8] (fp32).
//   (five-dword pieces: per dword the folded-out constant, 4 B; and a 512-byte decode table at the end)
//   Four-dword pieces hold a power-of-two number of fragments, which would put the eight pieces of a
//   segment (read together, one per A-operand lane) on the same LDS banks: their stride is one
//   fragment longer, except for pieces of four fragments (affine 4-bit), where pieces p and p + 4 are the
//   only ones to meet and the second half of a segment stores fragment d in slot d ^ 1 instead (a long
//   row's fragments are most of a workgroup's LDS: without the padding three workgroups of a
//   17408-column matrix fit a compute unit instead of two).  Five-dword pieces (160 bytes) spread over the
//   banks by themselves.
__host__ __device__ constexpr int mm1_piece_stride(int frags_per_piece, int dw = 4) {
    return dw == 4 ? (frags_per_piece == 4 ? 4 : frags_per_piece + 1) : frags_per_piece;
}
__host__ __device__ constexpr size_t mm1_wave_lds_bytes(int frags_per_piece, int nl, int dw = 4, int tok = 1) {
    return (size_t)tok * ((size_t)nl * 8 * mm1_piece_stride(frags_per_piece, dw) * 16 + (dw == 4 ? (size_t)nl * 8 * 8 : (size_t)nl * 8 * dw * 4)) +
           (size_t)frags_per_piece * 16;
}
__host__ __device__ constexpr size_t mm1_lds_bytes(int frags_per_piece, int nl, int waves, int nmat, int gpr, bool has_bias, int dw = 4, int tok = 1) {
    return (size_t)waves * mm1_wave_lds_bytes(frags_per_piece, nl, dw, tok) + (size_t)nmat * (has_bias ? 2 : 1) * 8 * gpr * 2 +
           (size_t)waves * nmat * tok * 32 + (dw == 4 ? 0 : 512);
}

// v[i] + v[i ^ 16] and v[i] + v[i ^ 32] in every lane, through the lane-swap instructions (no LDS
// round trip): the swap exchanges the odd rows (the upper half) of its first operand with the even
// rows (the lower half) of its second, so the two results hold the two addends in the same order in
// both partner lanes.
__device__ __forceinline__ float swap_sum16(float v) {
    const uint32_t b = __builtin_bit_cast(uint32_t, v);
    const auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}
__device__ __forceinline__ float swap_sum32(float v) {
    const uint32_t b = __builtin_bit_cast(uint32_t, v);
    const auto r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
    return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

__device__ __forceinline__ float quad_sum(float v) {
    v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    return dpp_add<0x4E>(v);  // quad_perm [2,3,0,1]
}

// One workgroup = one tile of eight rows; its kc waves split K: wave `chunk` owns the 128-byte
// segments [chunk * NL, chunk * NL + NL) of every row of the tile.
// NORM: 0 = x is multiplied as it is; 1 = the norm-scale prologue (what is multiplied is
// narrow((x * rs[token]) * (1 + weight)), the bits a staged norm would have stored; workgroup 0 also
// stores that row to ns.out); 2 = the same followed by the residual add of the norm_add_scale form.
// TOK = 2: two tokens per pass (grid row r takes tokens 2r and 2r + 1 of `tokens`).  With four-dword pieces the
// token slots 4q + 2 and 4q + 3 of an MFMA are free: they carry the second token's fragments, so the weights are
// unpacked and multiplied once for both tokens.
template <class F, class ActT, class ScaleT, int NMAT, int NL, class Epi, int NORM = 0, int TOK = 1>
__device__ __forceinline__ void mm1_body(const MatPtrs (&mats)[NMAT], const uint16_t* __restrict__ x_all, int rows,
                                         int cols, int row_stride, int group, const Epi& epi,
                                         const NormScale& ns = NormScale{}, int tokens = 0) {
    using E = Elem16<ActT>;
    constexpr int FPD = F::kFPD, FPL = F::kFPL, FIELDS = F::kFields, PAIRS = F::kPairs, DW = F::kDW;
    constexpr int PSTRIDE = mm1_piece_stride(FPL, DW);     // fragments from one piece to the next in LDS
    constexpr bool kSwizzle = DW == 4 && FPL == 4;         // unpadded pieces: slot d ^ 1 in the second half of a segment
    constexpr int NITEMS = NL * 8 * DW;                    // staging items of a wave: 8 pieces x DW dwords per segment
    constexpr int ITEMS = (NITEMS + kWave - 1) / kWave;    // per lane
    constexpr int PLANES = F::kHasBias ? 2 : 1;
    static_assert(TOK == 1 || (TOK == 2 && DW == 4 && NORM == 0 && !Epi::kTile), "two tokens per pass: four-dword pieces, no prologue");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_all[];
    // five-digit bytes: the 512-byte decode table sits at the start of LDS (a lookup address is the byte
    // value times two), everything else behind it
    unsigned char* const smem = smem_all + (F::kDecode ? 512 : 0);
    const int lane = threadIdx.x & (kWave - 1);
    const int chunk = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int kc = blockDim.x / kWave;
    const int n = lane & 15, q = lane >> 4;
    const int token = blockIdx.y * TOK;
    // (a second token past the batch re-reads the last one and is never stored)
    const int token_b = TOK == 2 && token + 1 < tokens ? token + 1 : token;
    const uint16_t* __restrict__ x = x_all + (size_t)token * cols;
    const uint16_t* __restrict__ x_b = x_all + (size_t)token_b * cols;
    const int pieces = row_stride >> 4;               // 16-byte pieces per packed row
    const int gshift = ilog2((uint32_t)group);
    const int gpr = (cols + group - 1) >> gshift;     // 16-byte pieces of one plane's scale block, too
    const int row0 = blockIdx.x * 8;
    const int piece0 = chunk * NL * 8;                // first piece of this wave's run
    // Weight loads are issued in memory order, eight consecutive lanes on the 128 bytes of one row
    // segment (lane = 8 * row-in-tile + piece); a cross-lane transpose then hands MFMA lane (n, q)
    // the piece 4 * (n / 8) + q of row n % 8.
    const int ld_q = lane & 7, ld_r = lane >> 3;
    const int hh = n >> 3, rn = n & 7;                // which half of the segment, which row of the tile
    const int xpose = (8 * rn + 4 * hh + q) * 4;      // byte address of the source lane for ds_bpermute

    // Nothing below branches or predicates a load until every load of the job is issued (a load
    // under a branch invites the compiler to move its consumer, and the wait, in there too).
    // Loads return in issue order, so what is needed first is asked for first: the activations (they
    // come from cache and are turned into fragments while the rest is still in flight), then the
    // scales, then the weights.  A row or piece past the end re-reads the last valid one and is
    // discarded later (zero scale, no store).
    //
    // ---- 1. this wave's slice of x ---------------------------------------------------------------
    // One item = the columns of one packed dword; item it = 4 * (piece within the run) + dword.
    uint32_t xe[TOK][ITEMS][FIELDS / 2];
    int item_piece[ITEMS], item_dword[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        int it = lane + k * kWave;
        if (it > NITEMS - 1) it = NITEMS - 1;
        item_piece[k] = DW == 4 ? it >> 2 : (it * 52429) >> 18;   // it / 5 for it < 2^14
        item_dword[k] = it - DW * item_piece[k];
        int col0 = (piece0 + item_piece[k]) * F::kPieceCols + item_dword[k] * FIELDS;
        // a dword past the end of the row (five-dword pieces end inside a piece) multiplies zeros
        const bool past = DW != 4 && col0 > cols - FIELDS;
        if (col0 > cols - FIELDS) col0 = cols - FIELDS;   // cols is a multiple of kFields
#pragma unroll
        for (int tk = 0; tk < TOK; ++tk)
#pragma unroll
        for (int v = 0; v < FIELDS / 8; ++v) {
            uint4_t t = *reinterpret_cast<const uint4_t*>((tk == 0 ? x : x_b) + col0 + 8 * v);
            if constexpr (NORM != 0) {
                // eight activations through the prologue, each rounded as the staged norm rounds it
                const float rs = ns.rs[token];
                const uint4_t w8 = *reinterpret_cast<const uint4_t*>(ns.weight + col0 + 8 * v);
                uint4_t r8 = uint4_t{0u, 0u, 0u, 0u};
                if constexpr (NORM == 2) r8 = *reinterpret_cast<const uint4_t*>(ns.residual + (size_t)token * cols + col0 + 8 * v);
                uint32_t out[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t pair = 0;
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        uint16_t e = norm_scale_value<ActT>((uint16_t)(t[j] >> (16 * h)), rs, (uint16_t)(w8[j] >> (16 * h)));
                        if constexpr (NORM == 2) e = ActT::narrow(ActT::widen(e) + ActT::widen((uint16_t)(r8[j] >> (16 * h))));
                        pair |= (uint32_t)e << (16 * h);
                    }
                    out[j] = pair;
                }
                t = uint4_t{out[0], out[1], out[2], out[3]};
                // (lanes past the last item hold the last item again and store the same bits again)
                if (blockIdx.x == 0 && ns.out != nullptr) *reinterpret_cast<uint4_t*>(ns.out + (size_t)token * cols + col0 + 8 * v) = t;
            }
            xe[tk][k][4 * v] = past ? 0u : t.x; xe[tk][k][4 * v + 1] = past ? 0u : t.y;
            xe[tk][k][4 * v + 2] = past ? 0u : t.z; xe[tk][k][4 * v + 3] = past ? 0u : t.w;
        }
    }
    // ---- 2. the scale (and bias) rows of the tile: one contiguous block per matrix and plane ----
    // Short affine rows (one or two segments per wave: the launches that are a single memory round
    // trip) skip the block: every lane fetches the two-byte scale and bias of the group it will apply,
    // no wave waits for another's loads and the workgroup meets only for its final sum.
    constexpr bool kDirectScales = F::kHasBias && DW == 4 && NL <= 2;
    const int plane_pieces = (rows * gpr * 2 + 15) >> 4;
    uint4_t sp[NMAT][PLANES];
    uint16_t sdir[NMAT][PLANES][NL];
    if constexpr (kDirectScales) {
        int srow = row0 + rn;
        if (srow > rows - 1) srow = rows - 1;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            int piece = piece0 + i * 8 + 4 * hh + q;
            if (piece > pieces - 1) piece = pieces - 1;
            const int g = (piece * F::kPieceCols) >> gshift;
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int pl = 0; pl < PLANES; ++pl) sdir[m][pl][i] = (pl == 0 ? mats[m].scales : mats[m].biases)[(size_t)srow * gpr + g];
        }
    } else {
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int pl = 0; pl < PLANES; ++pl) {
            const uint4_t* base = reinterpret_cast<const uint4_t*>(pl == 0 ? mats[m].scales : mats[m].biases);
            int idx = (int)threadIdx.x;
            if (idx > gpr - 1) idx = gpr - 1;
            int src = blockIdx.x * gpr + idx;         // row0 * gpr * 2 bytes = blockIdx.x * gpr pieces
            if (src > plane_pieces - 1) src = plane_pieces - 1;
            sp[m][pl] = base[src];
        }
    }
    // ---- 3. every weight load of the job -------------------------------------------------------------
    uint4_t codes[NMAT][NL];
    {
        int ld_row = row0 + ld_r;
        if (ld_row > rows - 1) ld_row = rows - 1;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            int piece = piece0 + i * 8 + ld_q;
            if (piece > pieces - 1) piece = pieces - 1;
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
                codes[m][i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(mats[m].codes + (size_t)ld_row * row_stride + (size_t)piece * 16));
        }
    }
    // the epilogue's operand, by every lane of every wave (clamped to the tile's rows): under a branch
    // the load brings its own wait on everything issued before it, and wave 0 would stage x only
    // after all its weights have arrived
    uint16_t res[TOK] = {};
    if constexpr (Epi::kPrefetch) {
        const int rr = row0 + (lane & 7);
        res[0] = epi.prefetch(token, rr < rows ? rr : rows - 1);
        if constexpr (TOK == 2) res[1] = epi.prefetch(token_b, rr < rows ? rr : rows - 1);
    }

    const size_t wave_bytes = mm1_wave_lds_bytes(FPL, NL, DW, TOK);
    constexpr int kTokStride = NL * 8 * PSTRIDE + (DW == 4 ? NL * 4 : 0);   // fragments and sums of one token, in 16-byte units
    uint4_t* lds_scales = reinterpret_cast<uint4_t*>(smem + (size_t)kc * wave_bytes);
    // ---- 4. x as operand fragments, wave-private in LDS --------------------------------------------
    // kFields consecutive activations become the kFPD fragments that dword's MFMAs take (k-slots
    // 2v, 2v+1 of fragment t = columns 4t+v, 4t+v+kPairs).  The four items of a 16-byte piece sit
    // in the four lanes of a quad, which add up their sum(base * x) and sum(x).
    uint4_t* wfrag = reinterpret_cast<uint4_t*>(smem + (size_t)chunk * wave_bytes);
    float* wsum = reinterpret_cast<float*>(wfrag + (size_t)NL * 8 * PSTRIDE);   // [piece][2]: constant, sum x ([piece][DW]: constants)
    // (a second token's fragments and sums follow the first's; the zero fragments come last)
    uint4_t* wzero = TOK == 2 ? wfrag + (size_t)TOK * kTokStride
                              : reinterpret_cast<uint4_t*>(wsum + (DW == 4 ? NL * 16 : NL * 8 * DW));   // FPL zero fragments
    // decode table of the five-digit bytes, copied from constant memory; visible after the barrier below
    uint16_t* lut = reinterpret_cast<uint16_t*>(smem_all);
    if constexpr (F::kDecode) {
        for (uint32_t i = threadIdx.x; i < 128; i += blockDim.x)
            reinterpret_cast<uint32_t*>(lut)[i] = reinterpret_cast<const uint32_t*>(kTrit5Lut.e)[i];
    }
    if (lane < FPL) wzero[lane] = uint4_t{0u, 0u, 0u, 0u};
#pragma unroll
    for (int tk = 0; tk < TOK; ++tk)
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        // lanes past the last item hold the last item again (whole quads of them: d == 3) and store
        // the same fragments again
        const int pl = item_piece[k], d = item_dword[k], it = pl * DW + d;
        uint4_t* const wfrag_t = wfrag + (size_t)tk * kTokStride;
        float* const wsum_t = wsum + (size_t)tk * kTokStride * 4;
        float cb = 0.0f, xs = 0.0f;
        constexpr uint32_t kOnes = F::both((uint32_t)E::kExpBias << E::kMant);   // (1.0, 1.0)
        uint32_t fr[PAIRS];
#pragma unroll
        for (int j = 0; j < PAIRS; ++j) {
            const uint32_t lo = xe[tk][k][j >> 1], hi = xe[tk][k][(PAIRS >> 1) + (j >> 1)];
            fr[j] = __builtin_amdgcn_perm(hi, lo, (j & 1) ? 0x07060302u : 0x05040100u);   // (x[j], x[j + kPairs])
            cb = E::dot2k(fr[j], F::base_pair(j), cb);
            xs = E::dot2k(fr[j], kOnes, xs);
        }
        if constexpr (DW == 4) {
            cb = quad_sum(cb);
            xs = quad_sum(xs);
        }
#pragma unroll
        for (int t = 0; t < FPD; ++t)
            wfrag_t[(size_t)pl * PSTRIDE + ((d * FPD + t) ^ (kSwizzle ? (pl >> 2) & 1 : 0))] = uint4_t{fr[4 * t], fr[4 * t + 1], fr[4 * t + 2], fr[4 * t + 3]};
        if constexpr (DW == 4) {
            if (d == 0) *reinterpret_cast<float2*>(wsum_t + 2 * pl) = float2{__builtin_fmaf(F::kOffset, xs, cb), xs};
        } else {
            wsum_t[it] = __builtin_fmaf(F::kOffset, xs, cb);   // one constant per dword: the job adds them per scale group
        }
    }
    // ---- 5. scales into LDS (they were asked for after the activations and arrive after them) ------
    if constexpr (kDirectScales) {
        // nothing to share; the fragments are this wave's own: LDS executes a wave's operations in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int pl = 0; pl < PLANES; ++pl) {
            // threads past the end of the block hold its last piece again and store it again
            int idx = (int)threadIdx.x;
            if (idx > gpr - 1) idx = gpr - 1;
            lds_scales[(m * PLANES + pl) * gpr + idx] = sp[m][pl];
        }

    __syncthreads();   // scales of every wave, fragments of this one
    }

    // ---- 6. the job --------------------------------------------------------------------------------
    // A-operand lanes 20q and 20q + 1 (token slots 4q and 4q + 1 in k-block q: the two halves of
    // the segment) read fragments; the others read the zero fragments, so no lane is masked off.
    // Five-dword pieces span up to two scale groups (a segment is five groups, eight pieces of five
    // dwords: piece p starts at dword 5p of forty, a group is eight dwords): the dwords of a piece's
    // second group go to token slots 4q + 2 and 4q + 3 instead, i.e. for those dwords A lanes 20q + 2
    // and 20q + 3 are the ones that read fragments.
    const int a_slot = n - 4 * q;                       // 0..3 for the lanes that ever read fragments
    const bool a_valid = DW == 4 && TOK == 1 ? (a_slot == 0 || a_slot == 1) : (a_slot >= 0 && a_slot < 4);
    const int a_half = a_slot & 1, a_second = a_slot >> 1;
    const int a_piece = 4 * a_half + q;                 // piece of the segment this lane feeds
    auto first_group_dwords = [](int piece_in_segment) {
        if (DW == 4) return 4;
        const int left = 8 - ((5 * piece_in_segment) & 7);
        return left < 5 ? left : 5;
    };
    const int a_split = first_group_dwords(a_piece);
    const uint16_t* lds_s16 = reinterpret_cast<const uint16_t*>(lds_scales);
    float y[TOK][NMAT];
#pragma unroll
    for (int tk = 0; tk < TOK; ++tk)
#pragma unroll
        for (int m = 0; m < NMAT; ++m) y[tk][m] = 0.0f;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        float4_t acc[NMAT];
#pragma unroll
        for (int m = 0; m < NMAT; ++m) acc[m] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        // the codes of this segment: as loaded, or decoded here (in load order, before the transpose)
        uint32_t cd[NMAT][DW];
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            if constexpr (F::kDecode) {
                FmtTrit5::decode(codes[m][i], lut, cd[m]);
            } else {
                cd[m][0] = codes[m][i].x; cd[m][1] = codes[m][i].y; cd[m][2] = codes[m][i].z; cd[m][3] = codes[m][i].w;
            }
        }
        // (two tokens: slots 4q + 2 and 4q + 3 read the second token's fragments of the same pieces)
        const uint4_t* piece_frags = wfrag + (TOK == 2 ? (size_t)a_second * kTokStride : (size_t)0) + (size_t)(i * 8 + a_piece) * PSTRIDE;
        if constexpr (DW * FPD <= 4 && !F::kDecode) {
            // few fragments per segment: all of them, and every transpose, are asked for before the first
            // MFMA, so the LDS round trips overlap each other (and, for the fragments, the weights' flight)
            uint4_t afr[DW][FPD];
#pragma unroll
            for (int d = 0; d < DW; ++d) {
                const bool a_live = a_valid && (TOK == 2 || (d >= a_split) == (a_second == 1));
                const uint4_t* pf = a_live ? piece_frags + (kSwizzle ? d ^ a_half : d) * FPD : wzero;
#pragma unroll
                for (int f = 0; f < FPD; ++f) afr[d][f] = pf[f];
            }
            uint32_t cw[NMAT][DW];
#pragma unroll
            for (int d = 0; d < DW; ++d)
#pragma unroll
                for (int m = 0; m < NMAT; ++m) cw[m][d] = (uint32_t)__builtin_amdgcn_ds_bpermute(xpose, (int)cd[m][d]);
#pragma unroll
            for (int d = 0; d < DW; ++d)
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    uint4_t ops[FPD];
                    F::operands(cw[m][d], ops);
#pragma unroll
                    for (int f = 0; f < FPD; ++f) acc[m] = E::mfma(afr[d][f], ops[f], acc[m]);
                }
        } else {
#pragma unroll
        for (int d = 0; d < DW; ++d) {
            const bool a_live = a_valid && (TOK == 2 || (d >= a_split) == (a_second == 1));
            const uint4_t* pf = a_live ? piece_frags + (kSwizzle ? d ^ a_half : d) * FPD : wzero;
            uint4_t afr[FPD];
#pragma unroll
            for (int f = 0; f < FPD; ++f) afr[f] = pf[f];
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const uint32_t cw = (uint32_t)__builtin_amdgcn_ds_bpermute(xpose, (int)cd[m][d]);
                uint4_t ops[FPD];
                F::operands(cw, ops);
#pragma unroll
                for (int f = 0; f < FPD; ++f) acc[m] = E::mfma(afr[f], ops[f], acc[m]);
            }
        }
        }
        const int piece = piece0 + i * 8 + 4 * hh + q;
        const bool piece_ok = piece < pieces;
        const int g = ((piece_ok ? piece : pieces - 1) * F::kPieceCols) >> gshift;
        if constexpr (DW == 4) {
#pragma unroll
            for (int tk = 0; tk < TOK; ++tk) {
            const float2 cs = *reinterpret_cast<const float2*>(wsum + (size_t)tk * kTokStride * 4 + 2 * (i * 8 + 4 * hh + q));
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const int sidx = (m * PLANES) * (8 * gpr) + rn * gpr + g;
                const float sv = F::kSemMul * ScaleT::widen(kDirectScales ? sdir[m][0][i] : lds_s16[sidx]);
                // token slot 4q + hh (the second token: 4q + 2 + hh)
                const float dotp = tk == 0 ? (hh ? acc[m].y : acc[m].x) : (hh ? acc[m].w : acc[m].z);
                y[tk][m] = __builtin_fmaf(piece_ok ? sv : 0.0f, dotp - cs.x, y[tk][m]);
                if (F::kHasBias) {
                    const float bv = ScaleT::widen(kDirectScales ? sdir[m][PLANES - 1][i] : lds_s16[sidx + 8 * gpr]);
                    y[tk][m] = __builtin_fmaf(piece_ok ? bv : 0.0f, cs.y, y[tk][m]);
                }
            }
            }
        } else {
            // the folded-out constants of the piece's dwords, per scale group
            const int split = first_group_dwords(4 * hh + q);
            const float* cdw = wsum + (i * 8 + 4 * hh + q) * DW;
            float c_first = 0.0f, c_second = 0.0f;
#pragma unroll
            for (int d = 0; d < DW; ++d) {
                const float c = cdw[d];
                c_first += d < split ? c : 0.0f;
                c_second += d < split ? 0.0f : c;
            }
            const int g2 = g + 1 < gpr ? g + 1 : gpr - 1;   // unused (its sums are zero) when the piece has one group
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const int srow = (m * PLANES) * (8 * gpr) + rn * gpr;
                const float s1 = F::kSemMul * ScaleT::widen(lds_s16[srow + g]);
                const float s2 = F::kSemMul * ScaleT::widen(lds_s16[srow + g2]);
                const float d1 = hh ? acc[m].y : acc[m].x;   // token slot 4q + hh: first group
                const float d2 = hh ? acc[m].w : acc[m].z;   // token slot 4q + 2 + hh: second group
                y[0][m] = __builtin_fmaf(piece_ok ? s1 : 0.0f, d1 - c_first, y[0][m]);
                y[0][m] = __builtin_fmaf(piece_ok ? s2 : 0.0f, d2 - c_second, y[0][m]);
            }
        }
    }
    // the eight pieces of a segment: lanes rn + 8 * {0..7}
#pragma unroll
    for (int tk = 0; tk < TOK; ++tk)
#pragma unroll
    for (int m = 0; m < NMAT; ++m) {
        y[tk][m] = dpp_add<0x128>(y[tk][m]);   // row_ror:8: lane i of a row of sixteen takes lane i ^ 8
        y[tk][m] = swap_sum16(y[tk][m]);
        y[tk][m] = swap_sum32(y[tk][m]);
    }

    // ---- 7. the kc waves of the workgroup -----------------------------------------------------------
    if (kc > 1) {
        float* red = reinterpret_cast<float*>(smem + (size_t)kc * wave_bytes + (size_t)NMAT * PLANES * 8 * gpr * 2);
        if (lane < 8) {
#pragma unroll
            for (int tk = 0; tk < TOK; ++tk)
#pragma unroll
            for (int m = 0; m < NMAT; ++m) red[((chunk * TOK + tk) * NMAT + m) * 8 + lane] = y[tk][m];
        }
        __syncthreads();
        if (chunk == 0) {
            // lane 8 k + r takes wave k's sum of row r (zero past the last wave; waves 8 .. 15 in a second
            // value), and the lanes r, r + 8, ... add up as the pieces of a segment did above
#pragma unroll
            for (int tk = 0; tk < TOK; ++tk)
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const int k = lane >> 3, r = lane & 7;
                const int k0 = k < kc ? k : kc - 1, k1 = k + 8 < kc ? k + 8 : kc - 1;
                const float v0 = red[((k0 * TOK + tk) * NMAT + m) * 8 + r], v1 = red[((k1 * TOK + tk) * NMAT + m) * 8 + r];
                float sum = (k < kc ? v0 : 0.0f) + (k + 8 < kc ? v1 : 0.0f);
                sum = dpp_add<0x128>(sum);
                sum = swap_sum16(sum);
                y[tk][m] = swap_sum32(sum);
            }
        }
    }
    if constexpr (Epi::kTile) {
        if (chunk == 0) epi.tile(token, row0, rows, lane, y[0]);
    } else if (chunk == 0 && lane < 8 && row0 + lane < rows) {
        if constexpr (Epi::kPrefetch) epi.finish(token, row0 + lane, y[0], res[0]);
        else epi(token, row0 + lane, y[0]);
        if constexpr (TOK == 2) {
            if (token + 1 < tokens) {
                if constexpr (Epi::kPrefetch) epi.finish(token + 1, row0 + lane, y[1], res[1]);
                else epi(token + 1, row0 + lane, y[1]);
            }
        }
    }
}

// lm_head: argmax over the rounded logits, fused (affine_matvec_argmax, one token per grid row).  The
// pipeline's consumer reads `num_partials` keys per token, any partition of the rows; a tile holds eight
// rows, so the tiles t, t + num_partials, ... share partial t: each leaves its best key in the workspace
// and counts itself in, and the last to arrive writes the best of them (keys carry their row, so the
// result does not depend on the order of arrival).  Keys cross workgroups as agent-scope relaxed atomics
// (coherent across the compute dies); a tile's store is acknowledged before its arrival is counted, and
// the last arrival reads only after its count returned.  Counters are left at zero for the next launch.
template <class ActT>
struct EpiTileArgmax : EpiBase {
    static constexpr bool kTile = true;
    uint2_t* partials;                 // [token][num_partials]
    unsigned long long* tile_keys;     // workspace: [token][tiles]
    uint32_t* counters;                // workspace: [token][num_partials]
    uint32_t num_partials;
    float logit_cap;
    __device__ __forceinline__ void tile(int token, int row0, int rows, int lane, const float* y) const {
        float x = y[0];
        if (logit_cap > 0.0f) {
            // cap * tanh(x / cap) as cap * (1 - 2 / (1 + exp(2x / cap))); exp overflow gives +-cap
            const float e = expf(2.0f * x / logit_cap);
            x = logit_cap * (1.0f - 2.0f / (1.0f + e));
        }
        uint2_t key = {0u, 0u};
        if (lane < 8 && row0 + lane < rows) key = argmax_pack_key(ActT::narrow(x), (uint32_t)(row0 + lane));
#pragma unroll
        for (int off = 4; off > 0; off >>= 1) {
            uint2_t o;
            o.x = __shfl_xor(key.x, off);
            o.y = __shfl_xor(key.y, off);
            key = argmax_key_max(key, o);
        }
        const uint32_t tiles = gridDim.x, parts = num_partials;
        const uint32_t slot = blockIdx.x % parts;
        const uint32_t members = tiles / parts + (slot < tiles % parts ? 1u : 0u);
        uint2_t* out = partials + (size_t)token * parts + slot;
        if (members == 1u) {
            if (lane == 0) *out = key;
            return;
        }
        unsigned long long* keys = tile_keys + (size_t)token * tiles;
        uint32_t* counter = counters + (size_t)token * parts + slot;
        uint32_t last = 0u;
        if (lane == 0) {
            __hip_atomic_store(keys + blockIdx.x, ((unsigned long long)key.x << 32) | key.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): the store is acknowledged
            last = atomicAdd(counter, 1u) == members - 1u ? 1u : 0u;
        }
        if (!__builtin_amdgcn_readfirstlane(last)) return;
        uint2_t best = {0u, 0u};
        for (uint32_t j = (uint32_t)lane; j < members; j += kWave) {
            const unsigned long long v = __hip_atomic_load(keys + slot + (size_t)j * parts, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            best = argmax_key_max(best, uint2_t{(uint32_t)(v >> 32), (uint32_t)v});
        }
        best = wave_argmax_key(best);
        if (lane == 0) {
            *out = best;
            *counter = 0u;
        }
    }
};

}  // namespace smelt

#define SMELT_MM1_KERNEL extern "C" __global__ __launch_bounds__(1024)

// Signed g128 formats: same argument lists as the vector-ALU kernels of the pipelines.  The launch
// supplies the split: one workgroup per NT row tiles, one wave per NL segments of a row.
#define SMELT_SIGNED_MM1_KERNELS(FN, FMT, T, ACT, NLV)                                       \
    SMELT_MM1_KERNEL void smelt_signed_##FN##_mm1_nl##NLV##_matvec_##T(                  \
        const u8* C, const u16* S, const u16* X, u16* Y, u32 rows, u32 cols) {                    \
        using namespace smelt;                                                                    \
        using F = FMT<ACT>;                                                                       \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        mm1_body<F, ACT, F16, 1, NLV>(mats, X, rows, cols,                                   \
                                           F::row_stride((int)cols), 128, epi);  \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_signed_##FN##_mm1_nl##NLV##_matvec_add_##T(              \
        const u8* C, const u16* S, const u16* X, u16* Y, const u16* res, u32 rows, u32 cols) {    \
        using namespace smelt;                                                                    \
        using F = FMT<ACT>;                                                                       \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                   \
        mm1_body<F, ACT, F16, 1, NLV>(mats, X, rows, cols,                                   \
                                           F::row_stride((int)cols), 128, epi);  \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_signed_##FN##_mm1_nl##NLV##_gate_up_swiglu_##T(          \
        const u8* gC, const u16* gS, const u8* uC, const u16* uS, const u16* X, u16* Y, u32 rows, \
        u32 cols) {                                                                      \
        using namespace smelt;                                                                    \
        using F = FMT<ACT>;                                                                       \
        const MatPtrs mats[2] = {{gC, gS, nullptr}, {uC, uS, nullptr}};                           \
        EpiSignedSwiglu<ACT> epi{{}, Y, (int)rows};                                               \
        mm1_body<F, ACT, F16, 2, NLV>(mats, X, rows, cols,                                   \
                                           F::row_stride((int)cols), 128, epi);  \
    }

// Two tokens per pass (binary and ternary codes): the argument lists above plus the number of tokens; grid row r
// takes tokens 2r and 2r + 1.
#define SMELT_SIGNED_MM1_KERNELS_T2(FN, FMT, T, ACT, NLV)                                         \
    SMELT_MM1_KERNEL void smelt_signed_##FN##_mm1_nl##NLV##_t2_matvec_##T(                        \
        const u8* C, const u16* S, const u16* X, u16* Y, u32 rows, u32 cols, u32 tokens) {        \
        using namespace smelt;                                                                    \
        using F = FMT<ACT>;                                                                       \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        mm1_body<F, ACT, F16, 1, NLV, EpiStore<ACT>, 0, 2>(mats, X, rows, cols, F::row_stride((int)cols), 128, epi, \
                                                           NormScale{}, (int)tokens);             \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_signed_##FN##_mm1_nl##NLV##_t2_matvec_add_##T(                    \
        const u8* C, const u16* S, const u16* X, u16* Y, const u16* res, u32 rows, u32 cols,      \
        u32 tokens) {                                                                             \
        using namespace smelt;                                                                    \
        using F = FMT<ACT>;                                                                       \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                   \
        mm1_body<F, ACT, F16, 1, NLV, EpiAdd<ACT>, 0, 2>(mats, X, rows, cols, F::row_stride((int)cols), 128, epi, \
                                                         NormScale{}, (int)tokens);               \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_signed_##FN##_mm1_nl##NLV##_t2_gate_up_swiglu_##T(                \
        const u8* gC, const u16* gS, const u8* uC, const u16* uS, const u16* X, u16* Y, u32 rows, \
        u32 cols, u32 tokens) {                                                                   \
        using namespace smelt;                                                                    \
        using F = FMT<ACT>;                                                                       \
        const MatPtrs mats[2] = {{gC, gS, nullptr}, {uC, uS, nullptr}};                           \
        EpiSignedSwiglu<ACT> epi{{}, Y, (int)rows};                                               \
        mm1_body<F, ACT, F16, 2, NLV, EpiSignedSwiglu<ACT>, 0, 2>(mats, X, rows, cols, F::row_stride((int)cols), 128, \
                                                                  epi, NormScale{}, (int)tokens); \
    }

#define SMELT_TERAFF_MM1_KERNELS_T2(T, ACT, NLV)                                                  \
    SMELT_MM1_KERNEL void smelt_teraff_mm1_nl##NLV##_t2_matvec_##T(                               \
        const u8* C, const u16* S, const u16*, const u16* X, u16* Y, u32 rows, u32 cols,          \
        u32 tokens) {                                                                             \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        mm1_body<M1Ter2<ACT>, ACT, F16, 1, NLV, EpiStore<ACT>, 0, 2>(mats, X, rows, cols, cols / 4, 128, epi, \
                                                                     NormScale{}, (int)tokens);   \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_teraff_mm1_nl##NLV##_t2_matvec_add_##T(                           \
        const u8* C, const u16* S, const u16*, const u16* X, u16* Y, const u16* res, u32 rows,    \
        u32 cols, u32 tokens) {                                                                   \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                   \
        mm1_body<M1Ter2<ACT>, ACT, F16, 1, NLV, EpiAdd<ACT>, 0, 2>(mats, X, rows, cols, cols / 4, 128, epi, \
                                                                   NormScale{}, (int)tokens);     \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_teraff_mm1_nl##NLV##_t2_gate_up_swiglu_##T(                       \
        const u8* gC, const u16* gS, const u16*, const u8* uC, const u16* uS, const u16*,         \
        const u16* X, u16* Y, u32 rows, u32 cols, u32 tokens) {                                   \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gC, gS, nullptr}, {uC, uS, nullptr}};                           \
        EpiSignedSwiglu<ACT> epi{{}, Y, (int)rows};                                               \
        mm1_body<M1Ter2<ACT>, ACT, F16, 2, NLV, EpiSignedSwiglu<ACT>, 0, 2>(mats, X, rows, cols, cols / 4, 128, \
                                                                            epi, NormScale{}, (int)tokens); \
    }

// Affine 4-bit: argument lists of the vector-ALU kernels of the same pipelines.
#define SMELT_AFFINE_MM1_KERNELS(T, ACT, SC, NLV)                                            \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_matvec_##T(                         \
        const u8* W, const u16* S, const u16* B, const u16* X, u16* Y, u32 rows, u32 cols,        \
        u32 group) {                                                                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        mm1_body<M1U4<ACT>, ACT, SC, 1, NLV>(mats, X, rows, cols, cols / 2, group, epi);     \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_matvec_add_##T(                     \
        const u8* W, const u16* S, const u16* B, const u16* X, u16* Y, const u16* res, u32 rows,  \
        u32 cols, u32 group) {                                                                    \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                   \
        mm1_body<M1U4<ACT>, ACT, SC, 1, NLV>(mats, X, rows, cols, cols / 2, group, epi);     \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_gate_up_swiglu_##T(                 \
        const u8* gW, const u16* gS, const u16* gB, const u8* uW, const u16* uS, const u16* uB,   \
        const u16* X, u16* Y, u32 rows, u32 cols, u32 group) {                                    \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiAffineSwiglu<ACT> epi{{}, Y, (int)rows};                                               \
        mm1_body<M1U4<ACT>, ACT, SC, 2, NLV>(mats, X, rows, cols, cols / 2, group, epi);     \
    }

#define SMELT_AFFINE_MM1_BANK(T, ACT, SC, NLV)                                                    \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_bank4_matvec_##T(                            \
        const u8* W, const u16* S, const u16* B, const u16* X, u16* y0, u16* y1, u16* y2,         \
        u16* y3, u32 rows0, u32 rows1, u32 rows2, u32 rows3, u32 cols, u32 group) {               \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiBank4<ACT> epi{{}, {y0, y1, y2, y3}, {rows0, rows1, rows2, rows3}};                    \
        mm1_body<M1U4<ACT>, ACT, SC, 1, NLV>(mats, X, rows0 + rows1 + rows2 + rows3, cols,        \
                                             cols / 2, group, epi);                               \
    }

// The other fused affine forms of the vector-ALU kernels, same argument lists: two projections of one
// input, GeGLU, and the norm-scale prologue in front of a projection, a pair or a gate+up.
#define SMELT_AFFINE_MM1_FUSED(T, ACT, SC, NLV)                                                   \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_dual_matvec_##T(                             \
        const u8* W1, const u16* S1, const u16* B1, const u8* W2, const u16* S2, const u16* B2,   \
        const u16* X, u16* y1, u16* y2, u32 rows, u32 cols, u32 group) {                          \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{W1, S1, B1}, {W2, S2, B2}};                                     \
        EpiDual<ACT> epi{{}, y1, y2, (int)rows};                                                  \
        mm1_body<M1U4<ACT>, ACT, SC, 2, NLV>(mats, X, rows, cols, cols / 2, group, epi);          \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_dual_matvec_add_##T(                         \
        const u8* W1, const u16* S1, const u16* B1, const u8* W2, const u16* S2, const u16* B2,   \
        const u16* X, u16* y1, u16* y2, const u16* r1, const u16* r2, u32 rows, u32 cols,         \
        u32 group) {                                                                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{W1, S1, B1}, {W2, S2, B2}};                                     \
        EpiDualAdd<ACT> epi{{}, y1, y2, r1, r2, (int)rows};                                       \
        mm1_body<M1U4<ACT>, ACT, SC, 2, NLV>(mats, X, rows, cols, cols / 2, group, epi);          \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_gate_up_geglu_##T(                           \
        const u8* gW, const u16* gS, const u16* gB, const u8* uW, const u16* uS, const u16* uB,   \
        const u16* X, u16* Y, u32 rows, u32 cols, u32 group) {                                    \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiGeglu<ACT> epi{{}, Y, (int)rows};                                                      \
        mm1_body<M1U4<ACT>, ACT, SC, 2, NLV>(mats, X, rows, cols, cols / 2, group, epi);          \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_norm_scale_matvec_##T(                       \
        const float* rs, const u16* X, const u16* nw, u16* xn, const u8* W, const u16* S,         \
        const u16* B, u16* Y, u32 rows, u32 cols, u32 group) {                                    \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        mm1_body<M1U4<ACT>, ACT, SC, 1, NLV, EpiStore<ACT>, 1>(mats, X, rows, cols, cols / 2, group, epi, \
                                                               NormScale{rs, nw, xn});            \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_norm_add_scale_matvec_##T(                   \
        const float* rs, const u16* X, const u16* nw, const u16* res, u16* xn, const u8* W,       \
        const u16* S, const u16* B, u16* Y, u32 rows, u32 cols, u32 group) {                      \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        mm1_body<M1U4<ACT>, ACT, SC, 1, NLV, EpiStore<ACT>, 2>(mats, X, rows, cols, cols / 2, group, epi, \
                                                               NormScale{rs, nw, xn, res});       \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_norm_scale_dual_matvec_##T(                  \
        const float* rs, const u16* X, const u16* nw, const u8* W1, const u16* S1, const u16* B1, \
        const u8* W2, const u16* S2, const u16* B2, u16* y1, u16* y2, u32 rows, u32 cols,         \
        u32 group) {                                                                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{W1, S1, B1}, {W2, S2, B2}};                                     \
        EpiDual<ACT> epi{{}, y1, y2, (int)rows};                                                  \
        mm1_body<M1U4<ACT>, ACT, SC, 2, NLV, EpiDual<ACT>, 1>(mats, X, rows, cols, cols / 2, group, epi, \
                                                              NormScale{rs, nw, nullptr});        \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_norm_scale_gate_up_swiglu_##T(               \
        const float* rs, const u16* X, const u16* nw, const u8* gW, const u16* gS, const u16* gB, \
        const u8* uW, const u16* uS, const u16* uB, u16* Y, u32 rows, u32 cols, u32 group) {      \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiAffineSwiglu<ACT> epi{{}, Y, (int)rows};                                               \
        mm1_body<M1U4<ACT>, ACT, SC, 2, NLV, EpiAffineSwiglu<ACT>, 1>(mats, X, rows, cols, cols / 2, group, \
                                                                      epi, NormScale{rs, nw, nullptr}); \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_norm_scale_gate_up_geglu_##T(                \
        const float* rs, const u16* X, const u16* nw, const u8* gW, const u16* gS, const u16* gB, \
        const u8* uW, const u16* uS, const u16* uB, u16* Y, u32 rows, u32 cols, u32 group) {      \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiGeglu<ACT> epi{{}, Y, (int)rows};                                                      \
        mm1_body<M1U4<ACT>, ACT, SC, 2, NLV, EpiGeglu<ACT>, 1>(mats, X, rows, cols, cols / 2, group, epi, \
                                                               NormScale{rs, nw, nullptr});       \
    }

// lm_head: one launch, one token per grid row; the workspace holds a key per tile and a counter per partial.
#define SMELT_AFFINE_MM1_ARGMAX(T, ACT, SC, NLV)                                                  \
    SMELT_MM1_KERNEL void smelt_affine_mm1_nl##NLV##_matvec_argmax_##T(                           \
        const u8* W, const u16* S, const u16* B, const u16* X, smelt::uint2_t* keys,              \
        unsigned long long* tile_keys, u32* counters, u32 rows, u32 cols, u32 group,              \
        u32 num_partials, float logit_cap) {                                                      \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiTileArgmax<ACT> epi{{}, keys, tile_keys, counters, num_partials, logit_cap};           \
        mm1_body<M1U4<ACT>, ACT, SC, 1, NLV>(mats, X, rows, cols, cols / 2, group, epi);          \
    }

// Ternary "affine" pipelines bind the scale plane a second time where MLX binds a bias plane; it
// is ignored as in the vector-ALU kernels.
#define SMELT_TERAFF_MM1_KERNELS(T, ACT, NLV)                                                     \
    SMELT_MM1_KERNEL void smelt_teraff_mm1_nl##NLV##_matvec_##T(                                  \
        const u8* C, const u16* S, const u16*, const u16* X, u16* Y, u32 rows, u32 cols) {        \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        mm1_body<M1Ter2<ACT>, ACT, F16, 1, NLV>(mats, X, rows, cols, cols / 4, 128, epi);         \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_teraff_mm1_nl##NLV##_matvec_add_##T(                              \
        const u8* C, const u16* S, const u16*, const u16* X, u16* Y, const u16* res, u32 rows,    \
        u32 cols) {                                                                               \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                   \
        mm1_body<M1Ter2<ACT>, ACT, F16, 1, NLV>(mats, X, rows, cols, cols / 4, 128, epi);         \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_teraff_mm1_nl##NLV##_gate_up_swiglu_##T(                          \
        const u8* gC, const u16* gS, const u16*, const u8* uC, const u16* uS, const u16*,         \
        const u16* X, u16* Y, u32 rows, u32 cols) {                                               \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gC, gS, nullptr}, {uC, uS, nullptr}};                           \
        EpiSignedSwiglu<ACT> epi{{}, Y, (int)rows};                                               \
        mm1_body<M1Ter2<ACT>, ACT, F16, 2, NLV>(mats, X, rows, cols, cols / 4, 128, epi);         \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_teraff_mm1_nl##NLV##_bank4_matvec_##T(                            \
        const u8* C, const u16* S, const u16*, const u16* X, u16* y0, u16* y1, u16* y2, u16* y3,  \
        u32 rows0, u32 rows1, u32 rows2, u32 rows3, u32 cols) {                                   \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiBank4<ACT> epi{{}, {y0, y1, y2, y3}, {rows0, rows1, rows2, rows3}};                    \
        mm1_body<M1Ter2<ACT>, ACT, F16, 1, NLV>(mats, X, rows0 + rows1 + rows2 + rows3, cols,     \
                                                cols / 4, 128, epi);                              \
    }

#define SMELT_BINARY_MM1_BANKS(T, ACT, NLV)                                                       \
    SMELT_MM1_KERNEL void smelt_signed_binary_mm1_nl##NLV##_packed_bank_matvec_##T(               \
        const u8* C, const u16* S, const u16* X, u16* y0, u16* y1, u32 rows0, u32 rows1,          \
        u32 cols) {                                                                               \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiBank4<ACT> epi{{}, {y0, y1, nullptr, nullptr}, {rows0, rows1, 0u, 0u}};                \
        mm1_body<M1Bin<ACT>, ACT, F16, 1, NLV>(mats, X, rows0 + rows1, cols, cols / 8, 128, epi); \
    }                                                                                             \
    SMELT_MM1_KERNEL void smelt_signed_binary_mm1_nl##NLV##_packed_bank4_matvec_##T(              \
        const u8* C, const u16* S, const u16* X, u16* y0, u16* y1, u16* y2, u16* y3, u32 rows0,   \
        u32 rows1, u32 rows2, u32 rows3, u32 cols) {                                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiBank4<ACT> epi{{}, {y0, y1, y2, y3}, {rows0, rows1, rows2, rows3}};                    \
        mm1_body<M1Bin<ACT>, ACT, F16, 1, NLV>(mats, X, rows0 + rows1 + rows2 + rows3, cols,      \
                                               cols / 8, 128, epi);                               \
    }


#define SMELT_TRIT5_MM1_BANK(T, ACT, NLV)                                                         \
    SMELT_MM1_KERNEL void smelt_signed_trit5_mm1_nl##NLV##_packed_bank4_matvec_##T(               \
        const u8* C, const u16* S, const u16* X, u16* y0, u16* y1, u16* y2, u16* y3, u32 rows0,   \
        u32 rows1, u32 rows2, u32 rows3, u32 cols) {                                              \
        using namespace smelt;                                                                    \
        using F = M1Trit5<ACT>;                                                                   \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiBank4<ACT> epi{{}, {y0, y1, y2, y3}, {rows0, rows1, rows2, rows3}};                    \
        mm1_body<F, ACT, F16, 1, NLV>(mats, X, rows0 + rows1 + rows2 + rows3, cols,               \
                                      F::row_stride((int)cols), 128, epi);                        \
    }
