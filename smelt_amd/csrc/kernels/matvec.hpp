// Batch-1 / small-batch quantized matvec for gfx950 (wave64).
//
// y[b, r] = sum_c w(r, c) * x[b, c]   with w dequantised from packed codes and per-group scales.
//
// Shape of the computation
//   * A "unit" is 16 bytes of one row's packed codes (one 128-bit load per lane): 32 affine-u4
//     columns, 64 ternary2 columns or 128 binary1 columns.
//   * A wave owns R rows (x S rows side by side when a row is shorter than 64 units); lane l
//     walks units l, l+L, ... of each of its rows, so every load instruction of the wave reads
//     one contiguous run of a row.
//   * The activation vector is staged once per workgroup into LDS as fp16 *pairs* laid out to
//     match the bit positions the codes occupy, so codes are turned into fp16 operands with one
//     AND-OR each and multiplied two at a time by v_dot2c_f32_f16 (fp32 accumulate):
//         ((dword >> s) & mask) | magic  ==  half2(base + code_a, base + code_b)
//     The row-independent term  sum base * x  is computed at staging time and subtracted from
//     each unit's dot product before the group scale is applied.
//   * Per-row partial sums are reduced across the L lanes of a row with DPP adds.
#pragma once
#include "common.hpp"

namespace smelt {

// (code & mask) | magic in one full-rate instruction (v_bitop3_b32, truth table 0xEA).
__device__ __forceinline__ uint32_t and_or(uint32_t c, uint32_t mask, uint32_t magic) {
    return __builtin_amdgcn_bitop3_b32(c, mask, magic, 0xEA);
}

// ---------------------------------------------------------------------------------------
// Format traits. dot() consumes one dword of codes and kPairsPerDword fp16 pairs of x
// (pair i = columns (i, i + kPairsPerDword) of that dword's column run).
// pair_offset(i) = base_i + kSemShift, the constant folded out of pair i.
// The semantic weight is kSemMul * (code + pair terms - offset) * scale.
// ---------------------------------------------------------------------------------------
struct FmtU4 {
    static constexpr bool kBitplanes = false;
    static constexpr int kDwordsPerUnit = 4;
    static constexpr bool kPerDwordScale = false;
    static constexpr int kBitsPerCode = 4;
    static constexpr int kPairsPerDword = 4;
    static constexpr bool kHasBias = true;
    static constexpr float kSemMul = 1.0f;
    static __device__ __forceinline__ float pair_offset(int i) { return (i & 1) ? 64.0f : 1024.0f; }
    static __device__ __forceinline__ float dot(uint32_t c, const uint32_t* xp, float acc) {
        const uint32_t c8 = c >> 8;
        acc = dot2(and_or(c, 0x000F000Fu, 0x64006400u), xp[0], acc);   // nibbles 0,4 -> 1024+n
        acc = dot2(and_or(c, 0x00F000F0u, 0x54005400u), xp[1], acc);   // nibbles 1,5 -> 64+n
        acc = dot2(and_or(c8, 0x000F000Fu, 0x64006400u), xp[2], acc);  // nibbles 2,6
        acc = dot2(and_or(c8, 0x00F000F0u, 0x54005400u), xp[3], acc);  // nibbles 3,7
        return acc;
    }
};

struct FmtTer2 {
    static constexpr bool kBitplanes = false;
    static constexpr int kDwordsPerUnit = 4;
    static constexpr bool kPerDwordScale = false;
    static constexpr int kBitsPerCode = 2;
    static constexpr int kPairsPerDword = 8;
    static constexpr bool kHasBias = false;
    static constexpr float kSemMul = 1.0f;
    // semantic = code - 1; codes sit at mantissa bits 4, 6 or 8 -> bases 64, 16, 4
    static __device__ __forceinline__ float pair_offset(int i) {
        const int k = i % 3;
        return (k == 0 ? 64.0f : (k == 1 ? 16.0f : 4.0f)) + 1.0f;
    }
    static __device__ __forceinline__ float dot(uint32_t c, const uint32_t* xp, float acc) {
        const uint32_t a = c << 4, b = c >> 2, d = c >> 8;
        acc = dot2(and_or(a, 0x00300030u, 0x54005400u), xp[0], acc);
        acc = dot2(and_or(a, 0x00C000C0u, 0x4C004C00u), xp[1], acc);
        acc = dot2(and_or(a, 0x03000300u, 0x44004400u), xp[2], acc);
        acc = dot2(and_or(b, 0x00300030u, 0x54005400u), xp[3], acc);
        acc = dot2(and_or(b, 0x00C000C0u, 0x4C004C00u), xp[4], acc);
        acc = dot2(and_or(b, 0x03000300u, 0x44004400u), xp[5], acc);
        acc = dot2(and_or(d, 0x00300030u, 0x54005400u), xp[6], acc);
        acc = dot2(and_or(d, 0x00C000C0u, 0x4C004C00u), xp[7], acc);
        return acc;
    }
};

struct FmtBin {
    static constexpr bool kBitplanes = false;
    static constexpr int kDwordsPerUnit = 4;
    static constexpr bool kPerDwordScale = false;
    static constexpr int kBitsPerCode = 1;
    static constexpr int kPairsPerDword = 16;
    static constexpr bool kHasBias = false;
    static constexpr float kSemMul = 2.0f;
    // semantic = 2*bit - 1 = 2*(bit - 0.5); bits sit at mantissa bits 4..9 -> bases 64..2
    static __device__ __forceinline__ float pair_offset(int i) {
        const int k = i % 6;
        return (float)(64 >> k) + 0.5f;
    }
    static __device__ __forceinline__ float dot(uint32_t c, const uint32_t* xp, float acc) {
        const uint32_t a = c << 4, b = c >> 2, d = c >> 8;
        acc = dot2(and_or(a, 0x00100010u, 0x54005400u), xp[0], acc);
        acc = dot2(and_or(a, 0x00200020u, 0x50005000u), xp[1], acc);
        acc = dot2(and_or(a, 0x00400040u, 0x4C004C00u), xp[2], acc);
        acc = dot2(and_or(a, 0x00800080u, 0x48004800u), xp[3], acc);
        acc = dot2(and_or(a, 0x01000100u, 0x44004400u), xp[4], acc);
        acc = dot2(and_or(a, 0x02000200u, 0x40004000u), xp[5], acc);
        acc = dot2(and_or(b, 0x00100010u, 0x54005400u), xp[6], acc);
        acc = dot2(and_or(b, 0x00200020u, 0x50005000u), xp[7], acc);
        acc = dot2(and_or(b, 0x00400040u, 0x4C004C00u), xp[8], acc);
        acc = dot2(and_or(b, 0x00800080u, 0x48004800u), xp[9], acc);
        acc = dot2(and_or(b, 0x01000100u, 0x44004400u), xp[10], acc);
        acc = dot2(and_or(b, 0x02000200u, 0x40004000u), xp[11], acc);
        acc = dot2(and_or(d, 0x00100010u, 0x54005400u), xp[12], acc);
        acc = dot2(and_or(d, 0x00200020u, 0x50005000u), xp[13], acc);
        acc = dot2(and_or(d, 0x00400040u, 0x4C004C00u), xp[14], acc);
        acc = dot2(and_or(d, 0x00800080u, 0x48004800u), xp[15], acc);
        return acc;
    }
};

// trit5: five base-3 digits per byte, decoded through a 243-entry table into the ternary2 bit
// layout.  A 16-byte unit holds 80 columns = five 16-column dwords; a dword never straddles a
// 128-column scale group, a unit can, so the scale is applied per dword.
struct FmtTrit5 {
    static constexpr bool kBitplanes = false;
    static constexpr int kDwordsPerUnit = 5;
    static constexpr bool kPerDwordScale = true;
    static constexpr int kBitsPerCode = 2;
    static constexpr int kPairsPerDword = 8;
    static constexpr bool kHasBias = false;
    static constexpr float kSemMul = 1.0f;
    static __device__ __forceinline__ float pair_offset(int i) { return FmtTer2::pair_offset(i); }
    static __device__ __forceinline__ float dot(uint32_t c, const uint32_t* xp, float acc) {
        return FmtTer2::dot(c, xp, acc);
    }
    static __device__ __forceinline__ void decode(const uint4_t& raw, const uint16_t* lut, uint32_t (&dw)[5]) {
        uint32_t f[16];
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int k = 0; k < 16; ++k) f[k] = lut[(w[k >> 2] >> (8 * (k & 3))) & 0xFFu];
        dw[0] = f[0] | (f[1] << 10) | (f[2] << 20) | (f[3] << 30);
        dw[1] = (f[3] >> 2) | (f[4] << 8) | (f[5] << 18) | (f[6] << 28);
        dw[2] = (f[6] >> 4) | (f[7] << 6) | (f[8] << 16) | (f[9] << 26);
        dw[3] = (f[9] >> 6) | (f[10] << 4) | (f[11] << 14) | (f[12] << 24);
        dw[4] = (f[12] >> 8) | (f[13] << 2) | (f[14] << 12) | (f[15] << 22);
    }
};

// Signed activation views (signed_quant.metal:746-755): the activations of a 128-column group
// arrive as a 16-bit scale and sign-magnitude integers stored as bit planes (plane p < P-1 = bit p of
// |q|, plane P-1 = sign; word w, bit l = column 32 w + l).  A unit's dot product is then integer:
//     sum_p 2^p * (2 * popcount(agree & plane_p) - popcount(nonzero & plane_p))
// with `agree` the columns where weight and activation signs give a positive product.  Codes keep
// the binary1 / ternary2 layouts and geometry; only staging and the per-unit arithmetic differ.
struct FmtBinPlanes : FmtBin {
    static constexpr bool kBitplanes = true;
    static constexpr bool kTernaryPlanes = false;
};
struct FmtTerPlanes : FmtTer2 {
    static constexpr bool kBitplanes = true;
    static constexpr bool kTernaryPlanes = true;
};

// 16 bits -> the even bit positions of 32 (bit i -> bit 2 i)
__device__ __forceinline__ uint32_t spread16(uint32_t v) {
    v = (v | (v << 8)) & 0x00FF00FFu;
    v = (v | (v << 4)) & 0x0F0F0F0Fu;
    v = (v | (v << 2)) & 0x33333333u;
    v = (v | (v << 1)) & 0x55555555u;
    return v;
}

__device__ __forceinline__ int popcount128(const uint4_t& v) {
    return __builtin_popcount(v.x) + __builtin_popcount(v.y) + __builtin_popcount(v.z) + __builtin_popcount(v.w);
}

template <class F>
struct FmtGeom {
    static constexpr int kPPD = F::kPairsPerDword;
    static constexpr int kColsPerDword = 2 * kPPD;
    static constexpr int kDPU = F::kDwordsPerUnit;         // code dwords per 16-byte unit after decode
    static constexpr int kColsPerUnit = kDPU * kColsPerDword;
    static constexpr int kChunksPerDword = kPPD / 4;       // 16-byte LDS chunks (4 pairs each)
    static constexpr int kChunksPerUnit = kDPU * kChunksPerDword;
    static constexpr int kCorrStride = kDPU <= 4 ? 4 : 8;  // floats of per-dword corrections per unit
};

// LDS layout for one batch tile of MB activations over U units per row:
//   pairs : [MB][kChunksPerUnit][U] x 16 B   (chunk-major so consecutive lanes hit consecutive 16 B)
//   corr  : [MB][U][kCorrStride] floats (one per dword of the unit)
//   xsum  : [MB][U][kCorrStride] floats (affine only)
constexpr int kPlaneSlots = 8;   // 16-byte plane slots per token and unit for activation views (2..6 used)

template <class F>
__device__ __forceinline__ size_t lds_pairs_bytes(int U, int MB) {
    if constexpr (F::kBitplanes) return (size_t)MB * kPlaneSlots * U * 16;
    return (size_t)MB * FmtGeom<F>::kChunksPerUnit * U * 16;
}

// Stage x[b0 .. b0+nb) (nb <= MB, rows of `cols` elements of ActT) into LDS.
// Activation-view staging: plane p of unit u goes to lds_pairs[p * U + u] (binary: the group's four
// words; ternary: the unit's 64 columns spread to the even bits of four dwords, the layout of the
// 2-bit codes); lds_corr holds per unit the activation scale, the binary correction
// sum_p 2^p popcount(plane_p) and the plane count.
template <class F, class ActT, int MB>
__device__ __forceinline__ void stage_planes(const uint32_t* __restrict__ planes, const uint16_t* __restrict__ act_scales,
                                             int nplanes, int U, int b0, int nb, uint4_t* lds_pairs, float* lds_corr) {
    constexpr bool TER = F::kTernaryPlanes;
    constexpr int NCH = kPlaneSlots;
    const int groups = TER ? U / 2 : U;
    for (int item = threadIdx.x; item < MB * U * nplanes; item += blockDim.x) {
        const int b = item / (U * nplanes), rest = item - b * U * nplanes;
        const int u = rest / nplanes, p = rest - u * nplanes;
        uint4_t v = {0u, 0u, 0u, 0u};
        if (b < nb) {
            const uint32_t* src = planes + (size_t)(b0 + b) * groups * nplanes * 4;
            if constexpr (!TER) {
                v = *reinterpret_cast<const uint4_t*>(src + ((size_t)u * nplanes + p) * 4);
            } else {
                const uint2_t w = *reinterpret_cast<const uint2_t*>(src + ((size_t)(u >> 1) * nplanes + p) * 4 + 2 * (u & 1));
                v.x = spread16(w.x & 0xFFFFu); v.y = spread16(w.x >> 16);
                v.z = spread16(w.y & 0xFFFFu); v.w = spread16(w.y >> 16);
            }
        }
        lds_pairs[((size_t)b * NCH + p) * U + u] = v;
    }
    for (int item = threadIdx.x; item < MB * U; item += blockDim.x) {
        const int b = item / U, u = item - b * U;
        const int g = TER ? u >> 1 : u;
        int bias = 0;
        float scale = 0.0f;
        if (b < nb) {
            const uint32_t* src = planes + (size_t)(b0 + b) * groups * nplanes * 4;
            if constexpr (!TER) {
                for (int p = 0; p < nplanes - 1; ++p)
                    bias += popcount128(*reinterpret_cast<const uint4_t*>(src + ((size_t)g * nplanes + p) * 4)) << p;
            }
            scale = ActT::widen(act_scales[(size_t)(b0 + b) * groups + g]);
        }
        float4_t c;
        c.x = scale;
        c.y = __builtin_bit_cast(float, bias);
        c.z = __builtin_bit_cast(float, nplanes);
        c.w = 0.0f;
        *reinterpret_cast<float4_t*>(lds_corr + ((size_t)b * U + u) * 4) = c;
    }
}

template <class F, class ActT, int MB>
__device__ __forceinline__ void stage_activations(const uint16_t* __restrict__ x, int cols, int U,
                                                  int b0, int nb, uint4_t* lds_pairs,
                                                  float* lds_corr, float* lds_xsum,
                                                  const uint16_t* x2 = nullptr, int nplanes = 0,
                                                  const NormScale& ns = NormScale{}) {
    if constexpr (F::kBitplanes) {
        stage_planes<F, ActT, MB>(reinterpret_cast<const uint32_t*>(x), x2, nplanes, U, b0, nb, lds_pairs, lds_corr);
        return;
    }
    using G = FmtGeom<F>;
    constexpr int PPD = G::kPPD;
    constexpr int CPD = G::kColsPerDword;
    constexpr int DPU = G::kDPU;
    const int dwords = U * DPU;
    float self_rs = 0.0f;
    if (ns.self_eps >= 0.0f) {   // uniform over the workgroup; one token (b0) per launch
        __shared__ float wave_sums[4];
        self_rs = row_inv_rms<ActT>(x + (size_t)b0 * cols, (uint32_t)cols, ns.self_eps, wave_sums);
        if (ns.publish != nullptr && blockIdx.x == 0 && threadIdx.x == 0) {
            ns.publish[0] = self_rs;
            reinterpret_cast<uint32_t*>(ns.publish)[1] = 1u;
        }
    }
    for (int item = threadIdx.x; item < MB * dwords; item += blockDim.x) {
        const int b = item / dwords;
        const int D = item - b * dwords;
        const int u = D / DPU, d = D - u * DPU;
        const int col0 = D * CPD;
        uint16_t v[CPD];
        if (b < nb && col0 + CPD <= cols) {
            const uint4_t* src = reinterpret_cast<const uint4_t*>(x + (size_t)(b0 + b) * cols + col0);
#pragma unroll
            for (int q = 0; q < CPD / 8; ++q) {
                uint4_t t = src[q];
                v[8 * q + 0] = (uint16_t)(t.x & 0xFFFF); v[8 * q + 1] = (uint16_t)(t.x >> 16);
                v[8 * q + 2] = (uint16_t)(t.y & 0xFFFF); v[8 * q + 3] = (uint16_t)(t.y >> 16);
                v[8 * q + 4] = (uint16_t)(t.z & 0xFFFF); v[8 * q + 5] = (uint16_t)(t.z >> 16);
                v[8 * q + 6] = (uint16_t)(t.w & 0xFFFF); v[8 * q + 7] = (uint16_t)(t.w >> 16);
            }
        } else {
#pragma unroll
            for (int i = 0; i < CPD; ++i) {
                const int c = col0 + i;
                v[i] = (b < nb && c < cols) ? x[(size_t)(b0 + b) * cols + c] : (uint16_t)0;
            }
        }
        if ((ns.rs != nullptr || ns.self_eps >= 0.0f) && b < nb) {
            const float rs = ns.self_eps >= 0.0f ? self_rs : ns.rs[b0 + b];
#pragma unroll
            for (int i = 0; i < CPD; ++i) {
                const int c = col0 + i;
                if (c < cols) {
                    v[i] = norm_scale_element<ActT>(ns, v[i], rs, (size_t)(b0 + b) * cols, c);
                    if (ns.out != nullptr && blockIdx.x == 0) ns.out[(size_t)(b0 + b) * cols + c] = v[i];
                }
            }
        }
        float corr = 0.0f, xsum = 0.0f;
        uint32_t pairs[PPD];
#pragma unroll
        for (int i = 0; i < PPD; ++i) {
            const uint16_t lo = ActT::to_f16_bits(v[i]);
            const uint16_t hi = ActT::to_f16_bits(v[i + PPD]);
            pairs[i] = (uint32_t)lo | ((uint32_t)hi << 16);
            const float s = F16::widen(lo) + F16::widen(hi);
            corr += F::pair_offset(i) * s;
            xsum += s;
        }
#pragma unroll
        for (int j = 0; j < G::kChunksPerDword; ++j) {
            uint4_t ch;
            ch.x = pairs[4 * j + 0]; ch.y = pairs[4 * j + 1];
            ch.z = pairs[4 * j + 2]; ch.w = pairs[4 * j + 3];
            lds_pairs[((size_t)b * G::kChunksPerUnit + d * G::kChunksPerDword + j) * U + u] = ch;
        }
        lds_corr[((size_t)b * U + u) * G::kCorrStride + d] = corr;
        if (F::kHasBias) lds_xsum[((size_t)b * U + u) * G::kCorrStride + d] = xsum;
    }
}

// One weight matrix as seen by the core.
struct MatPtrs {
    const uint8_t* codes;
    const uint16_t* scales;
    const uint16_t* biases;  // affine only
    // Optional second physical matrix that continues the row space at row `split` (two projections
    // driven as one matvec without moving their weights); split == 0 means there is none.
    const uint8_t* codes_hi = nullptr;
    const uint16_t* scales_hi = nullptr;
    int split = 0;
};

// Registers of one work item: the 16-byte unit `u` of R rows of NMAT matrices plus the group
// scale (and bias) each of them needs.
template <int R, int NMAT>
struct ItemRegs {
    uint4_t c[NMAT][R];
    uint16_t s[NMAT][R];
    uint16_t b[NMAT][R];   // affine bias; for per-dword-scale formats the next group's scale
    uint16_t res[R];       // epilogue operand fetched ahead with a row's last item (when the epilogue asks)
};

// Byte offsets of the R rows a lane owns inside a tile: codes and 16-bit scales.  They do not
// change from tile to tile, so the row * stride products are formed once per launch.
template <int R>
struct LaneRows {
    int rin0;               // first of the lane's rows within a tile
    uint32_t code[R];       // (rin0 + r) * row_stride
    uint32_t scale[R];      // (rin0 + r) * groups_per_row * 2
    __device__ __forceinline__ LaneRows(int first_row, int row_stride, int groups_per_row) : rin0(first_row) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            code[r] = (uint32_t)(first_row + r) * (uint32_t)row_stride;
            scale[r] = (uint32_t)(first_row + r) * (uint32_t)groups_per_row * 2u;
        }
    }
};

// Loads unit `u` of the R rows this lane owns in the tile that starts at row `row0`, clamped to
// the matrix in the last (partial) tile (clamped rows are computed, never stored).  row0 is
// uniform over the wave, so every address is a scalar tile base plus a 32-bit lane offset and the
// per-item address arithmetic stays off the vector ALU.
template <class F, int R, int NMAT>
__device__ __forceinline__ void load_item(const MatPtrs (&mats)[NMAT], int row0, int tile_rows, int rows,
                                          const LaneRows<R>& lr, int u, int row_stride,
                                          int groups_per_row, int gshift, ItemRegs<R, NMAT>& it) {
    const int g = (u * FmtGeom<F>::kColsPerUnit) >> gshift;
    const int g_next = g + 1 < groups_per_row ? g + 1 : g;
    const int last = rows - 1 - row0;
    const int max_rin = last < tile_rows - 1 ? last : tile_rows - 1;   // uniform
    const uint32_t max_code = (uint32_t)max_rin * (uint32_t)row_stride;
    const uint32_t max_scale = (uint32_t)max_rin * (uint32_t)groups_per_row * 2u;
    auto at = [](const uint16_t* base, uint32_t byte_off) {
        return reinterpret_cast<const uint16_t*>(reinterpret_cast<const uint8_t*>(base) + byte_off);
    };
#pragma unroll
    for (int m = 0; m < NMAT; ++m) {
        const uint8_t* codes = mats[m].codes;
        const uint16_t* scales = mats[m].scales;
        int base_row = row0;
        const int split = mats[m].split;
        if (split > 0 && row0 < split && row0 + tile_rows > split) {
            // the tile straddles the seam of a two-segment matrix: per-lane segment choice
#pragma unroll
            for (int r = 0; r < R; ++r) {
                int rr = row0 + (lr.rin0 + r < max_rin ? lr.rin0 + r : max_rin);
                const bool hi = rr >= split;
                const uint8_t* cb = hi ? mats[m].codes_hi : codes;
                const uint16_t* sb = hi ? mats[m].scales_hi : scales;
                if (hi) rr -= split;
                it.c[m][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(cb + (size_t)rr * row_stride + (size_t)u * 16));
                const size_t si = (size_t)rr * groups_per_row;
                it.s[m][r] = __builtin_nontemporal_load(sb + si + g);
                if (F::kHasBias) it.b[m][r] = __builtin_nontemporal_load(mats[m].biases + si + g);
                else if (F::kPerDwordScale) it.b[m][r] = __builtin_nontemporal_load(sb + si + g_next);
                else it.b[m][r] = 0;
            }
            continue;
        }
        if (split > 0 && row0 >= split) {
            codes = mats[m].codes_hi;
            scales = mats[m].scales_hi;
            base_row = row0 - split;
        }
        // weights are read once per launch: the streaming hint keeps them from displacing the
        // activations and the residual in the caches
        const uint8_t* tile_codes = codes + (size_t)base_row * row_stride;
        const uint16_t* tile_scales = scales + (size_t)base_row * groups_per_row;
        const uint16_t* tile_biases = F::kHasBias ? mats[m].biases + (size_t)base_row * groups_per_row : nullptr;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t code_off = (lr.code[r] < max_code ? lr.code[r] : max_code) + (uint32_t)u * 16u;
            const uint32_t scale_off = (lr.scale[r] < max_scale ? lr.scale[r] : max_scale) + (uint32_t)g * 2u;
            it.c[m][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(tile_codes + code_off));
            it.s[m][r] = __builtin_nontemporal_load(at(tile_scales, scale_off));
            if (F::kHasBias) it.b[m][r] = __builtin_nontemporal_load(at(tile_biases, scale_off));
            else if (F::kPerDwordScale) it.b[m][r] = __builtin_nontemporal_load(at(tile_scales, scale_off + (uint32_t)(g_next - g) * 2u));
            else it.b[m][r] = 0;
        }
    }
}

// The activation side of one unit for one token: the fp16 pairs, the folded-out constant and the
// plain sum of x (what a bias multiplies).  For a matrix whose rows fit one pass of the wave the
// unit of a lane never changes, so these registers are filled once per launch.
template <class F>
struct XUnit {
    using G = FmtGeom<F>;
    uint32_t xp[G::kChunksPerUnit * 4];
    float cr[G::kDPU];   // per dword (formats whose scale can change inside a unit)
    float corr;          // whole unit
    float xsum;
};

template <class F>
__device__ __forceinline__ void load_xunit(XUnit<F>& xu, int b, int u, int U, const uint4_t* lds_pairs,
                                           const float* lds_corr, const float* lds_xsum) {
    using G = FmtGeom<F>;
    constexpr int NCH = G::kChunksPerUnit;
    constexpr int DPU = G::kDPU;
#pragma unroll
    for (int q = 0; q < NCH; ++q) {
        const uint4_t t = lds_pairs[((size_t)b * NCH + q) * U + u];
        xu.xp[4 * q + 0] = t.x; xu.xp[4 * q + 1] = t.y; xu.xp[4 * q + 2] = t.z; xu.xp[4 * q + 3] = t.w;
    }
    const float4_t* c4 = reinterpret_cast<const float4_t*>(lds_corr + ((size_t)b * U + u) * G::kCorrStride);
    const float4_t lo = c4[0];
    xu.cr[0] = lo.x; xu.cr[1] = lo.y; xu.cr[2] = lo.z; xu.cr[3] = lo.w;
    if constexpr (DPU > 4) xu.cr[DPU - 1] = c4[1].x;
    xu.corr = (xu.cr[0] + xu.cr[1]) + (xu.cr[2] + xu.cr[3]);
    xu.xsum = 0.0f;
    if (F::kHasBias) {
        const float4_t xs = *reinterpret_cast<const float4_t*>(lds_xsum + ((size_t)b * U + u) * G::kCorrStride);
        xu.xsum = (xs.x + xs.y) + (xs.z + xs.w);
    }
}

// acc[m][r][b] += scale * (sum (base + code) * x  -  sum base * x) + bias * sum x   for unit u
template <class F, class ScaleT, int R, int MB, int NMAT>
__device__ __forceinline__ void compute_unit(const ItemRegs<R, NMAT>& it, const XUnit<F>& xu, int b, int u,
                                             int gshift, const uint16_t* lut, float (&acc)[NMAT][R][MB]) {
    using G = FmtGeom<F>;
    constexpr int DPU = G::kDPU;
    if constexpr (F::kPerDwordScale) {
        const int g0 = (u * G::kColsPerUnit) >> gshift;
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t dw[DPU];
                F::decode(it.c[m][r], lut, dw);
                const float s0 = F::kSemMul * ScaleT::widen(it.s[m][r]);
                const float s1 = F::kSemMul * ScaleT::widen(it.b[m][r]);
                float a = acc[m][r][b];
#pragma unroll
                for (int j = 0; j < DPU; ++j) {
                    const float d = F::dot(dw[j], xu.xp + j * G::kPPD, -xu.cr[j]);
                    const int gj = (u * G::kColsPerUnit + j * G::kColsPerDword) >> gshift;
                    a = __builtin_fmaf(gj == g0 ? s0 : s1, d, a);
                }
                acc[m][r][b] = a;
            }
    } else {
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float d = -xu.corr;
                d = F::dot(it.c[m][r].x, xu.xp + 0 * G::kPPD, d);
                d = F::dot(it.c[m][r].y, xu.xp + 1 * G::kPPD, d);
                d = F::dot(it.c[m][r].z, xu.xp + 2 * G::kPPD, d);
                d = F::dot(it.c[m][r].w, xu.xp + 3 * G::kPPD, d);
                float a = acc[m][r][b];
                if (F::kHasBias) a = __builtin_fmaf(ScaleT::widen(it.b[m][r]), xu.xsum, a);
                acc[m][r][b] = __builtin_fmaf(F::kSemMul * ScaleT::widen(it.s[m][r]), d, a);
            }
    }
}

// One work item against every token of the chunk.
template <class F, class ScaleT, int R, int MB, int NMAT>
__device__ __forceinline__ void compute_item(const ItemRegs<R, NMAT>& it, int u, int U, int gshift,
                                             const uint4_t* lds_pairs, const float* lds_corr,
                                             const float* lds_xsum, const uint16_t* lut,
                                             float (&acc)[NMAT][R][MB]) {
    if constexpr (F::kBitplanes) {
        constexpr int PCH = kPlaneSlots;
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const float4_t c4 = *reinterpret_cast<const float4_t*>(lds_corr + ((size_t)b * U + u) * 4);
            // (elements are copied out before the bit casts: a bit cast applied directly to a vector
            //  element reads the vector's first lane)
            const float act_scale = c4.x, bias_bits = c4.y, nplanes_bits = c4.z;
            const int bias = __builtin_bit_cast(int, bias_bits);
            const int nplanes = __builtin_bit_cast(int, nplanes_bits);
            const uint4_t* my_planes = lds_pairs + (size_t)b * PCH * U + u;
            const uint4_t sign = my_planes[(size_t)(nplanes - 1) * U];
            uint4_t agree[NMAT][R], nonzero[NMAT][R];
            int weighted[NMAT][R], active[NMAT][R];
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const uint4_t c = it.c[m][r];
                    if constexpr (!F::kTernaryPlanes) {
                        agree[m][r] = c ^ sign;          // weight +1 and activation >= 0, or -1 and < 0
                    } else {
                        const uint4_t even = {0x55555555u, 0x55555555u, 0x55555555u, 0x55555555u};
                        const uint4_t pos = (c >> 1) & even;   // code 2 = +1
                        nonzero[m][r] = ~c & even;             // code 1 = 0 has its low bit set
                        agree[m][r] = nonzero[m][r] & (pos ^ sign);
                    }
                    weighted[m][r] = 0;
                    active[m][r] = 0;
                }
            for (int p = 0; p < nplanes - 1; ++p) {
                const uint4_t plane = my_planes[(size_t)p * U];
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        weighted[m][r] += popcount128(agree[m][r] & plane) << p;
                        if constexpr (F::kTernaryPlanes) active[m][r] += popcount128(nonzero[m][r] & plane) << p;
                    }
            }
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const int dot = 2 * weighted[m][r] - (F::kTernaryPlanes ? active[m][r] : bias);
                    acc[m][r][b] = __builtin_fmaf((float)dot * act_scale, ScaleT::widen(it.s[m][r]), acc[m][r][b]);
                }
        }
        return;
    }
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        XUnit<F> xu;
        load_xunit<F>(xu, b, u, U, lds_pairs, lds_corr, lds_xsum);
        compute_unit<F, ScaleT, R, MB, NMAT>(it, xu, b, u, gshift, lut, acc);
    }
}

}  // namespace smelt
