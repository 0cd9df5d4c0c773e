// Matrix-core quantized matvec for gfx950: y[b, r] = sum_c w(r, c) * x[b, c] for up to 8 activation
// rows per pass, for matrices large enough that the packed weights stream from HBM.
//
// The vector-ALU matvec spends one AND-OR and one dot2 per pair of weights, which for binary and
// ternary codes (and, on long rows, 4-bit codes) is more issue time than the memory system needs
// to deliver them.  Here the multiply-accumulate and the cross-lane reduction move to
// v_mfma_f32_16x16x32_f16, leaving only the AND-OR operand formation on the vector ALU:
//   * A wave owns a tile of 32 weight rows.  MFMA lane (j = lane % 16, kb = lane / 16) supplies, as
//     the B operand, eight codes of row  j + 16 * (kb / 2)  taken from half  kb % 2  of a window
//     (one window = one scale group of one row, split in two halves).
//   * The MFMA contracts over all four kb, which would mix rows j and j + 16.  The A operand (the
//     activations) separates them: token slot i < 8 carries x only in k-slots kb < 2, slot i >= 8
//     only in kb >= 2, zero elsewhere.  Output D[i][j] is then row j for i < 8 and row j + 16 for
//     i >= 8: 32 rows x 8 tokens per instruction, one scale group per contraction.
//   * Codes enter the MFMA as (base + code) straight from the AND-OR; the row-independent
//     sum(base * x) per window and token is computed when the activations are staged and
//     subtracted before the group scale is applied in fp32.
//   * Packed codes go from global memory straight into a wave-private LDS ring (128-bit loads to
//     LDS), one item = 128 bytes of each of the tile's 32 rows, eight consecutive lanes per row
//     segment, so every load instruction reads whole cache lines whatever the MFMA lane layout
//     wants.  Lane l of load i lands in slot (row 8i + l/8, l%8) and fetches piece
//     (l%8) ^ f(row), f(row) = (row/2) % 8; the MFMA lane of row r finds piece q in slot q ^ f(r),
//     and the sixteen rows a 16-lane group reads fall in sixteen different bank groups.
//   * Activations are staged once per workgroup into LDS as fp16 operand fragments.
// K can be split over `kw` waves of a workgroup (partials meet in LDS); with kw = 1 every wave
// streams whole rows.
#pragma once
#include "matvec.hpp"

namespace smelt {

// ---- format traits: one packed dword -> kMPD MFMA B operands --------------------------------
// kCPD columns per dword, kDPL dwords an MFMA lane takes per window (the window is 2 * kDPL dwords
// of one row = one scale group).  col(m, q): column within the dword held by operand element q of
// MFMA m; base(m, q): what the AND-OR adds to that code, plus the offset of the semantic value.
struct MvU4 {
    using Valu = FmtU4;  // the vector-ALU format of the same bytes
    static constexpr int kCPD = 8, kMPD = 1, kDPL = 4;
    static constexpr bool kHasBias = true;
    static constexpr float kSemMul = 1.0f;
    static __device__ __forceinline__ constexpr int col(int, int q) { return (q >> 1) + 4 * (q & 1); }
    static __device__ __forceinline__ constexpr float base(int, int q) { return ((q >> 1) & 1) ? 64.0f : 1024.0f; }
    static __device__ __forceinline__ void operands(uint32_t c, uint4_t (&out)[kMPD]) {
        const uint32_t c8 = c >> 8;
        out[0].x = and_or(c, 0x000F000Fu, 0x64006400u);   // codes 0,4 -> 1024 + n
        out[0].y = and_or(c, 0x00F000F0u, 0x54005400u);   // codes 1,5 -> 64 + n
        out[0].z = and_or(c8, 0x000F000Fu, 0x64006400u);  // codes 2,6
        out[0].w = and_or(c8, 0x00F000F0u, 0x54005400u);  // codes 3,7
    }
};

struct MvTer2 {
    using Valu = FmtTer2;
    static constexpr int kCPD = 16, kMPD = 2, kDPL = 4;
    static constexpr bool kHasBias = false;
    static constexpr float kSemMul = 1.0f;
    // operand register v of MFMA m is pair p = 4m + v = codes (p, p + 8); semantic = code - 1
    static __device__ __forceinline__ constexpr int col(int m, int q) { return 4 * m + (q >> 1) + 8 * (q & 1); }
    static __device__ __forceinline__ constexpr float base(int m, int q) {
        const int p = 4 * m + (q >> 1), k = p % 3;
        return (k == 0 ? 64.0f : (k == 1 ? 16.0f : 4.0f)) + 1.0f;
    }
    static __device__ __forceinline__ void operands(uint32_t c, uint4_t (&out)[kMPD]) {
        const uint32_t a = c << 4, b = c >> 2, d = c >> 8;
        out[0].x = and_or(a, 0x00300030u, 0x54005400u);
        out[0].y = and_or(a, 0x00C000C0u, 0x4C004C00u);
        out[0].z = and_or(a, 0x03000300u, 0x44004400u);
        out[0].w = and_or(b, 0x00300030u, 0x54005400u);
        out[1].x = and_or(b, 0x00C000C0u, 0x4C004C00u);
        out[1].y = and_or(b, 0x03000300u, 0x44004400u);
        out[1].z = and_or(d, 0x00300030u, 0x54005400u);
        out[1].w = and_or(d, 0x00C000C0u, 0x4C004C00u);
    }
};

struct MvBin {
    using Valu = FmtBin;
    static constexpr int kCPD = 32, kMPD = 4, kDPL = 2;
    static constexpr bool kHasBias = false;
    static constexpr float kSemMul = 2.0f;
    // operand register v of MFMA m is pair p = 4m + v = bits (p, p + 16); semantic = 2 * (bit - 0.5)
    static __device__ __forceinline__ constexpr int col(int m, int q) { return 4 * m + (q >> 1) + 16 * (q & 1); }
    static __device__ __forceinline__ constexpr float base(int m, int q) {
        return (float)(64 >> ((4 * m + (q >> 1)) % 6)) + 0.5f;
    }
    static __device__ __forceinline__ void operands(uint32_t c, uint4_t (&out)[kMPD]) {
        const uint32_t a = c << 4, b = c >> 2, d = c >> 8;
        out[0].x = and_or(a, 0x00100010u, 0x54005400u);
        out[0].y = and_or(a, 0x00200020u, 0x50005000u);
        out[0].z = and_or(a, 0x00400040u, 0x4C004C00u);
        out[0].w = and_or(a, 0x00800080u, 0x48004800u);
        out[1].x = and_or(a, 0x01000100u, 0x44004400u);
        out[1].y = and_or(a, 0x02000200u, 0x40004000u);
        out[1].z = and_or(b, 0x00100010u, 0x54005400u);
        out[1].w = and_or(b, 0x00200020u, 0x50005000u);
        out[2].x = and_or(b, 0x00400040u, 0x4C004C00u);
        out[2].y = and_or(b, 0x00800080u, 0x48004800u);
        out[2].z = and_or(b, 0x01000100u, 0x44004400u);
        out[2].w = and_or(b, 0x02000200u, 0x40004000u);
        out[3].x = and_or(d, 0x00100010u, 0x54005400u);
        out[3].y = and_or(d, 0x00200020u, 0x50005000u);
        out[3].z = and_or(d, 0x00400040u, 0x4C004C00u);
        out[3].w = and_or(d, 0x00800080u, 0x48004800u);
    }
};

template <class F>
struct MvGeom {
    static constexpr int kLaneBytes = 4 * F::kDPL;                 // bytes an MFMA lane reads per window
    static constexpr int kWindowBytes = 2 * kLaneBytes;             // one row's bytes per window
    static constexpr int kWindowCols = 2 * F::kDPL * F::kCPD;       // == the scale group
    static constexpr int kWPI = 128 / kWindowBytes;                 // windows per ring item (128 bytes per row)
    static constexpr int kMPW = F::kDPL * F::kMPD;                  // MFMAs per window
    static constexpr int kFPW = 2 * kMPW;                           // activation fragments per window
    static constexpr int kItemCols = kWPI * kWindowCols;
};

// LDS bytes: fragments [windows][kFPW][tokens] x 16 B, one zero slot, per-window corrections (and
// activation sums) for 8 token slots, wave partials when K is split, then the code rings
// (two 4 KB items per wave and matrix), 1 KB aligned.
template <class F>
__host__ __device__ inline size_t mfma_matvec_lds_bytes(int cols, int token_shift, int nmat, int waves, int kw) {
    const size_t nwin = (size_t)cols / MvGeom<F>::kWindowCols;
    size_t bytes = ((nwin * MvGeom<F>::kFPW * 16) << token_shift) + 16;
    bytes += nwin * 32 * (F::kHasBias ? 2 : 1);
    if (kw > 1) bytes += (size_t)waves * nmat * 1024;
    return ((bytes + 1023) & ~(size_t)1023) + (size_t)waves * nmat * 2 * 4096;
}

__host__ __device__ inline int mfma_token_shift(int tokens) {
    int shift = 0;
    while ((1 << shift) < tokens && shift < 3) ++shift;
    return shift;
}

// scales (and biases) of the windows of one ring item: kWPI 16-bit values per matrix
template <class F, int NMAT>
struct MvScales {
    uint32_t s[NMAT][MvGeom<F>::kWPI / 2];
    uint32_t b[NMAT][MvGeom<F>::kWPI / 2];
};

// STREAM: kw == 1 (no cross-wave reduction, no barriers in the tile loop).
// ONE: the launch carries a single activation row (decode): only token slot 0 is formed and used.
template <class F, class ActT, class ScaleT, int NMAT, bool STREAM, bool ONE, class Epi>
__device__ __forceinline__ void mfma_matvec_body(const MatPtrs (&mats)[NMAT], const uint16_t* x, int rows,
                                                 int cols, int row_stride, int kw, int batch_lo,
                                                 int batch_hi, const Epi& epi) {
    using G = MvGeom<F>;
    constexpr int MPD = F::kMPD, CPD = F::kCPD, DPL = F::kDPL, FPW = G::kFPW, MPW = G::kMPW, WPI = G::kWPI;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave, nwaves = blockDim.x / kWave;
    const int lj = lane & 15, kb = lane >> 4, half = kb & 1, rsel = kb >> 1;
    const int nwin = cols / G::kWindowCols;  // == scale groups per row
    const int tiles = (rows + 31) / 32;
    const int span = batch_hi - batch_lo;
    const int tshift = ONE ? 0 : mfma_token_shift(span < 8 ? span : 8);
    const int tmask = (1 << tshift) - 1;

    uint4_t* frags = reinterpret_cast<uint4_t*>(smem);
    const size_t nfrag = ((size_t)nwin * FPW) << tshift;
    uint4_t* zero_slot = frags + nfrag;
    float* corr = reinterpret_cast<float*>(zero_slot + 1);     // [nwin][8]
    float* xsum = corr + (size_t)nwin * 8;                     // [nwin][8], affine only
    float* red = xsum + (F::kHasBias ? (size_t)nwin * 8 : 0);  // [nwaves][NMAT][8][32], kw > 1 only
    unsigned char* ring = smem +
                          (((size_t)(reinterpret_cast<unsigned char*>(red + (STREAM ? 0 : (size_t)nwaves * NMAT * 256)) - smem) + 1023) & ~(size_t)1023) +
                          (size_t)wave * NMAT * 2 * 4096;

    // A-operand lane (token slot i = lane % 16, kb): live where the slot's row half matches kb's
    const bool a_live = ((lj >> 3) == rsel) && ((lj & 7) <= tmask) && (!ONE || (lj & 7) == 0);
    const int a_tok = lj & 7;
    const int my_r = lj + 16 * rsel;  // row of the tile this lane feeds to the MFMA
    const int my_f = (my_r >> 1) & 7;

    const int tpw = nwaves / kw;      // tiles a workgroup covers per step
    const int sub = wave / kw, kwi = wave % kw;
    const int nbatch = nwin / WPI;    // ring items per row
    const int my_batches = kwi < nbatch ? (nbatch - kwi + kw - 1) / kw : 0;  // >= 1: the host checks nbatch >= kw

    uint4_t fr[MPW];  // activation fragments of the window in hand
#pragma unroll
    for (int k = 0; k < MPW; ++k) fr[k] = uint4_t{0u, 0u, 0u, 0u};

    // y[m][v] += scale * (sum (base + code) * x - sum base * x) + bias * sum x  over one ring item
    auto compute = [&](const MvScales<F, NMAT>& cur, int batch, int slot, float4_t (&y)[NMAT]) {
#pragma unroll
        for (int i = 0; i < WPI; ++i) {
            const int w = batch * WPI + i;
            // activation fragments: dead lanes hold zeros (ONE: registers that are never written;
            // otherwise a zero slot in LDS)
            if constexpr (ONE) {
                if (a_live) {
#pragma unroll
                    for (int k = 0; k < MPW; ++k) fr[k] = frags[(size_t)w * FPW + half + 2 * k];
                }
            } else {
                const uint4_t* fw = a_live ? frags + (((size_t)w * FPW + half) << tshift) + a_tok : zero_slot;
                const size_t fstep = a_live ? ((size_t)2 << tshift) : 0;
#pragma unroll
                for (int k = 0; k < MPW; ++k) fr[k] = fw[(size_t)k * fstep];
            }
            float4_t acc[NMAT];
#pragma unroll
            for (int m = 0; m < NMAT; ++m) acc[m] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
            // this lane's DPL dwords of window i: byte i * kWindowBytes + half * kLaneBytes of its row
            uint32_t cw[NMAT][DPL];
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const int off = i * G::kWindowBytes + half * G::kLaneBytes;
                const unsigned char* src = ring + (size_t)(slot * NMAT + m) * 4096 +
                                           ((size_t)my_r * 8 + ((off >> 4) ^ my_f)) * 16 + (off & 15);
                if constexpr (DPL == 4) {
                    const uint4_t v = *reinterpret_cast<const uint4_t*>(src);
                    cw[m][0] = v.x; cw[m][1] = v.y; cw[m][2] = v.z; cw[m][3] = v.w;
                } else {
                    const uint2_t v = *reinterpret_cast<const uint2_t*>(src);
                    cw[m][0] = v.x; cw[m][1] = v.y;
                }
            }
#pragma unroll
            for (int t = 0; t < DPL; ++t) {
                uint4_t ops[NMAT][MPD];
#pragma unroll
                for (int m = 0; m < NMAT; ++m) F::operands(cw[m][t], ops[m]);
#pragma unroll
                for (int q = 0; q < MPD; ++q) {
                    const half8_t xa = __builtin_bit_cast(half8_t, fr[t * MPD + q]);
#pragma unroll
                    for (int m = 0; m < NMAT; ++m)
                        acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa, __builtin_bit_cast(half8_t, ops[m][q]), acc[m], 0, 0, 0);
                }
            }
            // D lane (row j, ib = kb): tokens 4 * (kb % 2) + v of row half kb / 2
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const uint32_t sp = cur.s[m][i >> 1];
                const float sv = F::kSemMul * ScaleT::widen((uint16_t)((i & 1) ? sp >> 16 : sp & 0xFFFFu));
                float bv = 0.0f;
                if (F::kHasBias) {
                    const uint32_t bp = cur.b[m][i >> 1];
                    bv = ScaleT::widen((uint16_t)((i & 1) ? bp >> 16 : bp & 0xFFFFu));
                }
                if constexpr (ONE) {
                    y[m].x = __builtin_fmaf(sv, acc[m].x - corr[(size_t)w * 8], y[m].x);
                    if (F::kHasBias) y[m].x = __builtin_fmaf(bv, xsum[(size_t)w * 8], y[m].x);
                } else {
                    const float4_t cr = *reinterpret_cast<const float4_t*>(corr + (size_t)w * 8 + 4 * half);
                    y[m].x = __builtin_fmaf(sv, acc[m].x - cr.x, y[m].x);
                    y[m].y = __builtin_fmaf(sv, acc[m].y - cr.y, y[m].y);
                    y[m].z = __builtin_fmaf(sv, acc[m].z - cr.z, y[m].z);
                    y[m].w = __builtin_fmaf(sv, acc[m].w - cr.w, y[m].w);
                    if (F::kHasBias) {
                        const float4_t xs4 = *reinterpret_cast<const float4_t*>(xsum + (size_t)w * 8 + 4 * half);
                        y[m].x = __builtin_fmaf(bv, xs4.x, y[m].x);
                        y[m].y = __builtin_fmaf(bv, xs4.y, y[m].y);
                        y[m].z = __builtin_fmaf(bv, xs4.z, y[m].z);
                        y[m].w = __builtin_fmaf(bv, xs4.w, y[m].w);
                    }
                }
            }
        }
    };

    for (int b0 = batch_lo; b0 < batch_hi; b0 += 8) {
        const int nb = batch_hi - b0 < 8 ? batch_hi - b0 : 8;
        // ---- stage the activations of this chunk ----------------------------------------------
        // One item = one packed dword's worth of columns of one token: CPD consecutive columns are
        // converted to fp16 and written as the kMPD operand fragments that dword feeds; the
        // 2 * DPL items of a (token, window) sit in consecutive lanes and reduce their
        // sum(base * x) and sum(x) with DPP adds.
        if (b0 != batch_lo) __syncthreads();
        if (tid == 0) *zero_slot = uint4_t{0u, 0u, 0u, 0u};
        constexpr int EPW = 2 * DPL, ESHIFT = DPL == 4 ? 3 : 2;
        const int nitems = (nwin * EPW) << tshift;
        for (int base_i = 0; base_i < nitems; base_i += blockDim.x) {
            const int idx = base_i + tid;
            const int e = idx & (EPW - 1), tok = (idx >> ESHIFT) & tmask, w = idx >> (ESHIFT + tshift);
            const bool on = idx < nitems && tok < nb;
            uint16_t h[CPD];
#pragma unroll
            for (int q = 0; q < CPD / 8; ++q) {
                uint4_t v = {0u, 0u, 0u, 0u};
                if (on) v = *reinterpret_cast<const uint4_t*>(x + (size_t)(b0 + tok) * cols + ((size_t)w * EPW + e) * CPD + q * 8);
                const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    h[8 * q + 2 * k] = ActT::to_f16_bits((uint16_t)(d[k] & 0xFFFF));
                    h[8 * q + 2 * k + 1] = ActT::to_f16_bits((uint16_t)(d[k] >> 16));
                }
            }
            float cs = 0.0f, xs1 = 0.0f;
            const int hsel = e / DPL, t = e % DPL;  // dword t of lane half hsel
#pragma unroll
            for (int m = 0; m < MPD; ++m) {
                uint32_t o[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const uint16_t lo = h[F::col(m, 2 * v)], hi = h[F::col(m, 2 * v + 1)];
                    o[v] = (uint32_t)lo | ((uint32_t)hi << 16);
                    cs += F::base(m, 2 * v) * F16::widen(lo) + F::base(m, 2 * v + 1) * F16::widen(hi);
                    xs1 += F16::widen(lo) + F16::widen(hi);
                }
                if (on) frags[(((size_t)w * FPW + (t * MPD + m) * 2 + hsel) << tshift) + tok] = uint4_t{o[0], o[1], o[2], o[3]};
            }
            cs = group_sum_last<EPW>(cs);
            xs1 = group_sum_last<EPW>(xs1);
            if (e == EPW - 1 && idx < nitems) {
                corr[(size_t)w * 8 + tok] = cs;
                if (F::kHasBias) xsum[(size_t)w * 8 + tok] = xs1;
            }
        }
        __syncthreads();

        // ---- items: (tile step, batch) pairs of this wave, ring two deep ------------------------
        // STREAM: every wave walks its own tiles.  Otherwise the kw waves of a tile take batches
        // kwi, kwi + kw, ... and every wave of the workgroup walks the same number of tile steps
        // (a wave whose tile lies past the end computes clamped rows and stores nothing).
        int first_tile, tile_stride, steps;
        if (STREAM) {
            first_tile = blockIdx.x * nwaves + wave;
            tile_stride = gridDim.x * nwaves;
            steps = first_tile < tiles ? (tiles - first_tile + tile_stride - 1) / tile_stride : 0;
        } else {
            first_tile = blockIdx.x * tpw + sub;
            tile_stride = gridDim.x * tpw;
            const int wg_first = blockIdx.x * tpw;
            steps = wg_first < tiles ? (tiles - wg_first + tile_stride - 1) / tile_stride : 0;
        }
        const int per_tile = STREAM ? nbatch : my_batches;
        const int nq = steps * per_tile;
        MvScales<F, NMAT> regs_a, regs_b;
        int tile_c = first_tile, bat_c = 0, tile_n = first_tile, bat_n = 0;  // bat_*: index among this wave's batches
        auto fetch = [&](MvScales<F, NMAT>& dst, int slot) {
            __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): reads of this ring slot have returned
            const int batch = STREAM ? bat_n : kwi + bat_n * kw;
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int rt = 8 * i + (lane >> 3);
                    int row = tile_n * 32 + rt;
                    if (row >= rows) row = rows - 1;  // clamped rows are computed, never stored
                    const int piece = (lane & 7) ^ ((rt >> 1) & 7);
                    const uint8_t* src = mats[m].codes + (size_t)row * row_stride + (size_t)batch * 128 + piece * 16;
                    __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void*)(ring + ((size_t)(slot * NMAT + m) * 4 + i) * 1024), 16, 0, 0);
                }
                int row = tile_n * 32 + my_r;
                if (row >= rows) row = rows - 1;
                const uint16_t* sp = mats[m].scales + (size_t)row * nwin + batch * WPI;
                if constexpr (WPI == 4) {
                    const uint2_t v = *reinterpret_cast<const uint2_t*>(sp);
                    dst.s[m][0] = v.x; dst.s[m][1] = v.y;
                    if (F::kHasBias) {
                        const uint2_t u = *reinterpret_cast<const uint2_t*>(mats[m].biases + (size_t)row * nwin + batch * WPI);
                        dst.b[m][0] = u.x; dst.b[m][1] = u.y;
                    }
                } else {
                    const uint4_t v = *reinterpret_cast<const uint4_t*>(sp);
                    dst.s[m][0] = v.x; dst.s[m][1] = v.y; dst.s[m][2] = v.z; dst.s[m][3] = v.w;
                }
            }
            if (++bat_n == per_tile) { bat_n = 0; tile_n += tile_stride; }
        };
        constexpr int kLoadsPerItem = NMAT * (4 + 1 + (F::kHasBias ? 1 : 0));
        float4_t y[NMAT];
        auto step = [&](const MvScales<F, NMAT>& cur, MvScales<F, NMAT>& nxt, int slot, int q) {
            if (q + 1 < nq) {
                fetch(nxt, slot ^ 1);
                // item q has arrived once at most the loads just issued are outstanding
                __builtin_amdgcn_s_waitcnt(0x0F70 | (kLoadsPerItem & 15) | ((kLoadsPerItem >> 4) << 14));
            } else {
                __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
            }
            if (bat_c == 0) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m) y[m] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
            }
            compute(cur, STREAM ? bat_c : kwi + bat_c * kw, slot, y);
            if (++bat_c == per_tile) {
                if constexpr (STREAM) {
                    const int row = tile_c * 32 + my_r;
                    if (row < rows) {
#pragma unroll
                        for (int v = 0; v < (ONE ? 1 : 4); ++v) {
                            const int tok = 4 * half + v;
                            if (tok < nb) {
                                float vals[NMAT];
#pragma unroll
                                for (int m = 0; m < NMAT; ++m) vals[m] = v == 0 ? y[m].x : (v == 1 ? y[m].y : (v == 2 ? y[m].z : y[m].w));
                                epi(b0 + tok, row, vals);
                            }
                        }
                    }
                } else {
                    // partial sums of the kw waves of each tile meet in LDS
#pragma unroll
                    for (int m = 0; m < NMAT; ++m) {
                        float* dst = red + ((size_t)(wave * NMAT + m) * 8 + 4 * half) * 32 + my_r;
                        dst[0] = y[m].x; dst[32] = y[m].y; dst[64] = y[m].z; dst[96] = y[m].w;
                    }
                    __syncthreads();
                    const int tbase = tile_c - sub;
                    for (int idx = tid; idx < tpw * 256; idx += blockDim.x) {
                        const int s = idx >> 8, tok = (idx >> 5) & 7, r32 = idx & 31;
                        const int row = (tbase + s) * 32 + r32;
                        if (tbase + s < tiles && row < rows && tok < nb) {
                            float vals[NMAT];
#pragma unroll
                            for (int m = 0; m < NMAT; ++m) {
                                float sum = 0.0f;
                                for (int k = 0; k < kw; ++k) sum += red[((size_t)((s * kw + k) * NMAT + m) * 8 + tok) * 32 + r32];
                                vals[m] = sum;
                            }
                            epi(b0 + tok, row, vals);
                        }
                    }
                    __syncthreads();
                }
                bat_c = 0;
                tile_c += tile_stride;
            }
        };
        if (nq > 0) fetch(regs_a, 0);
        for (int q = 0; q < nq; q += 2) {
            step(regs_a, regs_b, 0, q);
            if (q + 1 < nq) step(regs_b, regs_a, 1, q + 1);
        }
        epi.end_chunk(b0, nb);
    }
}

}  // namespace smelt
