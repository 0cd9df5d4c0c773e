// Matrix-core quantized matvec for gfx950: y[b, r] = sum_c w(r, c) * x[b, c] for up to 8 activation
// rows per pass, for matrices large enough that the packed weights stream from HBM.
//
// The VALU matvec spends about 32 issue cycles per packed dword (shift, AND-OR, dot2), which for
// 4-bit weights is more than the memory system needs to deliver that dword.  Here the multiply-
// accumulate and the cross-lane reduction move to v_mfma_f32_16x16x32_f16, leaving only the
// AND-OR operand formation on the vector ALU:
//   * A wave owns a tile of 32 weight rows.  Lane (j = lane % 16, kb = lane / 16) loads 16 bytes of
//     row  32 * tile + j + 16 * (kb / 2)  at column half  kb % 2  of a window (two 16-byte halves
//     of one row = one scale group).  Each dword of those 16 bytes is, unchanged, the eight
//     (or 2 x eight) k-values lane (j, kb) supplies as the B operand of one MFMA.
//   * The MFMA contracts over all four kb, which would mix rows j and j + 16.  The A operand (the
//     activations) separates them: token slot i < 8 carries x only in k-slots kb < 2, slot i >= 8
//     only in kb >= 2, zero elsewhere.  Output D[i][j] is then row j for i < 8 and row j + 16 for
//     i >= 8: 32 rows x 8 tokens per instruction, one scale group per contraction.
//   * Codes enter the MFMA as (base + code) straight from the AND-OR; the row-independent
//     sum(base * x) per window and token is computed when the activations are staged and
//     subtracted before the group scale is applied in fp32.
//   * Activations are staged once per workgroup into LDS as fp16 operand fragments.
// K can be split over `kw` waves of a workgroup (partials meet in LDS); with kw = 1 every wave
// streams whole rows and keeps two batches of four windows in flight.
#pragma once
#include "matvec.hpp"

namespace smelt {

// ---- format traits: one packed dword -> kMPD MFMA B operands --------------------------------
struct MvU4 {
    static constexpr int kCPD = 8;   // columns per dword
    static constexpr int kMPD = 1;   // MFMAs per dword
    static constexpr bool kHasBias = true;
    static constexpr float kSemMul = 1.0f;
    // column (within the dword) held by operand element q of MFMA m; its additive base
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
    static constexpr int kCPD = 16;
    static constexpr int kMPD = 2;
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

constexpr int kMvRing = 2;  // items of packed codes a streaming wave keeps in its LDS ring

template <class F>
struct MvGeom {
    static constexpr int kWindowCols = 8 * F::kCPD;  // 2 halves x 4 dwords: one scale group
    static constexpr int kFragsPerWindow = 8 * F::kMPD;
    static constexpr int kWB = 4;                    // windows per register batch
};

// LDS bytes: fragments [windows][4 dwords][kMPD][2 halves][tokens] x 16 B, one zero slot,
// per-window corrections (and activation sums) for 8 token slots, wave partials when K is split.
template <class F>
__host__ __device__ inline size_t mfma_matvec_lds_bytes(int cols, int token_shift, int nmat, int waves, int kw) {
    const size_t nwin = (size_t)cols / MvGeom<F>::kWindowCols;
    size_t bytes = ((nwin * MvGeom<F>::kFragsPerWindow * 16) << token_shift) + 16;
    bytes += nwin * 32 * (F::kHasBias ? 2 : 1);
    if (kw > 1) bytes += (size_t)waves * nmat * 1024;
    else bytes = ((bytes + 1023) & ~(size_t)1023) + (size_t)waves * nmat * kMvRing * 4096;  // code rings of the streaming form
    return bytes;
}

__host__ __device__ inline int mfma_token_shift(int tokens) {
    int shift = 0;
    while ((1 << shift) < tokens && shift < 3) ++shift;
    return shift;
}

template <class F, int NMAT>
struct MvBatch {
    uint4_t c[NMAT][MvGeom<F>::kWB];
    uint2_t s[NMAT];  // four 16-bit group scales
    uint2_t b[NMAT];  // four 16-bit group biases (affine)
};

// ONE: the launch carries a single activation row (decode): only token slot 0 is formed and used.
template <class F, class ActT, class ScaleT, int NMAT, bool STREAM, bool ONE, class Epi>
__device__ __forceinline__ void mfma_matvec_body(const MatPtrs (&mats)[NMAT], const uint16_t* x, int rows,
                                                 int cols, int row_stride, int kw, int batch_lo,
                                                 int batch_hi, const Epi& epi) {
    using G = MvGeom<F>;
    constexpr int WB = G::kWB, MPD = F::kMPD, CPD = F::kCPD, FPW = G::kFragsPerWindow;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave, nwaves = blockDim.x / kWave;
    const int lj = lane & 15, kb = lane >> 4, half = kb & 1, rsel = kb >> 1;
    const int nwin = cols / G::kWindowCols;  // == scale groups per row
    const int tiles = (rows + 31) / 32;
    const int span = batch_hi - batch_lo;
    const int tshift = mfma_token_shift(span < 8 ? span : 8);
    const int tmask = (1 << tshift) - 1;

    uint4_t* frags = reinterpret_cast<uint4_t*>(smem);
    const size_t nfrag = ((size_t)nwin * FPW) << tshift;
    uint4_t* zero_slot = frags + nfrag;
    float* corr = reinterpret_cast<float*>(zero_slot + 1);   // [nwin][8]
    float* xsum = corr + (size_t)nwin * 8;                   // [nwin][8], affine only
    float* red = xsum + (F::kHasBias ? (size_t)nwin * 8 : 0);  // [nwaves][NMAT][8][32], kw > 1 only

    // A-operand lane (token slot i = lane % 16, kb): live where the slot's row half matches kb's
    const bool a_live = ((lj >> 3) == rsel) && ((lj & 7) <= tmask) && (!ONE || (lj & 7) == 0);
    const int a_tok = lj & 7;

    const int tpw = nwaves / kw;         // tiles a workgroup covers per step
    const int sub = wave / kw, kwi = wave % kw;
    const int nbatch = nwin / WB;        // batches of four windows per row
    const int my_batches = kwi < nbatch ? (nbatch - kwi + kw - 1) / kw : 0;

    auto load = [&](MvBatch<F, NMAT>& dst, int row, int batch) {
        const int w0 = batch * WB;
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            const uint8_t* wrow = mats[m].codes + (size_t)row * row_stride + half * 16;
#pragma unroll
            for (int i = 0; i < WB; ++i) dst.c[m][i] = *reinterpret_cast<const uint4_t*>(wrow + (size_t)(w0 + i) * 32);
            dst.s[m] = *reinterpret_cast<const uint2_t*>(mats[m].scales + (size_t)row * nwin + w0);
            if (F::kHasBias) dst.b[m] = *reinterpret_cast<const uint2_t*>(mats[m].biases + (size_t)row * nwin + w0);
        }
    };
    uint4_t fr[4 * MPD];  // activation fragments of the window in hand
#pragma unroll
    for (int k = 0; k < 4 * MPD; ++k) fr[k] = uint4_t{0u, 0u, 0u, 0u};
    // y[m][v] += scale * (sum (base + code) * x - sum base * x) + bias * sum x  for four windows
    auto compute = [&](const MvBatch<F, NMAT>& cur, int batch, float4_t (&y)[NMAT], auto&& codes_of) {
        const int w0 = batch * WB;
#pragma unroll
        for (int i = 0; i < WB; ++i) {
            const int w = w0 + i;
            // activation fragments: dead lanes hold zeros (ONE: registers that are never written;
            // otherwise a zero slot in LDS)
            if constexpr (ONE) {
                if (a_live) {
#pragma unroll
                    for (int k = 0; k < 4 * MPD; ++k) fr[k] = frags[(size_t)w * FPW + half + 2 * k];
                }
            } else {
                const uint4_t* fw = a_live ? frags + (((size_t)w * FPW + half) << tshift) + a_tok : zero_slot;
                const size_t fstep = a_live ? ((size_t)2 << tshift) : 0;
#pragma unroll
                for (int k = 0; k < 4 * MPD; ++k) fr[k] = fw[(size_t)k * fstep];
            }
            float4_t acc[NMAT];
#pragma unroll
            for (int m = 0; m < NMAT; ++m) acc[m] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
            uint4_t cw[NMAT];
#pragma unroll
            for (int m = 0; m < NMAT; ++m) cw[m] = codes_of(m, i);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                uint4_t ops[NMAT][MPD];
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
                    F::operands(t == 0 ? cw[m].x : (t == 1 ? cw[m].y : (t == 2 ? cw[m].z : cw[m].w)), ops[m]);
#pragma unroll
                for (int q = 0; q < MPD; ++q) {
                    const half8_t xa = __builtin_bit_cast(half8_t, fr[t * MPD + q]);
#pragma unroll
                    for (int m = 0; m < NMAT; ++m)
                        acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa, __builtin_bit_cast(half8_t, ops[m][q]), acc[m], 0, 0, 0);
                }
            }
            // D lane (row j, ib = kb): tokens 4 * (kb % 2) + v of row half kb / 2
            if constexpr (ONE) {
                const float cr = corr[(size_t)w * 8];
                const float xs1 = F::kHasBias ? xsum[(size_t)w * 8] : 0.0f;
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    const uint32_t sp = i < 2 ? cur.s[m].x : cur.s[m].y;
                    const float sv = F::kSemMul * ScaleT::widen((uint16_t)((i & 1) ? sp >> 16 : sp & 0xFFFFu));
                    y[m].x = __builtin_fmaf(sv, acc[m].x - cr, y[m].x);
                    if (F::kHasBias) {
                        const uint32_t bp = i < 2 ? cur.b[m].x : cur.b[m].y;
                        y[m].x = __builtin_fmaf(ScaleT::widen((uint16_t)((i & 1) ? bp >> 16 : bp & 0xFFFFu)), xs1, y[m].x);
                    }
                }
            } else {
                const float4_t cr = *reinterpret_cast<const float4_t*>(corr + (size_t)w * 8 + 4 * half);
                float4_t xs4 = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
                if (F::kHasBias) xs4 = *reinterpret_cast<const float4_t*>(xsum + (size_t)w * 8 + 4 * half);
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    const uint32_t sp = i < 2 ? cur.s[m].x : cur.s[m].y;
                    const float sv = F::kSemMul * ScaleT::widen((uint16_t)((i & 1) ? sp >> 16 : sp & 0xFFFFu));
                    y[m].x = __builtin_fmaf(sv, acc[m].x - cr.x, y[m].x);
                    y[m].y = __builtin_fmaf(sv, acc[m].y - cr.y, y[m].y);
                    y[m].z = __builtin_fmaf(sv, acc[m].z - cr.z, y[m].z);
                    y[m].w = __builtin_fmaf(sv, acc[m].w - cr.w, y[m].w);
                    if (F::kHasBias) {
                        const uint32_t bp = i < 2 ? cur.b[m].x : cur.b[m].y;
                        const float bv = ScaleT::widen((uint16_t)((i & 1) ? bp >> 16 : bp & 0xFFFFu));
                        y[m].x = __builtin_fmaf(bv, xs4.x, y[m].x);
                        y[m].y = __builtin_fmaf(bv, xs4.y, y[m].y);
                        y[m].z = __builtin_fmaf(bv, xs4.z, y[m].z);
                        y[m].w = __builtin_fmaf(bv, xs4.w, y[m].w);
                    }
                }
            }
            // keep one window's fragments and operands live at a time: without this fence the
            // scheduler hoists all sixteen operand sets of a batch and halves the occupancy
            if constexpr (!STREAM) __builtin_amdgcn_sched_barrier(0);
        }
    };

    for (int b0 = batch_lo; b0 < batch_hi; b0 += 8) {
        const int nb = batch_hi - b0 < 8 ? batch_hi - b0 : 8;
        // ---- stage the activations of this chunk ----------------------------------------------
        // One item = one packed dword's worth of columns of one token: CPD consecutive columns are
        // converted to fp16 and written as the kMPD operand fragments that dword feeds; the eight
        // items of a (token, window) sit in consecutive lanes and reduce their sum(base * x) and
        // sum(x) with DPP adds.
        if (b0 != batch_lo) __syncthreads();
        if (tid == 0) *zero_slot = uint4_t{0u, 0u, 0u, 0u};
        const int nitems = (nwin * 8) << tshift;
        for (int base_i = 0; base_i < nitems; base_i += blockDim.x) {
            const int idx = base_i + tid;
            const int e = idx & 7, tok = (idx >> 3) & tmask, w = idx >> (3 + tshift);
            const bool on = idx < nitems && tok < nb;
            uint16_t h[CPD];
#pragma unroll
            for (int q = 0; q < CPD / 8; ++q) {
                uint4_t v = {0u, 0u, 0u, 0u};
                if (on) v = *reinterpret_cast<const uint4_t*>(x + (size_t)(b0 + tok) * cols + ((size_t)w * 8 + e) * CPD + q * 8);
                const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    h[8 * q + 2 * k] = ActT::to_f16_bits((uint16_t)(d[k] & 0xFFFF));
                    h[8 * q + 2 * k + 1] = ActT::to_f16_bits((uint16_t)(d[k] >> 16));
                }
            }
            float cs = 0.0f, xs1 = 0.0f;
            const int hsel = e >> 2, t = e & 3;  // dword t of lane half hsel
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
            cs = group_sum_last<8>(cs);
            xs1 = group_sum_last<8>(xs1);
            if (e == 7 && idx < nitems) {
                corr[(size_t)w * 8 + tok] = cs;
                if (F::kHasBias) xsum[(size_t)w * 8 + tok] = xs1;
            }
        }
        __syncthreads();

        if constexpr (STREAM) {
            // ---- streaming: every wave owns whole tiles; (tile, batch) items two deep ----------
            // The packed codes of an item go straight from global memory into a wave-private LDS
            // ring (128-bit loads to LDS), eight consecutive lanes per 128-byte row segment, so
            // every load instruction reads whole cache lines.  Lane l of load i lands in slot
            // (row 8i + l/8, l%8) and fetches piece (l%8) ^ f(row), f(row) = (row/2) % 8; the MFMA
            // lane of row r then finds piece q in slot q ^ f(r), and the sixteen rows a 16-lane
            // group reads fall in sixteen different bank groups.
            const int first = blockIdx.x * nwaves + wave, stride = gridDim.x * nwaves;
            const int my_tiles = first < tiles ? (tiles - first + stride - 1) / stride : 0;
            const int nq = my_tiles * nbatch;
            unsigned char* ring = smem + (((size_t)(reinterpret_cast<unsigned char*>(red) - smem) + 1023) & ~(size_t)1023) +
                                  (size_t)wave * NMAT * kMvRing * 4096;
            const int my_r = lj + 16 * rsel;                      // row of the tile this lane feeds to the MFMA
            const int my_f = (my_r >> 1) & 7;
            MvBatch<F, NMAT> regs_a, regs_b;                      // scales and biases only; codes live in the ring
            int tile_c = first, bat_c = 0, tile_n = first, bat_n = 0;
            auto fetch = [&](MvBatch<F, NMAT>& dst, int slot) {
                __builtin_amdgcn_s_waitcnt(0xC07F);               // lgkmcnt(0): reads of this ring slot have returned
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int rt = 8 * i + (lane >> 3);
                        int row = tile_n * 32 + rt;
                        if (row >= rows) row = rows - 1;         // clamped rows are computed, never stored
                        const int piece = (lane & 7) ^ ((rt >> 1) & 7);
                        const uint8_t* src = mats[m].codes + (size_t)row * row_stride + (size_t)bat_n * 128 + piece * 16;
                        __builtin_amdgcn_global_load_lds(src, (__attribute__((address_space(3))) void*)(ring + ((size_t)(slot * NMAT + m) * 4 + i) * 1024), 16, 0, 0);
                    }
                    int row = tile_n * 32 + my_r;
                    if (row >= rows) row = rows - 1;
                    dst.s[m] = *reinterpret_cast<const uint2_t*>(mats[m].scales + (size_t)row * nwin + bat_n * WB);
                    if (F::kHasBias) dst.b[m] = *reinterpret_cast<const uint2_t*>(mats[m].biases + (size_t)row * nwin + bat_n * WB);
                }
                if (++bat_n == nbatch) { bat_n = 0; tile_n += stride; }
            };
            constexpr int kLoadsPerItem = NMAT * (4 + 1 + (F::kHasBias ? 1 : 0));
            constexpr int kAhead = kMvRing - 1;                   // items in flight beyond the one computed
            float4_t y[NMAT];
            // item q lives in ring slot q % kMvRing and register set q % kMvRing
            auto step = [&](const MvBatch<F, NMAT>& cur, MvBatch<F, NMAT>& ahead, int slot, int q) {
                int newer = nq - 1 - q;                           // items requested after q
                if (q + kAhead < nq) fetch(ahead, (slot + kAhead) % kMvRing);
                if (newer > kAhead) newer = kAhead;
                // item q has arrived once at most the loads of the newer items are outstanding
                if (newer == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | (kLoadsPerItem & 15) | ((kLoadsPerItem >> 4) << 14));
                else __builtin_amdgcn_s_waitcnt(0x0F70);
                if (bat_c == 0) {
#pragma unroll
                    for (int m = 0; m < NMAT; ++m) y[m] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
                }
                compute(cur, bat_c, y, [&](int m, int i) {
                    return *reinterpret_cast<const uint4_t*>(ring + (size_t)(slot * NMAT + m) * 4096 + ((size_t)my_r * 8 + ((2 * i + half) ^ my_f)) * 16);
                });
                if (++bat_c == nbatch) {
                    const int row = tile_c * 32 + lj + 16 * rsel;
                    if (row < rows) {
#pragma unroll
                        for (int v = 0; v < 4; ++v) {
                            const int tok = 4 * half + v;
                            if (tok < nb) {
                                float vals[NMAT];
#pragma unroll
                                for (int m = 0; m < NMAT; ++m) vals[m] = v == 0 ? y[m].x : (v == 1 ? y[m].y : (v == 2 ? y[m].z : y[m].w));
                                epi(b0 + tok, row, vals);
                            }
                        }
                    }
                    bat_c = 0;
                    tile_c += stride;
                }
            };
            static_assert(kMvRing == 2, "the item loop below is unrolled for a ring of two");
            if (nq > 0) fetch(regs_a, 0);
            for (int q = 0; q < nq; q += 2) {
                step(regs_a, regs_b, 0, q);
                if (q + 1 < nq) step(regs_b, regs_a, 1, q + 1);
            }
        } else {
            // ---- K split over kw waves: per tile, load everything, compute, meet in LDS --------
            for (int tbase = blockIdx.x * tpw; tbase < tiles; tbase += gridDim.x * tpw) {
                const int tile = tbase + sub;
                float4_t y[NMAT];
#pragma unroll
                for (int m = 0; m < NMAT; ++m) y[m] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
                if (tile < tiles && sub < tpw) {
                    int row = tile * 32 + lj + 16 * rsel;
                    if (row >= rows) row = rows - 1;
                    for (int g0 = 0; g0 < my_batches; g0 += 2) {
                        MvBatch<F, NMAT> ra, rb;
                        load(ra, row, kwi + g0 * kw);
                        if (g0 + 1 < my_batches) load(rb, row, kwi + (g0 + 1) * kw);
                        compute(ra, kwi + g0 * kw, y, [&](int m, int i) { return ra.c[m][i]; });
                        if (g0 + 1 < my_batches) compute(rb, kwi + (g0 + 1) * kw, y, [&](int m, int i) { return rb.c[m][i]; });
                    }
                }
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    float* dst = red + ((size_t)(wave * NMAT + m) * 8 + 4 * half) * 32 + lj + 16 * rsel;
                    dst[0] = y[m].x; dst[32] = y[m].y; dst[64] = y[m].z; dst[96] = y[m].w;
                }
                __syncthreads();
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
        }
        epi.end_chunk(b0, nb);
    }
}

}  // namespace smelt
