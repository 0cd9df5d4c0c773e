// Skinny quantized matmul for gfx950: Y[M, N] = X[M, K] * W[N, K]^T with M <= 32 tokens per pass,
// affine u4 weights with one scale group per 64 columns.
//
// At this batch the weights still stream from HBM once and the arithmetic is small, so the kernel is
// organised around keeping every byte of W in flight rather than around tile reuse:
//   * v_mfma_f32_32x32x16_f16 with the tokens as the A operand and 32 weight rows as the B operand.
//     Lane (j = lane % 32, kb = lane / 32) loads 16 bytes = 32 codes of row j; dword t of those 16
//     bytes holds exactly the eight k-values lane (j, kb) supplies to the t-th MFMA of a 64-column
//     window, so a packed dword becomes a B operand with one shift, four v_bitop3 and four packed
//     subtracts, with no shuffles and no LDS round trip for the weights.
//   * The MFMA multiplies the exact integer codes; the per-(row, window) scale is applied in fp32
//     on the 32x32 accumulator (each lane owns one weight row, so it is one scalar per lane).
//   * The bias term  sum_g b[n, g] * xsum[m, g]  is itself a small matmul over scale groups and is
//     fed through the same MFMA, with xsum split into fp16 high and low parts (22 significant bits).
//   * Only the live tokens of a pass (rounded up to a power of two) are resident in LDS, so a small
//     batch leaves room for long K chunks and many workgroups per CU.
//   * K is split over the waves of a workgroup (4 to 8) and, for long rows, over `ksplit` workgroups
//     (gridDim.x = row tiles * ksplit).  Wave partials meet in LDS; workgroup partials meet in a
//     workspace where the last workgroup to arrive adds them in a fixed order, so results do not
//     depend on arrival order.
// Activations are staged once per workgroup into LDS as fp16 in the operand order of the code
// pairs (every run of 8 columns permuted to 0,4,1,5,2,6,3,7).
#pragma once
#include "common.hpp"
#include "matvec.hpp"
#include "qmm.hpp"

namespace smelt {

typedef float float16v_t __attribute__((ext_vector_type(16)));

constexpr int kSkRows = 32;  // weight rows per workgroup tile (MFMA N)
constexpr int kSkTok = 32;   // tokens per pass (MFMA M)

struct SkinnyWorkspace {
    float* partial;      // [gridDim.y][tiles][ksplit][NMAT][1024] (thread-major, see the hand-off below)
    uint32_t* counters;  // [gridDim.y][tiles], zero between launches
};

// eight codes of one dword -> fp16 values (0..15) in operand order (0,4,1,5,2,6,3,7)
__device__ __forceinline__ half8_t skinny_codes(uint32_t c) {
    const uint32_t c8 = c >> 8;
    const half2_t o1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    const half2_t o64 = {(_Float16)64.0f, (_Float16)64.0f};
    const half2_t a0 = as_half2(and_or(c, 0x000F000Fu, 0x64006400u)) - o1024;
    const half2_t a1 = as_half2(and_or(c, 0x00F000F0u, 0x54005400u)) - o64;
    const half2_t a2 = as_half2(and_or(c8, 0x000F000Fu, 0x64006400u)) - o1024;
    const half2_t a3 = as_half2(and_or(c8, 0x00F000F0u, 0x54005400u)) - o64;
    half8_t a;
    a[0] = a0.x; a[1] = a0.y; a[2] = a1.x; a[3] = a1.y;
    a[4] = a2.x; a[5] = a2.y; a[6] = a3.x; a[7] = a3.y;
    return a;
}

__device__ __forceinline__ uint32_t dword_of(const uint4_t& v, int t) {
    return t == 0 ? v.x : (t == 1 ? v.y : (t == 2 ? v.z : v.w));
}

// Windows per K chunk and LDS bytes; the host computes the same numbers to size the launch.
__host__ __device__ inline int skinny_chunk_windows(int cols, int ksplit) {
    const int nwin = cols / 64;
    return (nwin + ksplit - 1) / ksplit;
}
__host__ __device__ inline int skinny_bias_blocks(int chunk_windows) { return (chunk_windows + 15) / 16 + 1; }
// tokens resident per window in LDS: the live tokens of a pass rounded up to a power of two
__host__ __device__ inline int skinny_token_shift(int batch, int batch_tile) {
    const int live = batch < batch_tile ? batch : batch_tile;
    int shift = 0;
    while ((1 << shift) < live) ++shift;
    return shift;
}
// Per window: 8 operand rows of (tokens + 1) x 16 B (one slot of padding spreads the rows over
// the banks) and 8 rows of (tokens + 1) run sums.
__host__ __device__ inline size_t skinny_lds_bytes(int cols, int ksplit, int nmat, int token_shift, int waves) {
    const int cw = skinny_chunk_windows(cols, ksplit);
    const size_t stage = (size_t)cw * 8 * ((1 << token_shift) + 1) * 20 + (size_t)skinny_bias_blocks(cw) * 2048;
    const size_t reduce = (size_t)waves * nmat * 4096;
    return stage > reduce ? stage : reduce;
}

template <class ActT, class ScaleT, int NMAT, class Epi>
__device__ __forceinline__ void qmm_skinny_body(const uint8_t* const (&W)[NMAT], const uint16_t* const (&S)[NMAT],
                                                const uint16_t* const (&B)[NMAT], const uint16_t* X,
                                                int rows, int cols, int batch, int batch_tile,
                                                SkinnyWorkspace ws, const Epi& epi) {
    constexpr int PAIRS = NMAT == 1 ? 6 : 3;  // window pairs whose codes a wave holds in registers at once
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ uint32_t last_flag;
    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave, nwaves = blockDim.x / kWave;
    const int lj = lane & 31, kb = lane >> 5;
    const int tiles = (rows + kSkRows - 1) / kSkRows;
    const int ksplit = gridDim.x / tiles;
    const int tile = blockIdx.x / ksplit, ks = blockIdx.x % ksplit;
    const int nwin = cols / 64;  // == scale groups per row
    const int cw = skinny_chunk_windows(cols, ksplit);
    const int W0 = ks * cw < nwin ? ks * cw : nwin;
    const int W1 = W0 + cw < nwin ? W0 + cw : nwin;
    const int m0 = blockIdx.y * batch_tile;
    const int ntok = batch - m0 < batch_tile ? batch - m0 : batch_tile;  // <= 32
    const int rs = cols / 2;

    const int tshift = skinny_token_shift(batch, batch_tile);
    const int tmask = (1 << tshift) - 1;
    const int xr = (1 << tshift) + 1;                                        // row stride, in slots
    uint4_t* xs = reinterpret_cast<uint4_t*>(smem);                          // [cw][4 t][2 kb] rows of xr x 16 B
    float* psum = reinterpret_cast<float*>(xs + (size_t)cw * 8 * xr);        // [cw][8 runs] rows of xr floats
    uint4_t* xsum_hi = reinterpret_cast<uint4_t*>(psum + (size_t)cw * 8 * xr);  // [blocks][2][32] x 16 B
    uint4_t* xsum_lo = xsum_hi + (size_t)skinny_bias_blocks(cw) * 64;
    float* red = reinterpret_cast<float*>(smem);                             // aliases the staging area
    const int blk0 = W0 / 16, blk1 = (W1 + 15) / 16;

    // this wave's windows of the chunk
    const int pw = (W1 - W0 + nwaves - 1) / nwaves;
    const int w0 = W0 + wave * pw < W1 ? W0 + wave * pw : W1;
    const int w1 = w0 + pw < W1 ? w0 + pw : W1;
    int row = tile * kSkRows + lj;
    if (row >= rows) row = rows - 1;  // clamped rows are computed and never stored

    // Codes and scales of up to 2 * PAIRS windows, all requested before anything else happens so
    // that the whole matrix is in flight at once.  The second window of a pair may lie past the
    // wave's range: it is then a repeat of the last window with scale 0.
    uint4_t codes[NMAT][PAIRS][2];
    float scale[NMAT][PAIRS][2];
    auto load = [&](int base) {
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
            const int wa = base + 2 * p;
            if (wa < w1) {
                const int wb = wa + 1 < w1 ? wa + 1 : wa;
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    const uint8_t* wrow = W[m] + (size_t)row * rs + kb * 16;
                    codes[m][p][0] = *reinterpret_cast<const uint4_t*>(wrow + (size_t)wa * 32);
                    codes[m][p][1] = *reinterpret_cast<const uint4_t*>(wrow + (size_t)wb * 32);
                    scale[m][p][0] = ScaleT::widen(S[m][(size_t)row * nwin + wa]);
                    scale[m][p][1] = wa + 1 < w1 ? ScaleT::widen(S[m][(size_t)row * nwin + wb]) : 0.0f;
                }
            }
        }
    };
    load(w0);
    // bias rows of this wave's first block of 16 groups, also in flight from the start
    auto load_bias = [&](uint4_t (&dst)[NMAT], int blk) {
        const int g = blk * 16 + kb * 8;
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            dst[m] = uint4_t{0u, 0u, 0u, 0u};
            if (blk < blk1 && g < nwin) dst[m] = *reinterpret_cast<const uint4_t*>(B[m] + (size_t)row * nwin + g);
        }
    };
    uint4_t bias_regs[NMAT];
    load_bias(bias_regs, blk0 + wave);

    // ---- stage activations -------------------------------------------------------------------
    for (int i = tid; i < (blk1 - blk0) * 128; i += blockDim.x) {
        const uint4_t z = {0u, 0u, 0u, 0u};
        (i < (blk1 - blk0) * 64 ? xsum_hi[i] : xsum_lo[i - (blk1 - blk0) * 64]) = z;
    }
    // One item = one run of 8 columns of one live token: a 16-byte load (eight consecutive lanes
    // read one 128-byte window of one token), converted to fp16 in operand order.  Items are
    // taken four at a time with the loads issued first.  Slots of tokens beyond the batch stay
    // unwritten: they only feed output rows that are never stored.
    {
        const int nitems = ntok > 0 ? (W1 - W0) << (3 + tshift) : 0;
        for (int base = tid; base < nitems; base += 4 * blockDim.x) {
            uint4_t v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = base + u * blockDim.x;
                const int e = idx & 7, tok = (idx >> 3) & tmask, wl = idx >> (3 + tshift);
                v[u] = uint4_t{0u, 0u, 0u, 0u};
                if (idx < nitems && tok < ntok)
                    v[u] = *reinterpret_cast<const uint4_t*>(X + (size_t)(m0 + tok) * cols + (size_t)(W0 + wl) * 64 + e * 8);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = base + u * blockDim.x;
                const int e = idx & 7, tok = (idx >> 3) & tmask, wl = idx >> (3 + tshift);
                if (idx < nitems && tok < ntok) {
                    uint16_t h[8];
                    const uint32_t d[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        h[2 * q] = ActT::to_f16_bits((uint16_t)(d[q] & 0xFFFF));
                        h[2 * q + 1] = ActT::to_f16_bits((uint16_t)(d[q] >> 16));
                    }
                    float run = 0.0f;
#pragma unroll
                    for (int q = 0; q < 8; ++q) run += F16::widen(h[q]);
                    uint4_t o;
                    o.x = h[0] | ((uint32_t)h[4] << 16);
                    o.y = h[1] | ((uint32_t)h[5] << 16);
                    o.z = h[2] | ((uint32_t)h[6] << 16);
                    o.w = h[3] | ((uint32_t)h[7] << 16);
                    // run e feeds lane half e / 4 of MFMA e % 4
                    xs[(size_t)((wl * 4 + (e & 3)) * 2 + (e >> 2)) * xr + tok] = o;
                    psum[(size_t)(wl * 8 + e) * xr + tok] = run;
                }
            }
        }
        __syncthreads();
        // per-(token, window) activation sum: the eight run sums in column order, split into fp16
        // high and low parts for the bias MFMA
        for (int idx = tid; idx < ((W1 - W0) << tshift); idx += blockDim.x) {
            const int tok = idx & tmask, wl = idx >> tshift;
            if (tok < ntok) {
                float xsum = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; ++e) xsum += psum[(size_t)(wl * 8 + e) * xr + tok];
                const int w = W0 + wl;
                const uint16_t hi = F16::narrow(xsum);
                const uint16_t lo = F16::narrow(xsum - F16::widen(hi));
                const size_t at = ((size_t)((w >> 4) - blk0) * 2 + ((w >> 3) & 1)) * 32 + tok;
                reinterpret_cast<uint16_t*>(xsum_hi + at)[w & 7] = hi;
                reinterpret_cast<uint16_t*>(xsum_lo + at)[w & 7] = lo;
            }
        }
    }
    __syncthreads();

    // ---- main loop: the wave's windows two at a time, as two independent MFMA chains ------------
    float16v_t y[NMAT];
    float16v_t zero;
#pragma unroll
    for (int v = 0; v < 16; ++v) zero[v] = 0.0f;
#pragma unroll
    for (int m = 0; m < NMAT; ++m) y[m] = zero;
    const int tl = lj & tmask;  // lanes of tokens beyond the resident ones re-read a live slot; their rows are never stored
    for (int base = w0; base < w1; base += 2 * PAIRS) {
#pragma unroll
        for (int p = 0; p < PAIRS; ++p) {
            const int wa = base + 2 * p;
            if (wa < w1) {
                const int wb = wa + 1 < w1 ? wa + 1 : wa;
                const uint4_t* xa_row = xs + (size_t)((wa - W0) * 8 + kb) * xr + tl;
                const uint4_t* xb_row = xs + (size_t)((wb - W0) * 8 + kb) * xr + tl;
                float16v_t acc_a[NMAT], acc_b[NMAT];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const half8_t xa = *reinterpret_cast<const half8_t*>(xa_row + (size_t)(2 * t) * xr);
                    const half8_t xb = *reinterpret_cast<const half8_t*>(xb_row + (size_t)(2 * t) * xr);
#pragma unroll
                    for (int m = 0; m < NMAT; ++m) {
                        acc_a[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xa, skinny_codes(dword_of(codes[m][p][0], t)), t == 0 ? zero : acc_a[m], 0, 0, 0);
                        acc_b[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xb, skinny_codes(dword_of(codes[m][p][1], t)), t == 0 ? zero : acc_b[m], 0, 0, 0);
                    }
                }
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        y[m][v] = __builtin_fmaf(scale[m][p][1], acc_b[m][v], __builtin_fmaf(scale[m][p][0], acc_a[m][v], y[m][v]));
            }
        }
        if (base + 2 * PAIRS < w1) load(base + 2 * PAIRS);
    }

    // ---- bias term: blocks of 16 scale groups, one MFMA pair each, spread over the waves -------
    for (int blk = blk0 + wave; blk < blk1; blk += nwaves) {
        const half8_t ah = *reinterpret_cast<const half8_t*>(xsum_hi + ((size_t)(blk - blk0) * 2 + kb) * 32 + lj);
        const half8_t al = *reinterpret_cast<const half8_t*>(xsum_lo + ((size_t)(blk - blk0) * 2 + kb) * 32 + lj);
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            const uint32_t d[4] = {bias_regs[m].x, bias_regs[m].y, bias_regs[m].z, bias_regs[m].w};
            uint32_t p[4];
#pragma unroll
            for (int q = 0; q < 4; ++q)
                p[q] = (uint32_t)ScaleT::to_f16_bits((uint16_t)(d[q] & 0xFFFF)) |
                       ((uint32_t)ScaleT::to_f16_bits((uint16_t)(d[q] >> 16)) << 16);
            half8_t bq;
            {
                const half2_t b0 = as_half2(p[0]), b1 = as_half2(p[1]), b2 = as_half2(p[2]), b3 = as_half2(p[3]);
                bq[0] = b0.x; bq[1] = b0.y; bq[2] = b1.x; bq[3] = b1.y;
                bq[4] = b2.x; bq[5] = b2.y; bq[6] = b3.x; bq[7] = b3.y;
            }
            y[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bq, y[m], 0, 0, 0);
            y[m] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bq, y[m], 0, 0, 0);
        }
        load_bias(bias_regs, blk + nwaves);
    }

    // ---- reduce the waves through LDS --------------------------------------------------------------
    __syncthreads();  // every wave is done with the staged activations
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int tok = 8 * (v >> 2) + 4 * kb + (v & 3);
            red[((size_t)(wave * NMAT + m) * kSkTok + tok) * kSkRows + lj] = y[m][v];
        }
    __syncthreads();
    // the first 256 threads own four consecutive rows of one token each from here on
    const bool owner = tid < 256;
    const int tok = owner ? tid >> 3 : kSkTok, r4 = (tid & 7) * 4;
    float val[NMAT][4];
    if (owner) {
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            float4_t sum = *reinterpret_cast<const float4_t*>(red + ((size_t)m * kSkTok + tok) * kSkRows + r4);
            for (int wv = 1; wv < nwaves; ++wv) {
                const float4_t p = *reinterpret_cast<const float4_t*>(red + ((size_t)(wv * NMAT + m) * kSkTok + tok) * kSkRows + r4);
                sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
            }
            val[m][0] = sum.x; val[m][1] = sum.y; val[m][2] = sum.z; val[m][3] = sum.w;
        }
    }

    if (ksplit > 1) {
        // Workgroup partials meet in the workspace; the last to arrive adds them in chunk order.
        // Partials are written and read with agent-scope relaxed atomics (coherent across the
        // compute dies without cache write-backs), value i of owner thread t at [i * 256 + t] so
        // that every store instruction covers consecutive dwords.  A workgroup's stores are
        // complete before its arrival is counted, and the last arrival reads only after its count
        // returned.
        const size_t slot = (size_t)blockIdx.y * tiles + tile;
        float* mine = ws.partial + ((slot * ksplit + ks) * NMAT) * 1024;
        if (tok < ntok) {
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    __hip_atomic_store(mine + (size_t)m * 1024 + i * 256 + tid, val[m][i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): this wave's stores are acknowledged
        __syncthreads();
        if (tid == 0) last_flag = atomicAdd(ws.counters + slot, 1u) == (uint32_t)(ksplit - 1) ? 1u : 0u;
        __syncthreads();
        if (!last_flag) return;
        if (tok < ntok) {
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                for (int c = 0; c < ksplit; ++c) {
                    const float* theirs = ws.partial + ((slot * ksplit + c) * NMAT + m) * 1024 + tid;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        sum[i] += __hip_atomic_load(theirs + i * 256, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) val[m][i] = sum[i];
            }
        }
        if (tid == 0) ws.counters[slot] = 0u;  // ready for the next launch on this stream
    }
    if (tok < ntok) epi(m0 + tok, tile * kSkRows + r4, rows, val);
}

}  // namespace smelt

#define SMELT_SKINNY_KERNEL(MAXT) extern "C" __global__ __launch_bounds__(MAXT)

#define SMELT_AFFINE_QMM_SKINNY(T, ACT, SC)                                                        \
    SMELT_SKINNY_KERNEL(512) void smelt_affine_qmm_skinny_##T(                                             \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* Y,    \
        uint32_t batch, uint32_t rows, uint32_t cols, uint32_t group, uint32_t batch_tile,         \
        float* ws_partial, uint32_t* ws_counters) {                                                \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        QEpiStore<ACT> epi{Y};                                                                     \
        qmm_skinny_body<ACT, SC, 1>(w, s, b, X, rows, cols, batch, batch_tile,                     \
                                    SkinnyWorkspace{ws_partial, ws_counters}, epi);                \
    }                                                                                              \
    SMELT_SKINNY_KERNEL(512) void smelt_affine_qmm_add_skinny_##T(                                         \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* MV,   \
        const uint16_t* RES, uint16_t* OUT, uint32_t batch, uint32_t rows, uint32_t cols,          \
        uint32_t group, uint32_t batch_tile, float* ws_partial, uint32_t* ws_counters) {           \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        QEpiAdd<ACT> epi{MV, RES, OUT};                                                            \
        qmm_skinny_body<ACT, SC, 1>(w, s, b, X, rows, cols, batch, batch_tile,                     \
                                    SkinnyWorkspace{ws_partial, ws_counters}, epi);                \
    }                                                                                              \
    SMELT_SKINNY_KERNEL(512) void smelt_affine_qmm_gate_up_swiglu_skinny_##T(                              \
        const uint8_t* gW, const uint16_t* gS, const uint16_t* gB, const uint8_t* uW,              \
        const uint16_t* uS, const uint16_t* uB, const uint16_t* X, uint16_t* Y, uint32_t batch,    \
        uint32_t rows, uint32_t cols, uint32_t group, uint32_t batch_tile, float* ws_partial,      \
        uint32_t* ws_counters) {                                                                   \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        QEpiSwiglu<ACT> epi{Y};                                                                    \
        qmm_skinny_body<ACT, SC, 2>(w, s, b, X, rows, cols, batch, batch_tile,                     \
                                    SkinnyWorkspace{ws_partial, ws_counters}, epi);                \
    }

SMELT_AFFINE_QMM_SKINNY(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_QMM_SKINNY(bf16, smelt::BF16, smelt::BF16)
