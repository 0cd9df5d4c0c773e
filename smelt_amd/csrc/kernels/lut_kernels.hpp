// u4_lut family (Resources/Shaders/lut_matvec.metal:28-790, 967-992): weights are 4-bit indices
// [rows, cols / 2] (low nibble = even column) into a 16-entry fp16 table shared by `group`
// consecutive ROWS:  y[r] = sum_c lut[r / group][index(r, c)] * x[c].
//
// A wave owns S x R rows at a time (S row groups side by side when a row is shorter than 64 units
// of 16 bytes).  For the row groups its tile touches it expands each 16-entry table into a
// 256-entry table of fp16 pairs in LDS, so one byte of indices (two columns) is one LDS lookup that
// yields both weights, multiplied with the matching activation pair by one v_dot2 (fp32 accumulate).
// Activations are staged once per workgroup as fp16 pairs in column order.
#pragma once
#include "common.hpp"

namespace smelt {

constexpr int kLutMaxTables = 4;   // row groups one wave tile may touch
constexpr int kLutRows = 4;        // rows per lane group (R)

struct LutMat {
    const uint8_t* indices;
    const uint16_t* lut;   // fp16 [row groups, 16]
};

template <class ActT, int NMAT, int L, class Epi>
__device__ __forceinline__ void lut_tiles(const LutMat (&mats)[NMAT], int rows, int cols, int group,
                                          const uint32_t* lds_x, uint32_t* lds_tables, const Epi& epi) {
    constexpr int S = kWave / L;
    constexpr int R = kLutRows;
    constexpr int TILE = S * R;
    const int U = cols / 32;
    const int row_bytes = cols / 2;
    const int waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int sub = lane & (L - 1), side = lane / L;
    const int tiles = (rows + TILE - 1) / TILE;
    uint32_t* my_tables = lds_tables + (size_t)wave * NMAT * kLutMaxTables * 256;
    for (int tile = blockIdx.x * waves + wave; tile < tiles; tile += gridDim.x * waves) {
        const int row0 = tile * TILE;
        const int last = row0 + TILE - 1 < rows ? row0 + TILE - 1 : rows - 1;
        const int g0 = row0 / group, ntab = last / group - g0 + 1;   // the host guarantees ntab <= kLutMaxTables
        // expand the tables of this tile
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
            for (int t = 0; t < ntab; ++t) {
                const uint16_t* src = mats[m].lut + (size_t)(g0 + t) * 16;
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const int e = lane + 64 * k;
                    my_tables[(m * kLutMaxTables + t) * 256 + e] = (uint32_t)src[e & 15] | ((uint32_t)src[e >> 4] << 16);
                }
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        float acc[NMAT][R];
        const uint32_t* tab[NMAT][R];
        int row[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int rr = row0 + side * R + r;
            row[r] = rr < rows ? rr : rows - 1;   // clamped rows are computed, never stored
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                acc[m][r] = 0.0f;
                tab[m][r] = my_tables + (m * kLutMaxTables + (row[r] / group - g0)) * 256;
            }
        }
        for (int u = sub; u < U; u += L) {
            uint4_t c[NMAT][R];
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r)
                    c[m][r] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(mats[m].indices + (size_t)row[r] * row_bytes + (size_t)u * 16));
            uint32_t xp[16];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint4_t t = reinterpret_cast<const uint4_t*>(lds_x)[u * 4 + q];
                xp[4 * q] = t.x; xp[4 * q + 1] = t.y; xp[4 * q + 2] = t.z; xp[4 * q + 3] = t.w;
            }
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const uint32_t w[4] = {c[m][r].x, c[m][r].y, c[m][r].z, c[m][r].w};
                    float a = acc[m][r];
#pragma unroll
                    for (int d = 0; d < 4; ++d)
#pragma unroll
                        for (int b = 0; b < 4; ++b)
                            a = dot2(tab[m][r][(w[d] >> (8 * b)) & 0xFFu], xp[4 * d + b], a);
                    acc[m][r] = a;
                }
        }
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int r = 0; r < R; ++r) acc[m][r] = group_sum_last<L>(acc[m][r]);
        if (sub == L - 1) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int rr = row0 + side * R + r;
                if (rr < rows) {
                    float v[NMAT];
#pragma unroll
                    for (int m = 0; m < NMAT; ++m) v[m] = acc[m][r];
                    epi(rr, v);
                }
            }
        }
    }
}

template <class ActT, int NMAT, class Epi>
__device__ __forceinline__ void lut_matvec_body(const LutMat (&mats)[NMAT], const uint16_t* x, int rows, int cols,
                                                int group, const Epi& epi) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint32_t* lds_x = reinterpret_cast<uint32_t*>(smem);
    uint32_t* lds_tables = lds_x + cols / 2;
    for (int j = threadIdx.x; j < cols / 2; j += blockDim.x) {
        const uint32_t pair = reinterpret_cast<const uint32_t*>(x)[j];
        lds_x[j] = (uint32_t)ActT::to_f16_bits((uint16_t)(pair & 0xFFFFu)) | ((uint32_t)ActT::to_f16_bits((uint16_t)(pair >> 16)) << 16);
    }
    __syncthreads();
    const int U = cols / 32;
    if (U > 32) lut_tiles<ActT, NMAT, 64>(mats, rows, cols, group, lds_x, lds_tables, epi);
    else if (U > 16) lut_tiles<ActT, NMAT, 32>(mats, rows, cols, group, lds_x, lds_tables, epi);
    else lut_tiles<ActT, NMAT, 16>(mats, rows, cols, group, lds_x, lds_tables, epi);
}

}  // namespace smelt

#define SMELT_LUT_KERNEL extern "C" __global__ __launch_bounds__(256)

#define SMELT_LUT_KERNELS(T, ACT)                                                                 \
    SMELT_LUT_KERNEL void smelt_lut_matvec_##T(const uint8_t* W, const uint16_t* lut,             \
                                               const uint16_t* x, uint16_t* y, uint32_t rows,     \
                                               uint32_t cols, uint32_t group) {                   \
        const smelt::LutMat mats[1] = {{W, lut}};                                                 \
        auto epi = [=](int r, const float* v) { y[r] = ACT::narrow(v[0]); };                      \
        smelt::lut_matvec_body<ACT, 1>(mats, x, rows, cols, group, epi);                          \
    }                                                                                             \
    /* fused_lut_matmul (prefill_matmul.metal:13-62): grid.y = token, rows of X and Y per token */  \
    SMELT_LUT_KERNEL void smelt_lut_matmul_##T(const uint8_t* W, const uint16_t* lut,             \
                                               const uint16_t* X, uint16_t* Y, uint32_t cols,     \
                                               uint32_t group, uint32_t rows) {                   \
        const smelt::LutMat mats[1] = {{W, lut}};                                                 \
        uint16_t* y = Y + (size_t)blockIdx.y * rows;                                              \
        auto epi = [=](int r, const float* v) { y[r] = ACT::narrow(v[0]); };                      \
        smelt::lut_matvec_body<ACT, 1>(mats, X + (size_t)blockIdx.y * cols, rows, cols, group, epi); \
    }                                                                                             \
    /* half(float(residual) + acc): the sum is not rounded before the add (lut_matvec.metal:334-340) */ \
    SMELT_LUT_KERNEL void smelt_lut_matvec_add_##T(const uint8_t* W, const uint16_t* lut,         \
                                                   const uint16_t* x, uint16_t* y,                \
                                                   const uint16_t* res, uint32_t rows,            \
                                                   uint32_t cols, uint32_t group) {               \
        const smelt::LutMat mats[1] = {{W, lut}};                                                 \
        auto epi = [=](int r, const float* v) { y[r] = ACT::narrow(ACT::widen(res[r]) + v[0]); }; \
        smelt::lut_matvec_body<ACT, 1>(mats, x, rows, cols, group, epi);                          \
    }                                                                                             \
    SMELT_LUT_KERNEL void smelt_dual_lut_matvec_##T(const uint8_t* W1, const uint16_t* lut1,      \
                                                    const uint8_t* W2, const uint16_t* lut2,      \
                                                    const uint16_t* x, uint16_t* y1,              \
                                                    uint16_t* y2, uint32_t rows, uint32_t cols,   \
                                                    uint32_t group) {                             \
        const smelt::LutMat mats[2] = {{W1, lut1}, {W2, lut2}};                                   \
        auto epi = [=](int r, const float* v) { y1[r] = ACT::narrow(v[0]); y2[r] = ACT::narrow(v[1]); }; \
        smelt::lut_matvec_body<ACT, 2>(mats, x, rows, cols, group, epi);                          \
    }                                                                                             \
    /* half(g / (1 + exp(-g)) * u) on the fp32 sums (lut_matvec.metal:786-790) */                 \
    SMELT_LUT_KERNEL void smelt_lut_gate_up_swiglu_##T(const uint8_t* gW, const uint16_t* glut,   \
                                                       const uint8_t* uW, const uint16_t* ulut,   \
                                                       const uint16_t* x, uint16_t* y,            \
                                                       uint32_t rows, uint32_t cols,              \
                                                       uint32_t group) {                          \
        const smelt::LutMat mats[2] = {{gW, glut}, {uW, ulut}};                                   \
        auto epi = [=](int r, const float* v) { y[r] = ACT::narrow(v[0] / (1.0f + expf(-v[0])) * v[1]); }; \
        smelt::lut_matvec_body<ACT, 2>(mats, x, rows, cols, group, epi);                          \
    }

// lut_embedding_gather (lut_matvec.metal:967-992): table values are copied bit for bit
extern "C" __global__ __launch_bounds__(1024) void smelt_lut_embedding_gather(
    const uint8_t* indices, const uint16_t* lut, const int* token, uint16_t* out, uint32_t cols, uint32_t group) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= cols / 2) return;
    const uint32_t row = (uint32_t)token[0];
    const uint16_t* table = lut + (size_t)(row / group) * 16;
    const uint8_t packed = indices[(size_t)row * (cols / 2) + i];
    out[2 * i] = table[packed & 0xF];
    out[2 * i + 1] = table[packed >> 4];
}
