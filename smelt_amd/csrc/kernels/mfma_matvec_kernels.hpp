// __global__ entry points of the matrix-core matvec.  Argument lists are those of the vector-ALU
// kernels of the same pipelines followed by `kw`, the number of waves that share one row tile.
#pragma once
#include "matvec_kernels.hpp"
#include "mfma_matvec.hpp"

// Two kernels per pipeline: `stream` (kw == 1, every wave streams whole rows) and `split` (K split
// over kw waves of a workgroup), so that each keeps only its own registers live.
#define SMELT_AFFINE_MM_KERNELS(T, ACT, SC, MODE, STREAMV)                                                       \
    SMELT_KERNEL void smelt_affine_mm_matvec_##MODE##_##T(const u8* W, const u16* S, const u16* B,         \
                                                 const u16* x, u16* y, u32 rows, u32 cols,        \
                                                 u32 group, u32 kw) {                             \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, y, (int)rows};                                                      \
        mfma_matvec_body<MvU4, ACT, SC, 1, STREAMV, true>(mats, x, rows, cols, cols / 2, kw, blockIdx.y,         \
                                           blockIdx.y + 1, epi);                                  \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_mm_matvec_add_##MODE##_##T(const u8* W, const u16* S, const u16* B,     \
                                                     const u16* x, u16* y, const u16* res,        \
                                                     u32 rows, u32 cols, u32 group, u32 kw) {     \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiAdd<ACT> epi{{}, y, res, (int)rows};                                                   \
        mfma_matvec_body<MvU4, ACT, SC, 1, STREAMV, true>(mats, x, rows, cols, cols / 2, kw, blockIdx.y,         \
                                           blockIdx.y + 1, epi);                                  \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_mm_gate_up_swiglu_##MODE##_##T(                                         \
        const u8* gW, const u16* gS, const u16* gB, const u8* uW, const u16* uS, const u16* uB,   \
        const u16* x, u16* y, u32 rows, u32 cols, u32 group, u32 kw) {                            \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiAffineSwiglu<ACT> epi{{}, y, (int)rows};                                               \
        mfma_matvec_body<MvU4, ACT, SC, 2, STREAMV, true>(mats, x, rows, cols, cols / 2, kw, blockIdx.y,         \
                                           blockIdx.y + 1, epi);                                  \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_mm_matvec_batched_##MODE##_##T(                                         \
        const u8* W, const u16* S, const u16* B, const u16* X, u16* Y, u32 batch, u32 rows,       \
        u32 cols, u32 group, u32 batch_tile, u32 kw) {                                            \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        mfma_matvec_body<MvU4, ACT, SC, 1, STREAMV, false>(mats, X, rows, cols, cols / 2, kw, lo, hi, epi);       \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_mm_gate_up_swiglu_batched_##MODE##_##T(                                 \
        const u8* gW, const u16* gS, const u16* gB, const u8* uW, const u16* uS, const u16* uB,   \
        const u16* X, u16* Y, u32 batch, u32 rows, u32 cols, u32 group, u32 batch_tile,           \
        u32 kw) {                                                                                 \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiAffineSwiglu<ACT> epi{{}, Y, (int)rows};                                               \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        mfma_matvec_body<MvU4, ACT, SC, 2, STREAMV, false>(mats, X, rows, cols, cols / 2, kw, lo, hi, epi);       \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_mm_matvec_argmax_##MODE##_##T(                                          \
        const u8* W, const u16* S, const u16* B, const u16* X, smelt::uint2_t* keys, u32 batch,   \
        float logit_cap, u32 rows, u32 cols, u32 group, u32 batch_tile, u32 kw) {                 \
        using namespace smelt;                                                                    \
        __shared__ uint2_t wave_keys[4];                                                          \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        uint2_t best = {0u, 0u};                                                                  \
        float best_raw = __builtin_nanf("");                                                      \
        EpiArgmax<ACT> epi{keys, logit_cap, &best, &best_raw, wave_keys};                                    \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        /* one key per token and workgroup: tokens take their own pass over the rows */           \
        for (u32 b = lo; b < hi; ++b) {                                                           \
            if (b != lo) __syncthreads();                                                         \
            mfma_matvec_body<MvU4, ACT, SC, 1, STREAMV, true>(mats, X, rows, cols, cols / 2, kw, b, b + 1, epi); \
        }                                                                                         \
    }

SMELT_AFFINE_MM_KERNELS(f16, smelt::F16, smelt::F16, stream, true)
SMELT_AFFINE_MM_KERNELS(f16, smelt::F16, smelt::F16, split, false)
SMELT_AFFINE_MM_KERNELS(bf16, smelt::BF16, smelt::BF16, stream, true)
SMELT_AFFINE_MM_KERNELS(bf16, smelt::BF16, smelt::BF16, split, false)

// Signed g128 formats (scales are fp16; no bias plane).  Same argument lists as the vector-ALU
// kernels of the pipelines, followed by kw.  The ternary "affine" pipelines bind the scale plane
// a second time where MLX binds a bias plane; it is ignored as in the vector-ALU kernels.
#define SMELT_SIGNED_MM_KERNELS(FN, FMT, T, ACT, MODE, STREAMV)                                   \
    SMELT_KERNEL void smelt_signed_##FN##_mm_matvec_##MODE##_##T(                                 \
        const u8* C, const u16* S, const u16* X, u16* Y, u32 rows, u32 cols, u32 kw) {            \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        mfma_matvec_body<FMT, ACT, F16, 1, STREAMV, true>(mats, X, rows, cols,                    \
                                                          packed_row_stride<typename FMT::Valu>(cols, 128), kw, \
                                                          blockIdx.y, blockIdx.y + 1, epi);       \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_##FN##_mm_matvec_add_##MODE##_##T(                             \
        const u8* C, const u16* S, const u16* X, u16* Y, const u16* res, u32 rows, u32 cols,      \
        u32 kw) {                                                                                 \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                   \
        mfma_matvec_body<FMT, ACT, F16, 1, STREAMV, true>(mats, X, rows, cols,                    \
                                                          packed_row_stride<typename FMT::Valu>(cols, 128), kw, \
                                                          blockIdx.y, blockIdx.y + 1, epi);       \
    }

#define SMELT_TERAFF_MM_KERNELS(T, ACT, MODE, STREAMV)                                            \
    SMELT_KERNEL void smelt_teraff_mm_matvec_##MODE##_##T(                                        \
        const u8* C, const u16* S, const u16*, const u16* X, u16* Y, u32 rows, u32 cols,          \
        u32 kw) {                                                                                 \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        mfma_matvec_body<MvTer2, ACT, F16, 1, STREAMV, true>(mats, X, rows, cols, cols / 4, kw,   \
                                                             blockIdx.y, blockIdx.y + 1, epi);    \
    }                                                                                             \
    SMELT_KERNEL void smelt_teraff_mm_matvec_add_##MODE##_##T(                                    \
        const u8* C, const u16* S, const u16*, const u16* X, u16* Y, const u16* res, u32 rows,    \
        u32 cols, u32 kw) {                                                                       \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                   \
        mfma_matvec_body<MvTer2, ACT, F16, 1, STREAMV, true>(mats, X, rows, cols, cols / 4, kw,   \
                                                             blockIdx.y, blockIdx.y + 1, epi);    \
    }

#define SMELT_SIGNED_MM_ALL(T, ACT)                                                               \
    SMELT_SIGNED_MM_KERNELS(binary, smelt::MvBin, T, ACT, stream, true)                           \
    SMELT_SIGNED_MM_KERNELS(binary, smelt::MvBin, T, ACT, split, false)                           \
    SMELT_SIGNED_MM_KERNELS(ternary, smelt::MvTer2, T, ACT, stream, true)                         \
    SMELT_SIGNED_MM_KERNELS(ternary, smelt::MvTer2, T, ACT, split, false)                         \
    SMELT_TERAFF_MM_KERNELS(T, ACT, stream, true)                                                 \
    SMELT_TERAFF_MM_KERNELS(T, ACT, split, false)

SMELT_SIGNED_MM_ALL(f16, smelt::F16)
SMELT_SIGNED_MM_ALL(bf16, smelt::BF16)
