// __global__ entry points for the quantized matvec family.  Argument order of every kernel is
// the binding order of the Smelt dispatch record that drives it (buffers and 4-byte constants
// by ascending binding index), followed by the shape arguments the pipeline table appends.
#pragma once
#include <type_traits>
#include "matvec.hpp"
#include "misc_kernels.hpp"

namespace smelt {

// ---- epilogues ---------------------------------------------------------------------------
// Each epilogue receives the reduced fp32 sums of one (batch, row) for NMAT matrices.

// Epilogues may keep per-thread state; end_chunk() runs on every thread once all rows of a
// batch chunk are done.
struct EpiBase {
    // An epilogue that reads one 16-bit operand per output row can have it fetched together with
    // the row's last weight item instead of after the reduction (single-token launches only).
    static constexpr bool kPrefetch = false;
    // An epilogue of the single-pass kernel that works on a whole row tile with a whole wave
    // (tile(token, row0, rows, lane, sums)) instead of one row per lane.
    static constexpr bool kTile = false;
    __device__ __forceinline__ void end_chunk(int, int) const {}
};

template <class ActT>
struct EpiStore : EpiBase {
    uint16_t* y;
    int rows;
    __device__ __forceinline__ void operator()(int b, int row, const float* v) const {
        y[(size_t)b * rows + row] = ActT::narrow(v[0]);
    }
};

// project, round to the activation type, add the residual in that type
template <class ActT>
struct EpiAdd : EpiBase {
    uint16_t* y;
    const uint16_t* residual;
    int rows;
    static constexpr bool kPrefetch = true;
    __device__ __forceinline__ uint16_t prefetch(int b, int row) const { return residual[(size_t)b * rows + row]; }
    __device__ __forceinline__ void finish(int b, int row, const float* v, uint16_t res) const {
        const float projected = ActT::widen(ActT::narrow(v[0]));
        y[(size_t)b * rows + row] = ActT::narrow(projected + ActT::widen(res));
    }
    __device__ __forceinline__ void operator()(int b, int row, const float* v) const {
        finish(b, row, v, residual[(size_t)b * rows + row]);
    }
};

// affine SwiGLU: narrow(gate / (1 + exp(-gate)) * up) on the fp32 sums
template <class ActT>
struct EpiAffineSwiglu : EpiBase {
    uint16_t* y;
    int rows;
    __device__ __forceinline__ void operator()(int b, int row, const float* v) const {
        const float g = v[0], u = v[1];
        y[(size_t)b * rows + row] = ActT::narrow(g / (1.0f + expf(-g)) * u);
    }
};

// GeGLU (lut_matvec.metal:2235-2243): gate and up rounded to the 16-bit type, tanh-form GELU of the
// gate with its argument clamped to +-20, product clamped to the fp16 range
template <class ActT>
struct EpiGeglu : EpiBase {
    uint16_t* y;
    int rows;
    __device__ __forceinline__ void operator()(int b, int row, const float* v) const {
        const float g = ActT::widen(ActT::narrow(v[0])), u = ActT::widen(ActT::narrow(v[1]));
        float inner = 0.7978845608f * (g + 0.044715f * (g * g * g));
        inner = fminf(fmaxf(inner, -20.0f), 20.0f);
        const float gelu = 0.5f * g * (1.0f + tanhf(inner));
        y[(size_t)b * rows + row] = ActT::narrow(fminf(fmaxf(gelu * u, -65504.0f), 65504.0f));
    }
};

// signed SwiGLU: gate and up are first rounded to the activation type and every intermediate
// (exp, 1+e, reciprocal, 1-tail, gate*sigmoid, *up) is materialised in that type
template <class ActT>
struct EpiSignedSwiglu : EpiBase {
    uint16_t* y;
    int rows;
    static __device__ __forceinline__ float rt(float v) { return ActT::widen(ActT::narrow(v)); }
    __device__ __forceinline__ void operator()(int b, int row, const float* v) const {
        const float g = rt(v[0]), u = rt(v[1]);
        const float e = rt(expf(fabsf(g)));
        const float denom = rt(1.0f + e);
        const float tail = rt(1.0f / denom);
        const float sig = g < 0.0f ? tail : rt(1.0f - tail);
        const float act = rt(g * sig);
        y[(size_t)b * rows + row] = ActT::narrow(act * u);
    }
};

template <class ActT>
struct EpiDual : EpiBase {
    uint16_t* y1;
    uint16_t* y2;
    int rows;
    __device__ __forceinline__ void operator()(int b, int row, const float* v) const {
        y1[(size_t)b * rows + row] = ActT::narrow(v[0]);
        y2[(size_t)b * rows + row] = ActT::narrow(v[1]);
    }
};

// two projections, each rounded to the activation type and added to its own residual in that type
// (fused_dual_affine_matvec_add_fixed_rows4, lut_matvec.metal:4660-4733)
template <class ActT>
struct EpiDualAdd : EpiBase {
    uint16_t* y1;
    uint16_t* y2;
    const uint16_t* r1;
    const uint16_t* r2;
    int rows;
    __device__ __forceinline__ void operator()(int b, int row, const float* v) const {
        const size_t at = (size_t)b * rows + row;
        y1[at] = ActT::narrow(ActT::widen(ActT::narrow(v[0])) + ActT::widen(r1[at]));
        y2[at] = ActT::narrow(ActT::widen(ActT::narrow(v[1])) + ActT::widen(r2[at]));
    }
};

// ---- workgroup body ------------------------------------------------------------------------
//
// A wave walks its row tiles (grid-stride, so any grid covers every row) as a flat sequence of
// work items (tile, unit step).  Items are software-pipelined two deep: the loads of items q+1
// and q+2 are in flight while item q is computed, and the loads of the first two items are issued
// before the activations are staged, so a small matrix pays one memory latency, not two.

template <class F, class ActT, class ScaleT, int R, int MB, int NMAT, int L, class Epi>
__device__ __forceinline__ void run_tiles(const MatPtrs (&mats)[NMAT], const uint16_t* x, int rows,
                                          int cols, int U, int row_stride, int gpr, int gshift,
                                          int batch_lo, int batch_hi, uint4_t* lds_pairs,
                                          float* lds_corr, float* lds_xsum, const uint16_t* lut,
                                          const Epi& epi, const uint16_t* x2 = nullptr, int nplanes = 0,
                                          const NormScale& ns = NormScale{}) {
    constexpr int S = kWave / L;
    constexpr int TILE = S * R;
    const int waves = blockDim.x / kWave;
    // the wave index is uniform over the wave; saying so keeps the tile walk on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane & (L - 1);
    const int side = lane / L;
    const int tiles = (rows + TILE - 1) / TILE;
    const int nit = (U + L - 1) / L;
    const int first = blockIdx.x * waves + wave;
    const int stride = gridDim.x * waves;
    const int my_tiles = first < tiles ? (tiles - first + stride - 1) / stride : 0;
    const int nq = my_tiles * nit;
    const LaneRows<R> lane_rows(side * R, row_stride, gpr);

    for (int b0 = batch_lo; b0 < batch_hi; b0 += MB) {
        const int nb = batch_hi - b0 < MB ? batch_hi - b0 : MB;
        ItemRegs<R, NMAT> regs_a, regs_b;
        // (tile, step) of the item being computed and of the item being prefetched
        int tile_c = first, it_c = 0, tile_n = first, it_n = 0;
        auto load = [&](ItemRegs<R, NMAT>& dst) {
            const int u = sub + L * it_n;
            const int row0 = tile_n * TILE;
            if (u < U) load_item<F, R, NMAT>(mats, row0, TILE, rows, lane_rows, u, row_stride, gpr, gshift, dst);
            if constexpr (Epi::kPrefetch && MB == 1) {
                if (it_n == nit - 1 && sub == L - 1) {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const int rr = row0 + side * R + r;
                        dst.res[r] = epi.prefetch(b0, rr < rows ? rr : rows - 1);
                    }
                }
            }
            if (++it_n == nit) { it_n = 0; tile_n += stride; }
        };
        if (nq > 0) load(regs_a);
        if (nq > 1) load(regs_b);
        if (b0 != batch_lo) __syncthreads();
        stage_activations<F, ActT, MB>(x, cols, U, b0, nb, lds_pairs, lds_corr, lds_xsum, x2, nplanes, ns);
        __syncthreads();

        // activation registers held across the walk when the lane's unit never changes
        constexpr bool kHoldX = MB == 1 && !F::kBitplanes && FmtGeom<F>::kChunksPerUnit * 4 <= 16;
        XUnit<F> xu;
        if constexpr (kHoldX) {
            if (nit == 1 && sub < U) load_xunit<F>(xu, 0, sub, U, lds_pairs, lds_corr, lds_xsum);
        }

        float acc[NMAT][R][MB];
        auto step = [&](ItemRegs<R, NMAT>& cur, int q) {
            if (it_c == 0) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int r = 0; r < R; ++r)
#pragma unroll
                        for (int b = 0; b < MB; ++b) acc[m][r][b] = 0.0f;
            }
            const int u = sub + L * it_c;
            if (u < U) {
                if constexpr (kHoldX) {
                    if (nit > 1) load_xunit<F>(xu, 0, u, U, lds_pairs, lds_corr, lds_xsum);
                    compute_unit<F, ScaleT, R, MB, NMAT>(cur, xu, 0, u, gshift, lut, acc);
                } else {
                    compute_item<F, ScaleT, R, MB, NMAT>(cur, u, U, gshift, lds_pairs, lds_corr, lds_xsum, lut, acc);
                }
            }
            if (it_c == nit - 1) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int r = 0; r < R; ++r)
#pragma unroll
                        for (int b = 0; b < MB; ++b) acc[m][r][b] = group_sum_last<L>(acc[m][r][b]);
                if (sub == L - 1) {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const int row = tile_c * TILE + side * R + r;
                        if (row < rows) {
#pragma unroll
                            for (int b = 0; b < MB; ++b) {
                                if (b < nb) {
                                    float v[NMAT];
#pragma unroll
                                    for (int m = 0; m < NMAT; ++m) v[m] = acc[m][r][b];
                                    if constexpr (Epi::kPrefetch && MB == 1) epi.finish(b0 + b, row, v, cur.res[r]);
                                    else epi(b0 + b, row, v);
                                }
                            }
                        }
                    }
                }
                it_c = 0;
                tile_c += stride;
            } else {
                ++it_c;
            }
            if (q + 2 < nq) load(cur);  // refill the registers just consumed: two items stay in flight
        };
        for (int q = 0; q < nq; q += 2) {
            step(regs_a, q);
            if (q + 1 < nq) step(regs_b, q + 1);
        }
        epi.end_chunk(b0, nb);
    }
}

// Covers batch rows [batch_lo, batch_hi) in chunks of MB with the activations of one chunk
// resident in LDS.  x is [batch, cols]; row_stride is the byte stride of one packed row.
template <class F, class ActT, class ScaleT, int R, int MB, int NMAT, class Epi>
__device__ __forceinline__ void matvec_body(const MatPtrs (&mats)[NMAT], const uint16_t* x,
                                            int rows, int cols, int row_stride, int group,
                                            int batch_lo, int batch_hi, const Epi& epi,
                                            const uint16_t* x2 = nullptr, int nplanes = 0,
                                            const NormScale& ns = NormScale{}) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int U = row_stride / 16;
    const int gshift = ilog2((uint32_t)group);
    const int gpr = (cols + group - 1) / group;
    uint4_t* lds_pairs = reinterpret_cast<uint4_t*>(smem);
    float* lds_corr = reinterpret_cast<float*>(smem + lds_pairs_bytes<F>(U, MB));
    float* lds_xsum = lds_corr + (size_t)MB * U * FmtGeom<F>::kCorrStride;
    uint16_t* lut = reinterpret_cast<uint16_t*>(lds_xsum + (size_t)MB * U * FmtGeom<F>::kCorrStride);
    if (F::kPerDwordScale)  // decode table; visible to every wave after the staging barrier
        for (uint32_t i = threadIdx.x; i < 256; i += blockDim.x) lut[i] = trit5_lut_entry(i);
    // A grid with more waves than there are R-row tiles asks for finer work items: such launches
    // (small matrices, where one wave per SIMD would otherwise chew through R rows serially) run
    // one row per wave slot, which shortens the latency-bound tail of the kernel.
    const int total_waves = (int)(gridDim.x * (blockDim.x / kWave));
    auto go = [&](auto lanes) {
        constexpr int L = decltype(lanes)::value;
        if constexpr (R > 1 && MB == 1) {
            const int tiles = (rows + (kWave / L) * R - 1) / ((kWave / L) * R);
            if (tiles < total_waves) {
                run_tiles<F, ActT, ScaleT, 1, MB, NMAT, L>(mats, x, rows, cols, U, row_stride, gpr, gshift, batch_lo, batch_hi, lds_pairs, lds_corr, lds_xsum, lut, epi, x2, nplanes, ns);
                return;
            }
        }
        run_tiles<F, ActT, ScaleT, R, MB, NMAT, L>(mats, x, rows, cols, U, row_stride, gpr, gshift, batch_lo, batch_hi, lds_pairs, lds_corr, lds_xsum, lut, epi, x2, nplanes, ns);
    };
    if (U > 32) go(std::integral_constant<int, 64>{});
    else if (U > 16) go(std::integral_constant<int, 32>{});
    else go(std::integral_constant<int, 16>{});
}

template <class F>
__device__ __forceinline__ int packed_row_stride(int cols, int group) {
    if (F::kPerDwordScale) return (((cols + 4) / 5) + 15) & ~15;  // trit5: 5 digits per byte, 16-byte rows
    const int padded = F::kHasBias ? cols : (cols + group - 1) / group * group;
    return (padded * F::kBitsPerCode + 7) / 8;
}

}  // namespace smelt

// ---- entry points ---------------------------------------------------------------------------
#define SMELT_KERNEL extern "C" __global__ __launch_bounds__(256)
// single-token streaming kernels: registers are held to what five waves per SIMD allow
#define SMELT_KERNEL_W5 extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(5)))
using u16 = uint16_t;
using u8 = uint8_t;
using u32 = uint32_t;

#define SMELT_AFFINE_KERNELS(T, ACT, SC)                                                          \
    SMELT_KERNEL_W5 void smelt_affine_matvec_##T(const u8* W, const u16* S, const u16* B,            \
                                              const u16* x, u16* y, u32 rows, u32 cols,           \
                                              u32 group) {                                        \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, y, (int)rows};                                                          \
        matvec_body<FmtU4, ACT, SC, 2, 1, 1>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi);                    \
    }                                                                                             \
    SMELT_KERNEL_W5 void smelt_affine_matvec_add_##T(const u8* W, const u16* S, const u16* B,        \
                                                  const u16* x, u16* y, const u16* res, u32 rows, \
                                                  u32 cols, u32 group) {                          \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiAdd<ACT> epi{{}, y, res, (int)rows};                                                       \
        matvec_body<FmtU4, ACT, SC, 2, 1, 1>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi);                    \
    }                                                                                             \
    SMELT_KERNEL_W5 void smelt_affine_gate_up_swiglu_##T(                                         \
        const u8* gW, const u16* gS, const u16* gB, const u8* uW, const u16* uS, const u16* uB,   \
        const u16* x, u16* y, u32 rows, u32 cols, u32 group) {                                    \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiAffineSwiglu<ACT> epi{{}, y, (int)rows};                                                   \
        matvec_body<FmtU4, ACT, SC, 2, 1, 2>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi);                    \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_dual_matvec_##T(                                               \
        const u8* W1, const u16* S1, const u16* B1, const u8* W2, const u16* S2, const u16* B2,   \
        const u16* x, u16* y1, u16* y2, u32 rows, u32 cols, u32 group) {                          \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{W1, S1, B1}, {W2, S2, B2}};                                     \
        EpiDual<ACT> epi{{}, y1, y2, (int)rows};                                                      \
        matvec_body<FmtU4, ACT, SC, 2, 1, 2>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi);                    \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_dual_matvec_add_##T(                                           \
        const u8* W1, const u16* S1, const u16* B1, const u8* W2, const u16* S2, const u16* B2,   \
        const u16* x, u16* y1, u16* y2, const u16* r1, const u16* r2, u32 rows, u32 cols,         \
        u32 group) {                                                                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{W1, S1, B1}, {W2, S2, B2}};                                     \
        EpiDualAdd<ACT> epi{{}, y1, y2, r1, r2, (int)rows};                                       \
        matvec_body<FmtU4, ACT, SC, 2, 1, 2>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi);                    \
    }                                                                                             \
    SMELT_KERNEL_W5 void smelt_affine_gate_up_geglu_##T(                                          \
        const u8* gW, const u16* gS, const u16* gB, const u8* uW, const u16* uS, const u16* uB,   \
        const u16* x, u16* y, u32 rows, u32 cols, u32 group) {                                    \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiGeglu<ACT> epi{{}, y, (int)rows};                                                      \
        matvec_body<FmtU4, ACT, SC, 2, 1, 2>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi);                    \
    }                                                                                             \
    /* norm-scale prologue: rs holds one fp32 scale per token (grid.y) */                         \
    SMELT_KERNEL_W5 void smelt_norm_scale_affine_matvec_##T(                                      \
        const float* rs, const u16* x, const u16* nw, u16* xn, const u8* W, const u16* S,         \
        const u16* B, u16* y, u32 rows, u32 cols, u32 group) {                                    \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, y, (int)rows};                                                      \
        matvec_body<FmtU4, ACT, SC, 2, 1, 1>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi, nullptr, 0,         \
                                             NormScale{rs, nw, xn});                              \
    }                                                                                             \
    SMELT_KERNEL_W5 void smelt_norm_add_scale_affine_matvec_##T(                                  \
        const float* rs, const u16* x, const u16* nw, const u16* res, u16* xn, const u8* W,       \
        const u16* S, const u16* B, u16* y, u32 rows, u32 cols, u32 group) {                      \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, y, (int)rows};                                                      \
        matvec_body<FmtU4, ACT, SC, 2, 1, 1>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi, nullptr, 0,         \
                                             NormScale{rs, nw, xn, res});                         \
    }                                                                                             \
    SMELT_KERNEL void smelt_norm_scale_affine_dual_matvec_##T(                                    \
        const float* rs, const u16* x, const u16* nw, const u8* W1, const u16* S1, const u16* B1, \
        const u8* W2, const u16* S2, const u16* B2, u16* y1, u16* y2, u32 rows, u32 cols,         \
        u32 group) {                                                                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{W1, S1, B1}, {W2, S2, B2}};                                     \
        EpiDual<ACT> epi{{}, y1, y2, (int)rows};                                                  \
        matvec_body<FmtU4, ACT, SC, 2, 1, 2>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi, nullptr, 0,         \
                                             NormScale{rs, nw, nullptr});                         \
    }                                                                                             \
    SMELT_KERNEL_W5 void smelt_norm_scale_affine_gate_up_swiglu_##T(                              \
        const float* rs, const u16* x, const u16* nw, const u8* gW, const u16* gS, const u16* gB, \
        const u8* uW, const u16* uS, const u16* uB, u16* y, u32 rows, u32 cols, u32 group) {      \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiAffineSwiglu<ACT> epi{{}, y, (int)rows};                                               \
        matvec_body<FmtU4, ACT, SC, 2, 1, 2>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi, nullptr, 0,         \
                                             NormScale{rs, nw, nullptr});                         \
    }                                                                                             \
    SMELT_KERNEL_W5 void smelt_norm_scale_affine_gate_up_geglu_##T(                               \
        const float* rs, const u16* x, const u16* nw, const u8* gW, const u16* gS, const u16* gB, \
        const u8* uW, const u16* uS, const u16* uB, u16* y, u32 rows, u32 cols, u32 group) {      \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiGeglu<ACT> epi{{}, y, (int)rows};                                                      \
        matvec_body<FmtU4, ACT, SC, 2, 1, 2>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group,        \
                                             blockIdx.y, blockIdx.y + 1, epi, nullptr, 0,         \
                                             NormScale{rs, nw, nullptr});                         \
    }

// Norm fused into its consumer (fused_norm_matvec.metal:19-297).  The reference lets workgroup 0
// compute the RMS scale and makes every other workgroup spin on a flag; here each workgroup sums the
// squares of the (cache-resident, few-KB) row itself while its first weight loads are in flight, so no
// workgroup waits on another.  Workgroup 0
// still publishes the scale and the ready flag in the scratch pair the record binds.
#define SMELT_AFFINE_FUSED_NORM(T, ACT, SC)                                                       \
    SMELT_KERNEL void smelt_atomic_norm_affine_matvec_##T(                                        \
        const u16* x, const u16* nw, u16* xn, const u8* W, const u16* S, const u16* B, u16* y,    \
        float* scratch, u32 rows, float eps, u32 cols, u32 group) {                               \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, y, (int)rows};                                                      \
        matvec_body<FmtU4, ACT, SC, 2, 1, 1>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group, 0, 1,  \
                                             epi, nullptr, 0,                                     \
                                             NormScale{nullptr, nw, xn, nullptr, eps, scratch});  \
    }                                                                                             \
    SMELT_KERNEL void smelt_atomic_norm_affine_gate_up_swiglu_##T(                                \
        const u16* x, const u16* nw, const u8* gW, const u16* gS, const u16* gB, const u8* uW,    \
        const u16* uS, const u16* uB, u16* y, float* scratch, u32 rows, float eps, u32 cols,      \
        u32 group) {                                                                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiAffineSwiglu<ACT> epi{{}, y, (int)rows};                                               \
        matvec_body<FmtU4, ACT, SC, 2, 1, 2>(mats, x, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group, 0, 1,  \
                                             epi, nullptr, 0,                                     \
                                             NormScale{nullptr, nw, nullptr, nullptr, eps,        \
                                                       scratch});                                 \
    }

#define SMELT_AFFINE_BATCHED(T, ACT, SC, MBV)                                                     \
    SMELT_KERNEL void smelt_affine_matvec_batched_mb##MBV##_##T(                                  \
        const u8* W, const u16* S, const u16* B, const u16* X, u16* Y, u32 batch, u32 rows,       \
        u32 cols, u32 group, u32 batch_tile) {                                                    \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                          \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        matvec_body<FmtU4, ACT, SC, 4, MBV, 1>(mats, X, rows, cols,                               \
                                               packed_row_stride<FmtU4>(cols, group), group, lo,  \
                                               hi, epi);                                          \
    }                                                                                             \
    SMELT_KERNEL void smelt_norm_scale_affine_matvec_batched_mb##MBV##_##T(                       \
        const float* rs, const u16* X, const u16* nw, u16* XN, const u8* W, const u16* S,         \
        const u16* B, u16* Y, u32 batch, u32 rows, u32 cols, u32 group, u32 batch_tile) {         \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        matvec_body<FmtU4, ACT, SC, 4, MBV, 1>(mats, X, rows, cols,                               \
                                               packed_row_stride<FmtU4>(cols, group), group, lo,  \
                                               hi, epi, nullptr, 0, NormScale{rs, nw, XN});       \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_matvec_add_batched_mb##MBV##_##T(                              \
        const u8* W, const u16* S, const u16* B, const u16* X, u16* Y, const u16* res, u32 batch, \
        u32 rows, u32 cols, u32 group, u32 batch_tile) {                                          \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                       \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        matvec_body<FmtU4, ACT, SC, 4, MBV, 1>(mats, X, rows, cols,                               \
                                               packed_row_stride<FmtU4>(cols, group), group, lo,  \
                                               hi, epi);                                          \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_gate_up_geglu_batched_mb##MBV##_##T(                           \
        const u8* gW, const u16* gS, const u16* gB, const u8* uW, const u16* uS, const u16* uB,   \
        const u16* X, u16* Y, u32 batch, u32 rows, u32 cols, u32 group, u32 batch_tile) {         \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiGeglu<ACT> epi{{}, Y, (int)rows};                                                      \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        matvec_body<FmtU4, ACT, SC, 2, MBV, 2>(mats, X, rows, cols,                               \
                                               packed_row_stride<FmtU4>(cols, group), group, lo,  \
                                               hi, epi);                                          \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_dual_matvec_batched_mb##MBV##_##T(                             \
        const u8* W1, const u16* S1, const u16* B1, const u8* W2, const u16* S2, const u16* B2,   \
        const u16* X, u16* Y1, u16* Y2, u32 batch, u32 rows, u32 cols, u32 group,                 \
        u32 batch_tile) {                                                                         \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{W1, S1, B1}, {W2, S2, B2}};                                     \
        EpiDual<ACT> epi{{}, Y1, Y2, (int)rows};                                                  \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        matvec_body<FmtU4, ACT, SC, 2, MBV, 2>(mats, X, rows, cols,                               \
                                               packed_row_stride<FmtU4>(cols, group), group, lo,  \
                                               hi, epi);                                          \
    }                                                                                             \
    SMELT_KERNEL void smelt_affine_gate_up_swiglu_batched_mb##MBV##_##T(                          \
        const u8* gW, const u16* gS, const u16* gB, const u8* uW, const u16* uS, const u16* uB,   \
        const u16* X, u16* Y, u32 batch, u32 rows, u32 cols, u32 group, u32 batch_tile) {         \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gW, gS, gB}, {uW, uS, uB}};                                     \
        EpiAffineSwiglu<ACT> epi{{}, Y, (int)rows};                                                   \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        matvec_body<FmtU4, ACT, SC, 2, MBV, 2>(mats, X, rows, cols,                               \
                                               packed_row_stride<FmtU4>(cols, group), group, lo,  \
                                               hi, epi);                                          \
    }

// Signed kernels: batch row = blockIdx.y (M = 1 family) or a tile of 4 rows (_b4 family).
#define SMELT_SIGNED_KERNELS(FN, FMT, T, ACT)                                                     \
    SMELT_KERNEL void smelt_signed_##FN##_matvec_##T(const u8* C, const u16* S, const u16* X,     \
                                                     u16* Y, u32 rows, u32 cols) {                \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                          \
        matvec_body<FMT, ACT, F16, 4, 1, 1>(mats, X, rows, cols,                                  \
                                            packed_row_stride<FMT>(cols, 128), 128, blockIdx.y,   \
                                            blockIdx.y + 1, epi);                                 \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_##FN##_matvec_add_##T(const u8* C, const u16* S, const u16* X, \
                                                         u16* Y, const u16* res, u32 rows,        \
                                                         u32 cols) {                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                       \
        matvec_body<FMT, ACT, F16, 4, 1, 1>(mats, X, rows, cols,                                  \
                                            packed_row_stride<FMT>(cols, 128), 128, blockIdx.y,   \
                                            blockIdx.y + 1, epi);                                 \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_##FN##_gate_up_swiglu_##T(                                     \
        const u8* gC, const u16* gS, const u8* uC, const u16* uS, const u16* X, u16* Y, u32 rows, \
        u32 cols) {                                                                               \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gC, gS, nullptr}, {uC, uS, nullptr}};                           \
        EpiSignedSwiglu<ACT> epi{{}, Y, (int)rows};                                                   \
        matvec_body<FMT, ACT, F16, 2, 1, 2>(mats, X, rows, cols,                                  \
                                            packed_row_stride<FMT>(cols, 128), 128, blockIdx.y,   \
                                            blockIdx.y + 1, epi);                                 \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_##FN##_matvec_b4_##T(const u8* C, const u16* S, const u16* X,  \
                                                        u16* Y, u32 rows, u32 cols, u32 batch) {  \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                          \
        const u32 lo = blockIdx.y * 4;                                                            \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + 4 < batch ? lo + 4 : batch;                                           \
        matvec_body<FMT, ACT, F16, 4, 2, 1>(mats, X, rows, cols,                                  \
                                            packed_row_stride<FMT>(cols, 128), 128, lo, hi, epi); \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_##FN##_gate_up_swiglu_b4_##T(                                  \
        const u8* gC, const u16* gS, const u8* uC, const u16* uS, const u16* X, u16* Y, u32 rows, \
        u32 cols, u32 batch) {                                                                    \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gC, gS, nullptr}, {uC, uS, nullptr}};                           \
        EpiSignedSwiglu<ACT> epi{{}, Y, (int)rows};                                                   \
        const u32 lo = blockIdx.y * 4;                                                            \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + 4 < batch ? lo + 4 : batch;                                           \
        matvec_body<FMT, ACT, F16, 2, 2, 2>(mats, X, rows, cols,                                  \
                                            packed_row_stride<FMT>(cols, 128), 128, lo, hi, epi); \
    }

// Signed activation views: the activation operand is (planes, scales) instead of x
// (signed_{binary,ternary}_bitplane_i{N}_{matvec,matvec_add,gate_up_swiglu}_g128_rows8,
//  signed_quant.metal:1564-2260); batch row = blockIdx.y.
#define SMELT_BITPLANE_KERNELS(FN, FMT, T, ACT)                                                   \
    SMELT_KERNEL void smelt_signed_##FN##_bitplane_matvec_##T(                                    \
        const u8* C, const u16* S, const u32* P, const u16* AS, u16* Y, u32 rows, u32 cols,       \
        u32 nplanes) {                                                                            \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        matvec_body<FMT, ACT, F16, 4, 1, 1>(mats, reinterpret_cast<const u16*>(P), rows, cols,    \
                                            packed_row_stride<FMT>(cols, 128), 128, blockIdx.y,   \
                                            blockIdx.y + 1, epi, AS, (int)nplanes);               \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_##FN##_bitplane_matvec_add_##T(                                \
        const u8* C, const u16* S, const u32* P, const u16* AS, u16* Y, const u16* res, u32 rows, \
        u32 cols, u32 nplanes) {                                                                  \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                   \
        matvec_body<FMT, ACT, F16, 4, 1, 1>(mats, reinterpret_cast<const u16*>(P), rows, cols,    \
                                            packed_row_stride<FMT>(cols, 128), 128, blockIdx.y,   \
                                            blockIdx.y + 1, epi, AS, (int)nplanes);               \
    }                                                                                             \
    /* prompt rows: `tile` tokens per grid row, four at a time share every weight load          \
       (signed_binary_bitplane_i{N}_matvec_g128_rows8_batched_b{4,8,16}, :1350-1562) */          \
    SMELT_KERNEL void smelt_signed_##FN##_bitplane_matvec_batched_##T(                            \
        const u8* C, const u16* S, const u32* P, const u16* AS, u16* Y, u32 rows, u32 cols,       \
        u32 batch, u32 nplanes, u32 tile) {                                                       \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        const u32 lo = blockIdx.y * tile;                                                         \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + tile < batch ? lo + tile : batch;                                     \
        matvec_body<FMT, ACT, F16, 4, 4, 1>(mats, reinterpret_cast<const u16*>(P), rows, cols,    \
                                            packed_row_stride<FMT>(cols, 128), 128, lo, hi, epi,  \
                                            AS, (int)nplanes);                                    \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_##FN##_bitplane_bank4_matvec_##T(                              \
        const u8* C, const u16* S, const u32* P, const u16* AS, u16* y0, u16* y1, u16* y2,        \
        u16* y3, u32 rows0, u32 rows1, u32 rows2, u32 rows3, u32 cols, u32 nplanes) {             \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiBank4<ACT> epi{{}, {y0, y1, y2, y3}, {rows0, rows1, rows2, rows3}};                    \
        matvec_body<FMT, ACT, F16, 4, 1, 1>(mats, reinterpret_cast<const u16*>(P),                \
                                            rows0 + rows1 + rows2 + rows3, cols,                  \
                                            packed_row_stride<FMT>(cols, 128), 128, 0, 1, epi,    \
                                            AS, (int)nplanes);                                    \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_##FN##_bitplane_gate_up_swiglu_##T(                            \
        const u8* gC, const u16* gS, const u8* uC, const u16* uS, const u32* P, const u16* AS,    \
        u16* Y, u32 rows, u32 cols, u32 nplanes) {                                                \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gC, gS, nullptr}, {uC, uS, nullptr}};                           \
        EpiSignedSwiglu<ACT> epi{{}, Y, (int)rows};                                               \
        matvec_body<FMT, ACT, F16, 2, 1, 2>(mats, reinterpret_cast<const u16*>(P), rows, cols,    \
                                            packed_row_stride<FMT>(cols, 128), 128, blockIdx.y,   \
                                            blockIdx.y + 1, epi, AS, (int)nplanes);               \
    }

// Binary projection banks on the direct (fp16 activation) path, signed_quant.metal:2638-2935:
//   packed bank   one code slab whose rows belong to 2 or 4 consumers in order
//   dual/virtual  two separate matrices driven as one row space (rows of the first, then the second)
// Five-digit-byte projection bank: the binary packed bank's argument list over trit5 rows (this format is
// not in the reference; the bank is what lets q, k and v share one launch as they do for the other formats).
#define SMELT_TRIT5_BANK_KERNELS(T, ACT)                                                          \
    SMELT_KERNEL void smelt_signed_trit5_packed_bank4_matvec_##T(                                 \
        const u8* C, const u16* S, const u16* X, u16* y0, u16* y1, u16* y2, u16* y3, u32 rows0,   \
        u32 rows1, u32 rows2, u32 rows3, u32 cols) {                                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiBank4<ACT> epi{{}, {y0, y1, y2, y3}, {rows0, rows1, rows2, rows3}};                    \
        matvec_body<FmtTrit5, ACT, F16, 4, 1, 1>(mats, X, rows0 + rows1 + rows2 + rows3, cols,    \
                                                 packed_row_stride<FmtTrit5>(cols, 128), 128, 0, 1, \
                                                 epi);                                            \
    }

#define SMELT_BINARY_BANK_KERNELS(T, ACT)                                                         \
    SMELT_KERNEL void smelt_signed_binary_packed_bank_matvec_##T(                                 \
        const u8* C, const u16* S, const u16* X, u16* y0, u16* y1, u32 rows0, u32 rows1,          \
        u32 cols) {                                                                               \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiBank4<ACT> epi{{}, {y0, y1, nullptr, nullptr}, {rows0, rows1, 0u, 0u}};                \
        matvec_body<FmtBin, ACT, F16, 4, 1, 1>(mats, X, rows0 + rows1, cols,                      \
                                               packed_row_stride<FmtBin>(cols, 128), 128, 0, 1,   \
                                               epi);                                              \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_binary_packed_bank4_matvec_##T(                                \
        const u8* C, const u16* S, const u16* X, u16* y0, u16* y1, u16* y2, u16* y3, u32 rows0,   \
        u32 rows1, u32 rows2, u32 rows3, u32 cols) {                                              \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiBank4<ACT> epi{{}, {y0, y1, y2, y3}, {rows0, rows1, rows2, rows3}};                    \
        matvec_body<FmtBin, ACT, F16, 4, 1, 1>(mats, X, rows0 + rows1 + rows2 + rows3, cols,      \
                                               packed_row_stride<FmtBin>(cols, 128), 128, 0, 1,   \
                                               epi);                                              \
    }                                                                                             \
    SMELT_KERNEL void smelt_signed_binary_two_matrix_matvec_##T(                                  \
        const u8* C1, const u16* S1, const u8* C2, const u16* S2, const u16* X, u16* y1, u16* y2, \
        u32 rows1, u32 rows2, u32 cols) {                                                         \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C1, S1, nullptr, C2, S2, (int)rows1}};                          \
        EpiBank4<ACT> epi{{}, {y1, y2, nullptr, nullptr}, {rows1, rows2, 0u, 0u}};                \
        matvec_body<FmtBin, ACT, F16, 4, 1, 1>(mats, X, rows1 + rows2, cols,                      \
                                               packed_row_stride<FmtBin>(cols, 128), 128, 0, 1,   \
                                               epi);                                              \
    }

// ---- lm_head: matvec fused with argmax over the rounded logits -------------------------------
namespace smelt {

// Keeps the best (value, index) key per thread; end_chunk() reduces the workgroup and writes one
// partial key for the batch row at partials[batch * gridDim.x + blockIdx.x].
template <class ActT>
struct EpiArgmax {
    static constexpr bool kPrefetch = false;
    uint2_t* partials;
    float logit_cap;
    uint2_t* best;      // one per thread (register-resident in the caller)
    float* best_raw;    // unrounded sum of the row that holds `best`; NaN while there is none
    uint2_t* lds_keys;  // blockDim.x / 64 entries
    // A thread sees its rows in increasing order, and capping and rounding are monotonic, so a row
    // whose raw sum does not exceed the raw sum of the current best can at most tie with it and
    // lose on the index.  Only rows that pass this one comparison (and NaNs) form a key.
    __device__ __forceinline__ void operator()(int, int row, const float* v) const {
        float x = v[0];
        if (!(x <= *best_raw)) {
            const float raw = x;
            if (logit_cap > 0.0f) {
                // cap * tanh(x / cap) as cap * (1 - 2 / (1 + exp(2x / cap))); exp overflow gives +-cap
                const float e = expf(2.0f * x / logit_cap);
                x = logit_cap * (1.0f - 2.0f / (1.0f + e));
            }
            const uint2_t key = argmax_pack_key(ActT::narrow(x), (uint32_t)row);
            if (argmax_key_gt(key, *best)) {
                *best = key;
                *best_raw = raw;  // a NaN keeps every later row on this path, where keys decide
            }
        }
    }
    __device__ __forceinline__ void end_chunk(int b0, int) const {
        const uint2_t k = wave_argmax_key(*best);
        const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
        __syncthreads();
        if (lane == 0) lds_keys[wave] = k;
        __syncthreads();
        if (threadIdx.x == 0) {
            uint2_t b = lds_keys[0];
            for (int w = 1; w < (int)(blockDim.x / kWave); ++w) b = argmax_key_max(b, lds_keys[w]);
            partials[(size_t)b0 * gridDim.x + blockIdx.x] = b;
        }
        *best = uint2_t{0u, 0u};
        *best_raw = __builtin_nanf("");
    }
};

// Projection bank: up to four members share the input and one contiguous slab of code rows and
// scale rows; virtual row r belongs to the member whose row range contains it.
template <class ActT>
struct EpiBank4 : EpiBase {
    uint16_t* y[4];
    uint32_t rows_m[4];
    __device__ __forceinline__ void operator()(int b, int row, const float* v) const {
        uint32_t r = (uint32_t)row;
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            if (r < rows_m[m]) { y[m][(size_t)b * rows_m[m] + r] = ActT::narrow(v[0]); return; }
            r -= rows_m[m];
        }
    }
};

}  // namespace smelt

#define SMELT_AFFINE_ARGMAX(T, ACT, SC)                                                           \
    SMELT_KERNEL void smelt_affine_matvec_argmax_##T(                                             \
        const u8* W, const u16* S, const u16* B, const u16* X, smelt::uint2_t* keys, u32 batch,   \
        float logit_cap, u32 rows, u32 cols, u32 group, u32 batch_tile) {                         \
        using namespace smelt;                                                                    \
        __shared__ uint2_t wave_keys[4];                                                          \
        uint2_t best = {0u, 0u};                                                                  \
        float best_raw = __builtin_nanf("");                                                      \
        EpiArgmax<ACT> epi{keys, logit_cap, &best, &best_raw, wave_keys};                                    \
        const u32 lo = blockIdx.y * batch_tile;                                                   \
        if (lo >= batch) return;                                                                  \
        const u32 hi = lo + batch_tile < batch ? lo + batch_tile : batch;                         \
        /* One key per token and workgroup: tokens take their own pass over the rows.  The        \
           arguments are re-read as opaque values in every pass: otherwise everything derived     \
           from them is hoisted out of the token loop and kept live, which halves the occupancy. */ \
        for (u32 b = lo; b < hi; ++b) {                                                           \
            if (b != lo) __syncthreads();                                                         \
            const u8* w2 = W;                                                                     \
            const u16 *s2 = S, *b2 = B, *x2 = X;                                                  \
            u32 r2 = rows, c2 = cols, g2 = group;                                                 \
            asm volatile("" : "+s"(w2), "+s"(s2), "+s"(b2), "+s"(x2), "+s"(r2), "+s"(c2), "+s"(g2)); \
            const MatPtrs mats[1] = {{w2, s2, b2}};                                               \
            matvec_body<FmtU4, ACT, SC, 4, 1, 1>(mats, x2, r2, c2,                                \
                                                 packed_row_stride<FmtU4>(c2, g2), g2, b, b + 1,  \
                                                 epi);                                            \
        }                                                                                         \
    }

// Decode form of the fused argmax: exactly one token (batch == 1, one grid row), so no token loop
// and the register footprint of the plain matvec.
#define SMELT_AFFINE_ARGMAX_SINGLE(T, ACT, SC)                                                    \
    SMELT_KERNEL_W5 void smelt_affine_matvec_argmax_single_##T(                                      \
        const u8* W, const u16* S, const u16* B, const u16* X, smelt::uint2_t* keys, u32,         \
        float logit_cap, u32 rows, u32 cols, u32 group, u32) {                                    \
        using namespace smelt;                                                                    \
        __shared__ uint2_t wave_keys[4];                                                          \
        uint2_t best = {0u, 0u};                                                                  \
        float best_raw = __builtin_nanf("");                                                      \
        EpiArgmax<ACT> epi{keys, logit_cap, &best, &best_raw, wave_keys};                         \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        matvec_body<FmtU4, ACT, SC, 2, 1, 1>(mats, X, rows, cols,                                 \
                                             packed_row_stride<FmtU4>(cols, group), group, 0, 1,  \
                                             epi);                                                \
    }

// Affine projection bank: up to four same-input members whose packed rows, scale rows and bias
// rows each form one contiguous slab in member order (q | k | v ...), driven as one matvec over
// the virtual row space; member m's rows go to output m.
#define SMELT_AFFINE_BANK(T, ACT, SC)                                                             \
    SMELT_KERNEL void smelt_affine_bank4_matvec_##T(                                              \
        const u8* W, const u16* S, const u16* B, const u16* x, u16* y0, u16* y1, u16* y2,         \
        u16* y3, u32 rows0, u32 rows1, u32 rows2, u32 rows3, u32 cols, u32 group) {               \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{W, S, B}};                                                      \
        EpiBank4<ACT> epi{{}, {y0, y1, y2, y3}, {rows0, rows1, rows2, rows3}};                    \
        matvec_body<FmtU4, ACT, SC, 4, 1, 1>(mats, x, rows0 + rows1 + rows2 + rows3, cols,        \
                                             packed_row_stride<FmtU4>(cols, group), group, 0, 1,  \
                                             epi);                                                \
    }

// The ternary "affine" pipelines bind the scale plane a second time where MLX binds a bias
// plane (bias = -scale); the arithmetic here is scale * (code - 1), so it is ignored.
#define SMELT_TERAFF_KERNELS(T, ACT)                                                              \
    SMELT_KERNEL void smelt_teraff_matvec_##T(const u8* C, const u16* S, const u16*,              \
                                              const u16* X, u16* Y, u32 rows, u32 cols) {         \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiStore<ACT> epi{{}, Y, (int)rows};                                                      \
        matvec_body<FmtTer2, ACT, F16, 4, 1, 1>(mats, X, rows, cols,                              \
                                                packed_row_stride<FmtTer2>(cols, 128), 128,       \
                                                blockIdx.y, blockIdx.y + 1, epi);                 \
    }                                                                                             \
    SMELT_KERNEL void smelt_teraff_matvec_add_##T(const u8* C, const u16* S, const u16*,          \
                                                  const u16* X, u16* Y, const u16* res, u32 rows, \
                                                  u32 cols) {                                     \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiAdd<ACT> epi{{}, Y, res, (int)rows};                                                   \
        matvec_body<FmtTer2, ACT, F16, 4, 1, 1>(mats, X, rows, cols,                              \
                                                packed_row_stride<FmtTer2>(cols, 128), 128,       \
                                                blockIdx.y, blockIdx.y + 1, epi);                 \
    }                                                                                             \
    SMELT_KERNEL void smelt_teraff_gate_up_swiglu_##T(                                            \
        const u8* gC, const u16* gS, const u16*, const u8* uC, const u16* uS, const u16*,         \
        const u16* X, u16* Y, u32 rows, u32 cols) {                                               \
        using namespace smelt;                                                                    \
        const MatPtrs mats[2] = {{gC, gS, nullptr}, {uC, uS, nullptr}};                           \
        EpiSignedSwiglu<ACT> epi{{}, Y, (int)rows};                                               \
        matvec_body<FmtTer2, ACT, F16, 2, 1, 2>(mats, X, rows, cols,                              \
                                                packed_row_stride<FmtTer2>(cols, 128), 128,       \
                                                blockIdx.y, blockIdx.y + 1, epi);                 \
    }                                                                                             \
    SMELT_KERNEL void smelt_teraff_bank4_matvec_##T(                                              \
        const u8* C, const u16* S, const u16*, const u16* X, u16* y0, u16* y1, u16* y2, u16* y3,  \
        u32 rows0, u32 rows1, u32 rows2, u32 rows3, u32 cols) {                                   \
        using namespace smelt;                                                                    \
        const MatPtrs mats[1] = {{C, S, nullptr}};                                                \
        EpiBank4<ACT> epi{{}, {y0, y1, y2, y3}, {rows0, rows1, rows2, rows3}};                    \
        const u32 rows = rows0 + rows1 + rows2 + rows3;                                           \
        matvec_body<FmtTer2, ACT, F16, 4, 1, 1>(mats, X, rows, cols,                              \
                                                packed_row_stride<FmtTer2>(cols, 128), 128, 0, 1, \
                                                epi);                                             \
    }
