// Streaming small-batch quantized matmul for gfx950:  Y[M, N] = X[M, K] * W[N, K]^T for up to 16
// tokens per pass, affine u4 weights with one scale group per 64 (or 128) columns, rows of a multiple of 256 (512) columns.
//
// At this batch the weights still stream from HBM once and the arithmetic is small; the kernel is
// the multi-token form of the single-pass matvec.  A wave owns 16 * RT weight rows and, per round,
// P pairs of scale groups (128 columns each); it issues every load of a round (scales first, then
// activations and weights pair by pair) before it does anything else.  K is split over the waves
// of a workgroup (up to sixteen) and, for long rows, over rounds; the waves' partial sums meet in
// LDS and no workspace is used.
//
// Memory side: every load instruction covers whole runs of memory with adjacent lanes (four lanes
// on the 64 bytes a row holds for a pair, sixteen lanes on the 256 bytes of a token), because a
// load whose 64 lanes touch 64 different cache lines costs the memory pipeline four to eight
// times the cycles.  The MFMA wants another lane order, so each pair goes through a wave-private
// LDS buffer: written as loaded, read back in operand order.  LDS operations of one wave execute
// in order, so the exchange needs no barrier.
//
// Arithmetic: v_mfma_f32_16x16x32_{f16,bf16}, tokens as the A operand (rows), sixteen weight rows
// as the B operand (columns).
//   * MFMA lane (n = lane % 16, q = lane / 16) takes the eight bytes of row n that hold columns
//     16 q .. 16 q + 15 of a scale group: its two dwords are the lane's share of the B operands
//     of the group's two MFMAs.  A packed dword becomes four operand registers with three shifts
//     and four AND-ORs: codes (r, r + 4) of the dword land at one mantissa bit of the two halves
//     of register r as (base + code), exact in the 16-bit float type.
//   * The activations enter in their own type, unconverted; each 16-byte run is brought into the
//     operand order of the codes (0, 4, 1, 5, 2, 6, 3, 7) with four byte permutes.
//   * One more MFMA pair per group, against a B operand of ones, gives every lane the plain sum
//     of its four tokens' activations over the group; with it
//         y += s * sum((base + code) * x) + (b - base * s) * sum(x)
//     applies the group's scale and bias in fp32 on the accumulators (each lane owns one weight
//     row, so both are one scalar per lane).
// Tokens past the batch and rows past the matrix re-read the last valid one and are never stored;
// pairs past the end of a row re-read the last pair under a zero scale.
#pragma once
#include <type_traits>
#include "mm1_matvec.hpp"

namespace smelt {

template <class ActT>
struct QsCodes;
template <>
struct QsCodes<BF16> { static constexpr int kPos = 0; };   // base 128
template <>
struct QsCodes<F16> { static constexpr int kPos = 4; };    // base 64

template <class ActT>
struct QsOperand {
    using E = Elem16<ActT>;
    static constexpr int kPos = QsCodes<ActT>::kPos;
    static constexpr uint32_t kMask = (0xFu << kPos) | (0xFu << (kPos + 16));
    static constexpr uint32_t kBaseHalf = (uint32_t)(E::kExpBias + E::kMant - kPos) << E::kMant;
    static constexpr uint32_t kBasePair = kBaseHalf | (kBaseHalf << 16);
    static constexpr float kBase = (float)(1 << (E::kMant - kPos));
    static constexpr uint32_t kOnePair = ((uint32_t)E::kExpBias << E::kMant) | ((uint32_t)E::kExpBias << (E::kMant + 16));
    // eight codes of one dword -> B operand registers; register r holds codes (r, r + 4)
    static __device__ __forceinline__ uint4_t codes(uint32_t c) {
        uint32_t r[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int sh = 4 * j - kPos;
            const uint32_t src = sh == 0 ? c : (sh > 0 ? c >> sh : c << -sh);
            r[j] = and_or(src, kMask, kBasePair);
        }
        return uint4_t{r[0], r[1], r[2], r[3]};
    }
    // eight consecutive activations -> A operand registers in the order of the codes
    static __device__ __forceinline__ uint4_t activations(const uint4_t& x) {
        return uint4_t{__builtin_amdgcn_perm(x.z, x.x, 0x05040100u), __builtin_amdgcn_perm(x.z, x.x, 0x07060302u),
                       __builtin_amdgcn_perm(x.w, x.y, 0x05040100u), __builtin_amdgcn_perm(x.w, x.y, 0x07060302u)};
    }
};

// LDS: (scale, bias - base * scale) of every row of the tile and every group plus one zero column,
// then one staging buffer per wave: 16 token rows of one pair (256 B + 16 B of padding each) and
// 16 weight rows per tile (64 B + 8 B of padding each).  A wave's partial sums (1 KB per tile) go
// to its own staging buffer once it is done with it.
constexpr int kQsTokens = 16;          // tokens per pass (blockIdx.y)
constexpr int kQsXStride = 272;        // bytes per staged token row
constexpr int kQsWStride = 72;         // bytes per staged weight row
__host__ __device__ constexpr size_t qms_scale_lds_bytes(int tiles, int groups) { return (size_t)tiles * 16 * (groups + 1) * 8; }
__host__ __device__ constexpr size_t qms_wave_lds_bytes(int tiles, int token_rows = 16) {
    return (size_t)token_rows * kQsXStride + (size_t)tiles * 16 * kQsWStride;
}
__host__ __device__ constexpr size_t qms_lds_bytes(int tiles, int groups, int waves, int token_rows = 16) {
    return qms_scale_lds_bytes(tiles, groups) + (size_t)waves * qms_wave_lds_bytes(tiles, token_rows);
}

// G32: groups of 32 columns.  The four k-blocks of an MFMA are the lane quarters q, and q / 2 is the group within a
// 64-column half, so each half takes its MFMAs twice, once per group with the other group's activations zeroed.
template <class ActT, class ScaleT, int NMAT, int RT, int XR, class Epi, bool G32 = false>
__device__ __forceinline__ void qms_body(const uint8_t* const (&W)[NMAT], const uint16_t* const (&S)[NMAT],
                                         const uint16_t* const (&B)[NMAT], const uint16_t* __restrict__ X, int batch,
                                         int rows, int cols, int group, const Epi& epi) {
    using E = Elem16<ActT>;
    using O = QsOperand<ActT>;
    constexpr int T = NMAT * RT;   // 16-row tiles a wave multiplies by its slice of x
    static_assert(qms_wave_lds_bytes(T, 4 * XR) >= (size_t)T * 1024, "partial sums reuse the staging buffer");
    static_assert(XR == 2 || XR == 4, "a pass stages eight or sixteen token rows");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int chunk = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int kc = blockDim.x / kWave;
    const int n = lane & 15, q = lane >> 4;
    // (groups of 128 columns: a step is one group instead of two, everything else is the same)
    const int g64 = cols >> 6;         // 64-column halves of a step's 128 columns
    const int gshift = group == 128 ? 1 : 0;
    const int gt = G32 ? g64 << 1 : g64 >> gshift;      // scale groups per row
    const int npairs = g64 >> 1;
    const int rs = cols >> 1;          // bytes per packed row
    const int row0 = blockIdx.x * (16 * RT);
    const int m0 = blockIdx.y * kQsTokens;
    const int last_tok = (batch < m0 + kQsTokens ? batch : m0 + kQsTokens) - 1;

    // Nothing below predicates a load; loads return in issue order, so what is needed first is
    // asked for first.
    // ---- scales and biases of the tile: one run of eight groups of one row per thread ------------
    // (rows of a multiple of 256 but not of 512 columns hold an odd number of four-group halves: runs of four then,
    // eight bytes per plane and thread; their rows start on 8-byte boundaries only)
    const bool half_runs = (gt & 7) != 0;
    const int run_len = half_runs ? 4 : 8;
    const int runs = half_runs ? gt >> 2 : gt >> 3;
    const int items = T * 16 * runs;
    float2* lds_sb = reinterpret_cast<float2*>(smem);
    const int sstride = gt + 1;
    struct ScaleRun { uint4_t s, b; int at; };
    auto load_scales = [&](int item) {
        if (item > items - 1) item = items - 1;               // threads past the end repeat the last item
        const int srow = item / runs, run = item - srow * runs;   // srow = (matrix * RT + tile) * 16 + row in tile
        const int smat = srow / (16 * RT);
        int r = row0 + (srow - smat * 16 * RT);
        if (r > rows - 1) r = rows - 1;
        const uint16_t* sp = S[0];
        const uint16_t* bp = B[0];
        if (NMAT > 1 && smat == 1) { sp = S[NMAT - 1]; bp = B[NMAT - 1]; }
        ScaleRun out;
        if (half_runs) {
            const uint2_t s2 = *reinterpret_cast<const uint2_t*>(sp + (size_t)r * gt + 4 * run);
            const uint2_t b2 = *reinterpret_cast<const uint2_t*>(bp + (size_t)r * gt + 4 * run);
            out.s = uint4_t{s2.x, s2.y, 0u, 0u};
            out.b = uint4_t{b2.x, b2.y, 0u, 0u};
        } else {
            out.s = *reinterpret_cast<const uint4_t*>(sp + (size_t)r * gt + 8 * run);
            out.b = *reinterpret_cast<const uint4_t*>(bp + (size_t)r * gt + 8 * run);
        }
        out.at = srow * sstride + run_len * run;
        return out;
    };
    auto store_scales = [&](const ScaleRun& v) {
        const uint32_t sd[4] = {v.s.x, v.s.y, v.s.z, v.s.w}, bd[4] = {v.b.x, v.b.y, v.b.z, v.b.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float s = ScaleT::widen((uint16_t)(e & 1 ? sd[e >> 1] >> 16 : sd[e >> 1] & 0xFFFFu));
            const float b = ScaleT::widen((uint16_t)(e & 1 ? bd[e >> 1] >> 16 : bd[e >> 1] & 0xFFFFu));
            if (e < run_len) lds_sb[v.at + e] = float2{s, __builtin_fmaf(-O::kBase, s, b)};
        }
    };
    const ScaleRun first_run = load_scales((int)threadIdx.x);

    unsigned char* stage = smem + qms_scale_lds_bytes(T, gt) + (size_t)chunk * qms_wave_lds_bytes(T, 4 * XR);
    unsigned char* stage_w = stage + 4 * XR * kQsXStride;
    // load side: sixteen lanes per token row, four lanes per weight row
    const int x_tok = lane >> 4, x_piece = lane & 15;
    const int w_row = lane >> 2, w_piece = lane & 3;
    const float4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint4_t ones = {O::kOnePair, O::kOnePair, O::kOnePair, O::kOnePair};
    float4_t acc[NMAT][RT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int t = 0; t < RT; ++t) acc[m][t] = zero;

    // One step = one pair of scale groups (128 columns): XR loads of activations (four token rows
    // each) and one load per tile of weights.  Wave c takes pairs c, c + kc, c + 2 kc, ...
    struct Step { uint4_t x[XR]; uint4_t w[NMAT][RT]; };
    const uint16_t* x_base[XR];
#pragma unroll
    for (int r = 0; r < XR; ++r) {
        int tok = m0 + 4 * r + x_tok;
        if (tok > last_tok) tok = last_tok;
        x_base[r] = X + (size_t)tok * cols + 8 * x_piece;
    }
    const uint8_t* w_base[NMAT][RT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            int r = row0 + 16 * t + w_row;
            if (r > rows - 1) r = rows - 1;
            w_base[m][t] = W[m] + (size_t)r * rs + 16 * w_piece;
        }
    auto issue = [&](Step& st, int pair) {
        if (pair > npairs - 1) pair = npairs - 1;   // past the end: the last pair again, under a zero scale
#pragma unroll
        for (int r = 0; r < XR; ++r) st.x[r] = *reinterpret_cast<const uint4_t*>(x_base[r] + 128 * pair);
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int t = 0; t < RT; ++t) st.w[m][t] = *reinterpret_cast<const uint4_t*>(w_base[m][t] + 64 * pair);
    };
    // through the wave's staging buffer: written as loaded, read back in operand order
    auto consume = [&](const Step& st, int pair) {
#pragma unroll
        for (int r = 0; r < XR; ++r)
            *reinterpret_cast<uint4_t*>(stage + (4 * r + x_tok) * kQsXStride + 16 * x_piece) = st.x[r];
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int t = 0; t < RT; ++t) {
                unsigned char* at = stage_w + ((m * RT + t) * 16 + w_row) * kQsWStride + 16 * w_piece;
                *reinterpret_cast<uint2_t*>(at) = uint2_t{st.w[m][t].x, st.w[m][t].y};
                *reinterpret_cast<uint2_t*>(at + 8) = uint2_t{st.w[m][t].z, st.w[m][t].w};
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        int gi = 2 * pair;
        if (gi > g64) gi = g64;   // past the end: the zero column below
        // with eight staged token rows, MFMA rows 8..15 re-read rows 0..7 (never stored)
        const int xrow = XR == 4 ? n : (n & 7);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const unsigned char* xr = stage + xrow * kQsXStride + 128 * e + 32 * q;
            const uint4_t a0 = O::activations(*reinterpret_cast<const uint4_t*>(xr));
            const uint4_t a1 = O::activations(*reinterpret_cast<const uint4_t*>(xr + 16));
            if constexpr (G32) {
                uint4_t cx[NMAT][RT], cy[NMAT][RT];
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int t = 0; t < RT; ++t) {
                        const uint2_t c = *reinterpret_cast<const uint2_t*>(stage_w + ((m * RT + t) * 16 + n) * kQsWStride + 32 * e + 8 * q);
                        cx[m][t] = O::codes(c.x);
                        cy[m][t] = O::codes(c.y);
                    }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const bool mine = (q >> 1) == h;
                    const uint4_t none = {0u, 0u, 0u, 0u};
                    const uint4_t a0h = mine ? a0 : none, a1h = mine ? a1 : none;
                    const float4_t xs = E::mfma(a1h, ones, E::mfma(a0h, ones, zero));
                    const int ge = gi + e < g64 ? 2 * (gi + e) + h : gt;
#pragma unroll
                    for (int m = 0; m < NMAT; ++m)
#pragma unroll
                        for (int t = 0; t < RT; ++t) {
                            const float4_t d = E::mfma(a1h, cy[m][t], E::mfma(a0h, cx[m][t], zero));
                            const float2 sb = lds_sb[((m * RT + t) * 16 + n) * sstride + ge];
                            acc[m][t].x = __builtin_fmaf(sb.x, d.x, __builtin_fmaf(sb.y, xs.x, acc[m][t].x));
                            acc[m][t].y = __builtin_fmaf(sb.x, d.y, __builtin_fmaf(sb.y, xs.y, acc[m][t].y));
                            acc[m][t].z = __builtin_fmaf(sb.x, d.z, __builtin_fmaf(sb.y, xs.z, acc[m][t].z));
                            acc[m][t].w = __builtin_fmaf(sb.x, d.w, __builtin_fmaf(sb.y, xs.w, acc[m][t].w));
                        }
                }
            } else {
            const float4_t xs = E::mfma(a1, ones, E::mfma(a0, ones, zero));
            const int ge = gi + e < g64 ? (gi + e) >> gshift : gt;
#pragma unroll
            for (int m = 0; m < NMAT; ++m)
#pragma unroll
                for (int t = 0; t < RT; ++t) {
                    const uint2_t c = *reinterpret_cast<const uint2_t*>(stage_w + ((m * RT + t) * 16 + n) * kQsWStride + 32 * e + 8 * q);
                    const float4_t d = E::mfma(a1, O::codes(c.y), E::mfma(a0, O::codes(c.x), zero));
                    const float2 sb = lds_sb[((m * RT + t) * 16 + n) * sstride + ge];
                    acc[m][t].x = __builtin_fmaf(sb.x, d.x, __builtin_fmaf(sb.y, xs.x, acc[m][t].x));
                    acc[m][t].y = __builtin_fmaf(sb.x, d.y, __builtin_fmaf(sb.y, xs.y, acc[m][t].y));
                    acc[m][t].z = __builtin_fmaf(sb.x, d.z, __builtin_fmaf(sb.y, xs.z, acc[m][t].z));
                    acc[m][t].w = __builtin_fmaf(sb.x, d.w, __builtin_fmaf(sb.y, xs.w, acc[m][t].w));
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    // One step is in flight while the other is consumed.  The first loads go out behind the scale
    // loads; the scales reach LDS while they fly.
    Step s0, s1;
    int pair = chunk;
    issue(s0, pair);
    issue(s1, pair + kc);
    store_scales(first_run);
    // a tile with more runs than the workgroup has threads takes more passes
    for (int base = (int)blockDim.x; base < items; base += (int)blockDim.x) store_scales(load_scales(base + (int)threadIdx.x));
    if (threadIdx.x < T * 16) lds_sb[threadIdx.x * sstride + gt] = float2{0.0f, 0.0f};
    __syncthreads();
    for (; pair < npairs; pair += 2 * kc) {
        consume(s0, pair);
        issue(s0, pair + 2 * kc);
        consume(s1, pair + kc);
        issue(s1, pair + 3 * kc);
    }

    // ---- the kc waves of the workgroup, in wave order -------------------------------------------------
    // each wave leaves its partial sums in its own staging buffer
    {
        float4_t* mine = reinterpret_cast<float4_t*>(stage);
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int t = 0; t < RT; ++t) mine[(m * RT + t) * kWave + lane] = acc[m][t];
    }
    __syncthreads();
    if (chunk < RT) {
        // wave t finishes tile t: lane (n, q) holds row 16 t + n of tokens 4 q .. 4 q + 3
        const int t = chunk;
        const unsigned char* first = smem + qms_scale_lds_bytes(T, gt);
        float4_t sum[NMAT];
#pragma unroll
        for (int m = 0; m < NMAT; ++m) sum[m] = zero;
        for (int c = 0; c < kc; ++c)
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const float4_t part = reinterpret_cast<const float4_t*>(first + (size_t)c * qms_wave_lds_bytes(T, 4 * XR))[(m * RT + t) * kWave + lane];
                sum[m].x += part.x; sum[m].y += part.y; sum[m].z += part.z; sum[m].w += part.w;
            }
        const int r = row0 + 16 * t + n;
        if (r < rows) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int tok = m0 + 4 * q + v;
                if (tok <= last_tok) {
                    float val[NMAT];
#pragma unroll
                    for (int m = 0; m < NMAT; ++m) val[m] = v == 0 ? sum[m].x : (v == 1 ? sum[m].y : (v == 2 ? sum[m].z : sum[m].w));
                    epi((size_t)tok * rows + r, val);
                }
            }
        }
    }
}

// ---- epilogues: (element index, values[NMAT]) -------------------------------------------------------
template <class ActT>
struct QsStore {
    uint16_t* y;
    __device__ __forceinline__ void operator()(size_t idx, const float (&v)[1]) const { y[idx] = ActT::narrow(v[0]); }
};
// matvec_out = narrow(acc); out = narrow(widen(matvec_out) + residual)
template <class ActT>
struct QsAdd {
    uint16_t* mv;
    const uint16_t* residual;
    uint16_t* out;
    __device__ __forceinline__ void operator()(size_t idx, const float (&v)[1]) const {
        const uint16_t p = ActT::narrow(v[0]);
        mv[idx] = p;
        out[idx] = ActT::narrow(ActT::widen(p) + ActT::widen(residual[idx]));
    }
};
template <class ActT>
struct QsSwiglu {
    uint16_t* y;
    __device__ __forceinline__ void operator()(size_t idx, const float (&v)[2]) const {
        const float g = v[0], u = v[1];
        y[idx] = ActT::narrow(g / (1.0f + expf(-g)) * u);
    }
};

// agent_geglu_product (lut_matvec.metal:2235-2243): gate and up rounded to the 16-bit type, tanh-form GELU of the
// gate with its argument clamped to +-20, product clamped to the fp16 range
template <class ActT>
struct QsGeglu {
    uint16_t* y;
    __device__ __forceinline__ void operator()(size_t idx, const float (&v)[2]) const {
        const float g = ActT::widen(ActT::narrow(v[0])), u = ActT::widen(ActT::narrow(v[1]));
        float inner = 0.7978845608f * (g + 0.044715f * (g * g * g));
        inner = fminf(fmaxf(inner, -20.0f), 20.0f);
        const float gelu = 0.5f * g * (1.0f + tanhf(inner));
        y[idx] = ActT::narrow(fminf(fmaxf(gelu * u, -65504.0f), 65504.0f));
    }
};

}  // namespace smelt

#define SMELT_QMS_KERNEL extern "C" __global__ __launch_bounds__(1024)

// Argument lists of the skinny kernels of the same pipelines (the workspace pointers are unused).
#define SMELT_AFFINE_QMS_PLAIN(T, ACT, SC, RTV, XRV)                                                \
    SMELT_QMS_KERNEL void smelt_affine_qms_r##RTV##_x##XRV##_store_##T(                             \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* Y,    \
        uint32_t batch, uint32_t rows, uint32_t cols, uint32_t group, uint32_t, float*, uint32_t*) { \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        qms_body<ACT, SC, 1, RTV, XRV>(w, s, b, X, batch, rows, cols, group, QsStore<ACT>{Y});      \
    }                                                                                              \
    SMELT_QMS_KERNEL void smelt_affine_qms_r##RTV##_x##XRV##_add_##T(                               \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* MV,   \
        const uint16_t* RES, uint16_t* OUT, uint32_t batch, uint32_t rows, uint32_t cols,          \
        uint32_t group, uint32_t, float*, uint32_t*) {                                             \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        qms_body<ACT, SC, 1, RTV, XRV>(w, s, b, X, batch, rows, cols, group, QsAdd<ACT>{MV, RES, OUT}); \
    }

#define SMELT_AFFINE_QMS_GATE_UP(T, ACT, SC, XRV)                                                   \
    SMELT_QMS_KERNEL void smelt_affine_qms_r1_x##XRV##_gate_up_swiglu_##T(                          \
        const uint8_t* gW, const uint16_t* gS, const uint16_t* gB, const uint8_t* uW,              \
        const uint16_t* uS, const uint16_t* uB, const uint16_t* X, uint16_t* Y, uint32_t batch,    \
        uint32_t rows, uint32_t cols, uint32_t group, uint32_t, float*, uint32_t*) {               \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        qms_body<ACT, SC, 2, 1, XRV>(w, s, b, X, batch, rows, cols, group, QsSwiglu<ACT>{Y});       \
    }                                                                                              \
    SMELT_QMS_KERNEL void smelt_affine_qms_r1_x##XRV##_gate_up_geglu_##T(                           \
        const uint8_t* gW, const uint16_t* gS, const uint16_t* gB, const uint8_t* uW,              \
        const uint16_t* uS, const uint16_t* uB, const uint16_t* X, uint16_t* Y, uint32_t batch,    \
        uint32_t rows, uint32_t cols, uint32_t group, uint32_t, float*, uint32_t*) {               \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        qms_body<ACT, SC, 2, 1, XRV>(w, s, b, X, batch, rows, cols, group, QsGeglu<ACT>{Y});        \
    }

// Groups of 32 columns: one row tile per wave.
#define SMELT_AFFINE_QMS_G32(T, ACT, SC, XRV)                                                       \
    SMELT_QMS_KERNEL void smelt_affine_qms_g32_x##XRV##_store_##T(                                  \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* Y,    \
        uint32_t batch, uint32_t rows, uint32_t cols, uint32_t group, uint32_t, float*, uint32_t*) { \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        qms_body<ACT, SC, 1, 1, XRV, QsStore<ACT>, true>(w, s, b, X, batch, rows, cols, group, QsStore<ACT>{Y}); \
    }                                                                                              \
    SMELT_QMS_KERNEL void smelt_affine_qms_g32_x##XRV##_add_##T(                                    \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* MV,   \
        const uint16_t* RES, uint16_t* OUT, uint32_t batch, uint32_t rows, uint32_t cols,          \
        uint32_t group, uint32_t, float*, uint32_t*) {                                             \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        qms_body<ACT, SC, 1, 1, XRV, QsAdd<ACT>, true>(w, s, b, X, batch, rows, cols, group, QsAdd<ACT>{MV, RES, OUT}); \
    }                                                                                              \
    SMELT_QMS_KERNEL void smelt_affine_qms_g32_x##XRV##_gate_up_swiglu_##T(                         \
        const uint8_t* gW, const uint16_t* gS, const uint16_t* gB, const uint8_t* uW,              \
        const uint16_t* uS, const uint16_t* uB, const uint16_t* X, uint16_t* Y, uint32_t batch,    \
        uint32_t rows, uint32_t cols, uint32_t group, uint32_t, float*, uint32_t*) {               \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        qms_body<ACT, SC, 2, 1, XRV, QsSwiglu<ACT>, true>(w, s, b, X, batch, rows, cols, group, QsSwiglu<ACT>{Y}); \
    }                                                                                              \
    SMELT_QMS_KERNEL void smelt_affine_qms_g32_x##XRV##_gate_up_geglu_##T(                          \
        const uint8_t* gW, const uint16_t* gS, const uint16_t* gB, const uint8_t* uW,              \
        const uint16_t* uS, const uint16_t* uB, const uint16_t* X, uint16_t* Y, uint32_t batch,    \
        uint32_t rows, uint32_t cols, uint32_t group, uint32_t, float*, uint32_t*) {               \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        qms_body<ACT, SC, 2, 1, XRV, QsGeglu<ACT>, true>(w, s, b, X, batch, rows, cols, group, QsGeglu<ACT>{Y}); \
    }

// ---- ternary codes (two bits, groups of 128 columns): the streaming form of the ternary qmm ------------
// The skeleton of qms_body with a dequantised fp16 weight operand in place of exact codes and scale FMAs: the
// value of an element is the token-slab kernel's (signed_quant_precise.metal:407-439), rounded to fp16 once:
// the two-bit field keeps its place inside its byte, byte lane k multiplies it by its own subscale
// fp16(scale / 4^k), and -bias (a plane of its own) is added.  Activations are multiplied as fp16 (bf16 rows are
// converted at staging, as that kernel does).  A wave owns sixteen rows and walks 128-column steps (one scale
// group each); the waves of a workgroup split K; tokens are the A operand in memory order, so lane (n, q) takes
// the four bytes of row n that hold columns 16 q .. 16 q + 15 of a 64-column half: byte j is registers 2 j
// (codes in byte lanes 0 and 1) and 2 j + 1 (lanes 2 and 3) of the two MFMAs' B operands.
namespace smelt {

typedef _Float16 half2v_t __attribute__((ext_vector_type(2)));
constexpr int kQtsWStride = 40;        // bytes per staged weight row of a step (32 + 8 of padding)
__host__ __device__ constexpr size_t qts_scale_lds_bytes(int groups) { return (size_t)16 * (groups + 1) * 4; }
__host__ __device__ constexpr size_t qts_wave_lds_bytes(int token_rows) {
    return (size_t)token_rows * kQsXStride + 16 * kQtsWStride < 1024 ? (size_t)1024 : (size_t)token_rows * kQsXStride + 16 * kQtsWStride;
}

template <class ActT, int XR>
__device__ __forceinline__ void qts_body(const uint8_t* __restrict__ W, const uint16_t* __restrict__ S,
                                         const uint16_t* __restrict__ B, const uint16_t* __restrict__ X,
                                         uint16_t* __restrict__ Y, int batch, int rows, int cols) {
    using E = Elem16<F16>;
    static_assert(XR == 2 || XR == 4, "a pass stages eight or sixteen token rows");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int chunk = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int kc = blockDim.x / kWave;
    const int n = lane & 15, q = lane >> 4;
    const int gt = cols >> 7;          // scale groups per row = steps
    const int rs = cols >> 2;          // bytes per packed row
    const int row0 = blockIdx.x * 16;
    const int m0 = blockIdx.y * kQsTokens;
    const int last_tok = (batch < m0 + kQsTokens ? batch : m0 + kQsTokens) - 1;

    // ---- (scale, -bias) of the sixteen rows and every group, plus one zero column: eight, four or two groups per
    // thread (rows of a multiple of 1024, 512 or 256 columns; the scale rows start on 16-, 8- or 4-byte boundaries)
    const bool half_runs = (gt & 7) != 0;
    const bool quarter_runs = (gt & 3) != 0;
    const int run_len = quarter_runs ? 2 : (half_runs ? 4 : 8);
    const int runs = gt / run_len;
    const int items = 16 * runs;
    uint32_t* lds_sb = reinterpret_cast<uint32_t*>(smem);
    const int sstride = gt + 1;
    struct ScaleRun { uint4_t s, b; int at; };
    auto load_scales = [&](int item) {
        if (item > items - 1) item = items - 1;
        const int srow = item / runs, run = item - srow * runs;
        int r = row0 + srow;
        if (r > rows - 1) r = rows - 1;
        ScaleRun out;
        if (quarter_runs) {
            out.s = uint4_t{*reinterpret_cast<const uint32_t*>(S + (size_t)r * gt + 2 * run), 0u, 0u, 0u};
            out.b = uint4_t{*reinterpret_cast<const uint32_t*>(B + (size_t)r * gt + 2 * run), 0u, 0u, 0u};
        } else if (half_runs) {
            const uint2_t s2 = *reinterpret_cast<const uint2_t*>(S + (size_t)r * gt + 4 * run);
            const uint2_t b2 = *reinterpret_cast<const uint2_t*>(B + (size_t)r * gt + 4 * run);
            out.s = uint4_t{s2.x, s2.y, 0u, 0u};
            out.b = uint4_t{b2.x, b2.y, 0u, 0u};
        } else {
            out.s = *reinterpret_cast<const uint4_t*>(S + (size_t)r * gt + 8 * run);
            out.b = *reinterpret_cast<const uint4_t*>(B + (size_t)r * gt + 8 * run);
        }
        out.at = srow * sstride + run_len * run;
        return out;
    };
    auto store_scales = [&](const ScaleRun& v) {
        const uint32_t sd[4] = {v.s.x, v.s.y, v.s.z, v.s.w}, bd[4] = {v.b.x, v.b.y, v.b.z, v.b.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint32_t sc = e & 1 ? sd[e >> 1] >> 16 : sd[e >> 1] & 0xFFFFu;
            const uint32_t bi = e & 1 ? bd[e >> 1] >> 16 : bd[e >> 1] & 0xFFFFu;
            if (e < run_len) lds_sb[v.at + e] = sc | ((bi ^ 0x8000u) << 16);   // (scale, -bias) as fp16
        }
    };
    const ScaleRun first_run = load_scales((int)threadIdx.x);

    unsigned char* stage = smem + qts_scale_lds_bytes(gt) + (size_t)chunk * qts_wave_lds_bytes(4 * XR);
    unsigned char* stage_w = stage + 4 * XR * kQsXStride;
    const int x_tok = lane >> 4, x_piece = lane & 15;
    const int w_row = lane >> 2, w_piece = lane & 3;
    float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};

    struct Step { uint4_t x[XR]; uint2_t w; };
    const uint16_t* x_base[XR];
#pragma unroll
    for (int r = 0; r < XR; ++r) {
        int tok = m0 + 4 * r + x_tok;
        if (tok > last_tok) tok = last_tok;
        x_base[r] = X + (size_t)tok * cols + 8 * x_piece;
    }
    const uint8_t* w_base;
    {
        int r = row0 + w_row;
        if (r > rows - 1) r = rows - 1;
        w_base = W + (size_t)r * rs + 8 * w_piece;
    }
    auto issue = [&](Step& st, int step) {
        if (step > gt - 1) step = gt - 1;   // past the end: the last step again, under a zero scale and bias
#pragma unroll
        for (int r = 0; r < XR; ++r) st.x[r] = *reinterpret_cast<const uint4_t*>(x_base[r] + 128 * step);
        st.w = *reinterpret_cast<const uint2_t*>(w_base + 32 * step);
    };
    auto consume = [&](const Step& st, int step) {
#pragma unroll
        for (int r = 0; r < XR; ++r) {
            uint4_t v = st.x[r];
            if (!ActT::kIsF16) {
                uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    p[i] = (uint32_t)ActT::to_f16_bits((uint16_t)(p[i] & 0xFFFFu)) | ((uint32_t)ActT::to_f16_bits((uint16_t)(p[i] >> 16)) << 16);
                v = uint4_t{p[0], p[1], p[2], p[3]};
            }
            *reinterpret_cast<uint4_t*>(stage + (4 * r + x_tok) * kQsXStride + 16 * x_piece) = v;
        }
        *reinterpret_cast<uint2_t*>(stage_w + w_row * kQtsWStride + 8 * w_piece) = st.w;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int gi = step < gt ? step : gt;   // the zero column
        const uint32_t sb = lds_sb[n * sstride + gi];
        const _Float16 sc = __builtin_bit_cast(_Float16, (uint16_t)(sb & 0xFFFFu));
        const _Float16 nb = __builtin_bit_cast(_Float16, (uint16_t)(sb >> 16));
        const half2v_t s01 = half2v_t{sc, sc} * half2v_t{(_Float16)1.0f, (_Float16)0.25f};
        const half2v_t s23 = half2v_t{sc, sc} * half2v_t{(_Float16)0.0625f, (_Float16)0.015625f};
        const half2v_t nb2 = {nb, nb};
        const half2v_t k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
        const int xrow = XR == 4 ? n : (n & 7);
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const unsigned char* xr = stage + xrow * kQsXStride + 128 * e + 32 * q;
            const uint4_t a0 = *reinterpret_cast<const uint4_t*>(xr);
            const uint4_t a1 = *reinterpret_cast<const uint4_t*>(xr + 16);
            const uint32_t c = *reinterpret_cast<const uint32_t*>(stage_w + n * kQtsWStride + 16 * e + 4 * q);
            uint32_t bw[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // byte j in both half-words, then its lanes 0|1 and 2|3 as (1024 + field) pairs
                const uint32_t rep = __builtin_amdgcn_perm(c, c, 0x0c000c00u | (uint32_t)j | ((uint32_t)j << 16));
                const half2v_t f01 = __builtin_bit_cast(half2v_t, and_or(rep, 0x000C0003u, 0x64006400u)) - k1024;
                const half2v_t f23 = __builtin_bit_cast(half2v_t, and_or(rep, 0x00C00030u, 0x64006400u)) - k1024;
                bw[2 * j] = __builtin_bit_cast(uint32_t, s01 * f01 + nb2);
                bw[2 * j + 1] = __builtin_bit_cast(uint32_t, s23 * f23 + nb2);
            }
            acc = E::mfma(a0, uint4_t{bw[0], bw[1], bw[2], bw[3]}, acc);
            acc = E::mfma(a1, uint4_t{bw[4], bw[5], bw[6], bw[7]}, acc);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    Step s0, s1;
    int step = chunk;
    issue(s0, step);
    issue(s1, step + kc);
    store_scales(first_run);
    for (int base = (int)blockDim.x; base < items; base += (int)blockDim.x) store_scales(load_scales(base + (int)threadIdx.x));
    if (threadIdx.x < 16) lds_sb[threadIdx.x * sstride + gt] = 0u;
    __syncthreads();
    for (; step < gt; step += 2 * kc) {
        consume(s0, step);
        issue(s0, step + 2 * kc);
        consume(s1, step + kc);
        issue(s1, step + 3 * kc);
    }

    // ---- the kc waves of the workgroup, in wave order ------------------------------------------------
    reinterpret_cast<float4_t*>(stage)[lane] = acc;
    __syncthreads();
    if (chunk == 0) {
        const unsigned char* first = smem + qts_scale_lds_bytes(gt);
        float4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int c = 0; c < kc; ++c) {
            const float4_t part = reinterpret_cast<const float4_t*>(first + (size_t)c * qts_wave_lds_bytes(4 * XR))[lane];
            sum.x += part.x; sum.y += part.y; sum.z += part.z; sum.w += part.w;
        }
        const int r = row0 + n;
        if (r < rows) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int tok = m0 + 4 * q + v;
                if (tok <= last_tok) Y[(size_t)tok * rows + r] = ActT::narrow(v == 0 ? sum.x : (v == 1 ? sum.y : (v == 2 ? sum.z : sum.w)));
            }
        }
    }
}

}  // namespace smelt

// Argument list of the ternary token-slab qmm (the bias plane is the scale plane bound a second time).
#define SMELT_TERNARY_QMS(T, ACT, XRV)                                                              \
    SMELT_QMS_KERNEL void smelt_ternary_qms_x##XRV##_##T(                                           \
        const uint8_t* C, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* Y,    \
        uint32_t rows, uint32_t cols, uint32_t batch) {                                            \
        smelt::qts_body<ACT, XRV>(C, S, B, X, Y, (int)batch, (int)rows, (int)cols);                \
    }

// ---- binary and ternary codes (groups of 128 columns) over many tokens ------------------------------
// The per-token records of the signed formats (one grid row per token) from eight tokens on (bf16 rows converted to fp16):
// the skeleton of qts_body with exact operands (2 code - 1 for one-bit codes, code - 1 for two-bit codes, as fp16)
// and the group's scale applied in fp32 to each step's sums, i.e. the arithmetic of the single-token kernels in
// another summation order.  NMAT = 2: gate and up of one tile (the fused SwiGLU form).  Epilogues are the
// single-token kernels' ((token, row, sums)).
namespace smelt {

template <class ActT, int BITS, int NMAT, int XR, class Epi>
__device__ __forceinline__ void qss_body(const uint8_t* const (&W)[NMAT], const uint16_t* const (&S)[NMAT],
                                         const uint16_t* __restrict__ X, int batch, int rows, int cols, const Epi& epi) {
    using E = Elem16<F16>;
    static_assert(BITS == 1 || BITS == 2, "one- or two-bit codes");
    constexpr int kWB = 16 * BITS;            // bytes of a row per 128-column step
    constexpr int kWStride = kWB + 8;         // staged, with padding
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & (kWave - 1);
    const int chunk = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int kc = blockDim.x / kWave;
    const int n = lane & 15, q = lane >> 4;
    const int gt = cols >> 7;
    const int rs = gt * kWB;
    const int row0 = blockIdx.x * 16;
    const int m0 = blockIdx.y * kQsTokens;
    const int last_tok = (batch < m0 + kQsTokens ? batch : m0 + kQsTokens) - 1;

    // ---- scales of the tile (fp32), plus one zero column: eight, four or two groups per thread
    const bool half_runs = (gt & 7) != 0, quarter_runs = (gt & 3) != 0;
    const int run_len = quarter_runs ? 2 : (half_runs ? 4 : 8);
    const int runs = gt / run_len;
    const int items = NMAT * 16 * runs;
    float* lds_s = reinterpret_cast<float*>(smem);
    const int sstride = gt + 1;
    struct ScaleRun { uint4_t s; int at; };
    auto load_scales = [&](int item) {
        if (item > items - 1) item = items - 1;
        const int srow = item / runs, run = item - srow * runs;   // srow = matrix * 16 + row in tile
        const int m = srow >> 4;
        int r = row0 + (srow & 15);
        if (r > rows - 1) r = rows - 1;
        const uint16_t* sp = NMAT > 1 && m == 1 ? S[NMAT - 1] : S[0];
        ScaleRun out;
        if (quarter_runs) out.s = uint4_t{*reinterpret_cast<const uint32_t*>(sp + (size_t)r * gt + 2 * run), 0u, 0u, 0u};
        else if (half_runs) {
            const uint2_t s2 = *reinterpret_cast<const uint2_t*>(sp + (size_t)r * gt + 4 * run);
            out.s = uint4_t{s2.x, s2.y, 0u, 0u};
        } else out.s = *reinterpret_cast<const uint4_t*>(sp + (size_t)r * gt + 8 * run);
        out.at = srow * sstride + run_len * run;
        return out;
    };
    auto store_scales = [&](const ScaleRun& v) {
        const uint32_t sd[4] = {v.s.x, v.s.y, v.s.z, v.s.w};
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (e < run_len) lds_s[v.at + e] = F16::widen((uint16_t)(e & 1 ? sd[e >> 1] >> 16 : sd[e >> 1] & 0xFFFFu));
    };
    const ScaleRun first_run = load_scales((int)threadIdx.x);

    constexpr size_t kWaveBytes = (size_t)4 * XR * kQsXStride + (size_t)NMAT * 16 * kWStride < (size_t)NMAT * 1024
                                      ? (size_t)NMAT * 1024 : (size_t)4 * XR * kQsXStride + (size_t)NMAT * 16 * kWStride;
    unsigned char* stage = smem + (size_t)NMAT * 16 * sstride * 4 + (size_t)chunk * kWaveBytes;
    unsigned char* stage_w = stage + 4 * XR * kQsXStride;
    const int x_tok = lane >> 4, x_piece = lane & 15;
    const int w_row = lane >> 2, w_piece = lane & 3;
    const float4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
    float4_t acc[NMAT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m) acc[m] = zero;

    struct Step { uint4_t x[XR]; uint32_t w[NMAT][BITS]; };
    const uint16_t* x_base[XR];
#pragma unroll
    for (int r = 0; r < XR; ++r) {
        int tok = m0 + 4 * r + x_tok;
        if (tok > last_tok) tok = last_tok;
        x_base[r] = X + (size_t)tok * cols + 8 * x_piece;
    }
    const uint8_t* w_base[NMAT];
    {
        int r = row0 + w_row;
        if (r > rows - 1) r = rows - 1;
#pragma unroll
        for (int m = 0; m < NMAT; ++m) w_base[m] = W[m] + (size_t)r * rs + 4 * BITS * w_piece;
    }
    auto issue = [&](Step& st, int step) {
        if (step > gt - 1) step = gt - 1;   // past the end: the last step again, under a zero scale
#pragma unroll
        for (int r = 0; r < XR; ++r) st.x[r] = *reinterpret_cast<const uint4_t*>(x_base[r] + 128 * step);
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int d = 0; d < BITS; ++d) st.w[m][d] = *reinterpret_cast<const uint32_t*>(w_base[m] + kWB * step + 4 * d);
    };
    auto consume = [&](const Step& st, int step) {
#pragma unroll
        for (int r = 0; r < XR; ++r) {
            uint4_t v = st.x[r];
            if (!ActT::kIsF16) {   // bf16 rows are multiplied as fp16, as in the vector kernels of these formats
                uint32_t p[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    p[i] = (uint32_t)ActT::to_f16_bits((uint16_t)(p[i] & 0xFFFFu)) | ((uint32_t)ActT::to_f16_bits((uint16_t)(p[i] >> 16)) << 16);
                v = uint4_t{p[0], p[1], p[2], p[3]};
            }
            *reinterpret_cast<uint4_t*>(stage + (4 * r + x_tok) * kQsXStride + 16 * x_piece) = v;
        }
#pragma unroll
        for (int m = 0; m < NMAT; ++m)
#pragma unroll
            for (int d = 0; d < BITS; ++d)
                *reinterpret_cast<uint32_t*>(stage_w + (m * 16 + w_row) * kWStride + 4 * BITS * w_piece + 4 * d) = st.w[m][d];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const int gi = step < gt ? step : gt;   // the zero column
        const half2v_t k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
        const half2v_t minus1 = {(_Float16)-1.0f, (_Float16)-1.0f};
        const int xrow = XR == 4 ? n : (n & 7);
        float4_t d[NMAT];
#pragma unroll
        for (int m = 0; m < NMAT; ++m) d[m] = zero;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const unsigned char* xr = stage + xrow * kQsXStride + 128 * e + 32 * q;
            const uint4_t a0 = *reinterpret_cast<const uint4_t*>(xr);
            const uint4_t a1 = *reinterpret_cast<const uint4_t*>(xr + 16);
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                uint32_t bw[8];
                if constexpr (BITS == 2) {
                    const uint32_t c = *reinterpret_cast<const uint32_t*>(stage_w + (m * 16 + n) * kWStride + 16 * e + 4 * q);
                    const half2v_t r01 = {(_Float16)1.0f, (_Float16)0.25f}, r23 = {(_Float16)0.0625f, (_Float16)0.015625f};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const uint32_t rep = __builtin_amdgcn_perm(c, c, 0x0c000c00u | (uint32_t)j | ((uint32_t)j << 16));
                        const half2v_t f01 = __builtin_bit_cast(half2v_t, and_or(rep, 0x000C0003u, 0x64006400u)) - k1024;
                        const half2v_t f23 = __builtin_bit_cast(half2v_t, and_or(rep, 0x00C00030u, 0x64006400u)) - k1024;
                        bw[2 * j] = __builtin_bit_cast(uint32_t, f01 * r01 + minus1);        // code - 1, exact
                        bw[2 * j + 1] = __builtin_bit_cast(uint32_t, f23 * r23 + minus1);
                    }
                } else {
                    const uint32_t c = *reinterpret_cast<const uint16_t*>(stage_w + (m * 16 + n) * kWStride + 8 * e + 2 * q);
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const uint32_t rep = __builtin_amdgcn_perm(c, c, 0x0c000c00u | (uint32_t)j | ((uint32_t)j << 16));
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const uint32_t mask = (1u << (2 * r)) | (1u << (2 * r + 1 + 16));
                            const half2v_t f = __builtin_bit_cast(half2v_t, and_or(rep, mask, 0x64006400u)) - k1024;
                            const half2v_t rc = {(_Float16)(2.0f / (float)(1 << (2 * r))), (_Float16)(2.0f / (float)(1 << (2 * r + 1)))};
                            bw[4 * j + r] = __builtin_bit_cast(uint32_t, f * rc + minus1);   // 2 bit - 1, exact
                        }
                    }
                }
                d[m] = E::mfma(a0, uint4_t{bw[0], bw[1], bw[2], bw[3]}, d[m]);
                d[m] = E::mfma(a1, uint4_t{bw[4], bw[5], bw[6], bw[7]}, d[m]);
            }
        }
#pragma unroll
        for (int m = 0; m < NMAT; ++m) {
            const float sc = lds_s[(m * 16 + n) * sstride + gi];
            acc[m].x = __builtin_fmaf(sc, d[m].x, acc[m].x);
            acc[m].y = __builtin_fmaf(sc, d[m].y, acc[m].y);
            acc[m].z = __builtin_fmaf(sc, d[m].z, acc[m].z);
            acc[m].w = __builtin_fmaf(sc, d[m].w, acc[m].w);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    Step s0, s1;
    int step = chunk;
    issue(s0, step);
    issue(s1, step + kc);
    store_scales(first_run);
    for (int base = (int)blockDim.x; base < items; base += (int)blockDim.x) store_scales(load_scales(base + (int)threadIdx.x));
    if (threadIdx.x < NMAT * 16) lds_s[threadIdx.x * sstride + gt] = 0.0f;
    __syncthreads();
    for (; step < gt; step += 2 * kc) {
        consume(s0, step);
        issue(s0, step + 2 * kc);
        consume(s1, step + kc);
        issue(s1, step + 3 * kc);
    }

    {
        float4_t* mine = reinterpret_cast<float4_t*>(stage);
#pragma unroll
        for (int m = 0; m < NMAT; ++m) mine[m * kWave + lane] = acc[m];
    }
    __syncthreads();
    if (chunk == 0) {
        const unsigned char* first = smem + (size_t)NMAT * 16 * sstride * 4;
        float4_t sum[NMAT];
#pragma unroll
        for (int m = 0; m < NMAT; ++m) sum[m] = zero;
        for (int c = 0; c < kc; ++c)
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const float4_t part = reinterpret_cast<const float4_t*>(first + (size_t)c * kWaveBytes)[m * kWave + lane];
                sum[m].x += part.x; sum[m].y += part.y; sum[m].z += part.z; sum[m].w += part.w;
            }
        const int r = row0 + n;
        if (r < rows) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int tok = m0 + 4 * q + v;
                if (tok <= last_tok) {
                    float val[NMAT];
#pragma unroll
                    for (int m = 0; m < NMAT; ++m) val[m] = v == 0 ? sum[m].x : (v == 1 ? sum[m].y : (v == 2 ? sum[m].z : sum[m].w));
                    epi(tok, r, val);
                }
            }
        }
    }
}

}  // namespace smelt

// Argument lists of the single-token kernels of the same pipelines plus the number of tokens.
#define SMELT_SIGNED_QSS(FN, BITSV, XRV, T, ACT)                                                            \
    SMELT_QMS_KERNEL void smelt_signed_##FN##_qss_x##XRV##_matvec_##T(                              \
        const uint8_t* C, const uint16_t* S, const uint16_t* X, uint16_t* Y, uint32_t rows,        \
        uint32_t cols, uint32_t tokens) {                                                          \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {C};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        qss_body<ACT, BITSV, 1, XRV>(w, s, X, (int)tokens, (int)rows, (int)cols, EpiStore<ACT>{{}, Y, (int)rows}); \
    }                                                                                              \
    SMELT_QMS_KERNEL void smelt_signed_##FN##_qss_x##XRV##_matvec_add_##T(                          \
        const uint8_t* C, const uint16_t* S, const uint16_t* X, uint16_t* Y, const uint16_t* res,  \
        uint32_t rows, uint32_t cols, uint32_t tokens) {                                           \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {C};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        qss_body<ACT, BITSV, 1, XRV>(w, s, X, (int)tokens, (int)rows, (int)cols, EpiAdd<ACT>{{}, Y, res, (int)rows}); \
    }                                                                                              \
    SMELT_QMS_KERNEL void smelt_signed_##FN##_qss_x##XRV##_gate_up_swiglu_##T(                      \
        const uint8_t* gC, const uint16_t* gS, const uint8_t* uC, const uint16_t* uS,              \
        const uint16_t* X, uint16_t* Y, uint32_t rows, uint32_t cols, uint32_t tokens) {           \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gC, uC};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        qss_body<ACT, BITSV, 2, XRV>(w, s, X, (int)tokens, (int)rows, (int)cols, EpiSignedSwiglu<ACT>{{}, Y, (int)rows}); \
    }

// the ternary-affine names: the scale plane bound a second time is ignored, as in the single-token kernels
#define SMELT_TERAFF_QSS(XRV, T, ACT)                                                                       \
    SMELT_QMS_KERNEL void smelt_teraff_qss_x##XRV##_matvec_##T(                                     \
        const uint8_t* C, const uint16_t* S, const uint16_t*, const uint16_t* X, uint16_t* Y,      \
        uint32_t rows, uint32_t cols, uint32_t tokens) {                                           \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {C};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        qss_body<ACT, 2, 1, XRV>(w, s, X, (int)tokens, (int)rows, (int)cols, EpiStore<ACT>{{}, Y, (int)rows}); \
    }                                                                                              \
    SMELT_QMS_KERNEL void smelt_teraff_qss_x##XRV##_matvec_add_##T(                                 \
        const uint8_t* C, const uint16_t* S, const uint16_t*, const uint16_t* X, uint16_t* Y,      \
        const uint16_t* res, uint32_t rows, uint32_t cols, uint32_t tokens) {                      \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {C};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        qss_body<ACT, 2, 1, XRV>(w, s, X, (int)tokens, (int)rows, (int)cols, EpiAdd<ACT>{{}, Y, res, (int)rows}); \
    }                                                                                              \
    SMELT_QMS_KERNEL void smelt_teraff_qss_x##XRV##_gate_up_swiglu_##T(                             \
        const uint8_t* gC, const uint16_t* gS, const uint16_t*, const uint8_t* uC,                 \
        const uint16_t* uS, const uint16_t*, const uint16_t* X, uint16_t* Y, uint32_t rows,        \
        uint32_t cols, uint32_t tokens) {                                                          \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gC, uC};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        qss_body<ACT, 2, 2, XRV>(w, s, X, (int)tokens, (int)rows, (int)cols, EpiSignedSwiglu<ACT>{{}, Y, (int)rows}); \
    }

// ---- token-tile form: prefill chunks ------------------------------------------------------------
// The same arithmetic for many tokens.  A workgroup of four waves (two along the rows, two along the
// tokens) owns 32 * RT weight rows times 32 * TB tokens and walks K one pair of scale groups at a time.
// Per step the threads bring the tile's activations (stored in the operand order of the codes), packed
// weights and (scale, bias - base * scale) pairs into one of two LDS buffers, shared by the waves, while
// the other buffer is multiplied; the global loads run two steps ahead in registers (buffer loads: a
// uniform descriptor per tensor, a 32-bit offset per thread), the scales for four steps at a time
// (16 bytes per row and tensor).  Each wave unpacks a 16-row B operand once per step and group and reuses
// it for its TB token blocks.  With KW = 2 the workgroup has eight waves: the second four take the second
// scale group of every step, and the two halves of K meet in LDS at the end; that halves the time of a
// workgroup when the matrix has too few tiles to give every compute unit two.
namespace smelt {

constexpr int kQtThreads = 256;
// one buffer of a tile of bn rows (per matrix) times bm tokens
__host__ __device__ constexpr size_t qmt_buffer_bytes(int nmat, int bn, int bm) {
    return (size_t)bm * kQsXStride + (size_t)nmat * bn * kQsWStride + (size_t)nmat * bn * 2 * 8;
}
__host__ __device__ constexpr size_t qmt_lds_bytes(int nmat, int bn, int bm) { return 2 * qmt_buffer_bytes(nmat, bn, bm); }

template <class ActT, class ScaleT, int NMAT, int RT, int TB, int KW, bool PERWAVE, class Epi>
__device__ __forceinline__ void qmt_body(const uint8_t* const (&W)[NMAT], const uint16_t* const (&S)[NMAT],
                                         const uint16_t* const (&B)[NMAT], const uint16_t* __restrict__ X, int batch,
                                         int rows, int cols, float* ws_partial, uint32_t* ws_counters, const Epi& epi) {
    using E = Elem16<ActT>;
    using O = QsOperand<ActT>;
    static_assert(KW == 1 || KW == 2, "one or two waves along K");
    // PERWAVE (two matrices): the two waves along the rows take one matrix each (RT row tiles of it) instead
    // of half the rows of both, so a wave's loop is that of the one-matrix kernel; gate and up of an element
    // meet in LDS at the end.
    static_assert(!PERWAVE || NMAT == 2, "one matrix per wave is for gate and up");
    constexpr int AM = PERWAVE ? 1 : NMAT;              // matrices a wave accumulates
    constexpr int BN = (PERWAVE ? 16 : 32) * RT, BM = 32 * TB;   // rows (per matrix) and tokens of the workgroup tile
    constexpr int NT = kQtThreads * KW;                 // threads of the workgroup
    constexpr int XI = BM * 16 / NT;                    // 16-byte activation loads per thread and step
    constexpr int WROWS = NMAT * BN;                    // staged weight rows
    constexpr int WI = (WROWS * 4 + NT - 1) / NT;       // 16-byte weight loads per thread and step
    static_assert(BM * 16 % NT == 0 && WROWS <= NT, "staging assignment");
    // a weight load of NT threads covers NT / 4 staged rows: all of one matrix
    static_assert(NMAT == 1 || BN % (NT / 4) == 0 || WI == 1, "a weight load stays within one matrix, or there is only one");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr size_t kBuf = qmt_buffer_bytes(NMAT, BN, BM);
    constexpr size_t kOffW = (size_t)BM * kQsXStride, kOffS = kOffW + (size_t)WROWS * kQsWStride;   // within a buffer
    constexpr int D = 2;                                // steps in flight in registers
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int wn = wave & 1, wm = (wave >> 1) & 1, wk = wave >> 2;
    const int n = lane & 15, q = lane >> 4;
    const int gt = cols >> 6, rs = cols >> 1;
    // gridDim.z workgroups share a tile: each takes a run of blocks of four steps (cols is a multiple of 512)
    const int nblocks = gt >> 3, ksplit = gridDim.z, ks = blockIdx.z;
    const int first_block = (int)((long)nblocks * ks / ksplit), end_block = (int)((long)nblocks * (ks + 1) / ksplit);
    const int first_pair = 4 * first_block, npairs = 4 * end_block;   // this workgroup's steps: [first_pair, npairs)
    const int row0 = blockIdx.x * BN;
    const int m0 = blockIdx.y * BM;
    const int last_tok = (batch < m0 + BM ? batch : m0 + BM) - 1;

    // staging assignment: sixteen lanes per token row, four lanes per weight row, one thread per
    // staged row for the scales (staged row = (matrix * 2 + row half) * 16 RT + row in half)
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(X), 0, 0xFFFFFFFF, 0x00027000);
    __amdgpu_buffer_rsrc_t w_rsrc[NMAT];
#pragma unroll
    for (int m = 0; m < NMAT; ++m) w_rsrc[m] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(W[m]), 0, 0xFFFFFFFF, 0x00027000);
    int x_off[XI], x_dst[XI];
#pragma unroll
    for (int j = 0; j < XI; ++j) {
        const int item = tid + NT * j, t = item >> 4, piece = item & 15;
        int tok = m0 + t;
        if (tok > last_tok) tok = last_tok;
        x_off[j] = (tok * cols + 8 * piece) * 2;
        x_dst[j] = t * kQsXStride + 16 * piece;
    }
    // a single weight load that spans both matrices takes its matrix from a pointer per thread
    constexpr bool kSplitLoad = NMAT > 1 && BN % (NT / 4) != 0;
    int w_off[WI], w_dst[WI];
    const uint8_t* w_ptr = nullptr;
#pragma unroll
    for (int j = 0; j < WI; ++j) {
        int item = tid + NT * j;
        if (item > WROWS * 4 - 1) item = WROWS * 4 - 1;
        const int sr = item >> 2, piece = item & 3, m = sr / BN;
        int r = row0 + (sr - m * BN);
        if (r > rows - 1) r = rows - 1;
        w_off[j] = r * rs + 16 * piece;
        w_dst[j] = sr * kQsWStride + 16 * piece;
        if (kSplitLoad) w_ptr = (m == 1 ? W[NMAT - 1] : W[0]) + w_off[j];
    }
    const uint16_t* s_src;
    const uint16_t* b_src;
    {
        int sr = tid;
        if (sr > WROWS - 1) sr = WROWS - 1;
        const int m = sr / BN;
        int r = row0 + (sr - m * BN);
        if (r > rows - 1) r = rows - 1;
        s_src = (NMAT > 1 && m == 1 ? S[NMAT - 1] : S[0]) + (size_t)r * gt;
        b_src = (NMAT > 1 && m == 1 ? B[NMAT - 1] : B[0]) + (size_t)r * gt;
    }
    const int s_dst = tid < WROWS ? tid : WROWS - 1;

    struct Step { uint4_t x[XI]; uint4_t w[WI]; };
    struct Scales { uint4_t s, b; };   // eight groups (four steps) of one staged row
    auto issue = [&](Step& st, int pair) {
#pragma unroll
        for (int j = 0; j < XI; ++j) st.x[j] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, x_off[j], 256 * pair, 0);
#pragma unroll
        for (int j = 0; j < WI; ++j) {
            constexpr int per = NT / 4;   // staged rows per load
            const int m = NMAT == 1 || kSplitLoad ? 0 : ((per * j) / BN < NMAT ? (per * j) / BN : NMAT - 1);
            if (kSplitLoad) st.w[j] = *reinterpret_cast<const uint4_t*>(w_ptr + 64 * pair);
            else st.w[j] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc[m], w_off[j], 64 * pair, 0);
        }
    };
    auto issue_scales = [&](Scales& sc, int block) {
        sc.s = *reinterpret_cast<const uint4_t*>(s_src + 8 * block);
        sc.b = *reinterpret_cast<const uint4_t*>(b_src + 8 * block);
    };
    auto stage = [&](const Step& st, uint32_t sp, uint32_t bp, unsigned char* buf) {
        float2* lds_sc = reinterpret_cast<float2*>(buf + kOffS);   // [staged row][2]
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const float s = ScaleT::widen((uint16_t)(e ? sp >> 16 : sp & 0xFFFFu));
            const float b = ScaleT::widen((uint16_t)(e ? bp >> 16 : bp & 0xFFFFu));
            lds_sc[s_dst * 2 + e] = float2{s, __builtin_fmaf(-O::kBase, s, b)};
        }
#pragma unroll
        for (int j = 0; j < XI; ++j) *reinterpret_cast<uint4_t*>(buf + x_dst[j]) = O::activations(st.x[j]);
#pragma unroll
        for (int j = 0; j < WI; ++j) {
            *reinterpret_cast<uint2_t*>(buf + kOffW + w_dst[j]) = uint2_t{st.w[j].x, st.w[j].y};
            *reinterpret_cast<uint2_t*>(buf + kOffW + w_dst[j] + 8) = uint2_t{st.w[j].z, st.w[j].w};
        }
    };

    const float4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint4_t ones = {O::kOnePair, O::kOnePair, O::kOnePair, O::kOnePair};
    float4_t acc[AM][RT][TB];
#pragma unroll
    for (int m = 0; m < AM; ++m)
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int u = 0; u < TB; ++u) acc[m][t][u] = zero;

    auto multiply = [&](const unsigned char* buf) {
        const float2* lds_sc = reinterpret_cast<const float2*>(buf + kOffS);
#pragma unroll
        for (int ee = 0; ee < 2 / KW; ++ee) {
            const int e = KW == 2 ? wk : ee;
            uint4_t a0[TB], a1[TB];
            float4_t xs[TB];
#pragma unroll
            for (int u = 0; u < TB; ++u) {
                const unsigned char* xr = buf + ((wm * TB + u) * 16 + n) * kQsXStride + 128 * e + 32 * q;
                a0[u] = *reinterpret_cast<const uint4_t*>(xr);
                a1[u] = *reinterpret_cast<const uint4_t*>(xr + 16);
                xs[u] = E::mfma(a1[u], ones, E::mfma(a0[u], ones, zero));
            }
#pragma unroll
            for (int m = 0; m < AM; ++m)
#pragma unroll
                for (int t = 0; t < RT; ++t) {
                    const int sr = PERWAVE ? (wn * RT + t) * 16 + n : ((m * 2 + wn) * RT + t) * 16 + n;
                    const uint2_t c = *reinterpret_cast<const uint2_t*>(buf + kOffW + sr * kQsWStride + 32 * e + 8 * q);
                    const uint4_t b0 = O::codes(c.x), b1 = O::codes(c.y);
                    const float2 sb = lds_sc[sr * 2 + e];
#pragma unroll
                    for (int u = 0; u < TB; ++u) {
                        const float4_t d = E::mfma(a1[u], b1, E::mfma(a0[u], b0, zero));
                        acc[m][t][u].x = __builtin_fmaf(sb.x, d.x, __builtin_fmaf(sb.y, xs[u].x, acc[m][t][u].x));
                        acc[m][t][u].y = __builtin_fmaf(sb.x, d.y, __builtin_fmaf(sb.y, xs[u].y, acc[m][t][u].y));
                        acc[m][t][u].z = __builtin_fmaf(sb.x, d.z, __builtin_fmaf(sb.y, xs[u].z, acc[m][t][u].z));
                        acc[m][t][u].w = __builtin_fmaf(sb.x, d.w, __builtin_fmaf(sb.y, xs[u].w, acc[m][t][u].w));
                    }
                }
        }
    };

    // Loads past the last pair repeat it (staged into the idle buffer, never multiplied), so that no
    // load sits under a branch.  `sc` holds the scales of the block of four steps being staged; it is
    // reloaded as soon as the block's last step is staged, one step before its next use.
    const int last_pair = npairs - 1, last_block = end_block - 1;
    Step st[D];
    Scales sc;
    issue_scales(sc, first_block);
#pragma unroll
    for (int d = 0; d < D; ++d) issue(st[d], first_pair + d < last_pair ? first_pair + d : last_pair);
    stage(st[0], sc.s.x, sc.b.x, smem);
    issue(st[0], first_pair + D < last_pair ? first_pair + D : last_pair);
    __syncthreads();
    for (int base = first_pair; base < npairs; base += 4) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int pair = base + d;
            // the next step's tile goes into the other buffer (everyone left it at the last barrier)
            unsigned char* to = smem + ((d + 1) & 1) * kBuf;
            if (d == 0) stage(st[(d + 1) % D], sc.s.y, sc.b.y, to);
            if (d == 1) stage(st[(d + 1) % D], sc.s.z, sc.b.z, to);
            if (d == 2) {
                stage(st[(d + 1) % D], sc.s.w, sc.b.w, to);
                const int block = (base >> 2) + 1;
                issue_scales(sc, block < last_block ? block : last_block);
            }
            if (d == 3) stage(st[(d + 1) % D], sc.s.x, sc.b.x, to);
            issue(st[(d + 1) % D], pair + 1 + D < last_pair ? pair + 1 + D : last_pair);
            multiply(smem + (d & 1) * kBuf);
            __syncthreads();
        }
    }

    constexpr int NV = AM * RT * TB * 4;   // accumulator values per lane
    if constexpr (KW == 2) {
        // the two halves of every step meet in LDS (all waves are past the last barrier of the loop):
        // value j of lane l of wave pair p at [(p * NV + j) * 64 + l]
        static_assert((size_t)4 * NV * kWave * sizeof(float) <= 2 * kBuf, "reduction fits the staging buffers");
        float* red = reinterpret_cast<float*>(smem) + (size_t)(wave & 3) * NV * kWave + lane;
        if (wk == 1) {
#pragma unroll
            for (int m = 0; m < AM; ++m)
#pragma unroll
                for (int t = 0; t < RT; ++t)
#pragma unroll
                    for (int u = 0; u < TB; ++u) {
                        float* at = red + (size_t)((m * RT + t) * TB + u) * 4 * kWave;
                        at[0] = acc[m][t][u].x; at[kWave] = acc[m][t][u].y; at[2 * kWave] = acc[m][t][u].z; at[3 * kWave] = acc[m][t][u].w;
                    }
        }
        __syncthreads();
        if (wk == 0) {
#pragma unroll
            for (int m = 0; m < AM; ++m)
#pragma unroll
                for (int t = 0; t < RT; ++t)
#pragma unroll
                    for (int u = 0; u < TB; ++u) {
                        const float* at = red + (size_t)((m * RT + t) * TB + u) * 4 * kWave;
                        acc[m][t][u].x += at[0]; acc[m][t][u].y += at[kWave]; acc[m][t][u].z += at[2 * kWave]; acc[m][t][u].w += at[3 * kWave];
                    }
        }
    }
    if (ksplit > 1) {
        // Workgroup partials meet in the workspace; the last to arrive adds them in slice order, so the
        // result does not depend on the order of arrival.  Partials are written and read with agent-scope
        // relaxed atomics (coherent across the compute dies without cache write-backs), value j of thread t
        // at [j * 256 + t].  A workgroup's stores are complete before its arrival is counted, and the last
        // arrival reads only after its count returned.  The counter is left at zero for the next launch.
        __shared__ uint32_t last_flag;
        const size_t tile = (size_t)blockIdx.y * gridDim.x + blockIdx.x;
        float* mine = ws_partial + (tile * ksplit + ks) * NV * kQtThreads + tid;
        if (wk == 0) {
#pragma unroll
            for (int m = 0; m < AM; ++m)
#pragma unroll
                for (int t = 0; t < RT; ++t)
#pragma unroll
                    for (int u = 0; u < TB; ++u) {
                        float* at = mine + (size_t)((m * RT + t) * TB + u) * 4 * kQtThreads;
                        __hip_atomic_store(at, acc[m][t][u].x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(at + kQtThreads, acc[m][t][u].y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(at + 2 * kQtThreads, acc[m][t][u].z, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(at + 3 * kQtThreads, acc[m][t][u].w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
        }
        __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0): this wave's stores are acknowledged
        __syncthreads();
        if (tid == 0) last_flag = atomicAdd(ws_counters + tile, 1u) == (uint32_t)(ksplit - 1) ? 1u : 0u;
        __syncthreads();
        if (!last_flag) return;
        if (wk == 0) {
#pragma unroll
            for (int m = 0; m < AM; ++m)
#pragma unroll
                for (int t = 0; t < RT; ++t)
#pragma unroll
                    for (int u = 0; u < TB; ++u) {
                        float4_t sum = zero;
                        for (int c = 0; c < ksplit; ++c) {
                            const float* at = ws_partial + (tile * ksplit + c) * NV * kQtThreads + tid + (size_t)((m * RT + t) * TB + u) * 4 * kQtThreads;
                            sum.x += __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            sum.y += __hip_atomic_load(at + kQtThreads, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            sum.z += __hip_atomic_load(at + 2 * kQtThreads, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            sum.w += __hip_atomic_load(at + 3 * kQtThreads, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        }
                        acc[m][t][u] = sum;
                    }
        }
        if (tid == 0) ws_counters[tile] = 0u;
    }
    if (wk != 0) return;

    if constexpr (PERWAVE) {
        // the waves that hold up hand their sums to the waves that hold gate of the same elements:
        // value j of lane l of token half wm at [(wm * NV + j) * 64 + l]
        static_assert((size_t)2 * NV * kWave * sizeof(float) <= 2 * kBuf, "the exchange fits the staging buffers");
        float* xch = reinterpret_cast<float*>(smem) + (size_t)wm * NV * kWave + lane;
        asm volatile("s_barrier" ::: "memory");   // the four waves that are left: everyone is done with LDS
        if (wn == 1) {
#pragma unroll
            for (int t = 0; t < RT; ++t)
#pragma unroll
                for (int u = 0; u < TB; ++u) {
                    float* at = xch + (size_t)(t * TB + u) * 4 * kWave;
                    at[0] = acc[0][t][u].x; at[kWave] = acc[0][t][u].y; at[2 * kWave] = acc[0][t][u].z; at[3 * kWave] = acc[0][t][u].w;
                }
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (wn == 1) return;
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            const int r = row0 + t * 16 + n;
            if (r < rows) {
#pragma unroll
                for (int u = 0; u < TB; ++u) {
                    const float* at = xch + (size_t)(t * TB + u) * 4 * kWave;
                    const float up[4] = {at[0], at[kWave], at[2 * kWave], at[3 * kWave]};
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int tok = m0 + (wm * TB + u) * 16 + 4 * q + v;
                        if (tok <= last_tok) {
                            const float val[2] = {v == 0 ? acc[0][t][u].x : (v == 1 ? acc[0][t][u].y : (v == 2 ? acc[0][t][u].z : acc[0][t][u].w)), up[v]};
                            epi((size_t)tok * rows + r, val);
                        }
                    }
                }
            }
        }
        return;
    } else {
    // lane (n, q) holds row n of tile t and tokens 4 q .. 4 q + 3 of block u
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int r = row0 + (wn * RT + t) * 16 + n;
        if (r < rows) {
#pragma unroll
            for (int u = 0; u < TB; ++u)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int tok = m0 + (wm * TB + u) * 16 + 4 * q + v;
                    if (tok <= last_tok) {
                        float val[NMAT];
#pragma unroll
                        for (int m = 0; m < NMAT; ++m)
                            val[m] = v == 0 ? acc[m][t][u].x : (v == 1 ? acc[m][t][u].y : (v == 2 ? acc[m][t][u].z : acc[m][t][u].w));
                        epi((size_t)tok * rows + r, val);
                    }
                }
        }
    }
    }
}

}  // namespace smelt

// Two workgroups per compute unit at least (the second launch-bound is in waves per SIMD): that caps the kernel at 256
// (four waves) or 128 (eight waves) registers, all of them VGPRs, so the MFMA results land where the fp32 FMAs read them
// (with the whole 512-register file on offer the compiler parks them in AGPRs and copies).
#define SMELT_QMT_KERNEL(KWV) extern "C" __global__ __launch_bounds__(256 * KWV, 2 * KWV)

// Argument lists of the token-slab qmm kernels of the same pipelines, plus the two workspace
// pointers of the skinny ones (used when gridDim.z workgroups split K).
#define SMELT_AFFINE_QMT_PLAIN(T, ACT, SC, RTV, TBV, KWV)                                          \
    SMELT_QMT_KERNEL(KWV) void smelt_affine_qmt_r##RTV##_t##TBV##_k##KWV##_store_##T(              \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* Y,    \
        uint32_t batch, uint32_t rows, uint32_t cols, uint32_t, uint32_t, float* WSP, uint32_t* WSC) { \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        qmt_body<ACT, SC, 1, RTV, TBV, KWV, false>(w, s, b, X, batch, rows, cols, WSP, WSC, QsStore<ACT>{Y}); \
    }                                                                                              \
    SMELT_QMT_KERNEL(KWV) void smelt_affine_qmt_r##RTV##_t##TBV##_k##KWV##_add_##T(                \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* MV,   \
        const uint16_t* RES, uint16_t* OUT, uint32_t batch, uint32_t rows, uint32_t cols,          \
        uint32_t, uint32_t, float* WSP, uint32_t* WSC) {                                           \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        qmt_body<ACT, SC, 1, RTV, TBV, KWV, false>(w, s, b, X, batch, rows, cols, WSP, WSC, QsAdd<ACT>{MV, RES, OUT}); \
    }

#define SMELT_AFFINE_QMT_GATE_UP(T, ACT, SC, RTV, TBV, KWV, PWV, TAG)                                        \
    SMELT_QMT_KERNEL(KWV) void smelt_affine_qmt_##TAG##RTV##_t##TBV##_k##KWV##_gate_up_swiglu_##T(     \
        const uint8_t* gW, const uint16_t* gS, const uint16_t* gB, const uint8_t* uW,              \
        const uint16_t* uS, const uint16_t* uB, const uint16_t* X, uint16_t* Y, uint32_t batch,    \
        uint32_t rows, uint32_t cols, uint32_t, uint32_t, float* WSP, uint32_t* WSC) {             \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        qmt_body<ACT, SC, 2, RTV, TBV, KWV, PWV>(w, s, b, X, batch, rows, cols, WSP, WSC, QsSwiglu<ACT>{Y}); \
    }                                                                                              \
    SMELT_QMT_KERNEL(KWV) void smelt_affine_qmt_##TAG##RTV##_t##TBV##_k##KWV##_gate_up_geglu_##T(      \
        const uint8_t* gW, const uint16_t* gS, const uint16_t* gB, const uint8_t* uW,              \
        const uint16_t* uS, const uint16_t* uB, const uint16_t* X, uint16_t* Y, uint32_t batch,    \
        uint32_t rows, uint32_t cols, uint32_t, uint32_t, float* WSP, uint32_t* WSC) {             \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        qmt_body<ACT, SC, 2, RTV, TBV, KWV, PWV>(w, s, b, X, batch, rows, cols, WSP, WSC, QsGeglu<ACT>{Y}); \
    }
