// Small-batch / prefill quantized matmul for gfx950:  Y[M, N] = X[M, K] * W[N, K]^T.
//
// A workgroup owns a 64-row slab of W and a tile of BM tokens.  Per K step of 128 columns it
//   1. dequantises the packed 64 x 128 weight tile into LDS as fp16, each element computed as
//      narrow_f16(float(code) * scale + bias) with one rounded multiply and one rounded add
//      (the embedding-row form of the per-element contract), so the tile is reused by every
//      token block and the dequant cost is amortised over BM tokens;
//   2. stages the BM x 128 activation tile into LDS as fp16;
//   3. feeds v_mfma_f32_16x16x32_f16 (fp32 accumulate): wave w owns weight rows 16w..16w+15 of
//      the slab and all BM/16 token blocks.
// Ternary2 weights {-s, 0, +s} are exact in fp16; affine weights carry one fp16 rounding
// (2^-12 relative), far inside the 2e-3 output tolerance.  bf16 activations are converted to
// fp16 on staging (exact for |x| in [2^-14, 65504]).
#pragma once
#include "common.hpp"

namespace smelt {

constexpr int kQmmBN = 64;    // weight rows per workgroup slab
constexpr int kQmmBK = 128;   // columns per K step
constexpr int kQmmPad = 8;    // fp16 elements of row padding in LDS (bank spread)
constexpr int kQmmLd = kQmmBK + kQmmPad;

struct QmmU4 {
    static constexpr bool kHasBias = true;
    static __device__ __forceinline__ int row_stride(int cols) { return cols / 2; }
    // 32 consecutive columns starting at k (k % 32 == 0) of one row -> 32 fp16 values
    template <class ScaleT>
    static __device__ __forceinline__ void dequant32(const uint8_t* row, int k, const uint16_t* srow,
                                                     const uint16_t* brow, int gshift, uint16_t* out) {
        const uint4_t c = *reinterpret_cast<const uint4_t*>(row + k / 2);
        const uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int g = (k + 8 * d) >> gshift;
            const float s = ScaleT::widen(srow[g]), b = ScaleT::widen(brow[g]);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float n = (float)((w[d] >> (4 * i)) & 0xFu);
                out[8 * d + i] = F16::narrow(__fadd_rn(__fmul_rn(n, s), b));
            }
        }
    }
};

struct QmmTer2 {
    static constexpr bool kHasBias = true;
    static __device__ __forceinline__ int row_stride(int cols) { return cols / 4; }
    // signed_quant_precise.metal:407-439: the two-bit field keeps its position inside the byte;
    // byte lane k multiplies it by its own fp16-rounded subscale fp16(scale / 4^k) and adds
    // -bias_scale. For scales whose quarter/sixteenth/sixty-fourth is not an fp16 value (small
    // scales reaching the subnormal range) this differs from (code - 1) * scale in the last bits.
    // The half-precision fused multiply-add rounds the exact value once; the unfused half form
    // gives the same bits because a subscale times a shifted ternary field is exact in fp16.
    template <class ScaleT>
    static __device__ __forceinline__ void dequant32(const uint8_t* row, int k, const uint16_t* srow,
                                                     const uint16_t* brow, int gshift, uint16_t* out) {
        const uint2_t c = *reinterpret_cast<const uint2_t*>(row + k / 4);
        const uint32_t w[2] = {c.x, c.y};
        const _Float16 s = __builtin_bit_cast(_Float16, srow[k >> gshift]);
        const _Float16 nb = -__builtin_bit_cast(_Float16, brow[k >> gshift]);
        const _Float16 sub[4] = {s, s * (_Float16)0.25f, s * (_Float16)0.0625f, s * (_Float16)0.015625f};
#pragma unroll
        for (int d = 0; d < 2; ++d)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int lane = i & 3;
                const _Float16 field = (_Float16)(int)(((w[d] >> (2 * i)) & 3u) << (2 * lane));
                out[16 * d + i] = __builtin_bit_cast(uint16_t, __builtin_fmaf16(sub[lane], field, nb));
            }
    }
};

// Accumulates acc[m][t] (t = token block) for weight slab rows [n0, n0+64) and tokens
// [m0, m0 + 16*MT) over the whole K range, for NMAT matrices sharing the activation tile.
template <class Q, class ActT, class ScaleT, int MT, int NMAT>
__device__ __forceinline__ void qmm_tile(const uint8_t* const (&W)[NMAT], const uint16_t* const (&S)[NMAT],
                                         const uint16_t* const (&B)[NMAT], const uint16_t* X,
                                         int rows, int cols, int gpr, int gshift, int batch, int n0,
                                         int m0, uint16_t* lds_w, uint16_t* lds_x,
                                         float4_t (&acc)[NMAT][MT]) {
    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int li = lane & 15, kb = lane >> 4;
    const int rs = Q::row_stride(cols);
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[m][t] = float4_t{0, 0, 0, 0};

    for (int k0 = 0; k0 < cols; k0 += kQmmBK) {
        __syncthreads();  // previous step's MFMA reads are done
        // ---- dequantise the weight tile(s): 64 rows x 4 segments of 32 columns = 256 work items
        {
            const int r = tid >> 2, seg = tid & 3;
            const int n = n0 + r;
            const int k = k0 + seg * 32;
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                uint16_t vals[32];
                if (n < rows && k < cols) {
                    Q::template dequant32<ScaleT>(W[m] + (size_t)n * rs, k, S[m] + (size_t)n * gpr,
                                                  Q::kHasBias ? B[m] + (size_t)n * gpr : nullptr, gshift, vals);
                } else {
#pragma unroll
                    for (int i = 0; i < 32; ++i) vals[i] = 0;
                }
                uint4_t* dst = reinterpret_cast<uint4_t*>(lds_w + ((size_t)m * kQmmBN + r) * kQmmLd + seg * 32);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint4_t v;
                    v.x = vals[8 * q + 0] | ((uint32_t)vals[8 * q + 1] << 16);
                    v.y = vals[8 * q + 2] | ((uint32_t)vals[8 * q + 3] << 16);
                    v.z = vals[8 * q + 4] | ((uint32_t)vals[8 * q + 5] << 16);
                    v.w = vals[8 * q + 6] | ((uint32_t)vals[8 * q + 7] << 16);
                    dst[q] = v;
                }
            }
        }
        // ---- stage the activation tile: 16*MT rows x 16 segments of 8 columns
        for (int item = tid; item < 16 * MT * 16; item += blockDim.x) {
            const int r = item >> 4, seg = item & 15;
            const int tok = m0 + r, k = k0 + seg * 8;
            uint4_t v = {0, 0, 0, 0};
            if (tok < batch && k < cols) {
                v = *reinterpret_cast<const uint4_t*>(X + (size_t)tok * cols + k);
                if (!ActT::kIsF16) {
                    uint32_t* p = reinterpret_cast<uint32_t*>(&v);
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        p[i] = (uint32_t)ActT::to_f16_bits((uint16_t)(p[i] & 0xFFFF)) |
                               ((uint32_t)ActT::to_f16_bits((uint16_t)(p[i] >> 16)) << 16);
                }
            }
            *reinterpret_cast<uint4_t*>(lds_x + (size_t)r * kQmmLd + seg * 8) = v;
        }
        __syncthreads();
        // ---- MFMA: A = weights (16 rows x 32 k), B = activations (32 k x 16 tokens)
#pragma unroll
        for (int ks = 0; ks < kQmmBK / 32; ++ks) {
            half8_t b[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t)
                b[t] = *reinterpret_cast<const half8_t*>(lds_x + (size_t)(t * 16 + li) * kQmmLd + ks * 32 + kb * 8);
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const half8_t a = *reinterpret_cast<const half8_t*>(
                    lds_w + ((size_t)m * kQmmBN + wave * 16 + li) * kQmmLd + ks * 32 + kb * 8);
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    acc[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[t], acc[m][t], 0, 0, 0);
            }
        }
    }
}

// Workgroup driver: grid-stride over 64-row slabs (x) and batch tiles of `batch_tile` tokens (y).
// The epilogue receives, per lane, token `tok` and 4 consecutive output rows n..n+3.
template <class Q, class ActT, class ScaleT, int MT, int NMAT, class Epi>
__device__ __forceinline__ void qmm_body(const uint8_t* const (&W)[NMAT], const uint16_t* const (&S)[NMAT],
                                         const uint16_t* const (&B)[NMAT], const uint16_t* X,
                                         int rows, int cols, int group, int batch, int batch_tile,
                                         const Epi& epi) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint16_t* lds_w = reinterpret_cast<uint16_t*>(smem);
    uint16_t* lds_x = lds_w + (size_t)NMAT * kQmmBN * kQmmLd;
    const int gshift = ilog2((uint32_t)group);
    const int gpr = (cols + group - 1) / group;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int li = lane & 15, nb = lane >> 4;
    const int slabs = (rows + kQmmBN - 1) / kQmmBN;
    const int m_lo = blockIdx.y * batch_tile;
    const int m_hi = m_lo + batch_tile < batch ? m_lo + batch_tile : batch;
    for (int slab = blockIdx.x; slab < slabs; slab += gridDim.x) {
        const int n0 = slab * kQmmBN;
        for (int m0 = m_lo; m0 < m_hi; m0 += 16 * MT) {
            float4_t acc[NMAT][MT];
            qmm_tile<Q, ActT, ScaleT, MT, NMAT>(W, S, B, X, rows, cols, gpr, gshift, batch, n0, m0, lds_w, lds_x, acc);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const int tok = m0 + t * 16 + li;
                const int n = n0 + wave * 16 + nb * 4;
                if (tok < m_hi) {
                    float v[NMAT][4];
#pragma unroll
                    for (int m = 0; m < NMAT; ++m) { v[m][0] = acc[m][t].x; v[m][1] = acc[m][t].y; v[m][2] = acc[m][t].z; v[m][3] = acc[m][t].w; }
                    epi(tok, n, rows, v);
                }
            }
        }
    }
}

// ---- qmm epilogues: (token, first row n, rows, values[NMAT][4]) ---------------------------------
template <class ActT>
struct QEpiStore {
    uint16_t* y;
    __device__ __forceinline__ void operator()(int tok, int n, int rows, const float (&v)[1][4]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n + i < rows) y[(size_t)tok * rows + n + i] = ActT::narrow(v[0][i]);
    }
};

// matvec_out = narrow(acc); out = narrow(widen(matvec_out) + residual)
template <class ActT>
struct QEpiAdd {
    uint16_t* mv;
    const uint16_t* residual;
    uint16_t* out;
    __device__ __forceinline__ void operator()(int tok, int n, int rows, const float (&v)[1][4]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n + i < rows) {
                const size_t idx = (size_t)tok * rows + n + i;
                const uint16_t p = ActT::narrow(v[0][i]);
                mv[idx] = p;
                out[idx] = ActT::narrow(ActT::widen(p) + ActT::widen(residual[idx]));
            }
    }
};

// agent_geglu_product (lut_matvec.metal:2235-2243)
template <class ActT>
struct QEpiGeglu {
    uint16_t* y;
    __device__ __forceinline__ void operator()(int tok, int n, int rows, const float (&v)[2][4]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n + i < rows) {
                const float g = ActT::widen(ActT::narrow(v[0][i])), u = ActT::widen(ActT::narrow(v[1][i]));
                float inner = 0.7978845608f * (g + 0.044715f * (g * g * g));
                inner = fminf(fmaxf(inner, -20.0f), 20.0f);
                const float gelu = 0.5f * g * (1.0f + tanhf(inner));
                y[(size_t)tok * rows + n + i] = ActT::narrow(fminf(fmaxf(gelu * u, -65504.0f), 65504.0f));
            }
    }
};

template <class ActT>
struct QEpiSwiglu {
    uint16_t* y;
    __device__ __forceinline__ void operator()(int tok, int n, int rows, const float (&v)[2][4]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (n + i < rows) {
                const float g = v[0][i], u = v[1][i];
                y[(size_t)tok * rows + n + i] = ActT::narrow(g / (1.0f + expf(-g)) * u);
            }
    }
};

}  // namespace smelt

// ---- affine qmm with exact weights -------------------------------------------------------------
// Rounding s*n+b to fp16 before the MFMA costs ~2^-12 per weight, which shows up on outputs that
// are small next to the row's largest terms.  The affine kernels therefore feed the MFMA the
// integer codes themselves (exact in fp16) one scale group at a time and apply the group's scale
// and bias in fp32 on the accumulators:
//     Y[m][n] += s[n,g] * sum_{k in g} code[n,k] * x[m,k]  +  b[n,g] * sum_{k in g} x[m,k]
// which is the grouped form of the reference matvec, with every product exact.
namespace smelt {

constexpr int kQxLdW = 64 + 16;  // bytes per slab row of packed codes in LDS (64 B data + pad)

template <class ActT, class ScaleT, int MT, int NMAT>
__device__ __forceinline__ void qmm_affine_tile(const uint8_t* const (&W)[NMAT], const uint16_t* const (&S)[NMAT],
                                                const uint16_t* const (&B)[NMAT], const uint16_t* X,
                                                int rows, int cols, int gpr, int gshift, int batch,
                                                int n0, int m0, unsigned char* smem,
                                                float4_t (&acc)[NMAT][MT], const NormScale& ns = NormScale{}) {
    // LDS: codes [NMAT][64][kQxLdW] bytes | x [16*MT][kQmmLd] fp16 (k permuted per 8) |
    //      xsum [16*MT][4] float (per 32-column quarter) | scale, bias [NMAT][4][64] float
    uint8_t* lds_c = smem;
    uint16_t* lds_x = reinterpret_cast<uint16_t*>(lds_c + (size_t)NMAT * kQmmBN * kQxLdW);
    float* lds_xs = reinterpret_cast<float*>(lds_x + (size_t)16 * MT * kQmmLd);
    float* lds_s = lds_xs + (size_t)16 * MT * 4;
    float* lds_b = lds_s + (size_t)NMAT * 4 * kQmmBN;
    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int li = lane & 15, kb = lane >> 4;
    const int rs = cols / 2;
    const int group = 1 << gshift;
    float4_t part[NMAT][MT];  // code-dot of the scale group in flight (may span K steps)
    float xg[MT];             // activation sum of that group
#pragma unroll
    for (int m = 0; m < NMAT; ++m)
#pragma unroll
        for (int t = 0; t < MT; ++t) { acc[m][t] = float4_t{0, 0, 0, 0}; part[m][t] = float4_t{0, 0, 0, 0}; }
#pragma unroll
    for (int t = 0; t < MT; ++t) xg[t] = 0.0f;

    for (int k0 = 0; k0 < cols; k0 += kQmmBK) {
        __syncthreads();
        // packed codes: 64 rows x 64 bytes, one 16-byte load per thread per matrix
        {
            const int r = tid >> 2, seg = tid & 3;
            const int n = n0 + r, k = k0 + seg * 32;
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                uint4_t v = {0, 0, 0, 0};
                if (n < rows && k < cols) v = *reinterpret_cast<const uint4_t*>(W[m] + (size_t)n * rs + k / 2);
                *reinterpret_cast<uint4_t*>(lds_c + ((size_t)m * kQmmBN + r) * kQxLdW + seg * 16) = v;
            }
        }
        // scales / biases of the (up to 4) 32-column quarters of this step, as fp32
        for (int item = tid; item < NMAT * 4 * kQmmBN; item += blockDim.x) {
            const int m = item / (4 * kQmmBN), rem = item % (4 * kQmmBN);
            const int q = rem / kQmmBN, r = rem % kQmmBN;
            const int n = n0 + r, k = k0 + q * 32;
            float sv = 0.0f, bv = 0.0f;
            if (n < rows && k < cols) {
                const size_t si = (size_t)n * gpr + (k >> gshift);
                sv = ScaleT::widen(S[m][si]);
                bv = ScaleT::widen(B[m][si]);
            }
            lds_s[item] = sv;
            lds_b[item] = bv;
        }
        // activations: 16*MT tokens x 4 quarters; each item converts 32 columns, permutes every
        // run of 8 to (0,4,1,5,2,6,3,7) to match the operand order of the code pairs, and sums them
        for (int item = tid; item < 16 * MT * 4; item += blockDim.x) {
            const int r = item >> 2, q = item & 3;
            const int tok = m0 + r, k = k0 + q * 32;
            float xsum = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint4_t v = {0, 0, 0, 0};
                if (tok < batch && k + e * 8 < cols) {
                    v = *reinterpret_cast<const uint4_t*>(X + (size_t)tok * cols + k + e * 8);
                    // norm-scale prologue: the tile multiplies the normalised row; the first row slab stores it
                    if (ns.rs != nullptr) {
                        uint32_t* p = reinterpret_cast<uint32_t*>(&v);
                        const float rs = ns.rs[tok];
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const uint16_t lo = norm_scale_element<ActT>(ns, (uint16_t)(p[i] & 0xFFFF), rs, (size_t)tok * cols, k + e * 8 + 2 * i);
                            const uint16_t hi = norm_scale_element<ActT>(ns, (uint16_t)(p[i] >> 16), rs, (size_t)tok * cols, k + e * 8 + 2 * i + 1);
                            p[i] = (uint32_t)lo | ((uint32_t)hi << 16);
                        }
                        if (ns.out != nullptr && n0 == 0) *reinterpret_cast<uint4_t*>(ns.out + (size_t)tok * cols + k + e * 8) = v;
                    }
                }
                uint16_t h[8];
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    h[2 * i] = ActT::to_f16_bits((uint16_t)(w[i] & 0xFFFF));
                    h[2 * i + 1] = ActT::to_f16_bits((uint16_t)(w[i] >> 16));
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) xsum += F16::widen(h[i]);
                uint4_t o;
                o.x = h[0] | ((uint32_t)h[4] << 16);
                o.y = h[1] | ((uint32_t)h[5] << 16);
                o.z = h[2] | ((uint32_t)h[6] << 16);
                o.w = h[3] | ((uint32_t)h[7] << 16);
                *reinterpret_cast<uint4_t*>(lds_x + (size_t)r * kQmmLd + q * 32 + e * 8) = o;
            }
            lds_xs[r * 4 + q] = xsum;
        }
        __syncthreads();
        // one 32-column MFMA step at a time; a scale group spans group/32 consecutive steps
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int k = k0 + ks * 32;
            const bool group_start = (k & (group - 1)) == 0;
            const bool group_end = ((k + 32) & (group - 1)) == 0 || k + 32 >= cols;
            if (group_start) {
#pragma unroll
                for (int m = 0; m < NMAT; ++m)
#pragma unroll
                    for (int t = 0; t < MT; ++t) part[m][t] = float4_t{0, 0, 0, 0};
#pragma unroll
                for (int t = 0; t < MT; ++t) xg[t] = 0.0f;
            }
            half8_t b[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                b[t] = *reinterpret_cast<const half8_t*>(lds_x + (size_t)(t * 16 + li) * kQmmLd + ks * 32 + kb * 8);
                xg[t] += lds_xs[(t * 16 + li) * 4 + ks];
            }
#pragma unroll
            for (int m = 0; m < NMAT; ++m) {
                const uint32_t c = *reinterpret_cast<const uint32_t*>(lds_c + ((size_t)m * kQmmBN + wave * 16 + li) * kQxLdW + ks * 16 + kb * 4);
                const uint32_t c8 = c >> 8;
                uint32_t p[4];
                p[0] = __builtin_amdgcn_bitop3_b32(c, 0x000F000Fu, 0x64006400u, 0xEA);
                p[1] = __builtin_amdgcn_bitop3_b32(c, 0x00F000F0u, 0x54005400u, 0xEA);
                p[2] = __builtin_amdgcn_bitop3_b32(c8, 0x000F000Fu, 0x64006400u, 0xEA);
                p[3] = __builtin_amdgcn_bitop3_b32(c8, 0x00F000F0u, 0x54005400u, 0xEA);
                half8_t a;
                {
                    const half2_t o1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
                    const half2_t o64 = {(_Float16)64.0f, (_Float16)64.0f};
                    const half2_t a0 = as_half2(p[0]) - o1024, a1 = as_half2(p[1]) - o64;
                    const half2_t a2 = as_half2(p[2]) - o1024, a3 = as_half2(p[3]) - o64;
                    a[0] = a0.x; a[1] = a0.y; a[2] = a1.x; a[3] = a1.y;
                    a[4] = a2.x; a[5] = a2.y; a[6] = a3.x; a[7] = a3.y;
                }
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    part[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b[t], part[m][t], 0, 0, 0);
            }
            if (group_end) {
                const int q = ks;  // scales are stored per quarter; all quarters of a group agree
#pragma unroll
                for (int m = 0; m < NMAT; ++m) {
                    const float4_t sv = *reinterpret_cast<const float4_t*>(lds_s + ((size_t)m * 4 + q) * kQmmBN + wave * 16 + kb * 4);
                    const float4_t bv = *reinterpret_cast<const float4_t*>(lds_b + ((size_t)m * 4 + q) * kQmmBN + wave * 16 + kb * 4);
#pragma unroll
                    for (int t = 0; t < MT; ++t) {
                        acc[m][t].x = __builtin_fmaf(sv.x, part[m][t].x, __builtin_fmaf(bv.x, xg[t], acc[m][t].x));
                        acc[m][t].y = __builtin_fmaf(sv.y, part[m][t].y, __builtin_fmaf(bv.y, xg[t], acc[m][t].y));
                        acc[m][t].z = __builtin_fmaf(sv.z, part[m][t].z, __builtin_fmaf(bv.z, xg[t], acc[m][t].z));
                        acc[m][t].w = __builtin_fmaf(sv.w, part[m][t].w, __builtin_fmaf(bv.w, xg[t], acc[m][t].w));
                    }
                }
            }
        }
    }
}

template <class ActT, class ScaleT, int MT, int NMAT, class Epi>
__device__ __forceinline__ void qmm_affine_body(const uint8_t* const (&W)[NMAT], const uint16_t* const (&S)[NMAT],
                                                const uint16_t* const (&B)[NMAT], const uint16_t* X,
                                                int rows, int cols, int group, int batch, int batch_tile,
                                                const Epi& epi, const NormScale& ns = NormScale{}) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int gshift = ilog2((uint32_t)group);
    const int gpr = (cols + group - 1) / group;
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int li = lane & 15, nb = lane >> 4;
    const int slabs = (rows + kQmmBN - 1) / kQmmBN;
    const int m_lo = blockIdx.y * batch_tile;
    const int m_hi = m_lo + batch_tile < batch ? m_lo + batch_tile : batch;
    for (int slab = blockIdx.x; slab < slabs; slab += gridDim.x) {
        const int n0 = slab * kQmmBN;
        for (int m0 = m_lo; m0 < m_hi; m0 += 16 * MT) {
            float4_t acc[NMAT][MT];
            qmm_affine_tile<ActT, ScaleT, MT, NMAT>(W, S, B, X, rows, cols, gpr, gshift, batch, n0, m0, smem, acc, ns);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const int tok = m0 + t * 16 + li;
                const int n = n0 + wave * 16 + nb * 4;
                if (tok < m_hi) {
                    float v[NMAT][4];
#pragma unroll
                    for (int m = 0; m < NMAT; ++m) { v[m][0] = acc[m][t].x; v[m][1] = acc[m][t].y; v[m][2] = acc[m][t].z; v[m][3] = acc[m][t].w; }
                    epi(tok, n, rows, v);
                }
            }
        }
    }
}

}  // namespace smelt

#define SMELT_QMM_KERNEL extern "C" __global__ __launch_bounds__(256)

#define SMELT_AFFINE_QMM(T, ACT, SC, MTV)                                                          \
    SMELT_QMM_KERNEL void smelt_affine_qmm_mt##MTV##_##T(                                          \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* Y,    \
        uint32_t batch, uint32_t rows, uint32_t cols, uint32_t group, uint32_t batch_tile) {       \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        QEpiStore<ACT> epi{Y};                                                                     \
        qmm_affine_body<ACT, SC, MTV, 1>(w, s, b, X, rows, cols, group, batch, batch_tile, epi);   \
    }                                                                                              \
    SMELT_QMM_KERNEL void smelt_affine_qmm_add_mt##MTV##_##T(                                      \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const uint16_t* X, uint16_t* MV,   \
        const uint16_t* RES, uint16_t* OUT, uint32_t batch, uint32_t rows, uint32_t cols,          \
        uint32_t group, uint32_t batch_tile) {                                                     \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        QEpiAdd<ACT> epi{MV, RES, OUT};                                                            \
        qmm_affine_body<ACT, SC, MTV, 1>(w, s, b, X, rows, cols, group, batch, batch_tile, epi);   \
    }                                                                                              \
    SMELT_QMM_KERNEL void smelt_affine_qmm_gate_up_swiglu_mt##MTV##_##T(                           \
        const uint8_t* gW, const uint16_t* gS, const uint16_t* gB, const uint8_t* uW,              \
        const uint16_t* uS, const uint16_t* uB, const uint16_t* X, uint16_t* Y, uint32_t batch,    \
        uint32_t rows, uint32_t cols, uint32_t group, uint32_t batch_tile) {                       \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        QEpiSwiglu<ACT> epi{Y};                                                                    \
        qmm_affine_body<ACT, SC, MTV, 2>(w, s, b, X, rows, cols, group, batch, batch_tile, epi);   \
    }                                                                                              \
    SMELT_QMM_KERNEL void smelt_affine_qmm_gate_up_geglu_mt##MTV##_##T(                            \
        const uint8_t* gW, const uint16_t* gS, const uint16_t* gB, const uint8_t* uW,              \
        const uint16_t* uS, const uint16_t* uB, const uint16_t* X, uint16_t* Y, uint32_t batch,    \
        uint32_t rows, uint32_t cols, uint32_t group, uint32_t batch_tile) {                       \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        QEpiGeglu<ACT> epi{Y};                                                                     \
        qmm_affine_body<ACT, SC, MTV, 2>(w, s, b, X, rows, cols, group, batch, batch_tile, epi);   \
    }                                                                                              \
    /* norm-scale prologue (agent_affine_qmm.h:790-...): rs[token], normalised rows stored by slab 0 */ \
    SMELT_QMM_KERNEL void smelt_norm_scale_affine_qmm_mt##MTV##_##T(                               \
        const float* rs, const uint16_t* X, const uint16_t* nw, uint16_t* XN, const uint8_t* W,    \
        const uint16_t* S, const uint16_t* B, uint16_t* Y, uint32_t batch, uint32_t rows,          \
        uint32_t cols, uint32_t group, uint32_t batch_tile) {                                      \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {W};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {B};                                                          \
        QEpiStore<ACT> epi{Y};                                                                     \
        qmm_affine_body<ACT, SC, MTV, 1>(w, s, b, X, rows, cols, group, batch, batch_tile, epi,    \
                                         NormScale{rs, nw, XN});                                   \
    }                                                                                              \
    SMELT_QMM_KERNEL void smelt_norm_scale_affine_qmm_gate_up_swiglu_mt##MTV##_##T(                \
        const float* rs, const uint16_t* X, const uint16_t* nw, const uint8_t* gW,                 \
        const uint16_t* gS, const uint16_t* gB, const uint8_t* uW, const uint16_t* uS,             \
        const uint16_t* uB, uint16_t* Y, uint32_t batch, uint32_t rows, uint32_t cols,             \
        uint32_t group, uint32_t batch_tile) {                                                     \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        QEpiSwiglu<ACT> epi{Y};                                                                    \
        qmm_affine_body<ACT, SC, MTV, 2>(w, s, b, X, rows, cols, group, batch, batch_tile, epi,    \
                                         NormScale{rs, nw, nullptr});                              \
    }                                                                                              \
    SMELT_QMM_KERNEL void smelt_norm_scale_affine_qmm_gate_up_geglu_mt##MTV##_##T(                 \
        const float* rs, const uint16_t* X, const uint16_t* nw, const uint8_t* gW,                 \
        const uint16_t* gS, const uint16_t* gB, const uint8_t* uW, const uint16_t* uS,             \
        const uint16_t* uB, uint16_t* Y, uint32_t batch, uint32_t rows, uint32_t cols,             \
        uint32_t group, uint32_t batch_tile) {                                                     \
        using namespace smelt;                                                                     \
        const uint8_t* const w[2] = {gW, uW};                                                      \
        const uint16_t* const s[2] = {gS, uS};                                                     \
        const uint16_t* const b[2] = {gB, uB};                                                     \
        QEpiGeglu<ACT> epi{Y};                                                                     \
        qmm_affine_body<ACT, SC, MTV, 2>(w, s, b, X, rows, cols, group, batch, batch_tile, epi,    \
                                         NormScale{rs, nw, nullptr});                              \
    }

#define SMELT_TERNARY_QMM(T, ACT, MTV)                                                             \
    SMELT_QMM_KERNEL void smelt_ternary_qmm_mt##MTV##_##T(                                         \
        const uint8_t* C, const uint16_t* S, const uint16_t* S2, const uint16_t* X, uint16_t* Y,   \
        uint32_t rows, uint32_t cols, uint32_t batch) {                                            \
        using namespace smelt;                                                                     \
        const uint8_t* const w[1] = {C};                                                           \
        const uint16_t* const s[1] = {S};                                                          \
        const uint16_t* const b[1] = {S2};                                                         \
        QEpiStore<ACT> epi{Y};                                                                     \
        qmm_body<QmmTer2, ACT, F16, MTV, 1>(w, s, b, X, rows, cols, 128, batch, 16 * MTV, epi);    \
    }

SMELT_AFFINE_QMM(f16, smelt::F16, smelt::F16, 1)
SMELT_AFFINE_QMM(f16, smelt::F16, smelt::F16, 4)
SMELT_AFFINE_QMM(bf16, smelt::BF16, smelt::BF16, 1)
SMELT_AFFINE_QMM(bf16, smelt::BF16, smelt::BF16, 4)
SMELT_TERNARY_QMM(f16, smelt::F16, 2)
SMELT_TERNARY_QMM(bf16, smelt::BF16, 2)
