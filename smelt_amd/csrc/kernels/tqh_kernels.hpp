// turbo_quant_h family (Resources/Shaders/lut_matvec.metal:1045-1079, 9207-9486): 2-bit codes index a
// four-entry fp16 codebook per 128-COLUMN group, and the group's values are the Sylvester-Hadamard
// rotation of the looked-up entries:
//     W[r, g*128 + p] = 1/sqrt(128) * sum_j sign(p, j) * cb[g][code(r, g, j)],  sign = (-1)^popcount(p & j).
// The matvec moves the rotation onto the activations once per token,
//     xhat[g, j] = sum_p sign(p, j) * x[g*128 + p],   y[r] = 1/sqrt(128) * sum_{g, j} cb[g][code(r, g, j)] * xhat[g, j],
// so the per-row work is one codebook lookup and one multiply-add per weight.
#pragma once
#include "common.hpp"

namespace smelt {
constexpr float kTqhInvSqrtG = 0.0883883476483184405f;
}

// xhat, fp32, summed over p in increasing order; columns beyond `cols` count as zero.  One thread
// per (group, j); grid.y = token.  Works for any 1-D launch that covers groups * 128 threads.
#define SMELT_TQH_KERNELS(T, ACT)                                                                  \
    extern "C" __global__ __launch_bounds__(1024) void smelt_tqh_matvec_prepare_input_##T(         \
        const uint16_t* x, float* xhat, uint32_t cols) {                                           \
        const uint32_t groups = (cols + 127u) / 128u;                                              \
        const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;                                \
        if (gid >= groups * 128u) return;                                                          \
        const uint32_t g = gid / 128u, j = gid % 128u, base = g * 128u;                            \
        x += (size_t)blockIdx.y * cols;                                                            \
        float acc = 0.0f;                                                                          \
        if (base + 128u <= cols && (reinterpret_cast<uintptr_t>(x + base) & 15u) == 0) {           \
            /* whole group: sixteen 16-byte loads, same additions in the same order */             \
            _Pragma("unroll 4") for (uint32_t q = 0; q < 16u; ++q) {                               \
                const smelt::uint4_t v = reinterpret_cast<const smelt::uint4_t*>(x + base)[q];     \
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};                                        \
                _Pragma("unroll") for (uint32_t k = 0; k < 8u; ++k) {                              \
                    const float xp = ACT::widen((uint16_t)(w[k >> 1] >> (16u * (k & 1u))));        \
                    acc += (__builtin_popcount((8u * q + k) & j) & 1) ? -xp : xp;                  \
                }                                                                                  \
            }                                                                                      \
        } else {                                                                                   \
            for (uint32_t p = 0; p < 128u && base + p < cols; ++p) {                               \
                const float xp = ACT::widen(x[base + p]);                                          \
                acc += (__builtin_popcount(p & j) & 1) ? -xp : xp;                                 \
            }                                                                                      \
        }                                                                                          \
        xhat[(size_t)blockIdx.y * groups * 128u + gid] = acc;                                      \
    }                                                                                              \
    /* codes [rows, codes_per_row] bytes (four codes per byte, LSB first), codebook [groups, 4] */ \
    extern "C" __global__ __launch_bounds__(256) void smelt_tqh_matvec_##T(                        \
        const uint8_t* codes, const uint16_t* codebook, const float* xhat, uint16_t* y,            \
        uint32_t rows, uint32_t cols, uint32_t codes_per_row) {                                    \
        using namespace smelt;                                                                     \
        extern __shared__ __attribute__((aligned(16))) unsigned char smem[];                       \
        float* lds_x = reinterpret_cast<float*>(smem);                                             \
        const uint32_t groups = (cols + 127u) / 128u;                                              \
        xhat += (size_t)blockIdx.y * groups * 128u;                                                \
        y += (size_t)blockIdx.y * rows;                                                            \
        for (uint32_t i = threadIdx.x; i < groups * 32u; i += blockDim.x)                          \
            reinterpret_cast<float4_t*>(lds_x)[i] = reinterpret_cast<const float4_t*>(xhat)[i];    \
        __syncthreads();                                                                           \
        const uint32_t waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x % kWave; \
        const uint32_t units = groups * 2u; /* 16 bytes = 64 codes = half a group */               \
        const uint32_t tiles = (rows + 3u) / 4u;                                                   \
        for (uint32_t tile = blockIdx.x * waves + wave; tile < tiles; tile += gridDim.x * waves) { \
            uint32_t row[4];                                                                       \
            float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};                                               \
            _Pragma("unroll") for (int r = 0; r < 4; ++r) {                                        \
                const uint32_t rr = tile * 4u + r;                                                 \
                row[r] = rr < rows ? rr : rows - 1u;                                               \
            }                                                                                      \
            for (uint32_t u = lane; u < units; u += kWave) {                                       \
                const uint32_t g = u >> 1;                                                         \
                /* the group's four fp16 entries as a byte table: low bytes in one dword, high */  \
                /* bytes in another, so that one byte permute looks up four codes at once */       \
                const uint2_t cbw = *reinterpret_cast<const uint2_t*>(codebook + g * 4u);          \
                const uint32_t cb_lo = __builtin_amdgcn_perm(cbw.y, cbw.x, 0x06040200u);           \
                const uint32_t cb_hi = __builtin_amdgcn_perm(cbw.y, cbw.x, 0x07050301u);           \
                uint4_t c[4];                                                                      \
                _Pragma("unroll") for (int r = 0; r < 4; ++r)                                      \
                    c[r] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(codes + (size_t)row[r] * codes_per_row + (size_t)u * 16u)); \
                const float4_t* xv4 = reinterpret_cast<const float4_t*>(lds_x + (size_t)u * 64u);  \
                _Pragma("unroll") for (int d = 0; d < 4; ++d) {                                    \
                    /* xs[i][k] = xhat of column 16 d + 4 i + k of this unit */                    \
                    float xs[4][4];                                                                \
                    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                \
                        const float4_t xv = xv4[4 * d + i];                                        \
                        xs[i][0] = xv.x; xs[i][1] = xv.y; xs[i][2] = xv.z; xs[i][3] = xv.w;        \
                    }                                                                              \
                    _Pragma("unroll") for (int r = 0; r < 4; ++r) {                                \
                        const uint32_t words[4] = {c[r].x, c[r].y, c[r].z, c[r].w};                \
                        _Pragma("unroll") for (int k = 0; k < 4; ++k) {                            \
                            /* byte i of sel = code of column 4 i + k (byte i of the dword) */     \
                            const uint32_t sel = (words[d] >> (2 * k)) & 0x03030303u;              \
                            const uint32_t lo = __builtin_amdgcn_perm(0u, cb_lo, sel);             \
                            const uint32_t hi = __builtin_amdgcn_perm(0u, cb_hi, sel);             \
                            const uint32_t w01 = __builtin_amdgcn_perm(hi, lo, 0x05010400u);       \
                            const uint32_t w23 = __builtin_amdgcn_perm(hi, lo, 0x07030602u);       \
                            const half2_t p01 = __builtin_bit_cast(half2_t, w01);                  \
                            const half2_t p23 = __builtin_bit_cast(half2_t, w23);                  \
                            acc[r] = __builtin_fmaf((float)p01.x, xs[0][k], acc[r]);               \
                            acc[r] = __builtin_fmaf((float)p01.y, xs[1][k], acc[r]);               \
                            acc[r] = __builtin_fmaf((float)p23.x, xs[2][k], acc[r]);               \
                            acc[r] = __builtin_fmaf((float)p23.y, xs[3][k], acc[r]);               \
                        }                                                                          \
                    }                                                                              \
                }                                                                                  \
            }                                                                                      \
            _Pragma("unroll") for (int r = 0; r < 4; ++r) acc[r] = group_sum_last<64>(acc[r]);     \
            if (lane == kWave - 1) {                                                               \
                _Pragma("unroll") for (int r = 0; r < 4; ++r)                                      \
                    if (tile * 4u + r < rows) y[tile * 4u + r] = ACT::narrow(acc[r] * kTqhInvSqrtG); \
            }                                                                                      \
        }                                                                                          \
    }                                                                                              \
    /* one dequantised row: thread gid = column (lut_matvec.metal:1045-1079) */                    \
    extern "C" __global__ __launch_bounds__(1024) void smelt_tqh_embedding_gather_##T(             \
        const uint8_t* codes, const uint16_t* codebook, const int* token, uint16_t* out,           \
        uint32_t codes_per_row, uint32_t cols) {                                                   \
        using namespace smelt;                                                                     \
        const uint32_t gid = blockIdx.x * blockDim.x + threadIdx.x;                                \
        if (gid >= cols) return;                                                                   \
        const uint32_t g = gid / 128u, p = gid % 128u;                                             \
        const uint8_t* src = codes + (size_t)(uint32_t)token[0] * codes_per_row + (size_t)g * 32u; \
        float acc = 0.0f;                                                                          \
        for (uint32_t j = 0; j < 128u; ++j) {                                                      \
            const uint32_t code = (src[j >> 2] >> ((j & 3u) * 2u)) & 3u;                           \
            const float c = F16::widen(codebook[g * 4u + code]);                                   \
            acc += (__builtin_popcount(p & j) & 1) ? -c : c;                                       \
        }                                                                                          \
        out[gid] = ACT::narrow(acc * kTqhInvSqrtG);                                                \
    }
