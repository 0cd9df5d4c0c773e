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

namespace smelt {
// Upper bound on the row quads (4 rows) a wave handles per tile.  A lane works on one
// (quad, 16-byte unit) item, so the quad count is chosen to make quads * units a multiple of the wave
// size where a small count does it (units = 40 for 2560 columns leaves 24 of 64 lanes idle with one
// quad), within a partial-sum budget of 32 KB of LDS per workgroup.  The host sizes the LDS with the
// same rule; the kernel may use fewer quads when the matrix has too few rows to occupy the grid.
__device__ __forceinline__ uint32_t tqh_max_quads_per_tile(uint32_t units, uint32_t waves) {
    uint32_t low = units & (0u - units);
    if (low > 64u) low = 64u;
    uint32_t q = 64u / low;
    if (q > 8u) q = 8u;
    while (q > 1u && (size_t)q * units * 16u * waves > 32768u) q >>= 1;
    return q;
}

// One lane's item: rows row0 .. row0 + 3 (clamped to the last row) against the 64 columns of unit u,
// added into acc.
__device__ __forceinline__ void tqh_item(const uint8_t* codes, const uint16_t* codebook, const float4_t* lds_x,
                                         uint32_t row0, uint32_t rows, uint32_t u, uint32_t codes_per_row,
                                         float (&acc)[4]) {
            const uint32_t g = u >> 1;
            const uint2_t cbw = *reinterpret_cast<const uint2_t*>(codebook + g * 4u);
            const uint32_t cb_lo = __builtin_amdgcn_perm(cbw.y, cbw.x, 0x06040200u);
            const uint32_t cb_hi = __builtin_amdgcn_perm(cbw.y, cbw.x, 0x07050301u);
            uint4_t c[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t rr = row0 + r < rows ? row0 + r : rows - 1u;
                c[r] = __builtin_nontemporal_load(
                    reinterpret_cast<const uint4_t*>(codes + (size_t)rr * codes_per_row + (size_t)u * 16u));
            }
            const float4_t* xv4 = lds_x + (size_t)u * 17u;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                float xs[4][4];  // xs[i][k] = xhat of column 16 d + 4 i + k of this unit
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float4_t xv = xv4[4 * d + i];
                    xs[i][0] = xv.x; xs[i][1] = xv.y; xs[i][2] = xv.z; xs[i][3] = xv.w;
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t words[4] = {c[r].x, c[r].y, c[r].z, c[r].w};
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        // byte i of sel = code of column 4 i + k (byte i of the dword)
                        const uint32_t sel = (words[d] >> (2 * k)) & 0x03030303u;
                        const uint32_t lo = __builtin_amdgcn_perm(0u, cb_lo, sel);
                        const uint32_t hi = __builtin_amdgcn_perm(0u, cb_hi, sel);
                        const half2_t p01 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(hi, lo, 0x05010400u));
                        const half2_t p23 = __builtin_bit_cast(half2_t, __builtin_amdgcn_perm(hi, lo, 0x07030602u));
                        acc[r] = __builtin_fmaf((float)p01.x, xs[0][k], acc[r]);
                        acc[r] = __builtin_fmaf((float)p01.y, xs[1][k], acc[r]);
                        acc[r] = __builtin_fmaf((float)p23.x, xs[2][k], acc[r]);
                        acc[r] = __builtin_fmaf((float)p23.y, xs[3][k], acc[r]);
                    }
                }
            }
}

// y[r] = 1/sqrt(128) * sum_j cb[g(j)][code(r, j)] * xhat[j].  The codebook lookup is a byte permute:
// the group's four fp16 entries are held as a low-byte table and a high-byte table, a dword of sixteen
// codes shifted by 2k and masked with 0x03030303 is the selector for the four columns 4i + k, and two
// more permutes interleave the looked-up bytes into fp16 pairs.
template <class ActT>
__device__ __forceinline__ void tqh_matvec_body(const uint8_t* codes, const uint16_t* codebook, const float* xhat,
                                                uint16_t* y, uint32_t rows, uint32_t cols, uint32_t codes_per_row,
                                                unsigned char* smem) {
    float4_t* lds_x = reinterpret_cast<float4_t*>(smem);
    const uint32_t groups = (cols + 127u) / 128u;
    xhat += (size_t)blockIdx.y * groups * 128u;
    y += (size_t)blockIdx.y * rows;
    // a lane reads the 256 bytes of its own unit: units sit 272 bytes apart so that the lanes of a
    // wave fall on different banks
    for (uint32_t i = threadIdx.x; i < groups * 32u; i += blockDim.x)
        lds_x[(i >> 4) * 17u + (i & 15u)] = reinterpret_cast<const float4_t*>(xhat)[i];
    __syncthreads();
    const uint32_t waves = blockDim.x / kWave, wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const uint32_t units = groups * 2u;  // 16 bytes = 64 codes = half a group
    const uint32_t max_quads = tqh_max_quads_per_tile(units, waves);
    uint32_t quads = max_quads;
    // keep a tile for every launched wave, up to two waves per SIMD of the 256-CU part
    const uint32_t want_tiles = gridDim.x * waves < 2048u ? gridDim.x * waves : 2048u;
    while (quads > 1u && (rows + quads * 4u - 1u) / (quads * 4u) < want_tiles) quads >>= 1;
    if (quads == 1u) {
        // one quad per wave tile: lanes stride over the units, partial sums stay in registers
        const uint32_t tiles4 = (rows + 3u) / 4u;
        for (uint32_t tile = blockIdx.x * waves + wave; tile < tiles4; tile += gridDim.x * waves) {
            float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (uint32_t u = lane; u < units; u += kWave)
                tqh_item(codes, codebook, lds_x, tile * 4u, rows, u, codes_per_row, acc);
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] = group_sum_last<64>(acc[r]);
            if (lane == kWave - 1) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (tile * 4u + r < rows) y[tile * 4u + r] = ActT::narrow(acc[r] * kTqhInvSqrtG);
            }
        }
        return;
    }
    const uint32_t items = quads * units, tile_rows = quads * 4u;
    float4_t* part = lds_x + (size_t)units * 17u + (size_t)wave * max_quads * units;
    const uint32_t tiles = (rows + tile_rows - 1u) / tile_rows;
    for (uint32_t tile = blockIdx.x * waves + wave; tile < tiles; tile += gridDim.x * waves) {
        for (uint32_t item = lane; item < items; item += kWave) {
            const uint32_t quad = item / units, u = item - quad * units;
            const uint32_t row0 = tile * tile_rows + quad * 4u;
            float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            tqh_item(codes, codebook, lds_x, row0, rows, u, codes_per_row, acc);
            part[item] = float4_t{acc[0], acc[1], acc[2], acc[3]};
        }
        // the wave's own LDS writes, read back by other lanes of the same wave
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        // lane = (sub, row of the tile): the 64 / tile_rows lanes of a row each sum a strided share of
        // its units, then meet through xor shuffles (tile_rows is 4, 8, 16 or 32)
        const uint32_t lanes_per_row = kWave / tile_rows;
        const uint32_t tr = lane & (tile_rows - 1u), sub = lane / tile_rows;
        float sum = 0.0f;
        {
            const float* col = reinterpret_cast<const float*>(part + (size_t)(tr >> 2) * units) + (tr & 3u);
            for (uint32_t u = sub; u < units; u += lanes_per_row) sum += col[(size_t)u * 4u];
        }
        for (uint32_t off = tile_rows; off < kWave; off <<= 1) sum += __shfl_xor(sum, (int)off);
        const uint32_t out_row = tile * tile_rows + tr;
        if (sub == 0u && out_row < rows) y[out_row] = ActT::narrow(sum * kTqhInvSqrtG);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}
}  // namespace smelt

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
        extern __shared__ __attribute__((aligned(16))) unsigned char smem[];                       \
        smelt::tqh_matvec_body<ACT>(codes, codebook, xhat, y, rows, cols, codes_per_row, smem);    \
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
