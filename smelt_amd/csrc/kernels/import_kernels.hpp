// Build-time producers of the packed formats the matvec kernels read, on the GPU:
//   * group-wise affine 4-bit quantisation of an fp32 / fp16 / bf16 tensor
//     (SmeltAffineU4.quantizeRow, SmeltAffineU4.swift:94-136; endpoint search :59-91;
//      per-tensor driver SmeltAffineQuantizer.swift:399-513),
//   * validation of signed code streams (SmeltSignedQuantCodec.swift:128-145),
//   * MLX (scale, bias) pair -> canonical signed scale (SmeltSignedQuantCodec.swift:154-215).
// All results are bit-identical to the host algorithms: every fp32 operation below is a single
// correctly rounded operation in the reference's order (no contraction into fused multiply-adds).
#pragma once
#include "common.hpp"

namespace smelt {

enum ImportSrcDType : uint32_t { kSrcF32 = 0, kSrcF16 = 1, kSrcBF16 = 2 };

__device__ __forceinline__ float import_load(const void* src, size_t i, uint32_t dtype) {
    if (dtype == kSrcF32) return reinterpret_cast<const float*>(src)[i];
    const uint16_t b = reinterpret_cast<const uint16_t*>(src)[i];
    return dtype == kSrcF16 ? F16::widen(b) : BF16::widen(b);
}

// One thread quantises one (row, group): n <= G values held in registers.
//   scale = (hi - lo) / 15 (1 when the range is below 1e-12), bias = lo,
//   nibble = round(clamp((v - bias) * (1 / scale), 0, 15)).
// clip == 1 searches nine shrink factors of [min, max] for the least reconstruction error through
// the rounded scale and bias (optionally weighted per column), summing the error in column order.
template <class ScaleT, int G>
__device__ __forceinline__ void quantize_group(const float (&v)[G], int n, uint32_t clip,
                                               const float* importance, uint16_t* scale_bits,
                                               uint16_t* bias_bits, uint8_t (&bytes)[G / 2]) {
#pragma clang fp contract(off)
    float minv = __builtin_inff(), maxv = -__builtin_inff();
#pragma unroll
    for (int c = 0; c < G; ++c)
        if (c < n) {
            if (v[c] < minv) minv = v[c];
            if (v[c] > maxv) maxv = v[c];
        }
    float lo = minv, hi = maxv;
    if (clip != 0) {
        const float half = (maxv - minv) / 2.0f;
        if (!(half < 1e-12f)) {
            float best_err = __builtin_inff();
            for (int step = 0; step <= 8; ++step) {
                const float c = 1.0f - (float)step * 0.075f;
                const float l = minv + (1.0f - c) * half, h = maxv - (1.0f - c) * half;
                const float scale = (h - l) / 15.0f;
                const float scale_r = ScaleT::widen(ScaleT::narrow(scale));
                const float lo_r = ScaleT::widen(ScaleT::narrow(l));
                const float inv = 1.0f / scale;
                float err = 0.0f;
#pragma unroll
                for (int k = 0; k < G; ++k)
                    if (k < n) {
                        const float nib = __builtin_fminf(__builtin_fmaxf(__builtin_roundf((v[k] - l) * inv), 0.0f), 15.0f);
                        const float d = v[k] - (nib * scale_r + lo_r);
                        const float w = importance ? importance[k] : 1.0f;
                        err += w * d * d;
                    }
                if (err < best_err) { best_err = err; lo = l; hi = h; }
            }
        }
    }
    const float range = hi - lo;
    const float scale = range < 1e-12f ? 1.0f : range / 15.0f;
    *scale_bits = ScaleT::narrow(scale);
    *bias_bits = ScaleT::narrow(lo);
    const float inv = 1.0f / scale;
#pragma unroll
    for (int b = 0; b < G / 2; ++b) {
        uint32_t byte = 0;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int c = 2 * b + h;
            if (c < n) {
                const float normalized = (v[c] - lo) * inv;
                const float clamped = __builtin_fminf(__builtin_fmaxf(normalized, 0.0f), 15.0f);
                byte |= (uint32_t)__builtin_roundf(clamped) << (4 * h);
            }
        }
        bytes[b] = (uint8_t)byte;
    }
}

// A wave owns 64 consecutive (row, group) cells at a time.  Their values are fetched with
// coalesced loads (consecutive lanes, consecutive elements) into a wave-private LDS tile whose
// rows are padded by one word, from which every lane then reads its own group without bank
// conflicts.  Lane l writes the packed bytes, scale and bias of cell first + l.
template <class ScaleT, int G>
__device__ __forceinline__ void affine_quantize_body(const void* src, uint8_t* packed, uint16_t* scales,
                                                     uint16_t* biases, const float* importance,
                                                     uint32_t rows, uint32_t src_dtype, uint32_t clip,
                                                     uint32_t cols) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    constexpr int STRIDE = G + 1;
    constexpr int LOG_G = G == 32 ? 5 : (G == 64 ? 6 : 7);
    const uint32_t waves = blockDim.x / kWave;
    const uint32_t wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    float* tile = reinterpret_cast<float*>(smem) + (size_t)wave * (kWave * STRIDE + 2 * kWave);
    uint32_t* cell_row = reinterpret_cast<uint32_t*>(tile + kWave * STRIDE);
    uint32_t* cell_col = cell_row + kWave;
    const uint32_t gpr = (cols + G - 1) / G;
    const uint32_t total = rows * gpr;  // the host checks that this fits 32 bits
    const uint32_t packed_stride = (cols + 1) / 2;
    const uint32_t step = gridDim.x * waves * kWave;
    for (uint32_t first = (blockIdx.x * waves + wave) * kWave; first < total; first += step) {
        const uint32_t cell = first + lane;
        const uint32_t row = cell < total ? cell / gpr : 0xFFFFFFFFu;
        const uint32_t col0 = cell < total ? (cell - row * gpr) * G : 0;
        cell_row[lane] = row;
        cell_col[lane] = col0;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if ((cols & 3u) == 0) {
            // four consecutive elements per lane and load (one group, one row: G and cols are
            // multiples of four), every load of the tile in flight at once
            uint4_t raw[G / 4];
#pragma unroll
            for (int i = 0; i < G / 4; ++i) {
                const uint32_t e = ((uint32_t)i * kWave + lane) * 4;
                const uint32_t j = e >> LOG_G, c = e & (G - 1);
                const uint32_t r = cell_row[j];
                const uint32_t col = cell_col[j] + c;
                raw[i] = uint4_t{0u, 0u, 0u, 0u};
                if (r != 0xFFFFFFFFu && col < cols) {
                    const size_t at = (size_t)r * cols + col;
                    if (src_dtype == kSrcF32) {
                        raw[i] = *reinterpret_cast<const uint4_t*>(reinterpret_cast<const float*>(src) + at);
                    } else {
                        const uint2_t h = *reinterpret_cast<const uint2_t*>(reinterpret_cast<const uint16_t*>(src) + at);
                        raw[i].x = h.x; raw[i].y = h.y;
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < G / 4; ++i) {
                const uint32_t e = ((uint32_t)i * kWave + lane) * 4;
                const uint32_t j = e >> LOG_G, c = e & (G - 1);
                // (elements are copied out first: a bit cast applied directly to a vector element
                //  reads the vector's first lane)
                const uint32_t r0 = raw[i].x, r1 = raw[i].y, r2 = raw[i].z, r3 = raw[i].w;
                float f[4];
                if (src_dtype == kSrcF32) {
                    f[0] = __builtin_bit_cast(float, r0); f[1] = __builtin_bit_cast(float, r1);
                    f[2] = __builtin_bit_cast(float, r2); f[3] = __builtin_bit_cast(float, r3);
                } else if (src_dtype == kSrcF16) {
                    f[0] = F16::widen((uint16_t)r0); f[1] = F16::widen((uint16_t)(r0 >> 16));
                    f[2] = F16::widen((uint16_t)r1); f[3] = F16::widen((uint16_t)(r1 >> 16));
                } else {
                    f[0] = BF16::widen((uint16_t)r0); f[1] = BF16::widen((uint16_t)(r0 >> 16));
                    f[2] = BF16::widen((uint16_t)r1); f[3] = BF16::widen((uint16_t)(r1 >> 16));
                }
#pragma unroll
                for (int k = 0; k < 4; ++k) tile[j * STRIDE + c + k] = f[k];
            }
        } else {
#pragma unroll 8
            for (int i = 0; i < G; ++i) {
                const uint32_t e = (uint32_t)i * kWave + lane;
                const uint32_t j = e >> LOG_G, c = e & (G - 1);
                const uint32_t r = cell_row[j];
                const uint32_t col = cell_col[j] + c;
                float val = 0.0f;
                if (r != 0xFFFFFFFFu && col < cols) val = import_load(src, (size_t)r * cols + col, src_dtype);
                tile[j * STRIDE + c] = val;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (cell < total) {
            float v[G];
#pragma unroll
            for (int c = 0; c < G; ++c) v[c] = tile[lane * STRIDE + c];
            const int n = cols - col0 < (uint32_t)G ? (int)(cols - col0) : G;
            uint16_t sb, bb;
            uint8_t bytes[G / 2];
            quantize_group<ScaleT, G>(v, n, clip, importance ? importance + col0 : nullptr, &sb, &bb, bytes);
            scales[cell] = sb;
            biases[cell] = bb;
            uint8_t* dst = packed + (size_t)row * packed_stride + col0 / 2;
            const int nbytes = (n + 1) / 2;
            if (n == G && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
#pragma unroll
                for (int q = 0; q < G / 32; ++q) {
                    uint4_t w;
                    uint32_t t[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        t[k] = (uint32_t)bytes[16 * q + 4 * k] | ((uint32_t)bytes[16 * q + 4 * k + 1] << 8) |
                               ((uint32_t)bytes[16 * q + 4 * k + 2] << 16) | ((uint32_t)bytes[16 * q + 4 * k + 3] << 24);
                    w.x = t[0]; w.y = t[1]; w.z = t[2]; w.w = t[3];
                    reinterpret_cast<uint4_t*>(dst)[q] = w;
                }
            } else {
#pragma unroll
                for (int b = 0; b < G / 2; ++b)
                    if (b < nbytes) dst[b] = bytes[b];
            }
        }
        // the tile is rewritten by the next round
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

// ---- signed code streams ------------------------------------------------------------------
// status[0..1] is a 64-bit word the caller initialises to all ones; kernels lower it to the first
// offending index (validation) or to (group << 8 | reason) of the first offending group (scales).

__device__ __forceinline__ void status_min(unsigned long long* status, unsigned long long v) {
    atomicMin(status, v);
}

}  // namespace smelt

#define SMELT_IMPORT_KERNEL extern "C" __global__ __launch_bounds__(256)

#define SMELT_AFFINE_QUANTIZE(T, SC, GV)                                                          \
    SMELT_IMPORT_KERNEL void smelt_affine_quantize_g##GV##_##T(                                   \
        const void* src, uint8_t* packed, uint16_t* scales, uint16_t* biases,                     \
        const float* importance, uint32_t rows, uint32_t src_dtype, uint32_t clip, uint32_t cols, \
        uint32_t) {                                                                               \
        smelt::affine_quantize_body<SC, GV>(src, packed, scales, biases, importance, rows,        \
                                            src_dtype, clip, cols);                               \
    }

// ternary2: a 2-bit field equal to 3 is invalid; trit5: a byte above 242 is invalid.
// `count` logical codes; format 1 = ternary2, 2 = trit5.  One 16-byte unit per lane and step.
SMELT_IMPORT_KERNEL void smelt_signed_validate_codes(const uint8_t* codes, unsigned long long* status,
                                                     uint32_t count_lo, uint32_t count_hi,
                                                     uint32_t format) {
    const unsigned long long count = ((unsigned long long)count_hi << 32) | count_lo;
    const unsigned long long nbytes = format == 2 ? (count + 4) / 5 : (count * 2 + 7) / 8;
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x * 16;
    unsigned long long bad = ~0ull;
    for (unsigned long long at = ((unsigned long long)blockIdx.x * blockDim.x + threadIdx.x) * 16; at < nbytes; at += stride) {
        uint32_t w[4] = {0, 0, 0, 0};
        if (at + 16 <= nbytes && (reinterpret_cast<uintptr_t>(codes + at) & 15u) == 0) {
            const smelt::uint4_t t = *reinterpret_cast<const smelt::uint4_t*>(codes + at);
            w[0] = t.x; w[1] = t.y; w[2] = t.z; w[3] = t.w;
        } else {
            for (int b = 0; b < 16; ++b)
                if (at + b < nbytes) w[b >> 2] |= (uint32_t)codes[at + b] << (8 * (b & 3));
                else if (format == 2) w[b >> 2] |= 121u << (8 * (b & 3));  // five zero trits
        }
        for (int k = 0; k < 4 && bad == ~0ull; ++k) {
            if (format == 2) {
                for (int b = 0; b < 4; ++b)
                    if (((w[k] >> (8 * b)) & 0xFFu) >= 243u) {
                        const unsigned long long idx = (at + 4 * k + b) * 5;
                        if (idx < count && idx < bad) bad = idx;
                    }
            } else {
                uint32_t both = w[k] & (w[k] >> 1) & 0x55555555u;
                while (both) {
                    const int bit = __builtin_ctz(both);
                    const unsigned long long idx = (at + 4 * k) * 4 + (unsigned)(bit >> 1);
                    if (idx < count) { if (idx < bad) bad = idx; break; }
                    both &= both - 1;
                }
            }
        }
    }
    if (bad != ~0ull) smelt::status_min(status, bad);
}

// MLX stores a signed group as an affine (scale, bias) pair.  The canonical signed scale is half
// the MLX scale (binary) or the MLX scale itself (ternary), and the pair is accepted only when the
// bias is the negation of that canonical scale, exactly or to within one ulp of it.
// reason codes: 1 = scale not finite or negative, 2 = bias does not match.
SMELT_IMPORT_KERNEL void smelt_signed_normalize_mlx_scales(const uint16_t* scales, const uint16_t* biases,
                                                           uint16_t* out, unsigned long long* status,
                                                           uint32_t groups, uint32_t format) {
    using smelt::F16;
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t g = blockIdx.x * blockDim.x + threadIdx.x; g < groups; g += stride) {
        const uint16_t sb = scales[g], bb = biases[g];
        const float source = F16::widen(sb);
        const bool s_finite = ((sb >> 10) & 0x1Fu) != 31u;
        if (!s_finite || !(source >= 0.0f)) {
            smelt::status_min(status, ((unsigned long long)g << 8) | 1ull);
            continue;
        }
        const uint16_t canonical = format == 0 ? F16::narrow(source * 0.5f) : sb;
        const float canonical_f = F16::widen(canonical);
        const uint16_t expected = F16::narrow(-canonical_f);
        const float actual = F16::widen(bb);
        const uint32_t exp = (canonical >> 10) & 0x1Fu;
        const float ulp = exp == 0 ? 5.9604644775390625e-08f : __builtin_ldexpf(1.0f, (int)exp - 25);
        const bool b_finite = ((bb >> 10) & 0x1Fu) != 31u;
        const bool equivalent = b_finite && actual <= 0.0f && __builtin_fabsf(actual - F16::widen(expected)) <= ulp;
        if (!(bb == expected || equivalent)) {
            smelt::status_min(status, ((unsigned long long)g << 8) | 2ull);
            continue;
        }
        out[g] = canonical;
    }
}
