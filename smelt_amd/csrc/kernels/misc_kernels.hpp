// Element-exact dequant (embedding gathers) and argmax kernels.
#pragma once
#include "common.hpp"

namespace smelt {

// w = float(code) * scale + bias with one rounded multiply and one rounded add (never fused),
// then narrowed to the output type: the per-element contract of the packed formats.
template <class ScaleT, class OutT>
__device__ __forceinline__ uint16_t dequant_affine(uint32_t nib, uint16_t s, uint16_t b) {
    const float p = __fmul_rn((float)nib, ScaleT::widen(s));
    return OutT::narrow(__fadd_rn(p, ScaleT::widen(b)));
}

template <class ScaleT, class OutT>
__device__ __forceinline__ void affine_gather_body(const uint8_t* W, const uint16_t* S,
                                                   const uint16_t* B, const int* token_ids,
                                                   uint16_t* out, uint32_t cols, uint32_t group,
                                                   uint32_t batch, uint32_t batch_count) {
    const uint32_t half_cols = cols / 2;
    const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= half_cols || batch >= batch_count) return;
    const size_t row = (size_t)(uint32_t)token_ids[batch];
    const uint32_t gpr = cols / group;
    const uint8_t packed = W[row * half_cols + t];
    const uint32_t c0 = t * 2, c1 = c0 + 1;
    const size_t sb = row * gpr;
    out[(size_t)batch * cols + c0] = dequant_affine<ScaleT, OutT>(packed & 0xFu, S[sb + c0 / group], B[sb + c0 / group]);
    out[(size_t)batch * cols + c1] = dequant_affine<ScaleT, OutT>(packed >> 4, S[sb + c1 / group], B[sb + c1 / group]);
}

// FORMAT: 0 binary1, 1 ternary2, 2 trit5 (5 base-3 digits per byte, LUT-decoded).
// trit5 rows are padded to a 16-byte multiple.
__device__ __forceinline__ uint32_t trit5_row_stride(uint32_t cols) {
    return (((cols + 4) / 5) + 15u) & ~15u;
}

template <int FORMAT, class OutT>
__device__ __forceinline__ void signed_gather_body(const uint8_t* codes, const uint16_t* scales,
                                                   const int* token_ids, uint16_t* out,
                                                   uint32_t hidden, const uint16_t* trit_lut) {
    const uint32_t col = blockIdx.x * blockDim.x + threadIdx.x;
    if (col >= hidden) return;
    const uint32_t b = blockIdx.y;
    const size_t row = (size_t)(uint32_t)token_ids[b];
    const uint32_t groups = hidden / 128;
    float value;
    if (FORMAT == 1) {
        const uint32_t packed = (codes[row * (hidden / 4) + col / 4] >> (2u * (col & 3u))) & 3u;
        value = (float)((int)packed - 1);
    } else if (FORMAT == 0) {
        const uint32_t packed = (codes[row * (hidden / 8) + col / 8] >> (col & 7u)) & 1u;
        value = packed == 0u ? -1.0f : 1.0f;
    } else {
        const uint32_t byte = codes[row * trit5_row_stride(hidden) + col / 5];
        const uint32_t packed = (trit_lut[byte] >> (2u * (col % 5u))) & 3u;
        value = (float)((int)packed - 1);
    }
    out[(size_t)b * hidden + col] = OutT::narrow(__fmul_rn(value, F16::widen(scales[row * groups + col / 128])));
}

// 243-entry decode table: five 2-bit codes (digit i at bits 2i..2i+1) per byte value.
__device__ __forceinline__ uint16_t trit5_lut_entry(uint32_t b) {
    if (b >= 243u) return 0x0155u;  // invalid bytes decode to five semantic zeros
    uint32_t e = 0;
#pragma unroll
    for (int i = 0; i < 5; ++i) { e |= (b % 3u) << (2 * i); b /= 3u; }
    return (uint16_t)e;
}

}  // namespace smelt

#define SMELT_MISC_KERNEL extern "C" __global__ __launch_bounds__(256)

#define SMELT_GATHER_KERNELS(T, ACT)                                                              \
    SMELT_MISC_KERNEL void smelt_affine_embedding_gather_##T(                                     \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const int* token_id,              \
        uint16_t* out, uint32_t cols, uint32_t group) {                                           \
        smelt::affine_gather_body<ACT, ACT>(W, S, B, token_id, out, cols, group, 0, 1);           \
    }                                                                                             \
    SMELT_MISC_KERNEL void smelt_affine_embedding_gather_batched_##T(                             \
        const uint8_t* W, const uint16_t* S, const uint16_t* B, const int* token_ids,             \
        uint16_t* out, uint32_t cols, uint32_t batch, uint32_t group) {                           \
        smelt::affine_gather_body<ACT, ACT>(W, S, B, token_ids, out, cols, group, blockIdx.y,     \
                                            batch);                                               \
    }                                                                                             \
    SMELT_MISC_KERNEL void smelt_signed_binary_embedding_gather_##T(                              \
        const uint8_t* C, const uint16_t* S, const int* ids, uint16_t* out, uint32_t hidden) {    \
        smelt::signed_gather_body<0, ACT>(C, S, ids, out, hidden, nullptr);                       \
    }                                                                                             \
    SMELT_MISC_KERNEL void smelt_signed_ternary_embedding_gather_##T(                             \
        const uint8_t* C, const uint16_t* S, const int* ids, uint16_t* out, uint32_t hidden) {    \
        smelt::signed_gather_body<1, ACT>(C, S, ids, out, hidden, nullptr);                       \
    }                                                                                             \
    SMELT_MISC_KERNEL void smelt_signed_trit5_embedding_gather_##T(                               \
        const uint8_t* C, const uint16_t* S, const int* ids, uint16_t* out, uint32_t hidden) {    \
        __shared__ uint16_t lut[256];                                                             \
        lut[threadIdx.x & 255] = smelt::trit5_lut_entry(threadIdx.x & 255);                       \
        if (blockDim.x < 256)                                                                     \
            for (uint32_t i = threadIdx.x; i < 256; i += blockDim.x)                              \
                lut[i] = smelt::trit5_lut_entry(i);                                               \
        __syncthreads();                                                                          \
        smelt::signed_gather_body<2, ACT>(C, S, ids, out, hidden, lut);                           \
    }

// The rows a norm-scale qmm multiplies, written out once for all of the matrix's workgroups:
// out[t][c] = narrow((x[t][c] * rs[t]) * (1 + w[c])), the bits a staged norm stores.  Eight columns per thread
// (cols is a multiple of eight), grid (columns / 2048 rounded up, tokens).
#define SMELT_NORM_SCALE_ROWS(T, ACT)                                                             \
    SMELT_MISC_KERNEL void smelt_norm_scale_rows_##T(                                             \
        const float* rs, const uint16_t* x, const uint16_t* w, uint16_t* out, uint32_t batch, uint32_t cols) { \
        using namespace smelt;                                                                    \
        const uint32_t tok = blockIdx.y, c0 = (blockIdx.x * blockDim.x + threadIdx.x) * 8;        \
        if (tok >= batch || c0 >= cols) return;                                                   \
        const float r = rs[tok];                                                                  \
        const uint4_t xv = *reinterpret_cast<const uint4_t*>(x + (size_t)tok * cols + c0);        \
        const uint4_t wv = *reinterpret_cast<const uint4_t*>(w + c0);                             \
        uint32_t o[4];                                                                            \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                           \
            const uint16_t lo = norm_scale_value<ACT>((uint16_t)(xv[j] & 0xFFFFu), r, (uint16_t)(wv[j] & 0xFFFFu)); \
            const uint16_t hi = norm_scale_value<ACT>((uint16_t)(xv[j] >> 16), r, (uint16_t)(wv[j] >> 16));         \
            o[j] = (uint32_t)lo | ((uint32_t)hi << 16);                                           \
        }                                                                                         \
        *reinterpret_cast<uint4_t*>(out + (size_t)tok * cols + c0) = uint4_t{o[0], o[1], o[2], o[3]}; \
    }

#ifndef SMELT_NO_INCLUDE_INSTANCES
SMELT_GATHER_KERNELS(f16, smelt::F16)
SMELT_GATHER_KERNELS(bf16, smelt::BF16)
SMELT_NORM_SCALE_ROWS(f16, smelt::F16)
SMELT_NORM_SCALE_ROWS(bf16, smelt::BF16)
#endif

#ifndef SMELT_NO_INCLUDE_INSTANCES
// ---- argmax over materialised 16-bit logits ---------------------------------------------------
// Largest value wins, ties go to the lowest index, -0 equals +0.  The ordering of the 16-bit
// pattern is the same for fp16 and bf16 (sign + magnitude), so one kernel serves both.
SMELT_MISC_KERNEL void smelt_argmax16_partials(const uint16_t* logits, smelt::uint2_t* partials,
                                               uint32_t vocab, uint32_t chunk) {
    using namespace smelt;
    const uint32_t start = blockIdx.x * chunk;
    const uint32_t end = start + chunk < vocab ? start + chunk : vocab;
    uint2_t best = {0u, 0u};
    for (uint32_t i = start + threadIdx.x; i < end; i += blockDim.x)
        best = argmax_key_max(best, argmax_pack_key(logits[i], i));
    best = wave_argmax_key(best);
    __shared__ uint2_t wave_best[16];
    const uint32_t wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) wave_best[wave] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t waves = (blockDim.x + kWave - 1) / kWave;
        for (uint32_t w = 1; w < waves; ++w) best = argmax_key_max(best, wave_best[w]);
        partials[blockIdx.x] = best;
    }
}
#endif

// Best key of row[0 .. n) over the workgroup's threads, four independent loads in flight per
// thread (a one-load-per-iteration loop pays a full memory round trip per iteration).
namespace smelt {
__device__ __forceinline__ uint2_t strided_key_max(const uint2_t* row, uint32_t n) {
    uint2_t best = {0u, 0u};
    for (uint32_t base = threadIdx.x; base < n; base += 4 * blockDim.x) {
        uint2_t v[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const uint32_t i = base + j * blockDim.x;
            v[j] = i < n ? row[i] : uint2_t{0u, 0u};
        }
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) best = argmax_key_max(best, v[j]);
    }
    return best;
}
}  // namespace smelt

#ifndef SMELT_NO_INCLUDE_INSTANCES
// one block per batch row (blockIdx.x); partials are [batch, num_partials]
SMELT_MISC_KERNEL void smelt_argmax_key_reduce(const smelt::uint2_t* partials, int* output,
                                               uint32_t num_partials) {
    using namespace smelt;
    const uint2_t* row = partials + (size_t)blockIdx.x * num_partials;
    uint2_t best = strided_key_max(row, num_partials);
    best = wave_argmax_key(best);
    __shared__ uint2_t wave_best[16];
    const uint32_t wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) wave_best[wave] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t waves = (blockDim.x + kWave - 1) / kWave;
        for (uint32_t w = 1; w < waves; ++w) best = argmax_key_max(best, wave_best[w]);
        output[blockIdx.x] = (int)(kArgmaxMaxIndex - best.y);
    }
}

// lm_head reduce: same as above with the batch guard of the fused lm_head path
SMELT_MISC_KERNEL void smelt_lm_head_argmax_reduce(const smelt::uint2_t* partials, int* output,
                                                   uint32_t batch, uint32_t num_partials) {
    using namespace smelt;
    if (blockIdx.x >= batch) return;
    const uint2_t* row = partials + (size_t)blockIdx.x * num_partials;
    uint2_t best = strided_key_max(row, num_partials);
    best = wave_argmax_key(best);
    __shared__ uint2_t wave_best[16];
    const uint32_t wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) wave_best[wave] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t waves = (blockDim.x + kWave - 1) / kWave;
        for (uint32_t w = 1; w < waves; ++w) best = argmax_key_max(best, wave_best[w]);
        output[blockIdx.x] = (int)(kArgmaxMaxIndex - best.y);
    }
}

// lm_head over several tokens, second half: the streaming qmm has left the rounded logits of `batch`
// tokens in `logits` [batch][rows]; this forms the same partial keys the fused matvec+argmax kernel
// leaves (one per token and grid column, any partition of the rows gives the same final key), so the
// record's reduce launch reads them unchanged.  Grid (num_partials, batch), one wave per workgroup.
// The bits are ordered as 16-bit floats of either type (sign and magnitude), so one kernel serves both.
SMELT_MISC_KERNEL void smelt_logits_argmax_partials(const uint16_t* __restrict__ logits, smelt::uint2_t* partials,
                                                    uint32_t batch, uint32_t rows, uint32_t num_partials) {
    using namespace smelt;
    const uint32_t tok = blockIdx.y;
    if (tok >= batch || blockIdx.x >= num_partials) return;
    const uint32_t per = (rows + num_partials - 1) / num_partials;
    const uint32_t lo = blockIdx.x * per;
    const uint32_t hi = lo + per < rows ? lo + per : rows;
    const uint16_t* row = logits + (size_t)tok * rows;
    uint2_t best = uint2_t{0u, 0u};
    for (uint32_t r = lo + threadIdx.x; r < hi; r += blockDim.x) {
        const uint2_t key = argmax_pack_key(row[r], r);
        if (argmax_key_gt(key, best)) best = key;
    }
    best = wave_argmax_key(best);
    __shared__ uint2_t wave_best[16];
    const uint32_t wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == 0) wave_best[wave] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t waves = (blockDim.x + kWave - 1) / kWave;
        for (uint32_t w = 1; w < waves; ++w) best = argmax_key_max(best, wave_best[w]);
        partials[(size_t)tok * num_partials + blockIdx.x] = best;
    }
}

// Plain device copy of n16 16-byte elements (grid-stride).  It moves a known number of bytes
// each way, which makes it the calibration kernel for memory-traffic counters.
extern "C" __global__ __launch_bounds__(256) void smelt_copy_u128(const smelt::uint4_t* __restrict__ src,
                                                                  smelt::uint4_t* __restrict__ dst,
                                                                  uint32_t n16) {
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// Plain device read of n16 16-byte elements (grid-stride, four loads in flight per thread): every
// thread folds what it read into one element of dst (dst[global thread id], inside the first n16
// elements).  What this kernel reaches on a buffer is what a weight-streaming kernel can hope for
// on the same bytes.
extern "C" __global__ __launch_bounds__(256) void smelt_read_u128(const smelt::uint4_t* __restrict__ src,
                                                                  smelt::uint4_t* __restrict__ dst,
                                                                  uint32_t n16) {
    const uint32_t stride = gridDim.x * blockDim.x, first = blockIdx.x * blockDim.x + threadIdx.x;
    smelt::uint4_t acc = {0u, 0u, 0u, 0u};
    uint32_t i = first;
    for (; i + 3 * stride < n16; i += 4 * stride) {
        const smelt::uint4_t a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
        acc.x ^= a.x ^ b.x ^ c.x ^ d.x; acc.y ^= a.y ^ b.y ^ c.y ^ d.y;
        acc.z ^= a.z ^ b.z ^ c.z ^ d.z; acc.w ^= a.w ^ b.w ^ c.w ^ d.w;
    }
    for (; i < n16; i += stride) {
        const smelt::uint4_t a = src[i];
        acc.x ^= a.x; acc.y ^= a.y; acc.z ^= a.z; acc.w ^= a.w;
    }
    if (first < n16) dst[first] = acc;
}

// The same read with the streaming (non-temporal) hint the weight kernels use and U loads in flight
// per thread, and without the per-thread store of read_u128 (8 MB of writes per launch at 2048 workgroups).  Together with the launch grid (workgroups per compute unit) these are the knobs of a
// reader; the benchmark sweeps them to find what the memory system hands a kernel at each launch size.
template <int U>
__device__ __forceinline__ void smelt_read_stream(const smelt::uint4_t* __restrict__ src, smelt::uint4_t* __restrict__ dst, uint32_t n16) {
    const uint32_t stride = gridDim.x * blockDim.x, first = blockIdx.x * blockDim.x + threadIdx.x;
    smelt::uint4_t acc = {0u, 0u, 0u, 0u};
    uint32_t i = first;
    for (; i + (U - 1) * stride < n16; i += U * stride) {
        smelt::uint4_t v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < U; ++u) { acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w; }
    }
    for (; i < n16; i += stride) {
        const smelt::uint4_t a = __builtin_nontemporal_load(src + i);
        acc.x ^= a.x; acc.y ^= a.y; acc.z ^= a.z; acc.w ^= a.w;
    }
    // a reader writes nothing: the store below keeps the loads alive and (almost) never executes
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x5EED1E55u && first < n16) dst[first] = acc;
}
extern "C" __global__ __launch_bounds__(256) void smelt_read_u128_nt4(const smelt::uint4_t* __restrict__ src, smelt::uint4_t* __restrict__ dst, uint32_t n16) {
    smelt_read_stream<4>(src, dst, n16);
}
extern "C" __global__ __launch_bounds__(256) void smelt_read_u128_nt8(const smelt::uint4_t* __restrict__ src, smelt::uint4_t* __restrict__ dst, uint32_t n16) {
    smelt_read_stream<8>(src, dst, n16);
}
extern "C" __global__ __launch_bounds__(256) void smelt_read_u128_nt16(const smelt::uint4_t* __restrict__ src, smelt::uint4_t* __restrict__ dst, uint32_t n16) {
    smelt_read_stream<16>(src, dst, n16);
}
#endif
