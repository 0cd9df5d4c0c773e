// Producers of signed activation views (signed_quant.metal:746-1298): every group of 128
// activations becomes a 16-bit scale (largest magnitude / largest integer) and sign-magnitude
// integers stored as bit planes, [group][plane][4 words], word w bit l = value 32 w + l.
//   values   plain input, the staged SwiGLU of (gate, up), a * sigmoid(b), or rms_norm_1pw's two-step value
//            half(x * rs) * half(1 + w) from a precomputed scale
//   scale    i2 and i3 views quantise with the unrounded fp32 scale, i4..i6 with the stored one
//   integer  round-half-away(clamp(value / scale, -max, +max)), max = 1 (i2) or 2^(planes-1) - 1
// One wave per group, grid-strided; a 32-thread workgroup (the reference's launch shape) works too.
#pragma once
#include "common.hpp"

namespace smelt {

enum BitplaneSource : int { kPlaneSrcPlain = 0, kPlaneSrcSwiglu = 1, kPlaneSrcNormScale = 2, kPlaneSrcSigmoidMul = 3 };

template <class ActT, int SRC>
__device__ __forceinline__ float bitplane_value(const float* norm_scale, const uint16_t* a, const uint16_t* b, size_t i) {
    if constexpr (SRC == kPlaneSrcPlain) {
        return ActT::widen(a[i]);
    } else if constexpr (SRC == kPlaneSrcSwiglu) {
        auto rt = [](float v) { return ActT::widen(ActT::narrow(v)); };
        const float g = ActT::widen(a[i]), u = ActT::widen(b[i]);
        const float e = rt(expf(fabsf(g)));
        const float tail = rt(1.0f / rt(1.0f + e));
        const float sig = g < 0.0f ? tail : rt(1.0f - tail);
        return rt(rt(g * sig) * u);
    } else if constexpr (SRC == kPlaneSrcSigmoidMul) {
        // a * sigmoid(b) with the sigmoid's every step in the 16-bit type (signed_quant.metal:1000-1006)
        auto rt = [](float v) { return ActT::widen(ActT::narrow(v)); };
        const float x = ActT::widen(a[i]), gate = ActT::widen(b[i]);
        const float tail = rt(1.0f / rt(1.0f + rt(expf(fabsf(gate)))));
        const float sig = gate < 0.0f ? tail : rt(1.0f - tail);
        return rt(x * sig);
    } else {
        const float normalized = ActT::widen(ActT::narrow(ActT::widen(a[i]) * norm_scale[0]));
        const float direct = ActT::widen(ActT::narrow(1.0f + ActT::widen(b[i])));
        return ActT::widen(ActT::narrow(normalized * direct));
    }
}

// One group of 128 values held `per_lane` to a lane (value k * width + lane in v[k]) -> its stored
// scale and bit planes.  Runs on the first `width` lanes of a wave.
template <class ActT>
__device__ __forceinline__ void bitplane_store_group(const float (&v)[4], uint32_t per_lane, uint32_t width, uint32_t lane,
                                                     uint32_t nplanes, uint32_t* dst, uint16_t* scale_dst) {
    const int max_q = nplanes == 2 ? 1 : (1 << (nplanes - 1)) - 1;
    float max_abs = 0.0f;
    for (uint32_t k = 0; k < per_lane; ++k) max_abs = __builtin_fmaxf(max_abs, __builtin_fabsf(v[k]));
    for (uint32_t off = width / 2; off > 0; off >>= 1) max_abs = __builtin_fmaxf(max_abs, __shfl_xor(max_abs, (int)off));
    const float producer = max_abs > 0.0f ? max_abs / (float)max_q : 1.0f;
    const uint16_t stored = ActT::narrow(producer);
    const float scale = nplanes >= 4 ? ActT::widen(stored) : producer;
    if (lane == 0) *scale_dst = stored;
    for (uint32_t k = 0; k < per_lane; ++k) {
        float t = v[k] / scale;
        t = __builtin_fminf(__builtin_fmaxf(t, -(float)max_q), (float)max_q);
        const int q = (int)__builtin_roundf(t);
        const uint32_t mag = (uint32_t)(q < 0 ? -q : q);
        for (uint32_t p = 0; p < nplanes; ++p) {
            const bool bit = p == nplanes - 1 ? q < 0 : ((mag >> p) & 1u) != 0;
            const unsigned long long mask = __ballot(bit);
            if (lane == 0) {
                uint32_t* w = dst + (size_t)p * 4;
                if (width == 64u) {
                    w[2 * k] = (uint32_t)mask;
                    w[2 * k + 1] = (uint32_t)(mask >> 32);
                } else {
                    w[k] = (uint32_t)mask;
                }
            }
        }
    }
}

// rms_norm_gated value of one element.  precise (the d128 kernels, norms_gated_precise.metal:7-18):
// half(w) * half(x * rs) as a 16-bit product, SiLU from the stable sigmoid in fp32, one final narrowing;
// otherwise the generic kernel's half(w * (x * rs) * silu(g)) (norms.metal:1143-1151).
template <class ActT>
__device__ __forceinline__ uint16_t rms_norm_gated_value(uint16_t x, uint16_t gate, uint16_t w, float rs, bool precise) {
#pragma clang fp contract(off)
    const float g = ActT::widen(gate);
    if (precise) {
        const float normalized = ActT::widen(ActT::narrow(ActT::widen(w) * ActT::widen(ActT::narrow(ActT::widen(x) * rs))));
        const float tail = 1.0f / (1.0f + expf(fabsf(g)));
        const float sigmoid = g < 0.0f ? tail : 1.0f - tail;
        return ActT::narrow(normalized * (g * sigmoid));
    }
    const float silu = g / (1.0f + expf(-g));
    const float scaled = ActT::widen(x) * rs;
    return ActT::narrow((ActT::widen(w) * scaled) * silu);
}

template <class ActT>
__device__ __forceinline__ void rms_norm_gated_head(const uint16_t* x, const uint16_t* gate, const uint16_t* w, uint16_t* y,
                                                    uint32_t head_dim, float eps, bool precise, uint32_t heads_per_token);

// sum over the workgroup for any workgroup of 32 threads or whole waves
__device__ __forceinline__ float block_sum_any(float v, float* wave_sums) {
    const uint32_t width = blockDim.x < 64u ? blockDim.x : 64u;
    for (uint32_t off = width / 2; off > 0; off >>= 1) v += __shfl_xor(v, (int)off);
    const uint32_t waves = (blockDim.x + 63u) / 64u;
    if (threadIdx.x % 64u == 0) wave_sums[threadIdx.x / 64u] = v;
    __syncthreads();
    float total = 0.0f;
    for (uint32_t w = 0; w < waves; ++w) total += wave_sums[w];
    __syncthreads();
    return total;
}

// one workgroup per head; grid.y = token (heads_per_token heads each)
template <class ActT>
__device__ __forceinline__ void rms_norm_gated_head(const uint16_t* x, const uint16_t* gate, const uint16_t* w, uint16_t* y,
                                                    uint32_t head_dim, float eps, bool precise, uint32_t heads_per_token) {
    __shared__ float wave_sums[16];
    const size_t at = ((size_t)blockIdx.y * heads_per_token + blockIdx.x) * head_dim;
    float sum = 0.0f;
    for (uint32_t i = threadIdx.x; i < head_dim; i += blockDim.x) {
        const float v = ActT::widen(x[at + i]);
        sum = __builtin_fmaf(v, v, sum);
    }
    const float rs = 1.0f / __builtin_sqrtf(block_sum_any(sum, wave_sums) / (float)head_dim + eps);
    for (uint32_t i = threadIdx.x; i < head_dim; i += blockDim.x)
        y[at + i] = rms_norm_gated_value<ActT>(x[at + i], gate[at + i], w[i], rs, precise);
}

template <class ActT, int SRC>
__device__ __forceinline__ void activation_bitplanes_body(const float* norm_scale, const uint16_t* a, const uint16_t* b,
                                                          uint32_t* planes, uint16_t* scales, uint32_t cols,
                                                          uint32_t nplanes) {
    const uint32_t groups = cols / 128;
    const uint32_t width = blockDim.x < 64u ? blockDim.x : 64u;      // 32 or 64 live lanes per wave
    const uint32_t lane = threadIdx.x % 64u;
    const uint32_t waves = (blockDim.x + 63u) / 64u;
    const uint32_t batch = blockIdx.y;
    a += (size_t)batch * cols;
    if (SRC == kPlaneSrcSwiglu || SRC == kPlaneSrcSigmoidMul) b += (size_t)batch * cols;           // the norm weight is shared by every token
    planes += (size_t)batch * groups * nplanes * 4;
    scales += (size_t)batch * groups;
    const uint32_t per_lane = 128u / width;
    for (uint32_t g = blockIdx.x * waves + threadIdx.x / 64u; g < groups; g += gridDim.x * waves) {
        float v[4];
        for (uint32_t k = 0; k < per_lane; ++k)
            v[k] = bitplane_value<ActT, SRC>(norm_scale, a, b, (size_t)g * 128 + k * width + lane);
        bitplane_store_group<ActT>(v, per_lane, width, lane, nplanes, planes + (size_t)g * nplanes * 4, scales + g);
    }
}

}  // namespace smelt

#define SMELT_PLANE_KERNEL extern "C" __global__ __launch_bounds__(1024)

// rms_norm_gated[_d128][_batched] and the fused gated-norm -> i6 view producer
// (signed_quant.metal:1029-1173): one workgroup per head of `head_dim` values; `precise` selects the
// d128 arithmetic, which the producer uses exactly when the reference does (32 threads, head_dim 128).
#define SMELT_GATED_NORM_KERNELS(T, ACT)                                                           \
    SMELT_PLANE_KERNEL void smelt_rms_norm_gated_##T(                                              \
        const uint16_t* x, const uint16_t* gate, const uint16_t* w, uint16_t* y, uint32_t head_dim, \
        float eps, uint32_t precise) {                                                             \
        smelt::rms_norm_gated_head<ACT>(x, gate, w, y, head_dim, eps, precise != 0, gridDim.x);    \
    }                                                                                              \
    SMELT_PLANE_KERNEL void smelt_rms_norm_gated_batched_##T(                                      \
        const uint16_t* x, const uint16_t* gate, const uint16_t* w, uint16_t* y,                   \
        uint32_t heads_per_token, uint32_t head_dim, float eps, uint32_t precise) {                \
        smelt::rms_norm_gated_head<ACT>(x, gate, w, y, head_dim, eps, precise != 0, heads_per_token); \
    }                                                                                              \
    SMELT_PLANE_KERNEL void smelt_rms_norm_gated_signed_activation_bitplanes_##T(                  \
        const uint16_t* x, const uint16_t* gate, const uint16_t* w, uint32_t* planes,              \
        uint16_t* scales, uint32_t head_dim, float eps) {                                          \
        __shared__ float wave_sums[16];                                                            \
        __shared__ uint16_t normalized[128];                                                       \
        const uint32_t g = blockIdx.x;                                                             \
        const size_t at = (size_t)g * head_dim;                                                    \
        const bool precise = blockDim.x == 32u && head_dim == 128u;                                \
        float sum = 0.0f;                                                                          \
        for (uint32_t i = threadIdx.x; i < head_dim; i += blockDim.x) {                            \
            const float v = ACT::widen(x[at + i]);                                                 \
            sum = __builtin_fmaf(v, v, sum);                                                       \
        }                                                                                          \
        const float rs = 1.0f / __builtin_sqrtf(smelt::block_sum_any(sum, wave_sums) / (float)head_dim + eps); \
        for (uint32_t i = threadIdx.x; i < head_dim; i += blockDim.x)                              \
            normalized[i] = smelt::rms_norm_gated_value<ACT>(x[at + i], gate[at + i], w[i], rs, precise); \
        __syncthreads();                                                                           \
        const uint32_t width = blockDim.x < 64u ? blockDim.x : 64u;                                \
        if (threadIdx.x >= width) return;                                                          \
        const uint32_t per_lane = 128u / width;                                                    \
        float v[4];                                                                                \
        for (uint32_t k = 0; k < per_lane; ++k) v[k] = ACT::widen(normalized[k * width + threadIdx.x]); \
        smelt::bitplane_store_group<ACT>(v, per_lane, width, threadIdx.x, 6u, planes + (size_t)g * 24, scales + g); \
    }

#define SMELT_ACTIVATION_BITPLANE_KERNELS(T, ACT)                                                  \
    SMELT_PLANE_KERNEL void smelt_signed_activation_bitplanes_##T(                                 \
        const uint16_t* x, uint32_t* planes, uint16_t* scales, uint32_t cols, uint32_t nplanes) {  \
        smelt::activation_bitplanes_body<ACT, smelt::kPlaneSrcPlain>(nullptr, x, nullptr, planes,  \
                                                                     scales, cols, nplanes);       \
    }                                                                                              \
    SMELT_PLANE_KERNEL void smelt_swiglu_signed_activation_bitplanes_##T(                          \
        const uint16_t* gate, const uint16_t* up, uint32_t* planes, uint16_t* scales,              \
        uint32_t cols, uint32_t nplanes) {                                                         \
        smelt::activation_bitplanes_body<ACT, smelt::kPlaneSrcSwiglu>(nullptr, gate, up, planes,   \
                                                                      scales, cols, nplanes);      \
    }                                                                                              \
    SMELT_PLANE_KERNEL void smelt_sigmoid_mul_signed_activation_bitplanes_##T(                     \
        const uint16_t* a, const uint16_t* b, uint32_t* planes, uint16_t* scales, uint32_t cols,   \
        uint32_t nplanes) {                                                                        \
        smelt::activation_bitplanes_body<ACT, smelt::kPlaneSrcSigmoidMul>(nullptr, a, b, planes,   \
                                                                          scales, cols, nplanes);  \
    }                                                                                              \
    SMELT_PLANE_KERNEL void smelt_norm_scale_signed_activation_bitplanes_##T(                      \
        const float* norm_scale, const uint16_t* x, const uint16_t* w, uint32_t* planes,           \
        uint16_t* scales, uint32_t cols, uint32_t nplanes) {                                       \
        smelt::activation_bitplanes_body<ACT, smelt::kPlaneSrcNormScale>(norm_scale, x, w, planes, \
                                                                         scales, cols, nplanes);   \
    }
