// The small decode ops that sit between the matvecs of a layer: RMS norms with the (1 + weight)
// convention, the staged SwiGLU and the elementwise add / multiply / copy
// (Resources/Shaders/norms.metal, activations_precise.metal, activations.metal).
// 16-bit values are fp16 or bf16 (template parameter); sums of squares are fp32.
#pragma once
#include "common.hpp"

namespace smelt {

// fp32 sum over the workgroup; every thread returns the total.  `scratch` holds one float per wave.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = group_sum_last<64>(v);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    const int waves = (blockDim.x + kWave - 1) / kWave;
    __syncthreads();
    if (lane == kWave - 1) scratch[wave] = v;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < waves; ++w) total += scratch[w];
    return total;
}

// One workgroup per row: the row is read once with 16-byte loads into LDS (two-byte loads for a
// ragged tail), squared and summed, and the second pass works from LDS.
template <class ActT>
__device__ __forceinline__ float stage_row_sum_squares(const uint16_t* x, uint32_t dim, uint16_t* row, float* scratch) {
    float sum = 0.0f;
    const bool vec = (dim & 7u) == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    if (vec) {
        for (uint32_t i = threadIdx.x; i < dim / 8; i += blockDim.x) {
            const uint4_t v = reinterpret_cast<const uint4_t*>(x)[i];
            reinterpret_cast<uint4_t*>(row)[i] = v;
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float a = ActT::widen((uint16_t)(w[k] & 0xFFFFu)), b = ActT::widen((uint16_t)(w[k] >> 16));
                sum = __builtin_fmaf(a, a, sum);
                sum = __builtin_fmaf(b, b, sum);
            }
        }
    } else {
        for (uint32_t i = threadIdx.x; i < dim; i += blockDim.x) {
            const uint16_t b = x[i];
            row[i] = b;
            const float a = ActT::widen(b);
            sum = __builtin_fmaf(a, a, sum);
        }
    }
    return block_sum(sum, scratch);
}

__device__ __forceinline__ float inv_rms(float sum_squares, uint32_t dim, float eps) {
    return 1.0f / __builtin_sqrtf(sum_squares / (float)dim + eps);
}

// mode 1 (two-step): half(1 + w) * half(x * rs), both factors materialised in the 16-bit type first (the
// generic rms_norm_1pw, norms.metal:54-62); mode 0: half(x * (rs * (1 + w))) (the vectorised
// fixed-dimension kernels, norms.metal:164-170); mode 2: half((x * rs) * (1 + w)), products left to
// right (the d256 kernels, norms.metal:213, 256).  residual != nullptr adds it to the rounded norm
// in the 16-bit type; scalar != nullptr then multiplies the rounded sum by scalar[0] (norms.metal:257-259).
enum NormMode : uint32_t { kNormScaleFirst = 0, kNormTwoStep = 1, kNormLeftToRight = 2 };

template <class ActT>
__device__ __forceinline__ void rms_norm_1pw_row(const uint16_t* x, const uint16_t* weight, const uint16_t* residual,
                                                 uint16_t* out, uint32_t dim, float eps, uint32_t mode,
                                                 const uint16_t* scalar = nullptr) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float* scratch = reinterpret_cast<float*>(smem);
    uint16_t* row = reinterpret_cast<uint16_t*>(smem + 64);
    const float rs = inv_rms(stage_row_sum_squares<ActT>(x, dim, row, scratch), dim, eps);
    for (uint32_t i = threadIdx.x; i < dim; i += blockDim.x) {
        const float v = ActT::widen(row[i]);
        const float w = ActT::widen(weight[i]);
        uint16_t y;
        if (mode == kNormTwoStep) {
            const float normalized = ActT::widen(ActT::narrow(v * rs));
            const float direct = ActT::widen(ActT::narrow(1.0f + w));
            y = ActT::narrow(direct * normalized);
        } else if (mode == kNormLeftToRight) {
            y = norm_scale_value<ActT>(row[i], rs, weight[i]);
        } else {
            y = ActT::narrow(v * (rs * (1.0f + w)));
        }
        if (residual) y = ActT::narrow(ActT::widen(y) + ActT::widen(residual[i]));
        if (scalar) y = ActT::narrow(ActT::widen(y) * ActT::widen(scalar[0]));
        out[i] = y;
    }
}

// rms_norm_1pw_from_fp32 (norms_fp32.metal:50-88): fp32 row in, 16-bit row out, the product clamped
// to the fp16 range before it is narrowed.
template <class ActT>
__device__ __forceinline__ void rms_norm_from_fp32_row(const float* x, const uint16_t* weight, uint16_t* out,
                                                       uint32_t dim, float eps) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float* scratch = reinterpret_cast<float*>(smem);
    float sum = 0.0f;
    for (uint32_t i = threadIdx.x; i < dim; i += blockDim.x) sum = __builtin_fmaf(x[i], x[i], sum);
    const float rs = inv_rms(block_sum(sum, scratch), dim, eps);
    for (uint32_t i = threadIdx.x; i < dim; i += blockDim.x) {
        float v;
        {
#pragma clang fp contract(off)
            const float scaled = x[i] * rs;
            v = scaled * (1.0f + ActT::widen(weight[i]));
        }
        out[i] = ActT::narrow(__builtin_fminf(__builtin_fmaxf(v, -65504.0f), 65504.0f));
    }
}

}  // namespace smelt

#define SMELT_LAYER_KERNEL extern "C" __global__ __launch_bounds__(1024)

// grid.x = row (token) index; `batch` guards launches whose grid is wider than the live rows
#define SMELT_LAYER_KERNELS(T, ACT)                                                               \
    SMELT_LAYER_KERNEL void smelt_rms_norm_1pw_##T(const uint16_t* x, const uint16_t* w,          \
                                                   uint16_t* y, uint32_t dim, float eps,          \
                                                   uint32_t two_step) {                           \
        const size_t at = (size_t)blockIdx.x * dim;                                               \
        smelt::rms_norm_1pw_row<ACT>(x + at, w, nullptr, y + at, dim, eps, two_step);        \
    }                                                                                             \
    SMELT_LAYER_KERNEL void smelt_rms_norm_1pw_add_##T(const uint16_t* x, const uint16_t* w,      \
                                                       const uint16_t* res, uint16_t* y,          \
                                                       uint32_t dim, float eps,                   \
                                                       uint32_t two_step) {                       \
        const size_t at = (size_t)blockIdx.x * dim;                                               \
        smelt::rms_norm_1pw_row<ACT>(x + at, w, res + at, y + at, dim, eps, two_step);       \
    }                                                                                             \
    SMELT_LAYER_KERNEL void smelt_rms_norm_1pw_add_scalar_##T(                                    \
        const uint16_t* x, const uint16_t* w, const uint16_t* res, const uint16_t* scalar,        \
        uint16_t* y, uint32_t dim, float eps, uint32_t mode) {                                    \
        const size_t at = (size_t)blockIdx.x * dim;                                               \
        smelt::rms_norm_1pw_row<ACT>(x + at, w, res + at, y + at, dim, eps, mode, scalar);        \
    }                                                                                             \
    SMELT_LAYER_KERNEL void smelt_rms_norm_1pw_from_fp32_##T(const float* x, const uint16_t* w,   \
                                                             uint16_t* y, uint32_t dim, float eps) { \
        const size_t at = (size_t)blockIdx.x * dim;                                               \
        smelt::rms_norm_from_fp32_row<ACT>(x + at, w, y + at, dim, eps);                          \
    }                                                                                             \
    SMELT_LAYER_KERNEL void smelt_rms_norm_scale_only_##T(const uint16_t* x, float* scale,        \
                                                          uint32_t dim, float eps) {              \
        extern __shared__ __attribute__((aligned(16))) unsigned char smem[];                      \
        const float ss = smelt::stage_row_sum_squares<ACT>(                                       \
            x + (size_t)blockIdx.x * dim, dim, reinterpret_cast<uint16_t*>(smem + 64),            \
            reinterpret_cast<float*>(smem));                                                      \
        if (threadIdx.x == 0) scale[blockIdx.x] = smelt::inv_rms(ss, dim, eps);                   \
    }                                                                                             \
    /* out = a + b in the 16-bit type, then the scale of the updated row (norms.metal:1059-1091) */ \
    SMELT_LAYER_KERNEL void smelt_residual_add_rms_norm_scale_only_##T(                           \
        const uint16_t* a, const uint16_t* b, uint16_t* out, float* scale, uint32_t dim,          \
        float eps) {                                                                              \
        extern __shared__ __attribute__((aligned(16))) unsigned char smem[];                      \
        float sum = 0.0f;                                                                         \
        const size_t at = (size_t)blockIdx.x * dim;                                               \
        for (uint32_t i = threadIdx.x; i < dim; i += blockDim.x) {                                \
            const uint16_t v = ACT::narrow(ACT::widen(a[at + i]) + ACT::widen(b[at + i]));        \
            out[at + i] = v;                                                                      \
            const float f = ACT::widen(v);                                                        \
            sum = __builtin_fmaf(f, f, sum);                                                      \
        }                                                                                         \
        const float ss = smelt::block_sum(sum, reinterpret_cast<float*>(smem));                   \
        if (threadIdx.x == 0) scale[blockIdx.x] = smelt::inv_rms(ss, dim, eps);                   \
    }                                                                                             \
    /* silu(gate) * up with every intermediate in the 16-bit type (activations_precise.metal:9-22) */ \
    SMELT_LAYER_KERNEL void smelt_swiglu_fused_##T(const uint16_t* gate, const uint16_t* up,      \
                                                   uint16_t* out, uint32_t count) {               \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i >= count) return;                                                                   \
        auto rt = [](float v) { return ACT::widen(ACT::narrow(v)); };                             \
        const float g = ACT::widen(gate[i]), u = ACT::widen(up[i]);                               \
        const float e = rt(expf(fabsf(g)));                                                       \
        const float tail = rt(1.0f / rt(1.0f + e));                                               \
        const float sig = g < 0.0f ? tail : rt(1.0f - tail);                                      \
        out[i] = ACT::narrow(rt(g * sig) * u);                                                    \
    }                                                                                             \
    /* pointwise activations of activations.metal:5-40, 98-177 and activations_precise.metal:26-38;     \
       op: 0 silu, 1 sigmoid, 2 softplus, 3 x * param, 4 param * tanh(x / param) */                  \
    SMELT_LAYER_KERNEL void smelt_unary_##T(const uint16_t* in, uint16_t* out, uint32_t count,    \
                                            float param, uint32_t op) {                           \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i >= count) return;                                                                   \
        const float x = ACT::widen(in[i]);                                                        \
        float v;                                                                                  \
        switch (op) {                                                                             \
            case 0: v = x / (1.0f + expf(-x)); break;                                             \
            case 1: v = 1.0f / (1.0f + expf(-x)); break;                                          \
            case 2: v = x > 20.0f ? x : logf(1.0f + expf(x)); break;                              \
            case 3: v = x * param; break;                                                         \
            default: v = param * tanhf(x / param); break;                                         \
        }                                                                                         \
        out[i] = ACT::narrow(v);                                                                  \
    }                                                                                             \
    SMELT_LAYER_KERNEL void smelt_scalar_mul_param_first_##T(const uint16_t* in, uint16_t* out,   \
                                                             float scalar, uint32_t count) {      \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i < count) out[i] = ACT::narrow(ACT::widen(in[i]) * scalar);                          \
    }                                                                                             \
    SMELT_LAYER_KERNEL void smelt_scalar_mul_weight_##T(const uint16_t* in, const uint16_t* s,    \
                                                        uint16_t* out, uint32_t count) {          \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i < count) out[i] = ACT::narrow(ACT::widen(in[i]) * ACT::widen(s[0]));                \
    }                                                                                             \
    /* attention * sigmoid(gate), the sigmoid staged in the 16-bit type (activations_precise.metal:26-38) */ \
    SMELT_LAYER_KERNEL void smelt_sigmoid_mul_##T(const uint16_t* a, const uint16_t* gate,        \
                                                  uint16_t* out, uint32_t count) {                \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i >= count) return;                                                                   \
        auto rt = [](float v) { return ACT::widen(ACT::narrow(v)); };                             \
        const float g = ACT::widen(gate[i]);                                                      \
        const float tail = rt(1.0f / rt(1.0f + rt(expf(fabsf(g)))));                              \
        const float sig = g < 0.0f ? tail : rt(1.0f - tail);                                      \
        out[i] = ACT::narrow(ACT::widen(a[i]) * sig);                                             \
    }                                                                                             \
    /* gelu(gate) * up, tanh form, clamped (activations.metal:124-140) */                         \
    SMELT_LAYER_KERNEL void smelt_geglu_fused_##T(const uint16_t* gate, const uint16_t* up,       \
                                                  uint16_t* out, uint32_t count) {                \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i >= count) return;                                                                   \
        const float g = ACT::widen(gate[i]), u = ACT::widen(up[i]);                               \
        float inner = 0.7978845608f * (g + 0.044715f * (g * g * g));                              \
        inner = fminf(fmaxf(inner, -20.0f), 20.0f);                                               \
        const float gelu = 0.5f * g * (1.0f + tanhf(inner));                                      \
        out[i] = ACT::narrow(fminf(fmaxf(gelu * u, -65504.0f), 65504.0f));                        \
    }                                                                                             \
    /* the same over [batch, count] with the up operand at its own row stride; grid.y = token       \
       (activations.metal:142-163) */                                                             \
    SMELT_LAYER_KERNEL void smelt_geglu_fused_strided_batched_##T(                                \
        const uint16_t* gate, const uint16_t* up, uint16_t* out, uint32_t count,                  \
        uint32_t up_stride) {                                                                     \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i >= count) return;                                                                   \
        const size_t at = (size_t)blockIdx.y * count + i;                                         \
        const float g = ACT::widen(gate[at]), u = ACT::widen(up[(size_t)blockIdx.y * up_stride + i]); \
        float inner = 0.7978845608f * (g + 0.044715f * (g * g * g));                              \
        inner = fminf(fmaxf(inner, -20.0f), 20.0f);                                               \
        const float gelu = 0.5f * g * (1.0f + tanhf(inner));                                      \
        out[at] = ACT::narrow(fminf(fmaxf(gelu * u, -65504.0f), 65504.0f));                       \
    }                                                                                             \
    /* out[token, row] = in[token, row] + bias[row]; grid.y = token (activations.metal:69-82) */  \
    SMELT_LAYER_KERNEL void smelt_projection_bias_add_batched_##T(                                \
        const uint16_t* in, const uint16_t* bias, uint16_t* out, uint32_t rows) {                 \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i >= rows) return;                                                                    \
        const size_t at = (size_t)blockIdx.y * rows + i;                                          \
        out[at] = ACT::narrow(ACT::widen(in[at]) + ACT::widen(bias[i]));                          \
    }                                                                                             \
    SMELT_LAYER_KERNEL void smelt_elementwise_add_##T(const uint16_t* a, const uint16_t* b,       \
                                                      uint16_t* out, uint32_t count) {            \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i < count) out[i] = ACT::narrow(ACT::widen(a[i]) + ACT::widen(b[i]));                 \
    }                                                                                             \
    SMELT_LAYER_KERNEL void smelt_elementwise_mul_##T(const uint16_t* a, const uint16_t* b,       \
                                                      uint16_t* out, uint32_t count) {            \
        const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;                                 \
        if (i < count) out[i] = ACT::narrow(ACT::widen(a[i]) * ACT::widen(b[i]));                 \
    }

extern "C" __global__ __launch_bounds__(1024) void smelt_buffer_copy16(const uint16_t* src, uint16_t* dst, uint32_t count) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) dst[i] = src[i];
}
