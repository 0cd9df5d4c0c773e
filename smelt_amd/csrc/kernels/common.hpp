// Shared device helpers for the gfx950 quantized matvec / qmm kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace smelt {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// Element types of activations / scales as stored in memory (raw 16-bit patterns).
struct F16 {
    static constexpr bool kIsF16 = true;
    static __device__ __forceinline__ float widen(uint16_t b) {
        return (float)__builtin_bit_cast(_Float16, b);
    }
    // Round-to-nearest-even narrowing of a value that has already been rounded to fp32, which is
    // what half(float) means in the reference.  The empty asm keeps the conversion apart from the
    // arithmetic that produced v: folded into a mixed-precision multiply-add (v_fma_mixlo_f16) the
    // exact product would be rounded once, and results on fp16 ties would differ by an ulp.
    static __device__ __forceinline__ uint16_t narrow(float v) {
        asm("" : "+v"(v));
        return __builtin_bit_cast(uint16_t, (_Float16)v);
    }
    // bits of the same value as fp16 (identity)
    static __device__ __forceinline__ uint16_t to_f16_bits(uint16_t b) { return b; }
};

struct BF16 {
    static constexpr bool kIsF16 = false;
    static __device__ __forceinline__ float widen(uint16_t b) {
        return __builtin_bit_cast(float, (uint32_t)b << 16);
    }
    static __device__ __forceinline__ uint16_t narrow(float v) {
        uint32_t bits = __builtin_bit_cast(uint32_t, v);
        uint32_t rounded = bits + 0x7FFFu + ((bits >> 16) & 1u);
        return (uint16_t)(rounded >> 16);
    }
    // bf16 -> fp16: exact for |v| in [2^-14, 65504]; smaller values round to the fp16
    // subnormal grid (absolute error <= 2^-25), larger ones saturate to +-65504.
    static __device__ __forceinline__ uint16_t to_f16_bits(uint16_t b) {
        float v = widen(b);
        v = __builtin_fminf(__builtin_fmaxf(v, -65504.0f), 65504.0f);
        return __builtin_bit_cast(uint16_t, (_Float16)v);
    }
};

// Prologue of the norm-scale kernels (lut_matvec.metal:1288-1292): with rs != nullptr the staged
// activation is narrow((x * rs[token]) * (1 + weight)), rounded to the 16-bit type exactly as a
// staged norm would store it; the launch's first workgroup also writes that row to `out`.
struct NormScale {
    const float* rs = nullptr;
    const uint16_t* weight = nullptr;
    uint16_t* out = nullptr;
    // norm_add_scale form (lut_matvec.metal:2896-2990): the rounded norm plus this row, added and
    // rounded in the 16-bit type, is what the kernel multiplies and stores
    const uint16_t* residual = nullptr;
    // self_eps >= 0: there is no precomputed scale; the workgroup forms 1 / sqrt(mean(x^2) + self_eps)
    // itself when it stages the row, and the launch's first workgroup publishes {scale, 1u} to `publish`
    float self_eps = -1.0f;
    float* publish = nullptr;
};




// (x * rs) * (1 + w) with each product and the sum rounded on its own: without the pragma the
// compiler folds t * (1 + w) into fma(w, t, t), one rounding fewer than the staged norm performs.
template <class ActT>
__device__ __forceinline__ uint16_t norm_scale_value(uint16_t x, float rs, uint16_t w) {
#pragma clang fp contract(off)
    const float scaled = ActT::widen(x) * rs;
    const float direct = 1.0f + ActT::widen(w);
    return ActT::narrow(scaled * direct);
}

// one element of the prologue: norm, then the optional residual add
template <class ActT>
__device__ __forceinline__ uint16_t norm_scale_element(const NormScale& ns, uint16_t x, float rs, size_t token_offset, int c) {
    uint16_t v = norm_scale_value<ActT>(x, rs, ns.weight[c]);
    if (ns.residual != nullptr) v = ActT::narrow(ActT::widen(v) + ActT::widen(ns.residual[token_offset + c]));
    return v;
}

__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }

// D = a.x*b.x + a.y*b.y + acc with fp32 accumulation (v_dot2c_f32_f16).
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(as_half2(a), as_half2(b), acc, false);
}

// ---- wave64 reductions with DPP (no LDS) ---------------------------------------------
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_add(float v) {
    int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, true);
    return v + __builtin_bit_cast(float, moved);
}

// Sum over aligned groups of LANES consecutive lanes; the total is valid in the LAST lane
// of each group (lane % LANES == LANES-1).
template <int LANES>
__device__ __forceinline__ float group_sum_last(float v) {
    static_assert(LANES == 64 || LANES == 32 || LANES == 16 || LANES == 8 || LANES == 4 ||
                  LANES == 2 || LANES == 1, "power of two");
    if (LANES >= 2) v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    if (LANES >= 4) v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    if (LANES >= 8) v = dpp_add<0x141>(v);  // row_half_mirror
    if (LANES >= 16) v = dpp_add<0x140>(v); // row_mirror
    if (LANES >= 32) v = dpp_add<0x142, 0xA>(v);  // row_bcast:15 into rows 1,3
    if (LANES >= 64) v = dpp_add<0x143, 0xC>(v);  // row_bcast:31 into rows 2,3
    return v;
}

// ---- argmax key (value in the high word, inverted index in the low word) ---------------
constexpr uint32_t kArgmaxIndexBits = 18;
constexpr uint32_t kArgmaxMaxIndex = (1u << kArgmaxIndexBits) - 1u;

__device__ __forceinline__ uint32_t ordered_key16(uint32_t bits) {
    if ((bits & 0x7FFFu) == 0u) bits = 0u;  // -0 == +0
    return (bits & 0x8000u) ? (0xFFFFu - bits) : (bits ^ 0x8000u);
}

__device__ __forceinline__ uint2_t argmax_pack_key(uint16_t value_bits, uint32_t index) {
    uint2_t k;
    k.x = ordered_key16(value_bits);
    k.y = (kArgmaxMaxIndex - index) & kArgmaxMaxIndex;
    return k;
}

__device__ __forceinline__ bool argmax_key_gt(uint2_t a, uint2_t b) {
    return a.x > b.x || (a.x == b.x && a.y > b.y);
}
__device__ __forceinline__ uint2_t argmax_key_max(uint2_t a, uint2_t b) {
    return argmax_key_gt(a, b) ? a : b;
}

__device__ __forceinline__ uint2_t wave_argmax_key(uint2_t k) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        uint2_t o;
        o.x = __shfl_xor(k.x, off);
        o.y = __shfl_xor(k.y, off);
        k = argmax_key_max(k, o);
    }
    return k;
}

__device__ __forceinline__ int ilog2(uint32_t v) { return 31 - __builtin_clz(v); }

// 1 / sqrt(mean(x^2) + eps) of one row, every thread of the workgroup returning the same value:
// threads stride over the row, waves reduce with DPP adds, wave totals meet in `wave_sums`.
template <class ActT>
__device__ __forceinline__ float row_inv_rms(const uint16_t* x, uint32_t cols, float eps, float* wave_sums) {
    float sum = 0.0f;
    for (uint32_t i = threadIdx.x; i < cols; i += blockDim.x) {
        const float v = ActT::widen(x[i]);
        sum = __builtin_fmaf(v, v, sum);
    }
    sum = group_sum_last<64>(sum);
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    if (lane == kWave - 1) wave_sums[wave] = sum;
    __syncthreads();
    float total = 0.0f;
    for (int w = 0; w < (int)(blockDim.x / kWave); ++w) total += wave_sums[w];
    return 1.0f / __builtin_sqrtf(total / (float)cols + eps);
}

}  // namespace smelt
