/*
 * smelt_oracle.c — CPU restatement of Smelt's quantized-weight numerics.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the HIP kernels are
 * compared against; nothing that ships (the C-ABI runtime, the kernels, the
 * record emitters) links, loads or calls it.  Only tests/, the smoke check and
 * the benchmark's cpu_baseline leg may use it.
 *
 * Every function cites the reference file:line it restates (paths relative to
 * the Smelt repository root).  Scalar C, no dependencies, one translation unit.
 *
 * Pin status (what fixes each function independently of this file):
 *   - f16/bf16 conversions ........ exhaustive vs numpy float16 / closed form
 *   - affine_u4 pack + dequant .... SmeltAffineU4Tests.swift:67-80,120-128
 *   - binary1/ternary2 codec ...... SmeltSignedQuantCodecTests.swift:16-107
 *   - MLX scale normalisation ..... SmeltSignedQuantCodecTests.swift:109-204
 *   - ternary affine QMV .......... MLX golden bits, SignedQuantKernelTests.swift:87-199
 *   - ternary affine QMM .......... MLX golden bits, SignedQuantKernelTests.swift:527-601, and
 *                                   an independent numpy float16 evaluation of the weight tile
 *   - affine / signed matvec ...... exact-rational recomputation on dyadic fixtures,
 *                                   brute-force dequant-then-dot cross-check
 *   - argmax key .................. special cases (ties, signed zero) + brute force
 *   - trit5 codec ................. PARITY UNPINNED BY THE REFERENCE: the format does
 *                                   not exist there; pinned by closed form, exhaustive
 *                                   243-entry check and agreement with ternary2
 *   - signed SwiGLU epilogue ...... PARITY UNPINNED: Metal's half-precision exp() is not
 *                                   specified bit-exactly; restated with fp32 expf rounded
 *                                   to fp16 at each materialisation point
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define SO_EXPORT __attribute__((visibility("default")))

/* error codes mirror SmeltSignedQuantError (SmeltSignedQuantCodec.swift:38-68) */
enum {
    SO_OK = 0,
    SO_ERR_GEOMETRY = -1,
    SO_ERR_BUFFER_TOO_SMALL = -2,
    SO_ERR_INVALID_CODE = -3,
    SO_ERR_MLX_SCALE = -4,
    SO_ERR_MLX_BIAS = -5,
};

/* element types for activations / scales */
enum { SO_F16 = 0, SO_BF16 = 1, SO_F32 = 2 };
/* signed formats: binary1 / ternary2 follow SmeltSignedQuantFormat; trit5 is new */
enum { SO_BINARY1 = 0, SO_TERNARY2 = 1, SO_TRIT5 = 2 };

/* ------------------------------------------------------------------------- */
/* IEEE conversions. Swift Float16(x) is round-to-nearest-even narrowing and   */
/* Float(Float16) is exact widening.                                           */
/* ------------------------------------------------------------------------- */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

SO_EXPORT float so_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return (sign ? -v : v);
    }
    if (exp == 31) return bits_f32(sign | 0x7F800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

SO_EXPORT uint16_t so_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) { /* inf / nan */
        if (absx > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((absx >> 13) & 0x3FFu));
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* rounds to inf: >= 65520 */
    if (absx < 0x33000001u) return sign;                          /* <= 2^-25 rounds to zero */
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    uint32_t shift;
    uint32_t base;
    if (e < -14) { /* subnormal result: units of 2^-24 */
        shift = (uint32_t)(13 + (-14 - e));
        base = 0;
    } else {
        shift = 13;
        base = ((uint32_t)(e + 15) << 10) - 0x400u; /* hidden bit adds 0x400 back */
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q += 1;
    return (uint16_t)(sign | (base + q));
}

/* SmeltBF16.swift:6-15 */
SO_EXPORT uint16_t so_f32_to_bf16(float f) {
    uint32_t bits = f32_bits(f);
    uint32_t rounded = bits + 0x7FFFu + ((bits >> 16) & 1u);
    return (uint16_t)(rounded >> 16);
}
SO_EXPORT float so_bf16_to_f32(uint16_t v) { return bits_f32((uint32_t)v << 16); }

static inline float widen(uint16_t bits, int dtype) {
    return dtype == SO_BF16 ? so_bf16_to_f32(bits) : so_f16_to_f32(bits);
}
static inline uint16_t narrow(float v, int dtype) {
    return dtype == SO_BF16 ? so_f32_to_bf16(v) : so_f32_to_f16(v);
}
SO_EXPORT float so_round_through(float v, int dtype) {
    if (dtype == SO_F32) return v;
    return widen(narrow(v, dtype), dtype);
}

/* ------------------------------------------------------------------------- */
/* affine_u4 — SmeltAffineU4.swift                                             */
/* ------------------------------------------------------------------------- */

/* SmeltAffineU4.swift:17-19 */
SO_EXPORT int so_affine_num_groups(int cols, int group) { return (cols + group - 1) / group; }
/* SmeltAffineU4.swift:22-23 */
SO_EXPORT int so_affine_packed_row_stride(int cols) { return (cols + 1) / 2; }

/* SmeltAffineU4.swift:30-34 — scale = (hi-lo)/15, bias = lo, degenerate range -> scale 1 */
SO_EXPORT void so_affine_params(float lo, float hi, int dtype, float *scale, float *bias,
                                uint16_t *scale_bits, uint16_t *bias_bits) {
    float range = hi - lo;
    float s = range < 1e-12f ? 1.0f : range / 15.0f;
    *scale = s;
    *bias = lo;
    *scale_bits = narrow(s, dtype);
    *bias_bits = narrow(lo, dtype);
}

/* SmeltAffineU4.swift:59-91 — endpoint choice; clip 0 = minMax, 1 = mseOptimal */
static void clip_endpoints(const float *values, int c0, int c1, float minv, float maxv, int clip,
                           const float *importance, int dtype, float *lo_out, float *hi_out) {
    if (clip == 0) { *lo_out = minv; *hi_out = maxv; return; }
    float half = (maxv - minv) / 2;
    if (half < 1e-12f) { *lo_out = minv; *hi_out = maxv; return; }
    float best_lo = minv, best_hi = maxv, best_err = INFINITY;
    for (int step = 0; step <= 8; ++step) {
        float c = 1.0f - (float)step * 0.075f;
        float lo = minv + (1 - c) * half, hi = maxv - (1 - c) * half;
        float scale = (hi - lo) / 15.0f;
        float scale_f = so_round_through(scale, dtype), lo_f = so_round_through(lo, dtype);
        float inv = 1.0f / scale;
        float err = 0;
        for (int k = c0; k < c1; ++k) {
            float v = values[k];
            float nib = fminf(fmaxf(roundf((v - lo) * inv), 0.0f), 15.0f);
            float d = v - (nib * scale_f + lo_f);
            err += (importance ? importance[k] : 1.0f) * d * d;
        }
        if (err < best_err) { best_err = err; best_lo = lo; best_hi = hi; }
    }
    *lo_out = best_lo; *hi_out = best_hi;
}

/* SmeltAffineU4.swift:94-136. Swift's .rounded() is round-half-away-from-zero = roundf. */
SO_EXPORT void so_affine_quantize_row(const float *values, int cols, int group, int clip,
                                      const float *importance, int dtype, uint8_t *packed,
                                      uint16_t *scales, uint16_t *biases) {
    int groups = so_affine_num_groups(cols, group);
    for (int g = 0; g < groups; ++g) {
        int c0 = g * group;
        int c1 = c0 + group < cols ? c0 + group : cols;
        float minv = INFINITY, maxv = -INFINITY;
        for (int c = c0; c < c1; ++c) {
            float v = values[c];
            if (v < minv) minv = v;
            if (v > maxv) maxv = v;
        }
        float lo, hi, scale, bias;
        clip_endpoints(values, c0, c1, minv, maxv, clip, importance, dtype, &lo, &hi);
        so_affine_params(lo, hi, dtype, &scale, &bias, &scales[g], &biases[g]);
        float inv = 1.0f / scale;
        for (int c = c0; c < c1; ++c) {
            float normalized = (values[c] - bias) * inv;
            float clamped = fminf(fmaxf(normalized, 0.0f), 15.0f);
            uint8_t nib = (uint8_t)roundf(clamped);
            int bi = c >> 1;
            if ((c & 1) == 0) packed[bi] = nib;
            else packed[bi] |= (uint8_t)(nib << 4);
        }
    }
}

/* SmeltAffineU4.swift:141-161: out[c] = Float(nibble) * scale + bias (one mul, one add). */
SO_EXPORT void so_affine_dequantize_row(const uint8_t *packed, const uint16_t *scales,
                                        const uint16_t *biases, int cols, int group, int dtype,
                                        float *out) {
    int groups = so_affine_num_groups(cols, group);
    for (int g = 0; g < groups; ++g) {
        int c0 = g * group;
        int c1 = c0 + group < cols ? c0 + group : cols;
        float scale = widen(scales[g], dtype);
        float bias = widen(biases[g], dtype);
        for (int c = c0; c < c1; ++c) {
            uint8_t byte = packed[c >> 1];
            uint8_t nib = (c & 1) == 0 ? (byte & 0x0F) : (byte >> 4);
            volatile float prod = (float)nib * scale; /* forbid fma contraction */
            out[c] = prod + bias;
        }
    }
}

/* SmeltRuntime.swift:2522-2595 — embedding-row form: Float16(Float(nib)*scale+bias) */
SO_EXPORT void so_affine_dequantize_row_narrow(const uint8_t *packed, const uint16_t *scales,
                                               const uint16_t *biases, int cols, int group,
                                               int dtype, int out_dtype, uint16_t *out) {
    int groups = so_affine_num_groups(cols, group);
    int stride = so_affine_packed_row_stride(cols);
    int bytes_per_group = group / 2;
    for (int g = 0; g < groups; ++g) {
        float scale = widen(scales[g], dtype);
        float bias = widen(biases[g], dtype);
        int c1 = (g + 1) * group < cols ? (g + 1) * group : cols;
        int b0 = g * bytes_per_group;
        int b1 = b0 + bytes_per_group < stride ? b0 + bytes_per_group : stride;
        for (int b = b0; b < b1; ++b) {
            uint8_t byte = packed[b];
            int col0 = b * 2;
            if (col0 < c1) {
                volatile float p = (float)(byte & 0x0F) * scale;
                out[col0] = narrow(p + bias, out_dtype);
            }
            if (col0 + 1 < c1) {
                volatile float p = (float)(byte >> 4) * scale;
                out[col0 + 1] = narrow(p + bias, out_dtype);
            }
        }
    }
}

/* MetalKernelTestSupport.swift:396-428 / PrefillKernelTests.swift:266-300.
 * Group-wise  acc += scale*dot + bias*xsum  in fp32, sequential order; result unrounded. */
SO_EXPORT void so_affine_matvec(const uint8_t *packed, const uint16_t *scales,
                                const uint16_t *biases, const float *x, int rows, int cols,
                                int group, int dtype, float *out) {
    int gpr = cols / group;
    int stride = cols / 2;
    for (int r = 0; r < rows; ++r) {
        const uint8_t *w = packed + (size_t)r * stride;
        float acc = 0;
        for (int g = 0; g < gpr; ++g) {
            float scale = widen(scales[(size_t)r * gpr + g], dtype);
            float bias = widen(biases[(size_t)r * gpr + g], dtype);
            int cb = g * group;
            float dot = 0, xsum = 0;
            for (int i = 0; i < group; ++i) {
                int col = cb + i;
                uint8_t byte = w[col / 2];
                uint8_t nib = (col & 1) == 0 ? (byte & 0x0F) : (byte >> 4);
                dot += (float)nib * x[col];
                xsum += x[col];
            }
            acc += scale * dot + bias * xsum;
        }
        out[r] = acc;
    }
}

/* Independent formulation used to cross-check so_affine_matvec: dequantise each
 * element (SmeltAffineU4.swift:141-161) and accumulate the dot product in double. */
SO_EXPORT void so_affine_matvec_dequant_f64(const uint8_t *packed, const uint16_t *scales,
                                            const uint16_t *biases, const float *x, int rows,
                                            int cols, int group, int dtype, double *out) {
    int gpr = so_affine_num_groups(cols, group);
    int stride = so_affine_packed_row_stride(cols);
    for (int r = 0; r < rows; ++r) {
        double acc = 0;
        for (int c = 0; c < cols; ++c) {
            uint8_t byte = packed[(size_t)r * stride + (c >> 1)];
            uint8_t nib = (c & 1) == 0 ? (byte & 0x0F) : (byte >> 4);
            float s = widen(scales[(size_t)r * gpr + c / group], dtype);
            float b = widen(biases[(size_t)r * gpr + c / group], dtype);
            volatile float p = (float)nib * s;
            float w = p + b;
            acc += (double)w * (double)x[c];
        }
        out[r] = acc;
    }
}

/* ------------------------------------------------------------------------- */
/* signed codec — SmeltSignedQuantCodec.swift                                  */
/* ------------------------------------------------------------------------- */

static inline int bits_per_code(int format) { return format == SO_BINARY1 ? 1 : 2; }

/* SmeltSignedQuantCodec.swift:72-84 (trit5: ceil(n/5) bytes) */
SO_EXPORT int64_t so_signed_packed_byte_count(int64_t logical_count, int format) {
    if (logical_count < 0) return SO_ERR_GEOMETRY;
    if (format == SO_TRIT5) return (logical_count + 4) / 5;
    return (logical_count * bits_per_code(format) + 7) / 8;
}

/* SmeltSignedQuantCodec.swift:88-98 */
SO_EXPORT int so_signed_groups_per_row(int padded_cols, int group) {
    if (padded_cols <= 0) return SO_ERR_GEOMETRY;
    if (group <= 0 || padded_cols % group != 0) return SO_ERR_GEOMETRY;
    return padded_cols / group;
}

/* SmeltSignedQuantCodec.swift:102-124 — LSB-first code extraction */
SO_EXPORT int so_signed_code_at(int64_t index, const uint8_t *bytes, int64_t byte_count,
                                int format) {
    if (index < 0) return SO_ERR_GEOMETRY;
    if (format == SO_TRIT5) {
        int64_t bi = index / 5;
        if (bi >= byte_count) return SO_ERR_BUFFER_TOO_SMALL;
        unsigned v = bytes[bi];
        if (v >= 243) return SO_ERR_INVALID_CODE;
        for (int i = (int)(index % 5); i > 0; --i) v /= 3;
        return (int)(v % 3);
    }
    int bpc = bits_per_code(format);
    int64_t bit = index * bpc;
    int64_t bi = bit >> 3;
    if (bi >= byte_count) return SO_ERR_BUFFER_TOO_SMALL;
    int shift = (int)(bit & 7);
    int mask = (1 << bpc) - 1;
    return (bytes[bi] >> shift) & mask;
}

/* SmeltSignedQuantCodec.swift:22-35 */
SO_EXPORT int so_signed_semantic(int format, int packed_code, int *out) {
    if (format == SO_BINARY1) {
        if (packed_code >= 2 || packed_code < 0) return SO_ERR_INVALID_CODE;
        *out = packed_code == 0 ? -1 : 1;
        return SO_OK;
    }
    if (packed_code >= 3 || packed_code < 0) return SO_ERR_INVALID_CODE;
    *out = packed_code - 1;
    return SO_OK;
}

/* SmeltSignedQuantCodec.swift:128-145; on failure *bad_index = first offending index */
SO_EXPORT int so_signed_validate_codes(const uint8_t *bytes, int64_t byte_count,
                                       int64_t logical_count, int format, int64_t *bad_index) {
    int64_t need = so_signed_packed_byte_count(logical_count, format);
    if (need < 0) return (int)need;
    if (byte_count < need) return SO_ERR_BUFFER_TOO_SMALL;
    if (format == SO_BINARY1) return SO_OK;
    for (int64_t i = 0; i < logical_count; ++i) {
        int v = so_signed_code_at(i, bytes, byte_count, format);
        if (v == 3 || v == SO_ERR_INVALID_CODE) {
            if (bad_index) *bad_index = i;
            return SO_ERR_INVALID_CODE;
        }
    }
    return SO_OK;
}

static int f16_is_finite(uint16_t h) { return ((h >> 10) & 0x1F) != 31; }
static float f16_ulp(uint16_t h) {
    /* Swift Float16.ulp: spacing at |h|; for zero/subnormal it is the least nonzero value */
    uint32_t exp = (h >> 10) & 0x1Fu;
    if (exp == 0) return 5.9604644775390625e-08f;
    return ldexpf(1.0f, (int)exp - 15 - 10);
}

/* SmeltSignedQuantCodec.swift:180-215 */
SO_EXPORT int so_signed_canonical_mlx_scale_bits(int format, uint16_t source_scale_bits,
                                                 uint16_t bias_bits, uint16_t *out) {
    float source = so_f16_to_f32(source_scale_bits);
    if (!f16_is_finite(source_scale_bits) || !(source >= 0)) return SO_ERR_MLX_SCALE;
    uint16_t canonical = format == SO_BINARY1 ? so_f32_to_f16(source * 0.5f) : source_scale_bits;
    float canonical_f = so_f16_to_f32(canonical);
    uint16_t expected_bias = so_f32_to_f16(-canonical_f);
    float actual = so_f16_to_f32(bias_bits);
    int equivalent = f16_is_finite(bias_bits) && actual <= 0 &&
                     fabsf(actual - so_f16_to_f32(expected_bias)) <= f16_ulp(canonical);
    if (!(bias_bits == expected_bias || equivalent)) return SO_ERR_MLX_BIAS;
    *out = canonical;
    return SO_OK;
}

/* SmeltSignedQuantCodec.swift:154-176; on failure *bad_group is the failing group */
SO_EXPORT int so_signed_normalize_mlx_scales(int format, const uint16_t *scales,
                                             const uint16_t *biases, int group_count,
                                             uint16_t *out, int *bad_group) {
    if (group_count < 0) return SO_ERR_GEOMETRY;
    for (int g = 0; g < group_count; ++g) {
        int rc = so_signed_canonical_mlx_scale_bits(format, scales[g], biases[g], &out[g]);
        if (rc != SO_OK) { if (bad_group) *bad_group = g; return rc; }
    }
    return SO_OK;
}

/* SmeltSignedQuantCodec.swift:219-257 (fp32 row) */
SO_EXPORT int so_signed_dequantize_row(int format, const uint8_t *codes, int64_t code_bytes,
                                       const uint16_t *scales, int64_t scale_bytes, int cols,
                                       int padded_cols, int group, float *out) {
    if (cols <= 0 || cols > padded_cols) return SO_ERR_GEOMETRY;
    int groups = so_signed_groups_per_row(padded_cols, group);
    if (groups < 0) return groups;
    int64_t need = so_signed_packed_byte_count(padded_cols, format);
    if (code_bytes < need) return SO_ERR_BUFFER_TOO_SMALL;
    if (scale_bytes < (int64_t)groups * 2) return SO_ERR_BUFFER_TOO_SMALL;
    int rc = so_signed_validate_codes(codes, code_bytes, padded_cols, format, NULL);
    if (rc != SO_OK) return rc;
    for (int col = 0; col < cols; ++col) {
        int packed = so_signed_code_at(col, codes, code_bytes, format);
        int sem;
        rc = so_signed_semantic(format, packed, &sem);
        if (rc != SO_OK) return rc;
        out[col] = (float)sem * so_f16_to_f32(scales[col / group]);
    }
    return SO_OK;
}

/* SmeltSignedQuantCodec.swift:262-324 (fp16 row) */
SO_EXPORT int so_signed_dequantize_row_f16(int format, const uint8_t *codes, int64_t code_bytes,
                                           const uint16_t *scales, int64_t scale_bytes, int cols,
                                           int padded_cols, int group, uint16_t *out) {
    if (cols <= 0 || cols > padded_cols) return SO_ERR_GEOMETRY;
    int groups = so_signed_groups_per_row(padded_cols, group);
    if (groups < 0) return groups;
    int64_t need = so_signed_packed_byte_count(padded_cols, format);
    if (code_bytes < need) return SO_ERR_BUFFER_TOO_SMALL;
    if (scale_bytes < (int64_t)groups * 2) return SO_ERR_BUFFER_TOO_SMALL;
    int rc = so_signed_validate_codes(codes, code_bytes, padded_cols, format, NULL);
    if (rc != SO_OK) return rc;
    for (int col = 0; col < cols; ++col) {
        int packed = so_signed_code_at(col, codes, code_bytes, format);
        int sem;
        rc = so_signed_semantic(format, packed, &sem);
        if (rc != SO_OK) return rc;
        out[col] = so_f32_to_f16((float)sem * so_f16_to_f32(scales[col / group]));
    }
    return SO_OK;
}

/* Test-fixture packer, SignedQuantKernelTests.swift:7-22 (LSB-first, row stride
 * cols*bits/8) and the trit5 closed form byte = sum d_i * 3^i (digit 0 = lowest
 * column; tail digits beyond cols encode 1, i.e. semantic zero). */
SO_EXPORT void so_signed_pack_row(int format, const uint8_t *codes, int cols, uint8_t *out,
                                  int64_t out_bytes) {
    memset(out, 0, (size_t)out_bytes);
    if (format == SO_TRIT5) {
        for (int64_t b = 0; b < out_bytes; ++b) {
            unsigned v = 0, p = 1;
            for (int i = 0; i < 5; ++i) {
                int64_t c = b * 5 + i;
                unsigned d = c < cols ? codes[c] : 1u;
                v += d * p;
                p *= 3;
            }
            out[b] = (uint8_t)v;
        }
        return;
    }
    int bpc = bits_per_code(format);
    for (int c = 0; c < cols; ++c) {
        int bit = c * bpc;
        out[bit / 8] |= (uint8_t)(codes[c] << (bit & 7));
    }
}

/* trit5 decode table: entry[byte] packs five 2-bit ternary2-style codes (digit i at
 * bits 2i..2i+1); bytes 243..255 are invalid and map to 0xFFFF. */
SO_EXPORT void so_trit5_build_lut(uint16_t *lut256) {
    for (unsigned b = 0; b < 256; ++b) {
        if (b >= 243) { lut256[b] = 0xFFFFu; continue; }
        unsigned v = b, e = 0;
        for (int i = 0; i < 5; ++i) { e |= (v % 3) << (2 * i); v /= 3; }
        lut256[b] = (uint16_t)e;
    }
}

/* SignedQuantKernelTests.swift:1030-1045: expected += x * semantic * scale, fp32, in
 * column order; result unrounded. x is [batch, cols] already widened to fp32. */
SO_EXPORT int so_signed_matvec(int format, const uint8_t *codes, int64_t row_stride,
                               const uint16_t *scales, const float *x, int rows, int cols,
                               int padded_cols, int group, int batch, float *out) {
    int groups = so_signed_groups_per_row(padded_cols, group);
    if (groups < 0) return groups;
    for (int b = 0; b < batch; ++b) {
        for (int r = 0; r < rows; ++r) {
            const uint8_t *row = codes + (size_t)r * row_stride;
            float expected = 0;
            for (int c = 0; c < cols; ++c) {
                int packed = so_signed_code_at(c, row, row_stride, format);
                int sem;
                int rc = so_signed_semantic(format, packed, &sem);
                if (rc != SO_OK) return rc;
                expected += x[(size_t)b * cols + c] * (float)sem *
                            so_f16_to_f32(scales[(size_t)r * groups + c / group]);
            }
            out[(size_t)b * rows + r] = expected;
        }
    }
    return SO_OK;
}

/* Cross-check formulation: per-group exact integer-weighted sums in double. */
SO_EXPORT int so_signed_matvec_f64(int format, const uint8_t *codes, int64_t row_stride,
                                   const uint16_t *scales, const float *x, int rows, int cols,
                                   int padded_cols, int group, int batch, double *out) {
    int groups = so_signed_groups_per_row(padded_cols, group);
    if (groups < 0) return groups;
    for (int b = 0; b < batch; ++b)
        for (int r = 0; r < rows; ++r) {
            const uint8_t *row = codes + (size_t)r * row_stride;
            double acc = 0;
            for (int g = 0; g < groups; ++g) {
                double part = 0;
                int c1 = (g + 1) * group < cols ? (g + 1) * group : cols;
                for (int c = g * group; c < c1; ++c) {
                    int packed = so_signed_code_at(c, row, row_stride, format);
                    int sem;
                    int rc = so_signed_semantic(format, packed, &sem);
                    if (rc != SO_OK) return rc;
                    part += (double)sem * (double)x[(size_t)b * cols + c];
                }
                acc += part * (double)so_f16_to_f32(scales[(size_t)r * groups + g]);
            }
            out[(size_t)b * rows + r] = acc;
        }
    return SO_OK;
}

/* ------------------------------------------------------------------------- */
/* Ternary "affine" QMV, the arithmetic of MLX affine_qmv_fast<half,128,2>     */
/* signed_quant_precise.metal:8-25 (qdot16) and :41-108 (kernel).              */
/* x is fp16 bits [batch, cols]; out fp16 bits [batch, rows].                  */
/* Lane l of a 32-wide simdgroup owns 16 columns of each 512-column block.     */
/* ------------------------------------------------------------------------- */

static inline float h2f(uint16_t h) { return so_f16_to_f32(h); }
static inline float hround(float v) { return so_f16_to_f32(so_f32_to_f16(v)); }

SO_EXPORT void so_ternary_affine_qmv(const uint8_t *codes, const uint16_t *scales,
                                     const uint16_t *bias_scales, const uint16_t *x, int rows,
                                     int cols, int batch, uint16_t *out) {
    const int G = 128, VPL = 16, BLOCK = VPL * 32;
    int groups = cols / G;
    int row_bytes = cols / 4;
    for (int b = 0; b < batch; ++b) {
        const uint16_t *xb = x + (size_t)b * cols;
        for (int r = 0; r < rows; ++r) {
            float lane_result[32];
            for (int lane = 0; lane < 32; ++lane) {
                float result = 0;
                for (int block = 0; block < cols; block += BLOCK) {
                    int col = block + lane * VPL;
                    if (col >= cols) continue;
                    float xt[16];
                    float sum = 0;
                    for (int i = 0; i < VPL; i += 4) {
                        /* half-typed a+b+c+d, then widened into the float accumulator */
                        float h = hround(h2f(xb[col + i]) + h2f(xb[col + i + 1]));
                        h = hround(h + h2f(xb[col + i + 2]));
                        h = hround(h + h2f(xb[col + i + 3]));
                        sum += h;
                        xt[i + 0] = h2f(xb[col + i + 0]);
                        xt[i + 1] = h2f(xb[col + i + 1]) / 4.0f;
                        xt[i + 2] = h2f(xb[col + i + 2]) / 16.0f;
                        xt[i + 3] = h2f(xb[col + i + 3]) / 64.0f;
                    }
                    uint32_t packed_codes;
                    memcpy(&packed_codes, codes + (size_t)r * row_bytes + col / 4, 4);
                    float scale = h2f(scales[(size_t)r * groups + col / G]);
                    float bias = -h2f(bias_scales[(size_t)r * groups + col / G]);
                    float accum = 0;
                    for (int i = 0; i < 4; ++i) {
                        uint32_t p = (packed_codes >> (i * 8)) & 0xFFu;
                        volatile float t0 = xt[4 * i + 0] * (float)(p & 0x03u);
                        volatile float t1 = xt[4 * i + 1] * (float)(p & 0x0Cu);
                        volatile float t2 = xt[4 * i + 2] * (float)(p & 0x30u);
                        volatile float t3 = xt[4 * i + 3] * (float)(p & 0xC0u);
                        volatile float s01 = t0 + t1;
                        volatile float s012 = s01 + t2;
                        volatile float s = s012 + t3;
                        accum += s;
                    }
                    volatile float sa = scale * accum;
                    volatile float sb = sum * bias;
                    result += sa + sb;
                }
                lane_result[lane] = result;
            }
            /* simd_sum: butterfly reduction (xor 16, 8, 4, 2, 1) */
            for (int off = 16; off > 0; off >>= 1)
                for (int lane = 0; lane < off; ++lane) lane_result[lane] += lane_result[lane + off];
            out[(size_t)b * rows + r] = so_f32_to_f16(lane_result[0]);
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Ternary "affine" QMM weight tile, the arithmetic of MLX affine_qmm_t<half,128,2> */
/* signed_quant_precise.metal:407-439. Each two-bit field stays at its position */
/* inside the byte; byte lane k multiplies it by a separately rounded fp16      */
/* subscale fp16(scale / 4^k) and adds -bias_scale, all in half arithmetic.     */
/* (The product of a subscale and a shifted ternary field is exact in fp16, so   */
/* a fused and an unfused half multiply-add round identically.)                */
/* out_bits: fp16 [rows, cols].                                               */
/* ------------------------------------------------------------------------- */
static float f64_to_f32_round_odd(double v) {
    float f = (float)v;
    if ((double)f == v || v != v) return f;
    uint32_t u;
    memcpy(&u, &f, 4);
    if (fabs((double)f) > fabs(v)) u -= 1; /* back to the truncated magnitude */
    u |= 1u;
    memcpy(&f, &u, 4);
    return f;
}

SO_EXPORT void so_ternary_affine_qmm_weights(const uint8_t *codes, const uint16_t *scales,
                                             const uint16_t *bias_scales, int rows, int cols,
                                             uint16_t *out_bits) {
    const int G = 128;
    int groups = cols / G;
    int row_bytes = cols / 4;
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c) {
            size_t si = (size_t)r * groups + c / G;
            float scale = h2f(scales[si]);
            float bias = -h2f(bias_scales[si]);
            int lane = c & 3;
            float sub = lane == 0 ? scale : hround(scale / (float)(1 << (2 * lane)));
            uint32_t field = (codes[(size_t)r * row_bytes + c / 4] >> (2 * lane)) & 3u;
            /* widened product and sum are exact in double; one rounding to half
             * (through a round-to-odd float so that the two-step narrowing cannot
             * double-round when scale and bias_scale differ widely in magnitude) */
            double v = (double)sub * (double)(field << (2 * lane)) + (double)bias;
            out_bits[(size_t)r * cols + c] = so_f32_to_f16(f64_to_f32_round_odd(v));
        }
}

/* QMM result over that tile (signed_quant_precise.metal:441-489): fp16 weights  */
/* times fp16 activations accumulated in fp32 by the 8x8 matrix unit, whose       */
/* internal order is not specified; restated as a double-precision dot rounded    */
/* once to float. x fp16 bits [batch, cols]; out float [batch, rows].            */
SO_EXPORT void so_ternary_affine_qmm(const uint8_t *codes, const uint16_t *scales,
                                     const uint16_t *bias_scales, const uint16_t *x, int rows,
                                     int cols, int batch, float *out) {
    uint16_t *w = (uint16_t *)malloc((size_t)rows * cols * sizeof(uint16_t));
    so_ternary_affine_qmm_weights(codes, scales, bias_scales, rows, cols, w);
    for (int b = 0; b < batch; ++b)
        for (int r = 0; r < rows; ++r) {
            double acc = 0;
            for (int c = 0; c < cols; ++c)
                acc += (double)h2f(w[(size_t)r * cols + c]) * (double)h2f(x[(size_t)b * cols + c]);
            out[(size_t)b * rows + r] = (float)acc;
        }
    free(w);
}

/* ------------------------------------------------------------------------- */
/* Epilogues                                                                   */
/* ------------------------------------------------------------------------- */

/* lut_matvec.metal:4574-4577, signed_quant.metal:277-284:
 * project, round to the activation type, then add the residual in that type. */
SO_EXPORT uint16_t so_epilogue_residual_add(float acc, uint16_t residual, int dtype) {
    float projected = so_round_through(acc, dtype);
    return narrow(projected + widen(residual, dtype), dtype);
}

/* lut_matvec.metal:5075, agent_affine_qmm.h:329: half(gate/(1+exp(-gate))*up), fp32 g,u */
SO_EXPORT uint16_t so_epilogue_affine_swiglu(float gate, float up, int dtype) {
    return narrow(gate / (1.0f + expf(-gate)) * up, dtype);
}

/* lut_matvec.metal:2235-2243 (agent_geglu_product): gate and up rounded to the 16-bit type, tanh
 * form of GELU with its argument clamped to +-20, product clamped to the fp16 range. */
SO_EXPORT uint16_t so_epilogue_geglu(float gate, float up, int dtype) {
    gate = so_round_through(gate, dtype);
    up = so_round_through(up, dtype);
    float gate3 = gate * gate * gate;
    float inner = 0.7978845608f * (gate + 0.044715f * gate3);
    inner = inner < -20.0f ? -20.0f : (inner > 20.0f ? 20.0f : inner);
    float gelu = 0.5f * gate * (1.0f + tanhf(inner));
    float prod = gelu * up;
    prod = prod < -65504.0f ? -65504.0f : (prod > 65504.0f ? 65504.0f : prod);
    return narrow(prod, dtype);
}

/* lut_matvec.metal:1347-1379 (norm_scale_affine_matvec and its gate/up forms): the activation a
 * norm-scale kernel multiplies is half((x * rs) * (1 + w)), products taken left to right. */
SO_EXPORT void so_norm_scale_input(const uint16_t *x, float rs, const uint16_t *weight, int dtype,
                                   int count, uint16_t *out) {
    for (int i = 0; i < count; ++i) {
        float scaled = widen(x[i], dtype) * rs;
        float direct = 1.0f + widen(weight[i], dtype);
        out[i] = narrow(scaled * direct, dtype);
    }
}

/* signed_quant.metal:15-20 / signed_quant_precise.metal:31-36: every intermediate is
 * materialised in the activation type. gate/up arrive already rounded to that type. */
SO_EXPORT uint16_t so_epilogue_signed_swiglu(uint16_t gate_bits, uint16_t up_bits, int dtype) {
    float gate = widen(gate_bits, dtype), up = widen(up_bits, dtype);
    float e = so_round_through(expf(fabsf(gate)), dtype);
    float denom = so_round_through(1.0f + e, dtype);
    float tail = so_round_through(1.0f / denom, dtype);
    float sigmoid = gate < 0.0f ? tail : so_round_through(1.0f - tail, dtype);
    float activated = so_round_through(gate * sigmoid, dtype);
    return narrow(activated * up, dtype);
}

/* ------------------------------------------------------------------------- */
/* Layer ops between the matvecs                                               */
/* ------------------------------------------------------------------------- */

/* 1 / sqrt(mean(x^2) + eps), fp32, summed in index order
 * (CPU mirror: Tests/SmeltCompilerTests/Helpers/MetalKernelTestSupport.swift:233-235;
 *  kernels: Resources/Shaders/norms.metal:991-1020). */
SO_EXPORT float so_rms_scale(const uint16_t *x, int n, float eps, int dtype) {
    float sum = 0.0f;
    for (int i = 0; i < n; ++i) {
        float v = widen(x[i], dtype);
        sum += v * v;
    }
    return 1.0f / sqrtf(sum / (float)n + eps);
}

/* rms_norm_1pw: x * rs * (1 + w) in the 16-bit type.
 * two_step != 0: half(1 + w) * half(x * rs) (norms.metal:54-62, 1537-1545);
 * two_step == 0: half(x * (rs * (1 + w))) (the fixed-dimension kernels, norms.metal:164-170).
 * residual (may be NULL) is added to the rounded result in the 16-bit type (norms.metal:412-445). */
SO_EXPORT void so_rms_norm_1pw(const uint16_t *x, const uint16_t *w, const uint16_t *residual, int n,
                               float eps, int dtype, int two_step, uint16_t *out) {
    float rs = so_rms_scale(x, n, eps, dtype);
    for (int i = 0; i < n; ++i) {
        float v = widen(x[i], dtype), wt = widen(w[i], dtype);
        uint16_t y;
        if (two_step == 1) {
            float normalized = so_round_through(v * rs, dtype);
            float direct = so_round_through(1.0f + wt, dtype);
            y = narrow(direct * normalized, dtype);
        } else if (two_step == 2) {   /* the d256 kernels: x * rs * (1 + w), left to right (norms.metal:213) */
            float scaled = v * rs;
            y = narrow(scaled * (1.0f + wt), dtype);
        } else {
            float scale = rs * (1.0f + wt);
            y = narrow(v * scale, dtype);
        }
        if (residual) y = narrow(widen(y, dtype) + widen(residual[i], dtype), dtype);
        out[i] = y;
    }
}

/* rms_norm_1pw_d256_add_scalar_weight (norms.metal:218-260): the d256 norm, + residual, * scalar[0],
 * each step rounded to the 16-bit type. */
SO_EXPORT void so_rms_norm_1pw_add_scalar(const uint16_t *x, const uint16_t *w, const uint16_t *residual,
                                          uint16_t scalar, int n, float eps, int dtype, uint16_t *out) {
    so_rms_norm_1pw(x, w, residual, n, eps, dtype, 2, out);
    for (int i = 0; i < n; ++i) out[i] = narrow(widen(out[i], dtype) * widen(scalar, dtype), dtype);
}

/* rms_norm_1pw_from_fp32 (norms_fp32.metal:50-88): fp32 input, running fp32 sum of squares,
 * half(clamp(x * rs * (1 + w), +-65504)). */
SO_EXPORT void so_rms_norm_1pw_from_fp32(const float *x, const uint16_t *w, int n, float eps, int dtype,
                                         uint16_t *out) {
    float sum = 0.0f;
    for (int i = 0; i < n; ++i) sum += x[i] * x[i];
    float rs = 1.0f / sqrtf(sum / (float)n + eps);
    for (int i = 0; i < n; ++i) {
        float scaled = x[i] * rs;
        float v = scaled * (1.0f + widen(w[i], dtype));
        v = v < -65504.0f ? -65504.0f : (v > 65504.0f ? 65504.0f : v);
        out[i] = narrow(v, dtype);
    }
}

/* rms_norm_gated (norms.metal:1093-1153): per head half(w * (x * rs) * silu(gate)), SiLU in fp32.
 * precise != 0: the d128 kernels (norms_gated_precise.metal:7-18): half(w) * half(x * rs) as a 16-bit
 * product, SiLU from the stable sigmoid in fp32, one final narrowing. */
static uint16_t rms_norm_gated_value(uint16_t x, uint16_t gate, uint16_t w, float rs, int precise, int dtype) {
    float g = widen(gate, dtype);
    if (precise) {
        float normalized = so_round_through(widen(w, dtype) * so_round_through(widen(x, dtype) * rs, dtype), dtype);
        float tail = 1.0f / (1.0f + expf(fabsf(g)));
        float sigmoid = g < 0.0f ? tail : 1.0f - tail;
        return narrow(normalized * (g * sigmoid), dtype);
    }
    float silu = g / (1.0f + expf(-g));
    float normalized = widen(x, dtype) * rs;
    float weighted = widen(w, dtype) * normalized;
    return narrow(weighted * silu, dtype);
}

SO_EXPORT void so_rms_norm_gated(const uint16_t *x, const uint16_t *gate, const uint16_t *w, int heads,
                                 int head_dim, float eps, int dtype, int precise, uint16_t *out) {
    for (int h = 0; h < heads; ++h) {
        const uint16_t *xr = x + (size_t)h * head_dim, *gr = gate + (size_t)h * head_dim;
        float rs = so_rms_scale(xr, head_dim, eps, dtype);
        for (int i = 0; i < head_dim; ++i)
            out[(size_t)h * head_dim + i] = rms_norm_gated_value(xr[i], gr[i], w[i], rs, precise, dtype);
    }
}

/* Pointwise activations (activations.metal:5-40, 98-108, 166-177), fp32 arithmetic, one narrowing:
 * op 0 silu, 1 sigmoid, 2 softplus (x itself above 20), 3 x * param, 4 param * tanh(x / param). */
SO_EXPORT uint16_t so_unary(int op, uint16_t x_bits, float param, int dtype) {
    float x = widen(x_bits, dtype), v;
    switch (op) {
        case 0: v = x / (1.0f + expf(-x)); break;
        case 1: v = 1.0f / (1.0f + expf(-x)); break;
        case 2: v = x > 20.0f ? x : logf(1.0f + expf(x)); break;
        case 3: v = x * param; break;
        default: v = param * tanhf(x / param); break;
    }
    return narrow(v, dtype);
}

/* swiglu_fused (activations_precise.metal:9-22), elementwise_add / _mul (activations.metal:56-66, 85-95) */
SO_EXPORT void so_swiglu_fused(const uint16_t *gate, const uint16_t *up, int n, int dtype, uint16_t *out) {
    for (int i = 0; i < n; ++i) out[i] = so_epilogue_signed_swiglu(gate[i], up[i], dtype);
}
SO_EXPORT void so_elementwise(const uint16_t *a, const uint16_t *b, int n, int dtype, int multiply, uint16_t *out) {
    for (int i = 0; i < n; ++i) {
        float x = widen(a[i], dtype), y = widen(b[i], dtype);
        out[i] = narrow(multiply ? x * y : x + y, dtype);
    }
}

/* ------------------------------------------------------------------------- */
/* Signed activation views (bit planes) — signed_quant.metal:746-2260          */
/* ------------------------------------------------------------------------- */

/* Largest magnitude of an i{planes} view: i2 keeps {-1, 0, +1} (signed_quant.metal:848-858),
 * the others 2^(planes-1) - 1 (:757-775, 836-846, 860-872, 918-930). */
SO_EXPORT int so_bitplane_max_q(int planes) { return planes == 2 ? 1 : (1 << (planes - 1)) - 1; }

/* One group of 128 values -> scale bits + quantised integers (signed_quant.metal:797-834).
 * i2 and i3 quantise with the unrounded scale, i4..i6 with the stored 16-bit scale. */
static uint16_t bitplane_quantize_group(const float *v, int planes, int dtype, int *q) {
    int max_q = so_bitplane_max_q(planes);
    float max_abs = 0.0f;
    for (int i = 0; i < 128; ++i) max_abs = fmaxf(max_abs, fabsf(v[i]));
    float producer = max_abs > 0.0f ? max_abs / (float)max_q : 1.0f;
    uint16_t stored = narrow(producer, dtype);
    float scale = planes >= 4 ? widen(stored, dtype) : producer;
    for (int i = 0; i < 128; ++i) {
        float t = v[i] / scale;
        t = fminf(fmaxf(t, -(float)max_q), (float)max_q);
        q[i] = (int)roundf(t);
    }
    return stored;
}

/* Plane p < planes-1 holds bit p of |q|, plane planes-1 the sign; word w, bit l = value w*32+l;
 * out_planes is [groups][planes][4] (signed_quant.metal:751-755, 786-794). */
static void bitplane_pack_group(const int *q, int planes, uint32_t *out) {
    for (int p = 0; p < planes; ++p)
        for (int w = 0; w < 4; ++w) {
            uint32_t word = 0;
            for (int l = 0; l < 32; ++l) {
                int v = q[w * 32 + l];
                uint32_t bit = p == planes - 1 ? (v < 0 ? 1u : 0u) : (((uint32_t)abs(v) >> p) & 1u);
                word |= bit << l;
            }
            out[p * 4 + w] = word;
        }
}

/* signed_activation_bitplanes_i{2..6}_g128: cols a multiple of 128. q_out (may be NULL) receives
 * the integers the planes encode. */
SO_EXPORT void so_signed_activation_bitplanes(const uint16_t *x, int cols, int planes, int dtype,
                                              uint32_t *out_planes, uint16_t *out_scales, int *q_out) {
    int groups = cols / 128;
    for (int g = 0; g < groups; ++g) {
        float v[128];
        int q[128];
        for (int i = 0; i < 128; ++i) v[i] = widen(x[g * 128 + i], dtype);
        out_scales[g] = bitplane_quantize_group(v, planes, dtype, q);
        bitplane_pack_group(q, planes, out_planes + (size_t)g * planes * 4);
        if (q_out) memcpy(q_out + g * 128, q, sizeof(q));
    }
}

/* swiglu_signed_activation_bitplanes_i5_g128 (:876-916): the staged SwiGLU value, then the view. */
SO_EXPORT void so_swiglu_signed_activation_bitplanes(const uint16_t *gate, const uint16_t *up, int cols,
                                                     int planes, int dtype, uint32_t *out_planes,
                                                     uint16_t *out_scales) {
    int groups = cols / 128;
    for (int g = 0; g < groups; ++g) {
        float v[128];
        int q[128];
        for (int i = 0; i < 128; ++i)
            v[i] = widen(so_epilogue_signed_swiglu(gate[g * 128 + i], up[g * 128 + i], dtype), dtype);
        out_scales[g] = bitplane_quantize_group(v, planes, dtype, q);
        bitplane_pack_group(q, planes, out_planes + (size_t)g * planes * 4);
    }
}

/* sigmoid_mul_signed_activation_bitplanes_i6_g128 (signed_quant.metal:985-1027): a * sigmoid(b) with
 * exp, 1 + e, the reciprocal, 1 - tail and the product each materialised in the 16-bit type, then the view. */
SO_EXPORT uint16_t so_sigmoid_mul(uint16_t a_bits, uint16_t b_bits, int dtype) {
    float a = widen(a_bits, dtype), b = widen(b_bits, dtype);
    float e = so_round_through(expf(fabsf(b)), dtype);
    float denom = so_round_through(1.0f + e, dtype);
    float tail = so_round_through(1.0f / denom, dtype);
    float sig = b < 0.0f ? tail : so_round_through(1.0f - tail, dtype);
    return narrow(a * sig, dtype);
}

SO_EXPORT void so_sigmoid_mul_signed_activation_bitplanes(const uint16_t *a, const uint16_t *b, int cols,
                                                          int planes, int dtype, uint32_t *out_planes,
                                                          uint16_t *out_scales) {
    int groups = cols / 128;
    for (int g = 0; g < groups; ++g) {
        float v[128];
        int q[128];
        for (int i = 0; i < 128; ++i) v[i] = widen(so_sigmoid_mul(a[g * 128 + i], b[g * 128 + i], dtype), dtype);
        out_scales[g] = bitplane_quantize_group(v, planes, dtype, q);
        bitplane_pack_group(q, planes, out_planes + (size_t)g * planes * 4);
    }
}

/* rms_norm_gated_d128_signed_activation_bitplanes_i6_g128 (signed_quant.metal:1029-1173): the gated norm of
 * one 128-value head (precise or generic arithmetic, as the launch selects), then its i6 view. */
SO_EXPORT void so_rms_norm_gated_signed_activation_bitplanes(const uint16_t *x, const uint16_t *gate, const uint16_t *w,
                                                             int heads, float eps, int dtype, int precise,
                                                             uint32_t *out_planes, uint16_t *out_scales) {
    for (int h = 0; h < heads; ++h) {
        uint16_t row[128];
        float v[128];
        int q[128];
        so_rms_norm_gated(x + (size_t)h * 128, gate + (size_t)h * 128, w, 1, 128, eps, dtype, precise, row);
        for (int i = 0; i < 128; ++i) v[i] = widen(row[i], dtype);
        out_scales[h] = bitplane_quantize_group(v, 6, dtype, q);
        bitplane_pack_group(q, 6, out_planes + (size_t)h * 24);
    }
}

/* norm_scale_signed_activation_bitplanes_i{2..6}_g128 (:1175-1223): rms_norm_1pw's two-step value
 * half(x * rs) * half(1 + w) from a precomputed scale, then the view. */
SO_EXPORT void so_norm_scale_signed_activation_bitplanes(float rs, const uint16_t *x, const uint16_t *w,
                                                         int cols, int planes, int dtype,
                                                         uint32_t *out_planes, uint16_t *out_scales) {
    int groups = cols / 128;
    for (int g = 0; g < groups; ++g) {
        float v[128];
        int q[128];
        for (int i = 0; i < 128; ++i) {
            float normalized = so_round_through(widen(x[g * 128 + i], dtype) * rs, dtype);
            float direct = so_round_through(1.0f + widen(w[g * 128 + i], dtype), dtype);
            v[i] = so_round_through(normalized * direct, dtype);
        }
        out_scales[g] = bitplane_quantize_group(v, planes, dtype, q);
        bitplane_pack_group(q, planes, out_planes + (size_t)g * planes * 4);
    }
}

static int popc32(uint32_t v) { return __builtin_popcount(v); }

/* signed_{binary,ternary}_bitplane_i{N}_matvec_g128_rows8 (:1564-1636, 2054-2104): per (row, group)
 * an integer dot of signed weights with the quantised activations, formed from popcounts
 * (:1300-1348), times activation scale, times weight scale; fp32 sum over groups in group order. */
SO_EXPORT void so_signed_bitplane_matvec(int format, const uint8_t *codes, const uint16_t *weight_scales,
                                         const uint32_t *act_planes, const uint16_t *act_scales, int rows,
                                         int cols, int planes, int dtype, float *out) {
    int groups = cols / 128;
    int row_bytes = format == SO_BINARY1 ? cols / 8 : cols / 4;
    for (int r = 0; r < rows; ++r) {
        float acc = 0.0f;
        for (int g = 0; g < groups; ++g) {
            uint32_t pos[4] = {0, 0, 0, 0}, neg[4] = {0, 0, 0, 0};
            for (int c = 0; c < 128; ++c) {
                int code = so_signed_code_at((int64_t)g * 128 + c, codes + (size_t)r * row_bytes, row_bytes, format);
                int sem = 0;
                so_signed_semantic(format, code, &sem);
                if (sem > 0) pos[c >> 5] |= 1u << (c & 31);
                if (sem < 0) neg[c >> 5] |= 1u << (c & 31);
            }
            const uint32_t *pl = act_planes + (size_t)g * planes * 4;
            const uint32_t *sign = pl + (planes - 1) * 4;
            int dot = 0;
            for (int b = 0; b < planes - 1; ++b) {
                int agreement = 0, active = 0;
                for (int w = 0; w < 4; ++w) {
                    uint32_t mask = (pos[w] & ~sign[w]) | (neg[w] & sign[w]);
                    agreement += popc32(mask & pl[b * 4 + w]);
                    active += popc32((pos[w] | neg[w]) & pl[b * 4 + w]);
                }
                dot += (1 << b) * (2 * agreement - active);
            }
            volatile float scaled = (float)dot * widen(act_scales[g], dtype);
            volatile float term = scaled * so_f16_to_f32(weight_scales[(size_t)r * groups + g]);
            acc += term;
        }
        out[r] = acc;
    }
}

/* ------------------------------------------------------------------------- */
/* u4_lut — lut_matvec.metal:28-790, 967-992                                   */
/* ------------------------------------------------------------------------- */

/* y[r] = sum_c lut[r / group][index(r, c)] * x[c]: fp32, products accumulated in column order
 * (lut_matvec.metal:86-140; the kernel's lanes each take every 32nd 16-column run, the scalar
 * restatement keeps one running sum). lut is fp16 [ceil(rows / group), 16]. */
SO_EXPORT void so_lut_matvec(const uint8_t *indices, const uint16_t *lut, const float *x, int rows,
                             int cols, int group, float *out) {
    int half_cols = cols / 2;
    for (int r = 0; r < rows; ++r) {
        const uint16_t *table = lut + (size_t)(r / group) * 16;
        float acc = 0.0f;
        for (int c = 0; c < cols; ++c) {
            uint8_t byte = indices[(size_t)r * half_cols + (c >> 1)];
            uint8_t idx = (c & 1) ? (byte >> 4) : (byte & 0x0F);
            volatile float prod = so_f16_to_f32(table[idx]) * x[c];
            acc += prod;
        }
        out[r] = acc;
    }
}

/* fused_lut_matvec_add: half(float(residual) + acc) (lut_matvec.metal:334-340) */
SO_EXPORT uint16_t so_epilogue_lut_add(float acc, uint16_t residual, int dtype) {
    return narrow(widen(residual, dtype) + acc, dtype);
}

/* lut_embedding_gather (lut_matvec.metal:967-992) */
SO_EXPORT void so_lut_gather(const uint8_t *indices, const uint16_t *lut, int row, int cols, int group,
                             uint16_t *out) {
    const uint16_t *table = lut + (size_t)(row / group) * 16;
    for (int i = 0; i < cols / 2; ++i) {
        uint8_t byte = indices[(size_t)row * (cols / 2) + i];
        out[2 * i] = table[byte & 0x0F];
        out[2 * i + 1] = table[byte >> 4];
    }
}

/* ------------------------------------------------------------------------- */
/* turbo_quant_h — lut_matvec.metal:1045-1079, 9207-9355                       */
/* ------------------------------------------------------------------------- */

#define SO_TQH_INV_SQRT_G 0.0883883476483184405f

static int tqh_code(const uint8_t *row_codes, int g, int j) {
    return (row_codes[g * 32 + (j >> 2)] >> ((j & 3) * 2)) & 3;
}

/* tqh_matvec_prepare_input (:9222-9244): xhat[g, j] = sum_p (-1)^popcount(p & j) x[g*128 + p], fp32,
 * p increasing, columns beyond cols skipped. xhat is [ceil(cols/128) * 128]. */
SO_EXPORT void so_tqh_prepare(const uint16_t *x, int cols, int dtype, float *xhat) {
    int groups = (cols + 127) / 128;
    for (int g = 0; g < groups; ++g)
        for (int j = 0; j < 128; ++j) {
            float acc = 0.0f;
            for (int p = 0; p < 128 && g * 128 + p < cols; ++p) {
                float xp = widen(x[g * 128 + p], dtype);
                acc += (__builtin_popcount((unsigned)(p & j)) & 1) ? -xp : xp;
            }
            xhat[g * 128 + j] = acc;
        }
}

/* tqh_matvec (:9250-9343): acc = sum_{g, j} cb[g][code] * xhat[g, j] (fp32), out = acc / sqrt(128). */
SO_EXPORT void so_tqh_matvec(const uint8_t *codes, const uint16_t *codebook, const float *xhat, int rows,
                             int cols, float *out) {
    int groups = (cols + 127) / 128;
    int codes_per_row = groups * 32;
    for (int r = 0; r < rows; ++r) {
        float acc = 0.0f;
        for (int g = 0; g < groups; ++g)
            for (int j = 0; j < 128; ++j) {
                volatile float prod = so_f16_to_f32(codebook[g * 4 + tqh_code(codes + (size_t)r * codes_per_row, g, j)]) * xhat[g * 128 + j];
                acc += prod;
            }
        volatile float scaled = acc * SO_TQH_INV_SQRT_G;
        out[r] = scaled;
    }
}

/* tqh_embedding_gather (:1045-1079): one dequantised row in fp32 before the final rounding:
 * W[p] = (sum_j (-1)^popcount(p & j) cb[g][code_j]) / sqrt(128). */
SO_EXPORT void so_tqh_dequantize_row(const uint8_t *row_codes, const uint16_t *codebook, int cols, float *out) {
    for (int c = 0; c < cols; ++c) {
        int g = c / 128, p = c % 128;
        float acc = 0.0f;
        for (int j = 0; j < 128; ++j) {
            float v = so_f16_to_f32(codebook[g * 4 + tqh_code(row_codes, g, j)]);
            acc += (__builtin_popcount((unsigned)(p & j)) & 1) ? -v : v;
        }
        volatile float scaled = acc * SO_TQH_INV_SQRT_G;
        out[c] = scaled;
    }
}

/* ------------------------------------------------------------------------- */
/* Argmax key — lut_matvec.metal:4045-4074                                     */
/* ------------------------------------------------------------------------- */

#define SO_ARGMAX_INDEX_BITS 18
#define SO_ARGMAX_MAX_INDEX ((1u << SO_ARGMAX_INDEX_BITS) - 1u)

SO_EXPORT uint32_t so_argmax_ordered_key16(uint16_t bits16) {
    uint32_t bits = bits16;
    if ((bits & 0x7FFFu) == 0u) bits = 0u;
    return (bits & 0x8000u) != 0u ? (0xFFFFu - bits) : (bits ^ 0x8000u);
}

SO_EXPORT uint64_t so_argmax_pack_key(uint16_t value_bits, uint32_t index) {
    uint32_t ordered = so_argmax_ordered_key16(value_bits);
    uint32_t inverse = (SO_ARGMAX_MAX_INDEX - index) & SO_ARGMAX_MAX_INDEX;
    return ((uint64_t)ordered << 32) | inverse;
}

/* argmax over 16-bit float patterns (fp16, or bf16 — same sign/magnitude ordering):
 * largest value wins, ties to the lowest index, -0 == +0. */
SO_EXPORT int so_argmax16(const uint16_t *values, int count) {
    uint64_t best = 0;
    for (int i = 0; i < count; ++i) {
        uint64_t k = so_argmax_pack_key(values[i], (uint32_t)i);
        if (k > best) best = k;
    }
    return (int)(SO_ARGMAX_MAX_INDEX - (uint32_t)(best & 0xFFFFFFFFu));
}

/* ------------------------------------------------------------------------- */
/* Threaded driver for the benchmark's cpu_baseline leg: rows split over       */
/* threads with OpenMP if built with -fopenmp; the arithmetic is the scalar    */
/* restatement above.                                                          */
/* ------------------------------------------------------------------------- */

SO_EXPORT void so_affine_matvec_mt(const uint8_t *packed, const uint16_t *scales,
                                   const uint16_t *biases, const float *x, int rows, int cols,
                                   int group, int dtype, float *out) {
    int gpr = cols / group;
    size_t stride = (size_t)cols / 2;
#pragma omp parallel for schedule(static)
    for (int r0 = 0; r0 < rows; r0 += 64) {
        int n = rows - r0 < 64 ? rows - r0 : 64;
        so_affine_matvec(packed + (size_t)r0 * stride, scales + (size_t)r0 * gpr,
                         biases + (size_t)r0 * gpr, x, n, cols, group, dtype, out + r0);
    }
}

SO_EXPORT int so_signed_matvec_mt(int format, const uint8_t *codes, int64_t row_stride,
                                  const uint16_t *scales, const float *x, int rows, int cols,
                                  int padded_cols, int group, float *out) {
    int groups = so_signed_groups_per_row(padded_cols, group);
    if (groups < 0) return groups;
    int rc_all = SO_OK;
#pragma omp parallel for schedule(static)
    for (int r0 = 0; r0 < rows; r0 += 64) {
        int n = rows - r0 < 64 ? rows - r0 : 64;
        int rc = so_signed_matvec(format, codes + (size_t)r0 * row_stride, row_stride,
                                  scales + (size_t)r0 * groups, x, n, cols, padded_cols, group, 1,
                                  out + r0);
        if (rc != SO_OK) rc_all = rc;
    }
    return rc_all;
}
