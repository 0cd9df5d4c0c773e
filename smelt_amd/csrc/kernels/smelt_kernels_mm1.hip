// Translation unit 9 of the gfx950 code objects (smelt_kernels_mm1.hsaco): the single-pass
// matrix-core matvec kernels, one instance per number of 128-byte segments a wave owns.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#define SMELT_NO_INCLUDE_INSTANCES
#include "mm1_matvec.hpp"

#define SMELT_MM1_ALL(T, ACT, NLV)                                                                \
    SMELT_SIGNED_MM1_KERNELS(binary, smelt::M1Bin, T, ACT, NLV)                                   \
    SMELT_SIGNED_MM1_KERNELS(ternary, smelt::M1Ter2, T, ACT, NLV)                                 \
    SMELT_TERAFF_MM1_KERNELS(T, ACT, NLV)                                                         \
    SMELT_BINARY_MM1_BANKS(T, ACT, NLV)                                                           \
    SMELT_AFFINE_MM1_KERNELS(T, ACT, ACT, NLV)                                                    \
    SMELT_AFFINE_MM1_BANK(T, ACT, ACT, NLV)

#define SMELT_MM1_EVERY_NL(T, ACT)                                                                \
    SMELT_MM1_ALL(T, ACT, 1) SMELT_MM1_ALL(T, ACT, 2) SMELT_MM1_ALL(T, ACT, 3)                    \
    SMELT_MM1_ALL(T, ACT, 4) SMELT_MM1_ALL(T, ACT, 5) SMELT_MM1_ALL(T, ACT, 6)

SMELT_MM1_EVERY_NL(f16, smelt::F16)
SMELT_MM1_EVERY_NL(bf16, smelt::BF16)

// affine rows of more than 24576 columns (96 segments: sixteen waves of six) need seven or eight per wave
#define SMELT_MM1_AFFINE_LONG(T, ACT)                                                             \
    SMELT_AFFINE_MM1_KERNELS(T, ACT, ACT, 7) SMELT_AFFINE_MM1_BANK(T, ACT, ACT, 7)                 \
    SMELT_AFFINE_MM1_KERNELS(T, ACT, ACT, 8) SMELT_AFFINE_MM1_BANK(T, ACT, ACT, 8)
SMELT_MM1_AFFINE_LONG(f16, smelt::F16)
SMELT_MM1_AFFINE_LONG(bf16, smelt::BF16)

// two tokens per pass: binary and ternary codes (the per-row and four-token forms from two tokens on)
#define SMELT_MM1_T2(T, ACT, NLV)                                                                 \
    SMELT_SIGNED_MM1_KERNELS_T2(binary, smelt::M1Bin, T, ACT, NLV)                                \
    SMELT_SIGNED_MM1_KERNELS_T2(ternary, smelt::M1Ter2, T, ACT, NLV)                              \
    SMELT_TERAFF_MM1_KERNELS_T2(T, ACT, NLV)
#define SMELT_MM1_T2_EVERY_NL(T, ACT)                                                             \
    SMELT_MM1_T2(T, ACT, 1) SMELT_MM1_T2(T, ACT, 2) SMELT_MM1_T2(T, ACT, 3)                       \
    SMELT_MM1_T2(T, ACT, 4) SMELT_MM1_T2(T, ACT, 5) SMELT_MM1_T2(T, ACT, 6)
SMELT_MM1_T2_EVERY_NL(f16, smelt::F16)
SMELT_MM1_T2_EVERY_NL(bf16, smelt::BF16)

#define SMELT_MM1_TRIT5(T, ACT)                                                                   \
    SMELT_SIGNED_MM1_KERNELS(trit5, smelt::M1Trit5, T, ACT, 1) SMELT_SIGNED_MM1_KERNELS(trit5, smelt::M1Trit5, T, ACT, 2) \
    SMELT_SIGNED_MM1_KERNELS(trit5, smelt::M1Trit5, T, ACT, 3)                                    \
    SMELT_TRIT5_MM1_BANK(T, ACT, 1) SMELT_TRIT5_MM1_BANK(T, ACT, 2) SMELT_TRIT5_MM1_BANK(T, ACT, 3)
SMELT_MM1_TRIT5(f16, smelt::F16)
SMELT_MM1_TRIT5(bf16, smelt::BF16)
