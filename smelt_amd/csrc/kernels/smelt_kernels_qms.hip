// Translation unit 10 of the gfx950 code objects (smelt_kernels_qms.hsaco): the streaming
// small-batch affine qmm, one instance per (row tiles per wave, eight or sixteen staged token rows), and the
// forms for groups of 32 columns and for ternary codes.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#define SMELT_NO_INCLUDE_INSTANCES
#include "qmm_stream.hpp"

#define SMELT_QMS_ALL(T, ACT)                                                                      \
    SMELT_AFFINE_QMS_PLAIN(T, ACT, ACT, 1, 2) SMELT_AFFINE_QMS_PLAIN(T, ACT, ACT, 1, 4)            \
    SMELT_AFFINE_QMS_PLAIN(T, ACT, ACT, 2, 2) SMELT_AFFINE_QMS_PLAIN(T, ACT, ACT, 2, 4)            \
    SMELT_AFFINE_QMS_GATE_UP(T, ACT, ACT, 2) SMELT_AFFINE_QMS_GATE_UP(T, ACT, ACT, 4)              \
    SMELT_AFFINE_QMS_G32(T, ACT, ACT, 2) SMELT_AFFINE_QMS_G32(T, ACT, ACT, 4)                      \
    SMELT_TERNARY_QMS(T, ACT, 2) SMELT_TERNARY_QMS(T, ACT, 4)

SMELT_QMS_ALL(f16, smelt::F16)
SMELT_QMS_ALL(bf16, smelt::BF16)

// binary and ternary per-token records over many tokens
#define SMELT_QSS_ALL(T, ACT)                                                                      \
    SMELT_SIGNED_QSS(binary, 1, 2, T, ACT) SMELT_SIGNED_QSS(binary, 1, 4, T, ACT)                  \
    SMELT_SIGNED_QSS(ternary, 2, 2, T, ACT) SMELT_SIGNED_QSS(ternary, 2, 4, T, ACT)                \
    SMELT_TERAFF_QSS(2, T, ACT) SMELT_TERAFF_QSS(4, T, ACT)
SMELT_QSS_ALL(f16, smelt::F16)
SMELT_QSS_ALL(bf16, smelt::BF16)
