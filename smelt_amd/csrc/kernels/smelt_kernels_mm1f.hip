// Translation unit 12 of the gfx950 code objects (smelt_kernels_mm1f.hsaco): the single-pass
// matrix-core matvec in the fused affine forms (two projections of one input, GeGLU, norm-scale
// prologue, the lm_head's argmax), one instance per number of 128-byte segments a wave owns.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#define SMELT_NO_INCLUDE_INSTANCES
#include "mm1_matvec.hpp"

#define SMELT_MM1F_EVERY_NL(T, ACT)                                                               \
    SMELT_AFFINE_MM1_ARGMAX(T, ACT, ACT, 1) SMELT_AFFINE_MM1_ARGMAX(T, ACT, ACT, 2)               \
    SMELT_AFFINE_MM1_ARGMAX(T, ACT, ACT, 3) SMELT_AFFINE_MM1_ARGMAX(T, ACT, ACT, 4)               \
    SMELT_AFFINE_MM1_ARGMAX(T, ACT, ACT, 5) SMELT_AFFINE_MM1_ARGMAX(T, ACT, ACT, 6)               \
    SMELT_AFFINE_MM1_ARGMAX(T, ACT, ACT, 7) SMELT_AFFINE_MM1_ARGMAX(T, ACT, ACT, 8)               \
    SMELT_AFFINE_MM1_FUSED(T, ACT, ACT, 1) SMELT_AFFINE_MM1_FUSED(T, ACT, ACT, 2)                 \
    SMELT_AFFINE_MM1_FUSED(T, ACT, ACT, 3) SMELT_AFFINE_MM1_FUSED(T, ACT, ACT, 4)                 \
    SMELT_AFFINE_MM1_FUSED(T, ACT, ACT, 5) SMELT_AFFINE_MM1_FUSED(T, ACT, ACT, 6)                 \
    SMELT_AFFINE_MM1_FUSED(T, ACT, ACT, 7) SMELT_AFFINE_MM1_FUSED(T, ACT, ACT, 8)

SMELT_MM1F_EVERY_NL(f16, smelt::F16)
SMELT_MM1F_EVERY_NL(bf16, smelt::BF16)
