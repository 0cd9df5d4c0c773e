// Translation unit 1 of the gfx950 code objects (smelt_kernels.hsaco): single-token affine 4-bit matvec kernels, gathers, copy.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#include "matvec_kernels.hpp"

SMELT_AFFINE_KERNELS(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_KERNELS(bf16, smelt::BF16, smelt::BF16)
SMELT_AFFINE_FUSED_NORM(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_FUSED_NORM(bf16, smelt::BF16, smelt::BF16)
SMELT_AFFINE_BANK(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_BANK(bf16, smelt::BF16, smelt::BF16)
