// Translation unit 3 of the gfx950 code objects (smelt_kernels_batched_bf16.hsaco): token-tile affine matvec kernels and the fused argmax, bf16.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#define SMELT_NO_INCLUDE_INSTANCES
#include "matvec_kernels.hpp"

SMELT_AFFINE_BATCHED(bf16, smelt::BF16, smelt::BF16, 1)
SMELT_AFFINE_BATCHED(bf16, smelt::BF16, smelt::BF16, 2)
SMELT_AFFINE_BATCHED(bf16, smelt::BF16, smelt::BF16, 4)
SMELT_AFFINE_ARGMAX(bf16, smelt::BF16, smelt::BF16)
SMELT_AFFINE_ARGMAX_SINGLE(bf16, smelt::BF16, smelt::BF16)
