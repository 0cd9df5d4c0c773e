// Translation unit 2 of the gfx950 code objects (smelt_kernels_batched_f16.hsaco): token-tile affine matvec kernels and the fused argmax, fp16.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#define SMELT_NO_INCLUDE_INSTANCES
#include "matvec_kernels.hpp"

SMELT_AFFINE_BATCHED(f16, smelt::F16, smelt::F16, 1)
SMELT_AFFINE_BATCHED(f16, smelt::F16, smelt::F16, 2)
SMELT_AFFINE_BATCHED(f16, smelt::F16, smelt::F16, 4)
SMELT_AFFINE_ARGMAX(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_ARGMAX_SINGLE(f16, smelt::F16, smelt::F16)
