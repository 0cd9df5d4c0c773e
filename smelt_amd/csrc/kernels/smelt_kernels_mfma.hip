// Translation unit 6 of the gfx950 code objects (smelt_kernels_mfma.hsaco): ring-buffered matrix-core matvec kernels.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#define SMELT_NO_INCLUDE_INSTANCES
#include "mfma_matvec_kernels.hpp"
