// Translation unit 5 of the gfx950 code objects (smelt_kernels_planes.hsaco): signed activation views: producers and popcount matvec consumers.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#define SMELT_NO_INCLUDE_INSTANCES
#include "matvec_kernels.hpp"
#include "bitplane_kernels.hpp"

SMELT_BITPLANE_KERNELS(binary, smelt::FmtBinPlanes, f16, smelt::F16)
SMELT_BITPLANE_KERNELS(binary, smelt::FmtBinPlanes, bf16, smelt::BF16)
SMELT_BITPLANE_KERNELS(ternary, smelt::FmtTerPlanes, f16, smelt::F16)
SMELT_BITPLANE_KERNELS(ternary, smelt::FmtTerPlanes, bf16, smelt::BF16)
SMELT_ACTIVATION_BITPLANE_KERNELS(f16, smelt::F16)
SMELT_ACTIVATION_BITPLANE_KERNELS(bf16, smelt::BF16)
SMELT_GATED_NORM_KERNELS(f16, smelt::F16)
SMELT_GATED_NORM_KERNELS(bf16, smelt::BF16)
