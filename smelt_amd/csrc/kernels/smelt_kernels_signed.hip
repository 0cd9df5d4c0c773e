// Translation unit 4 of the gfx950 code objects (smelt_kernels_signed.hsaco): binary, ternary, ternary-affine and trit5 vector-ALU matvec kernels.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#define SMELT_NO_INCLUDE_INSTANCES
#include "matvec_kernels.hpp"

SMELT_SIGNED_KERNELS(binary, smelt::FmtBin, f16, smelt::F16)
SMELT_SIGNED_KERNELS(binary, smelt::FmtBin, bf16, smelt::BF16)
SMELT_SIGNED_KERNELS(ternary, smelt::FmtTer2, f16, smelt::F16)
SMELT_SIGNED_KERNELS(ternary, smelt::FmtTer2, bf16, smelt::BF16)
SMELT_TERAFF_KERNELS(f16, smelt::F16)
SMELT_TERAFF_KERNELS(bf16, smelt::BF16)
SMELT_SIGNED_KERNELS(trit5, smelt::FmtTrit5, f16, smelt::F16)
SMELT_SIGNED_KERNELS(trit5, smelt::FmtTrit5, bf16, smelt::BF16)
SMELT_BINARY_BANK_KERNELS(f16, smelt::F16)
SMELT_BINARY_BANK_KERNELS(bf16, smelt::BF16)
SMELT_TRIT5_BANK_KERNELS(f16, smelt::F16)
SMELT_TRIT5_BANK_KERNELS(bf16, smelt::BF16)
