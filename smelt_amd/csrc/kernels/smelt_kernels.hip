// Single translation unit for the gfx950 code object (smelt_kernels.hsaco).
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#include "matvec_kernels.hpp"
#include "mfma_matvec_kernels.hpp"
#include "misc_kernels.hpp"
#include "qmm.hpp"
#include "qmm_skinny.hpp"
#include "import_kernels.hpp"
#include "layer_kernels.hpp"
#include "bitplane_kernels.hpp"
#include "lut_kernels.hpp"
#include "tqh_kernels.hpp"

SMELT_AFFINE_KERNELS(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_KERNELS(bf16, smelt::BF16, smelt::BF16)
SMELT_AFFINE_FUSED_NORM(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_FUSED_NORM(bf16, smelt::BF16, smelt::BF16)
SMELT_AFFINE_BATCHED(f16, smelt::F16, smelt::F16, 1)
SMELT_AFFINE_BATCHED(f16, smelt::F16, smelt::F16, 2)
SMELT_AFFINE_BATCHED(f16, smelt::F16, smelt::F16, 4)
SMELT_AFFINE_BATCHED(bf16, smelt::BF16, smelt::BF16, 1)
SMELT_AFFINE_BATCHED(bf16, smelt::BF16, smelt::BF16, 2)
SMELT_AFFINE_BATCHED(bf16, smelt::BF16, smelt::BF16, 4)

SMELT_SIGNED_KERNELS(binary, smelt::FmtBin, f16, smelt::F16)
SMELT_SIGNED_KERNELS(binary, smelt::FmtBin, bf16, smelt::BF16)
SMELT_SIGNED_KERNELS(ternary, smelt::FmtTer2, f16, smelt::F16)
SMELT_SIGNED_KERNELS(ternary, smelt::FmtTer2, bf16, smelt::BF16)

SMELT_AFFINE_ARGMAX(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_ARGMAX_SINGLE(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_ARGMAX(bf16, smelt::BF16, smelt::BF16)
SMELT_AFFINE_ARGMAX_SINGLE(bf16, smelt::BF16, smelt::BF16)
SMELT_TERAFF_KERNELS(f16, smelt::F16)
SMELT_TERAFF_KERNELS(bf16, smelt::BF16)
SMELT_SIGNED_KERNELS(trit5, smelt::FmtTrit5, f16, smelt::F16)
SMELT_SIGNED_KERNELS(trit5, smelt::FmtTrit5, bf16, smelt::BF16)
SMELT_AFFINE_BANK(f16, smelt::F16, smelt::F16)
SMELT_AFFINE_BANK(bf16, smelt::BF16, smelt::BF16)

SMELT_AFFINE_QUANTIZE(f16, smelt::F16, 32)
SMELT_AFFINE_QUANTIZE(f16, smelt::F16, 64)
SMELT_AFFINE_QUANTIZE(f16, smelt::F16, 128)
SMELT_AFFINE_QUANTIZE(bf16, smelt::BF16, 32)
SMELT_AFFINE_QUANTIZE(bf16, smelt::BF16, 64)
SMELT_AFFINE_QUANTIZE(bf16, smelt::BF16, 128)

SMELT_LAYER_KERNELS(f16, smelt::F16)
SMELT_LAYER_KERNELS(bf16, smelt::BF16)

SMELT_BITPLANE_KERNELS(binary, smelt::FmtBinPlanes, f16, smelt::F16)
SMELT_BITPLANE_KERNELS(binary, smelt::FmtBinPlanes, bf16, smelt::BF16)
SMELT_BITPLANE_KERNELS(ternary, smelt::FmtTerPlanes, f16, smelt::F16)
SMELT_BITPLANE_KERNELS(ternary, smelt::FmtTerPlanes, bf16, smelt::BF16)
SMELT_ACTIVATION_BITPLANE_KERNELS(f16, smelt::F16)
SMELT_ACTIVATION_BITPLANE_KERNELS(bf16, smelt::BF16)
SMELT_GATED_NORM_KERNELS(f16, smelt::F16)
SMELT_GATED_NORM_KERNELS(bf16, smelt::BF16)
SMELT_LUT_KERNELS(f16, smelt::F16)
SMELT_LUT_KERNELS(bf16, smelt::BF16)
SMELT_TQH_KERNELS(f16, smelt::F16)
SMELT_TQH_KERNELS(bf16, smelt::BF16)
SMELT_BINARY_BANK_KERNELS(f16, smelt::F16)
SMELT_BINARY_BANK_KERNELS(bf16, smelt::BF16)
