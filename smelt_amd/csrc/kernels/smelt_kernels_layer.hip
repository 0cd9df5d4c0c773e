// Translation unit 8 of the gfx950 code objects (smelt_kernels_layer.hsaco): weight-import producers, layer ops, u4_lut and turbo_quant_h kernels.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#include "import_kernels.hpp"
#include "layer_kernels.hpp"
#include "lut_kernels.hpp"
#include "tqh_kernels.hpp"

SMELT_AFFINE_QUANTIZE(f16, smelt::F16, 32)
SMELT_AFFINE_QUANTIZE(f16, smelt::F16, 64)
SMELT_AFFINE_QUANTIZE(f16, smelt::F16, 128)
SMELT_AFFINE_QUANTIZE(bf16, smelt::BF16, 32)
SMELT_AFFINE_QUANTIZE(bf16, smelt::BF16, 64)
SMELT_AFFINE_QUANTIZE(bf16, smelt::BF16, 128)

SMELT_LAYER_KERNELS(f16, smelt::F16)
SMELT_LAYER_KERNELS(bf16, smelt::BF16)
SMELT_LUT_KERNELS(f16, smelt::F16)
SMELT_LUT_KERNELS(bf16, smelt::BF16)
SMELT_TQH_KERNELS(f16, smelt::F16)
SMELT_TQH_KERNELS(bf16, smelt::BF16)
