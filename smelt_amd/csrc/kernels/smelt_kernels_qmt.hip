// Translation unit 11 of the gfx950 code objects (smelt_kernels_qmt.hsaco): the token-tile affine
// qmm (two or three row tiles and two token blocks per wave, eight waves; gate+up: two row tiles of each matrix
// per wave and four waves, or three row tiles of one matrix per wave and eight waves).
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#define SMELT_NO_INCLUDE_INSTANCES
#include "qmm_stream.hpp"

#define SMELT_QMT_ALL(T, ACT)                                                                      \
    SMELT_AFFINE_QMT_PLAIN(T, ACT, ACT, 2, 2, 2) SMELT_AFFINE_QMT_PLAIN(T, ACT, ACT, 3, 2, 2)      \
    SMELT_AFFINE_QMT_GATE_UP(T, ACT, ACT, 2, 2, 1, false, r)                                         \
    SMELT_AFFINE_QMT_GATE_UP(T, ACT, ACT, 3, 2, 2, true, w)

SMELT_QMT_ALL(f16, smelt::F16)
SMELT_QMT_ALL(bf16, smelt::BF16)
