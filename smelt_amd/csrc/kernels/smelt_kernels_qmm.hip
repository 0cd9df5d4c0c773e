// Translation unit 7 of the gfx950 code objects (smelt_kernels_qmm.hsaco): MFMA qmm kernels: token slabs and the split-K skinny form.
// Built with:  hipcc --offload-arch=gfx950 --genco -O3 -Xclang -target-feature -Xclang -packed-fp32-ops
#include "qmm.hpp"
#include "qmm_skinny.hpp"
