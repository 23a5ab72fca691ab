// f32 instantiations of the implicit-GEMM kernel whose store adds a residual operand (the last convolution of a
// residual block with the Add, and the Relu, after it): kernels of their own because the addends of a tile are all
// requested at once, which takes registers the plain kernels keep for occupancy.
#include "igemm_kernel.hpp"

namespace onhip {

int igemm_launch_f32_res(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    switch (cfg.bl) {
        case BL_GATHER: return launch_tile<DT_F32, BL_GATHER, 1, true>(cfg, p, stream);
        case BL_PLAIN: return launch_tile<DT_F32, BL_PLAIN, 1, true>(cfg, p, stream);
        case BL_TAPC: return launch_tile<DT_F32, BL_TAPC, 1, true>(cfg, p, stream);
        default: return set_error(ONHIP_ERR_ARG, "igemm f32: unsupported loader %d", cfg.bl);
    }
}

}  // namespace onhip
