// int8 instantiations of the implicit-GEMM kernel whose fp32 store adds a residual operand (the last convolution of a
// residual block of W8A32 convolutions with the Add, and the Relu, after it): kernels of their own, like the fp32 ones,
// because a row tile's addends are all requested at once, which takes registers the plain kernels keep for occupancy.
#include "igemm_kernel.hpp"

namespace onhip {

int igemm_launch_i8_res(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    if (p.out_s8 || p.acc_out) return set_error(ONHIP_ERR_ARG, "igemm i8: the residual store is for fp32 results");
    if (cfg.bl == BL_KVEC_TAP) {
        if (!p.use_tapmask || p.units_per_tap % 4) return set_error(ONHIP_ERR_ARG, "igemm i8: K tiles straddle filter taps");
        return launch_tile<DT_I8, BL_KVEC_TAP, 1, true>(cfg, p, stream);
    }
    if (cfg.bl != BL_KVEC) return set_error(ONHIP_ERR_ARG, "igemm i8: unsupported loader %d", cfg.bl);
    return launch_tile<DT_I8, BL_KVEC, 1, true>(cfg, p, stream);
}

}  // namespace onhip
