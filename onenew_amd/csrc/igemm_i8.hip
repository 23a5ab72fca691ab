// int8 instantiations of the implicit-GEMM kernel (NHWC 16-byte vector loader).
#include "igemm_kernel.hpp"

namespace onhip {

int igemm_launch_i8(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    if (cfg.bl != BL_KVEC) return set_error(ONHIP_ERR_ARG, "igemm i8: unsupported loader %d", cfg.bl);
    return launch_tile<DT_I8, BL_KVEC>(cfg, p, stream);
}

}  // namespace onhip
