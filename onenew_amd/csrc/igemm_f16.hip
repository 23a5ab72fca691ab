// f16 instantiations of the implicit-GEMM kernel (element gather and plain 1x1 / matrix loaders).
#include "igemm_kernel.hpp"

namespace onhip {

int igemm_launch_f16(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    switch (cfg.bl) {
        case BL_GATHER: return launch_tile<DT_F16, BL_GATHER>(cfg, p, stream);
        case BL_PLAIN: return launch_tile<DT_F16, BL_PLAIN>(cfg, p, stream);
        case BL_TAPC: return launch_tile<DT_F16, BL_TAPC>(cfg, p, stream);
        default: return set_error(ONHIP_ERR_ARG, "igemm f16: unsupported loader %d", cfg.bl);
    }
}

}  // namespace onhip
