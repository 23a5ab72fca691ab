// f32 instantiations of the implicit-GEMM kernel (element gather and plain 1x1 / matrix loaders).
#include "igemm_kernel.hpp"

namespace onhip {

int igemm_launch_f32_res(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream);   // igemm_f32_res.hip

int igemm_launch_f32(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    if (p.res) return igemm_launch_f32_res(cfg, p, stream);
    switch (cfg.bl) {
        case BL_GATHER: return launch_tile<DT_F32, BL_GATHER>(cfg, p, stream);
        case BL_PLAIN: return launch_tile<DT_F32, BL_PLAIN>(cfg, p, stream);
        case BL_TAPC: return launch_tile<DT_F32, BL_TAPC>(cfg, p, stream);
        default: return set_error(ONHIP_ERR_ARG, "igemm f32: unsupported loader %d", cfg.bl);
    }
}

}  // namespace onhip
