// int8 instantiations of the implicit-GEMM kernel (NHWC 16-byte vector loader, with and without per-lane taps).
#include "igemm_kernel.hpp"

namespace onhip {

// One register set of tiles in flight (PF = 1): two and four sets were measured on the YOLOv8s layers and changed
// nothing, the K loop of these kernels is bound by LDS traffic and instruction issue, not by memory latency.
int igemm_launch_i8_res(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream);   // igemm_i8_res.hip

int igemm_launch_i8(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    if (p.res) return igemm_launch_i8_res(cfg, p, stream);
    if (cfg.bl == BL_KVEC_TAP) {
        if (!p.use_tapmask || p.units_per_tap % 4) return set_error(ONHIP_ERR_ARG, "igemm i8: K tiles straddle filter taps");
        return launch_tile<DT_I8, BL_KVEC_TAP>(cfg, p, stream);
    }
    if (cfg.bl != BL_KVEC) return set_error(ONHIP_ERR_ARG, "igemm i8: unsupported loader %d", cfg.bl);
    return launch_tile<DT_I8, BL_KVEC>(cfg, p, stream);
}

}  // namespace onhip
