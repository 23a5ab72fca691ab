// Dispatch of the implicit-GEMM kernel family: picks the tile and the (element type, B loader)
// variant; the kernels themselves are instantiated per element type in igemm_{f32,bf16,f16,i8}.hip.
#include <stdio.h>
#include <stdlib.h>

#include "onhip_internal.hpp"

namespace onhip {

int igemm_launch_f32(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream);
int igemm_launch_bf16(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream);
int igemm_launch_f16(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream);
int igemm_launch_i8(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream);

int igemm_launch(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    if (p.M < 1 || p.N < 1 || p.k_units < 1 || cfg.batch < 1 || cfg.split < 1)
        return set_error(ONHIP_ERR_ARG, "igemm: empty problem M=%d N=%d units=%d", p.M, p.N, p.k_units);
    if (cfg.batch > 65535 || cfg.split > 65535) return set_error(ONHIP_ERR_ARG, "igemm: grid too large");
    if (cfg.split > 1 && !p.partial) return set_error(ONHIP_ERR_WORKSPACE, "igemm: split-K without workspace");
    // every byte offset a lane or a scalar register carries must stay below 2 GiB
    if (p.a_slice_bytes >= (1LL << 31) || p.b_slice_bytes + 2 * p.b_shift_bytes >= (1LL << 31) ||
        p.c_slice_bytes >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "igemm: an operand slice of 2 GiB or more is not supported");
    if (p.res && cfg.dtype != DT_F32 && cfg.dtype != DT_I8)
        return set_error(ONHIP_ERR_ARG, "igemm: the residual store exists for fp32 and int8 operands");
    if (p.res && cfg.dtype == DT_I8 && cfg.split > 1) return set_error(ONHIP_ERR_ARG, "igemm i8: no split-K with a residual operand");
    switch (cfg.dtype) {
        case DT_F32: return igemm_launch_f32(cfg, p, stream);
        case DT_BF16: return igemm_launch_bf16(cfg, p, stream);
        case DT_F16: return igemm_launch_f16(cfg, p, stream);
        case DT_I8: return igemm_launch_i8(cfg, p, stream);
        default: return set_error(ONHIP_ERR_ARG, "igemm: unsupported element type %d", cfg.dtype);
    }
}

}  // namespace onhip
