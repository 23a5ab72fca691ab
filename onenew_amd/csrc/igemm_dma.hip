// The direct-to-LDS kernel (igemm_dma_kernel.hpp): which problems it takes, the int8 instantiations, and the dispatch
// over operand types (the bf16 and fp16 instantiations are translation units of their own).
#include "igemm_dma_kernel.hpp"

namespace onhip {

bool dma_ok(const IgemmLaunch &cfg, const IgemmParams &p) {
    if (cfg.dtype != DT_I8 && cfg.dtype != DT_BF16 && cfg.dtype != DT_F16) return false;
    if (cfg.batch != 1 || (cfg.bl != BL_KVEC && cfg.bl != BL_KVEC_TAP)) return false;
    if (!p.use_tapmask || p.units_per_tap < 1 || p.k_units != p.khkw * p.units_per_tap) return false;
    if (p.lda != p.k_units * 16 || (p.pix_stride != p.units_per_tap * 16 && !p.tap_spans_pixels)) return false;
    if (reinterpret_cast<uintptr_t>(p.A) % 16 || reinterpret_cast<uintptr_t>(p.B) % 16) return false;
    return dma_stage_bytes(p) != 0 || dma_multi_tap(cfg.dtype, p);
}

bool dma_tile_ok(int bm, int bn) {
    return (bm == 128 && bn == 128) || (bm == 128 && bn == 64) || (bm == 64 && bn == 128) || (bm == 64 && bn == 64);
}

template int dma_launch_dt<DT_I8>(const IgemmLaunch &, const IgemmParams &, hipStream_t);
extern template int dma_launch_dt<DT_BF16>(const IgemmLaunch &, const IgemmParams &, hipStream_t);
extern template int dma_launch_dt<DT_F16>(const IgemmLaunch &, const IgemmParams &, hipStream_t);

int dma_launch(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    if (!dma_ok(cfg, p)) return set_error(ONHIP_ERR_ARG, "igemm: not a problem for the direct-to-LDS kernel");
    switch (cfg.dtype) {
        case DT_I8: return dma_launch_dt<DT_I8>(cfg, p, stream);
        case DT_BF16: return dma_launch_dt<DT_BF16>(cfg, p, stream);
        default: return dma_launch_dt<DT_F16>(cfg, p, stream);
    }
}

}  // namespace onhip
