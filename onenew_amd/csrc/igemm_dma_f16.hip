// f16 instantiations of the direct-to-LDS kernel: operands stored in 16 bits (NHWC activations, tap-major weights),
// fp32 accumulation in v_mfma_f32_32x32x16_f16.
#include "igemm_dma_kernel.hpp"

namespace onhip {
template int dma_launch_dt<DT_F16>(const IgemmLaunch &, const IgemmParams &, hipStream_t);
}
