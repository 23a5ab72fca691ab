// f32 instantiations of the implicit-GEMM kernel that multiply the finished tile by a second, 1x1 weight matrix before
// storing it (a convolution with at most 64 output channels followed by a 1x1 convolution, in one launch): the
// tap-major packed loader on the 64 x 64 tile, with and without the residual operand of the second result.
#include "igemm_kernel.hpp"

namespace onhip {

int igemm_launch_f32_pw(const IgemmParams &p_in, hipStream_t stream) {
    constexpr int BM = 64, BN = 64;
    IgemmParams p = p_in;
    if (p.M < 1 || p.M > BM || p.N < 1 || p.k_units < 1 || p.m2 < 1 || !p.w2 || reinterpret_cast<uintptr_t>(p.w2) % 16)
        return set_error(ONHIP_ERR_ARG, "conv + 1x1: %d rows of the first product (1 to 64), %d of the second", p.M, p.m2);
    if (p.partial || p.dp_tiles || p.out_mode != OUT_CONV)
        return set_error(ONHIP_ERR_ARG, "conv + 1x1: whole-K launches of convolutions only");
    if (p.a_slice_bytes >= (1LL << 31) || p.b_slice_bytes + 2 * p.b_shift_bytes >= (1LL << 31) || p.c_slice_bytes >= (1LL << 31) ||
        (long long) p.m2 * 64 * 4 >= (1LL << 30))
        return set_error(ONHIP_ERR_ARG, "conv + 1x1: an operand of 2 GiB or more is not supported");
    const int tiles = (p.N + BN - 1) / BN;
    p.k_split_units = p.k_units;
    p.div_ohw = make_div31((unsigned) (p.OHW > 0 ? p.OHW : 1));
    p.div_ow = make_div31((unsigned) (p.OW > 0 ? p.OW : 1));
    p.div_tiles_m = make_div31(1u);
    p.div_tiles_n = make_div31((unsigned) tiles);
    p.n_fast = 0;
    const dim3 grid(tiles, 1, 1);
    if (p.res)
        hipLaunchKernelGGL((igemm_kernel<DT_F32, BL_TAPC, BM, BN, 2, 2, 1, true, true>), grid, dim3(THREADS), 0, stream, p);
    else
        hipLaunchKernelGGL((igemm_kernel<DT_F32, BL_TAPC, BM, BN, 2, 2, 1, false, true>), grid, dim3(THREADS), 0, stream, p);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

}  // namespace onhip
