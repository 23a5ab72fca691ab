// Layout and type conversions of the 16-bit storage path (bf16 / fp16 operands, NHWC activations with the channel count
// padded to a pitch of 32 channels, tap-major weights): what a caller runs once per weight tensor and at the two ends
// of a chain of layers that stays in 16 bits.  Rounding is to nearest even, the conversion the hardware does
// (v_cvt_pk_bf16_f32, v_cvt_pkrtz is not used).  All of them are bound by memory traffic.
#include "igemm_kernel.hpp"

namespace onhip {

// ---- fp32 weights -> [rows][taps][cp] 16-bit, channels zero-padded to cp -------------------------------------------
// the source element of (row, tap, channel) is w[row * s_row + channel * s_ch + tap * s_tap]: OIHW convolution weights
// (s_row = cin * taps, s_ch = taps, s_tap = 1) or the right operand [K][N] of a MatMul (row = column n: s_row = 1,
// s_ch = N, one tap)
template <int DT>
__global__ __launch_bounds__(256) void pack_w16_kernel(const float *w, int cin, int taps, int cp, long long s_row, long long s_ch,
                                                       long long s_tap, unsigned short *packed, long long total_pairs) {
    const long long idx = (long long) blockIdx.x * blockDim.x + threadIdx.x;   // one pair of channels per thread
    if (idx >= total_pairs) return;
    const int half_cp = cp / 2;
    const int c = (int) (idx % half_cp) * 2;
    const long long t = idx / half_cp;
    const int tap = (int) (t % taps);
    const long long row = t / taps;
    const float lo = c < cin ? w[row * s_row + c * s_ch + tap * s_tap] : 0.0f;
    const float hi = c + 1 < cin ? w[row * s_row + (c + 1) * s_ch + tap * s_tap] : 0.0f;
    reinterpret_cast<unsigned *>(packed)[idx] = pack_h16<DT>(lo, hi);
}

int pack_w16_launch(int dt, const float *w, long long rows, int cin, int taps, int cp, long long s_row, long long s_ch,
                    long long s_tap, void *packed, hipStream_t stream) {
    const long long total = rows * taps * (cp / 2);
    const unsigned blocks = (unsigned) ((total + 255) / 256);
    unsigned short *out = reinterpret_cast<unsigned short *>(packed);
    if (dt == DT_BF16) hipLaunchKernelGGL(pack_w16_kernel<DT_BF16>, dim3(blocks), dim3(256), 0, stream, w, cin, taps, cp, s_row, s_ch, s_tap, out, total);
    else hipLaunchKernelGGL(pack_w16_kernel<DT_F16>, dim3(blocks), dim3(256), 0, stream, w, cin, taps, cp, s_row, s_ch, s_tap, out, total);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// ---- fp32 NCHW -> 16-bit NHWC (pitch cp, a multiple of 8) -------------------------------------------------------------
// One thread converts the 8 channels of one 16-byte block of one pixel.  A wavefront covers 4 neighbouring channel
// blocks of 16 consecutive pixels: stores are runs of 64 contiguous bytes per pixel, each of the 8 loads reads runs of
// 16 consecutive pixels of a channel plane.  Grid: (pixel blocks, groups of 4 channel blocks, images).
template <int DT>
__global__ __launch_bounds__(256) void nchw_to_nhwc16_kernel(const float *x, int c, int hw, int cp, unsigned short *y) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pix = (blockIdx.x * 4 + wave) * 16 + lane / 4;
    const int cb = blockIdx.y * 4 + lane % 4;
    if (pix >= hw || cb * 8 >= cp) return;
    const long long img = blockIdx.z;
    const float *src = x + (img * c + (long long) cb * 8) * hw + pix;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = cb * 8 + e < c ? src[(long long) e * hw] : 0.0f;
    *reinterpret_cast<uint4 *>(y + (img * hw + pix) * (long long) cp + cb * 8) =
        make_uint4(pack_h16<DT>(v[0], v[1]), pack_h16<DT>(v[2], v[3]), pack_h16<DT>(v[4], v[5]), pack_h16<DT>(v[6], v[7]));
}

int nchw_to_nhwc16_launch(int dt, const float *x, int n, int c, int h, int w, int cp, void *y, hipStream_t stream) {
    const int hw = h * w;
    if (n > 65535) return set_error(ONHIP_ERR_ARG, "16-bit conversion: batch of %d", n);
    const dim3 grid((hw + 63) / 64, (cp / 8 + 3) / 4, n);
    unsigned short *out = reinterpret_cast<unsigned short *>(y);
    if (dt == DT_BF16) hipLaunchKernelGGL(nchw_to_nhwc16_kernel<DT_BF16>, grid, dim3(256), 0, stream, x, c, hw, cp, out);
    else hipLaunchKernelGGL(nchw_to_nhwc16_kernel<DT_F16>, grid, dim3(256), 0, stream, x, c, hw, cp, out);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// ---- first layers: fp32 NCHW (at most 8 channels) -> 16-bit [n][h][wp][cpp], cpp = 4 or 8 channels per pixel ----------
// Stored column s holds image column s - pad_l (zeros outside the image, zeros in the channels past c), so that the 8
// stored pixels from column ow * stride_w on are the whole receptive-field row of output column ow: 16 cpp contiguous
// bytes.  One thread per stored pixel; the loads of a wavefront are runs of 64 pixels of a channel plane.
template <int DT, int CPP>
__global__ __launch_bounds__(256) void first_from_nchw_kernel(const float *x, int c, int h, int w, int wp, int pad_l, unsigned short *y) {
    const int s = blockIdx.x * 256 + threadIdx.x, row = blockIdx.y;
    const long long img = blockIdx.z;
    if (s >= wp) return;
    const int col = s - pad_l;
    float v[CPP];
#pragma unroll
    for (int e = 0; e < CPP; ++e) v[e] = e < c && col >= 0 && col < w ? x[((img * c + e) * h + row) * (long long) w + col] : 0.0f;
    unsigned short *dst = y + ((img * h + row) * (long long) wp + s) * CPP;
    if constexpr (CPP == 8)
        *reinterpret_cast<uint4 *>(dst) = make_uint4(pack_h16<DT>(v[0], v[1]), pack_h16<DT>(v[2], v[3]), pack_h16<DT>(v[4], v[5]), pack_h16<DT>(v[6], v[7]));
    else
        *reinterpret_cast<uint2 *>(dst) = make_uint2(pack_h16<DT>(v[0], v[1]), pack_h16<DT>(v[2], v[3]));
}

int first_from_nchw_launch(int dt, const float *x, int n, int c, int h, int w, int wp, int cpp, int pad_l, void *y, hipStream_t stream) {
    if (n > 65535 || h > 65535) return set_error(ONHIP_ERR_ARG, "16-bit first layer: %d images of %d rows", n, h);
    const dim3 grid((wp + 255) / 256, h, n);
    unsigned short *out = reinterpret_cast<unsigned short *>(y);
    if (dt == DT_BF16 && cpp == 8) hipLaunchKernelGGL((first_from_nchw_kernel<DT_BF16, 8>), grid, dim3(256), 0, stream, x, c, h, w, wp, pad_l, out);
    else if (dt == DT_BF16) hipLaunchKernelGGL((first_from_nchw_kernel<DT_BF16, 4>), grid, dim3(256), 0, stream, x, c, h, w, wp, pad_l, out);
    else if (cpp == 8) hipLaunchKernelGGL((first_from_nchw_kernel<DT_F16, 8>), grid, dim3(256), 0, stream, x, c, h, w, wp, pad_l, out);
    else hipLaunchKernelGGL((first_from_nchw_kernel<DT_F16, 4>), grid, dim3(256), 0, stream, x, c, h, w, wp, pad_l, out);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// fp32 OIHW weights -> [cout][kh][8 columns][cpp channels] 16-bit: filter row i of an output channel as the bytes that
// meet a receptive-field row of the layout above (columns past kw and channels past cin are zeros)
template <int DT, int CPP>
__global__ __launch_bounds__(256) void first_pack_w16_kernel(const float *w, int cin, int kh, int kw, unsigned short *packed, int total) {
    const int idx = blockIdx.x * 256 + threadIdx.x;   // one (row, filter row, column) per thread
    if (idx >= total) return;
    const int j = idx % 8, i = (idx / 8) % kh, row = idx / (8 * kh);
    float v[CPP];
#pragma unroll
    for (int e = 0; e < CPP; ++e) v[e] = e < cin && j < kw ? w[((long long) (row * cin + e) * kh + i) * kw + j] : 0.0f;
    unsigned short *dst = packed + (long long) idx * CPP;
    if constexpr (CPP == 8)
        *reinterpret_cast<uint4 *>(dst) = make_uint4(pack_h16<DT>(v[0], v[1]), pack_h16<DT>(v[2], v[3]), pack_h16<DT>(v[4], v[5]), pack_h16<DT>(v[6], v[7]));
    else
        *reinterpret_cast<uint2 *>(dst) = make_uint2(pack_h16<DT>(v[0], v[1]), pack_h16<DT>(v[2], v[3]));
}

int first_pack_w16_launch(int dt, const float *w, int cout, int cin, int kh, int kw, int cpp, void *packed, hipStream_t stream) {
    const int total = cout * kh * 8;
    const dim3 grid((total + 255) / 256);
    unsigned short *out = reinterpret_cast<unsigned short *>(packed);
    if (dt == DT_BF16 && cpp == 8) hipLaunchKernelGGL((first_pack_w16_kernel<DT_BF16, 8>), grid, dim3(256), 0, stream, w, cin, kh, kw, out, total);
    else if (dt == DT_BF16) hipLaunchKernelGGL((first_pack_w16_kernel<DT_BF16, 4>), grid, dim3(256), 0, stream, w, cin, kh, kw, out, total);
    else if (cpp == 8) hipLaunchKernelGGL((first_pack_w16_kernel<DT_F16, 8>), grid, dim3(256), 0, stream, w, cin, kh, kw, out, total);
    else hipLaunchKernelGGL((first_pack_w16_kernel<DT_F16, 4>), grid, dim3(256), 0, stream, w, cin, kh, kw, out, total);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// ---- 16-bit NHWC (pitch cp) -> fp32 NCHW ---------------------------------------------------------------------------
// The mirror image: a thread reads one 16-byte block and writes its 8 channels to 8 planes; the 16 lanes that share a
// channel block write 16 consecutive floats of a plane.
template <int DT>
__global__ __launch_bounds__(256) void nhwc16_to_nchw_kernel(const unsigned short *x, int c, int hw, int cp, float *y) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pix = (blockIdx.x * 4 + wave) * 16 + lane % 16;
    const int cb = blockIdx.y * 4 + lane / 16;
    if (pix >= hw || cb * 8 >= c) return;
    const long long img = blockIdx.z;
    const uint4 q = *reinterpret_cast<const uint4 *>(x + (img * hw + pix) * (long long) cp + cb * 8);
    const unsigned wds[4] = {q.x, q.y, q.z, q.w};
    float *dst = y + (img * c + (long long) cb * 8) * hw + pix;
#pragma unroll
    for (int e = 0; e < 8; ++e)
        if (cb * 8 + e < c) dst[(long long) e * hw] = unpack_h16<DT>(wds[e / 2], e & 1);
}

int nhwc16_to_nchw_launch(int dt, const void *x, int n, int c, int h, int w, int cp, float *y, hipStream_t stream) {
    const int hw = h * w;
    if (n > 65535) return set_error(ONHIP_ERR_ARG, "16-bit conversion: batch of %d", n);
    const dim3 grid((hw + 63) / 64, ((c + 7) / 8 + 3) / 4, n);
    const unsigned short *in = reinterpret_cast<const unsigned short *>(x);
    if (dt == DT_BF16) hipLaunchKernelGGL(nhwc16_to_nchw_kernel<DT_BF16>, grid, dim3(256), 0, stream, in, c, hw, cp, y);
    else hipLaunchKernelGGL(nhwc16_to_nchw_kernel<DT_F16>, grid, dim3(256), 0, stream, in, c, hw, cp, y);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// ---- rows of a matrix: fp32 [rows][k] <-> 16-bit [rows][kp] ----------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void rows_to_h16_kernel(const float *x, int k, int kp, unsigned short *y, long long total_pairs) {
    const long long idx = (long long) blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total_pairs) return;
    const int half = kp / 2;
    const int c = (int) (idx % half) * 2;
    const long long row = idx / half;
    const float lo = c < k ? x[row * k + c] : 0.0f, hi = c + 1 < k ? x[row * k + c + 1] : 0.0f;
    reinterpret_cast<unsigned *>(y)[idx] = pack_h16<DT>(lo, hi);
}

template <int DT>
__global__ __launch_bounds__(256) void rows_from_h16_kernel(const unsigned short *x, int k, int kp, float *y, long long total) {
    const long long idx = (long long) blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int c = (int) (idx % k);
    const long long row = idx / k;
    const unsigned short h = x[row * kp + c];
    y[idx] = unpack_h16<DT>((unsigned) h, 0);
}

int rows_to_h16_launch(int dt, const float *x, long long rows, int k, int kp, void *y, hipStream_t stream) {
    const long long total = rows * (kp / 2);
    const unsigned blocks = (unsigned) ((total + 255) / 256);
    unsigned short *out = reinterpret_cast<unsigned short *>(y);
    if (dt == DT_BF16) hipLaunchKernelGGL(rows_to_h16_kernel<DT_BF16>, dim3(blocks), dim3(256), 0, stream, x, k, kp, out, total);
    else hipLaunchKernelGGL(rows_to_h16_kernel<DT_F16>, dim3(blocks), dim3(256), 0, stream, x, k, kp, out, total);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int rows_from_h16_launch(int dt, const void *x, long long rows, int k, int kp, float *y, hipStream_t stream) {
    const long long total = rows * k;
    const unsigned blocks = (unsigned) ((total + 255) / 256);
    const unsigned short *in = reinterpret_cast<const unsigned short *>(x);
    if (dt == DT_BF16) hipLaunchKernelGGL(rows_from_h16_kernel<DT_BF16>, dim3(blocks), dim3(256), 0, stream, in, k, kp, y, total);
    else hipLaunchKernelGGL(rows_from_h16_kernel<DT_F16>, dim3(blocks), dim3(256), 0, stream, in, k, kp, y, total);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

}  // namespace onhip
