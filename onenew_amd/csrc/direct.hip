// Bandwidth-bound kernels where MFMA does not pay: depthwise convolution (fp32 and W8A32), the
// activation quantiser that stages NCHW fp32 as NHWC int8 for the int8 MFMA path, the int8 weight
// re-layout, and the skinny Gemm  out = A * W^T + bias  with a wavefront-shuffle reduction.
#include "onhip_internal.hpp"

namespace onhip {


// ---- fp32 NCHW activations -> int8 NHWC with the channel count padded to cp (a multiple of 16) -------------
// One thread quantises the 16 channels of one 16-byte block of one pixel (conv.c:961-973 per element).  A
// wavefront covers CBW neighbouring channel blocks of 64 / CBW consecutive pixels, so its stores are runs of
// CBW * 16 contiguous bytes per pixel (whole pixels when cp <= 64) and each of its 16 loads reads runs of
// 64 / CBW consecutive pixels of a channel plane.  Grid: (pixel blocks, channel block groups, images).
template <int CBW>
__global__ __launch_bounds__(256) void quantize_nhwc_kernel(const float *x, int c, int hw, int cp, float inv_scale,
                                                            int8_t *q) {
    constexpr int PIXW = 64 / CBW;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pix = (blockIdx.x * 4 + wave) * PIXW + lane / CBW;
    const int cb = blockIdx.y * CBW + lane % CBW;
    if (pix >= hw || cb * 16 >= cp) return;
    const long long img = blockIdx.z;
    const float *src = x + (img * c + (long long) cb * 16) * hw + pix;
    float v[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = cb * 16 + e < c ? src[(long long) e * hw] : 0.0f;
    unsigned out[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        unsigned word = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) word |= ((unsigned) quant_s8(v[g * 4 + e], inv_scale) & 0xffu) << (8 * e);
        out[g] = word;
    }
    *reinterpret_cast<uint4 *>(q + (img * hw + pix) * (long long) cp + cb * 16) = make_uint4(out[0], out[1], out[2], out[3]);
}

int quantize_nhwc_launch(const float *x, int n, int c, int h, int w, int cp, float inv_scale, int8_t *q,
                         hipStream_t stream) {
    const int hw = h * w, cblocks = cp / 16;
    if (n > 65535) return set_error(ONHIP_ERR_ARG, "quantize: batch of %d", n);
    const int cbw = cblocks >= 4 ? 4 : cblocks >= 2 ? 2 : 1;
    const dim3 grid((hw + 4 * (64 / cbw) - 1) / (4 * (64 / cbw)), (cblocks + cbw - 1) / cbw, n);
    if (cbw == 4) hipLaunchKernelGGL(quantize_nhwc_kernel<4>, grid, dim3(256), 0, stream, x, c, hw, cp, inv_scale, q);
    else if (cbw == 2) hipLaunchKernelGGL(quantize_nhwc_kernel<2>, grid, dim3(256), 0, stream, x, c, hw, cp, inv_scale, q);
    else hipLaunchKernelGGL(quantize_nhwc_kernel<1>, grid, dim3(256), 0, stream, x, c, hw, cp, inv_scale, q);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// ---- fp32 weights [cout][cin][kh*kw] -> [cout][kh*kw][cp]: tap-major, channels zero-padded to cp -------
__global__ __launch_bounds__(256) void pack_wf32_kernel(const float *w, int cin, int khkw, int cp, float *packed,
                                                        long long total) {
    const long long idx = (long long) blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int c = (int) (idx % cp);
    const long long t = idx / cp;
    const int tap = (int) (t % khkw);
    const long long oc = t / khkw;
    packed[idx] = c < cin ? w[(oc * cin + c) * khkw + tap] : 0.0f;
}

int pack_wf32_launch(const float *w, int cout, int cin, int khkw, int cp, float *packed, hipStream_t stream) {
    const long long total = (long long) cout * khkw * cp;
    const long long blocks = (total + 255) / 256;
    hipLaunchKernelGGL(pack_wf32_kernel, dim3((unsigned) blocks), dim3(256), 0, stream, w, cin, khkw, cp, packed, total);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// ---- fp32 1x1 weights [m2][cmid] (cmid <= 64) -> the A operand order of igemm_kernel's second product ---------------
// [block of 64 rows][half of 32 rows][step s < 8][lane (lh, li)][4 floats]: lane (li, lh) of half wm holds columns
// 4 (2 s + lh) .. + 3 of row block * 64 + wm * 32 + li; zeros beyond m2 rows and cmid columns
__global__ __launch_bounds__(256) void pack_pw2_kernel(const float *w, int m2, int cmid, float4 *packed, long long total) {
    const long long idx = (long long) blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int lane = (int) (idx % 64), s = (int) ((idx / 64) % 8);
    const int half = (int) (idx / 512);
    const int row = half * 32 + lane % 32, col = 4 * (2 * s + lane / 32);
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = (row < m2 && col + j < cmid) ? w[(long long) row * cmid + col + j] : 0.0f;
    packed[idx] = make_float4(v[0], v[1], v[2], v[3]);
}

int pack_pw2_launch(const float *w, int m2, int cmid, float *packed, hipStream_t stream) {
    const long long total = (long long) ((m2 + 63) / 64) * 2 * 8 * 64;
    hipLaunchKernelGGL(pack_pw2_kernel, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, stream, w, m2, cmid,
                       reinterpret_cast<float4 *>(packed), total);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// ---- int8 weights [cout][cin][kh][kw] -> [cout][k_units * 16], k = (tap * cp + channel), zero padded ---
__global__ __launch_bounds__(256) void pack_w8_kernel(const int8_t *w8, int cin, int khkw, int cp, int row_bytes,
                                                      int8_t *packed, long long total) {
    const long long idx = (long long) blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int kq = (int) (idx % row_bytes);
    const long long oc = idx / row_bytes;
    const int tap = kq / cp, ch = kq % cp;
    int8_t v = 0;
    if (tap < khkw && ch < cin) v = w8[(oc * cin + ch) * khkw + tap];
    packed[idx] = v;
}

int pack_w8_launch(const int8_t *w8, int cout, int cin, int kh, int kw, int cp, int k_units, int8_t *packed,
                   hipStream_t stream) {
    const long long total = (long long) cout * k_units * 16;
    const long long blocks = (total + 255) / 256;
    hipLaunchKernelGGL(pack_w8_kernel, dim3((unsigned) blocks), dim3(256), 0, stream, w8, cin, kh * kw, cp,
                       k_units * 16, packed, total);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// ---- the activation table through the output quantiser --------------------------------------------------
// qlut[i] = quantiser(lut[i]): what the int8 store of a table activation would compute per element, once per table
// entry.  requant_s8(0) is 0, so the table's "below -8" rule needs no entry of its own.
__global__ __launch_bounds__(256) void build_qlut_kernel(const float *__restrict__ lut, float out_inv_scale,
                                                         signed char *__restrict__ qlut) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < 8192) qlut[i] = (signed char) quant_s8(lut[i], out_inv_scale);
}

int build_qlut_launch(const float *lut, float out_inv_scale, signed char *qlut, hipStream_t stream) {
    hipLaunchKernelGGL(build_qlut_kernel, dim3(32), dim3(256), 0, stream, lut, out_inv_scale, qlut);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

// ---- skinny Gemm: out[m][n] = sum_k a[m][k] * w[n][k] + bias[n]  (device/x86/Gemm/gemm.c:9-79) ---------
// One wavefront per output column n; lanes stride over k, eight rows of A at a time share each
// weight load; butterfly reduction over the 64 lanes; the bias is added last.
constexpr int GEMM_ROWS = 8;
__global__ __launch_bounds__(256) void gemm_nt_kernel(int M, int K, int N, const float *a, const float *w,
                                                      const float *bias, float *out, int vec) {
    const int lane = threadIdx.x & 63;
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    const float *wr = w + (long long) n * K;
    for (int m0 = 0; m0 < M; m0 += GEMM_ROWS) {
        float acc[GEMM_ROWS];
#pragma unroll
        for (int r = 0; r < GEMM_ROWS; ++r) acc[r] = 0.0f;
        if (vec) {
            for (int k = lane * 4; k < K; k += 256) {
                const float4 wv = *reinterpret_cast<const float4 *>(wr + k);
#pragma unroll
                for (int r = 0; r < GEMM_ROWS; ++r) {
                    if (m0 + r < M) {
                        const float4 av = *reinterpret_cast<const float4 *>(a + (long long) (m0 + r) * K + k);
                        acc[r] = fmaf(av.x, wv.x, fmaf(av.y, wv.y, fmaf(av.z, wv.z, fmaf(av.w, wv.w, acc[r]))));
                    }
                }
            }
        } else {
            for (int k = lane; k < K; k += 64) {
                const float wv = wr[k];
#pragma unroll
                for (int r = 0; r < GEMM_ROWS; ++r)
                    if (m0 + r < M) acc[r] = fmaf(a[(long long) (m0 + r) * K + k], wv, acc[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < GEMM_ROWS; ++r) {
            float v = acc[r];
#pragma unroll
            for (int s = 32; s >= 1; s >>= 1) v += __shfl_xor(v, s, 64);
            if (lane == 0 && m0 + r < M) out[(long long) (m0 + r) * N + n] = __fadd_rn(v, bias[n]);
        }
    }
}

int gemm_nt_launch(int m, int k, int n, const float *a, const float *w, const float *bias, float *out,
                   hipStream_t stream) {
    const int vec = (k % 4 == 0) && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w)) % 16 == 0);
    hipLaunchKernelGGL(gemm_nt_kernel, dim3((n + 3) / 4), dim3(256), 0, stream, m, k, n, a, w, bias, out, vec);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

}  // namespace onhip

namespace onhip {

// ---- plain device copy: the yardstick that HBM traffic counters are scaled by ------------------------
__global__ __launch_bounds__(256) void copy_f32_kernel(const float4 *src, float4 *dst, long long n4) {
    const long long stride = (long long) gridDim.x * blockDim.x;
    for (long long i = (long long) blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) dst[i] = src[i];
}

int copy_f32_launch(const float *src, float *dst, long long n, hipStream_t stream) {
    if (n % 4 || (reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % 16)
        return set_error(ONHIP_ERR_ARG, "copy: element count must be a multiple of 4 and pointers 16-byte aligned");
    hipLaunchKernelGGL(copy_f32_kernel, dim3(256 * 8), dim3(256), 0, stream, reinterpret_cast<const float4 *>(src),
                       reinterpret_cast<float4 *>(dst), n / 4);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

}  // namespace onhip
