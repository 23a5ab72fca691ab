// Depthwise convolution (fp32 and W8A32) for gfx950: a bandwidth-bound kernel, so the design is about
// touching every input byte once with fully coalesced loads.
//
// A workgroup owns a chunk of the (image, channel) planes that is contiguous in memory: several
// whole planes when they are small (7x7 ... 28x28), or a band of rows of one large plane.  The 256
// threads copy the chunk into LDS with back-to-back coalesced loads (128-bit when the chunk is
// 16-byte aligned; the W8A32 form quantises on the way in), then every thread computes outputs
// from LDS: lanes run along `ow`, padding is a predicate on the read.  Taps are added in ascending
// (i, j) order to a zero sum with separately rounded multiply and add and the bias last, i.e. the
// arithmetic of device/x86/Conv/conv.c:597-612 and :853-894 (fp32) and :727-752 (W8A32) exactly, so
// results are bit-identical to the reference.
#include <string.h>

#include "onhip_internal.hpp"

namespace onhip {

constexpr int DW_THREADS = 256;
constexpr int DW_LDS_FLOATS = 8192;   // 32 KiB of LDS per workgroup: five workgroups per CU

struct DwParams {
    int C, H, W, OH, OW, kh, kw, sh, sw, pt, pl;
    int planes;          // batch * C
    int planes_per_wg;   // >= 1 when whole planes fit in LDS, else 0
    int band_rows;       // output rows per workgroup when a plane is split into bands
    int bands;           // bands per plane (1 when planes_per_wg >= 1)
    int strip_rows;      // 3x3 specialisation: output rows one thread walks down
    float in_scale, inv_in_scale, out_inv_scale;
    int out_s8;
};

// S3 > 0: 3x3 filter with stride S3, fully unrolled with a register window that slides down the
// column (a new output row costs one new input row of three LDS reads for stride 1, two for stride 2).
// S3 == 0: any filter, one output at a time.
template <bool INT8, int S3>
__global__ __launch_bounds__(DW_THREADS) void depthwise_tiled_kernel(DwParams p, const float *__restrict__ x,
                                                                     const void *__restrict__ wv,
                                                                     const void *__restrict__ bv,
                                                                     const float *__restrict__ weight_aux, Epilogue ep,
                                                                     void *__restrict__ y, int32_t *__restrict__ acc32) {
    __shared__ float tile[DW_LDS_FLOATS];
    const int tid = threadIdx.x;
    int plane0, nplanes, oh0, oh1, ih_lo, ih_hi;
    if (p.planes_per_wg >= 1) {
        plane0 = blockIdx.x * p.planes_per_wg;
        nplanes = min(p.planes_per_wg, p.planes - plane0);
        oh0 = 0; oh1 = p.OH; ih_lo = 0; ih_hi = p.H;
    } else {
        plane0 = blockIdx.x / p.bands;
        nplanes = 1;
        const int band = blockIdx.x - plane0 * p.bands;
        oh0 = band * p.band_rows;
        oh1 = min(p.OH, oh0 + p.band_rows);
        ih_lo = max(0, oh0 * p.sh - p.pt);
        ih_hi = min(p.H, (oh1 - 1) * p.sh - p.pt + p.kh);
    }
    const int rows = ih_hi - ih_lo;                 // input rows held per plane
    const int plane_elems = rows * p.W;
    // ---- stage the contiguous input chunk ---------------------------------------------------------
    if (p.planes_per_wg >= 1) {
        const long long start = (long long) plane0 * p.H * p.W;
        const int total = nplanes * p.H * p.W;
        const float *src = x + start;
        if (((start | total) & 3) == 0) {
            const float4 *s4 = reinterpret_cast<const float4 *>(src);
            for (int i = tid; i < total / 4; i += DW_THREADS) {
                float4 v = s4[i];
                if (INT8) { v.x = (float) quant_s8(v.x, p.inv_in_scale); v.y = (float) quant_s8(v.y, p.inv_in_scale);
                            v.z = (float) quant_s8(v.z, p.inv_in_scale); v.w = (float) quant_s8(v.w, p.inv_in_scale); }
                reinterpret_cast<float4 *>(tile)[i] = v;
            }
        } else {
            for (int i = tid; i < total; i += DW_THREADS) {
                const float v = src[i];
                tile[i] = INT8 ? (float) quant_s8(v, p.inv_in_scale) : v;
            }
        }
    } else {
        const long long start = ((long long) plane0 * p.H + ih_lo) * p.W;
        const float *src = x + start;
        if (((start | plane_elems) & 3) == 0) {
            const float4 *s4 = reinterpret_cast<const float4 *>(src);
            for (int i = tid; i < plane_elems / 4; i += DW_THREADS) {
                float4 v = s4[i];
                if (INT8) { v.x = (float) quant_s8(v.x, p.inv_in_scale); v.y = (float) quant_s8(v.y, p.inv_in_scale);
                            v.z = (float) quant_s8(v.z, p.inv_in_scale); v.w = (float) quant_s8(v.w, p.inv_in_scale); }
                reinterpret_cast<float4 *>(tile)[i] = v;
            }
        } else {
            for (int i = tid; i < plane_elems; i += DW_THREADS) {
                const float v = src[i];
                tile[i] = INT8 ? (float) quant_s8(v, p.inv_in_scale) : v;
            }
        }
    }
    __syncthreads();
    // ---- compute --------------------------------------------------------------------------------------
    const int out_rows = oh1 - oh0;
    const int khkw = p.kh * p.kw;
    if constexpr (S3 > 0) {
        // a thread owns a strip: one output column, p.strip_rows consecutive output rows of one plane
        const int nsr = (out_rows + p.strip_rows - 1) / p.strip_rows;
        const int strips_per_plane = nsr * p.OW;
        const int strips = nplanes * strips_per_plane;
        for (int sidx = tid; sidx < strips; sidx += DW_THREADS) {
            const int pl = sidx / strips_per_plane;
            const int rem = sidx - pl * strips_per_plane;
            const int sr = rem / p.OW;
            const int ow = rem - sr * p.OW;
            const int plane = plane0 + pl;
            const int c = plane % p.C;
            const float *tp = tile + pl * plane_elems;
            float wreg[9];
            float bias_f;
            if (INT8) {
                const int8_t *wc = reinterpret_cast<const int8_t *>(wv) + (long long) c * 9;
#pragma unroll
                for (int t = 0; t < 9; ++t) wreg[t] = (float) wc[t];
                bias_f = (float) reinterpret_cast<const int32_t *>(bv)[c];
            } else {
                const float *wc = reinterpret_cast<const float *>(wv) + (long long) c * 9;
#pragma unroll
                for (int t = 0; t < 9; ++t) wreg[t] = wc[t];
                bias_f = reinterpret_cast<const float *>(bv)[c];
            }
            const float coeff = INT8 ? __fdiv_rn(weight_aux[c], 127.0f) : 0.0f;
            const int iw0 = ow * p.sw - p.pl;
            bool col_ok[3];
#pragma unroll
            for (int j = 0; j < 3; ++j) col_ok[j] = (unsigned) (iw0 + j) < (unsigned) p.W;
            // a tap outside the image multiplies a zero, as the reference's zero padding does
            auto load_row = [&](int ih, float (&row)[3]) {
                const bool rok = (unsigned) ih < (unsigned) p.H;
                const int base = (ih - ih_lo) * p.W + iw0;
#pragma unroll
                for (int j = 0; j < 3; ++j) row[j] = (rok && col_ok[j]) ? tp[base + j] : 0.0f;
            };
            const int r_begin = oh0 + sr * p.strip_rows;
            const int r_end = min(oh1, r_begin + p.strip_rows);
            float win[3][3];
            int ih = r_begin * S3 - p.pt;
            load_row(ih, win[0]);
            load_row(ih + 1, win[1]);
            long long oidx = ((long long) plane * p.OH + r_begin) * p.OW + ow;
            for (int oh = r_begin; oh < r_end; ++oh, oidx += p.OW) {
                load_row(ih + 2, win[2]);
                float v;
                if (INT8) {
                    int acc = 0;
#pragma unroll
                    for (int i = 0; i < 3; ++i)
#pragma unroll
                        for (int j = 0; j < 3; ++j) acc += (int) wreg[i * 3 + j] * (int) win[i][j];
                    if (acc32) acc32[oidx] = acc;
                    // conv.c:739 and :746-752: acc * s + bias32, then * (aux / 127): separately rounded
                    const float f = __fadd_rn(__fmul_rn((float) acc, p.in_scale), bias_f);
                    v = apply_act(__fmul_rn(f, coeff), ep);
                } else {
                    float acc = 0.0f;
#pragma unroll
                    for (int i = 0; i < 3; ++i)
#pragma unroll
                        for (int j = 0; j < 3; ++j) acc = __fadd_rn(acc, __fmul_rn(wreg[i * 3 + j], win[i][j]));
                    v = apply_act(__fadd_rn(acc, bias_f), ep);
                }
                if (INT8 && p.out_s8) reinterpret_cast<int8_t *>(y)[oidx] = (int8_t) quant_s8(v, p.out_inv_scale);
                else reinterpret_cast<float *>(y)[oidx] = v;
                // slide the window down by the stride
                if (S3 == 1) {
#pragma unroll
                    for (int j = 0; j < 3; ++j) { win[0][j] = win[1][j]; win[1][j] = win[2][j]; }
                    ih += 1;
                } else {
#pragma unroll
                    for (int j = 0; j < 3; ++j) win[0][j] = win[2][j];
                    ih += 2;
                    load_row(ih + 1, win[1]);
                }
            }
        }
        return;
    }
    const int per_plane = out_rows * p.OW;
    const int total_out = nplanes * per_plane;
    for (int o = tid; o < total_out; o += DW_THREADS) {
        const int pl = o / per_plane;
        const int rem = o - pl * per_plane;
        const int r = rem / p.OW;
        const int ow = rem - r * p.OW;
        const int oh = oh0 + r;
        const int plane = plane0 + pl;
        const int c = plane % p.C;
        const float *tp = tile + pl * plane_elems;
        const int ihb = oh * p.sh - p.pt, iwb = ow * p.sw - p.pl;
        const long long oidx = ((long long) plane * p.OH + oh) * p.OW + ow;
        if (INT8) {
            const int8_t *wc = reinterpret_cast<const int8_t *>(wv) + (long long) c * khkw;
            int acc = 0;
            for (int i = 0; i < p.kh; ++i) {
                const int ih = ihb + i;
                if ((unsigned) ih >= (unsigned) p.H) continue;
                for (int j = 0; j < p.kw; ++j) {
                    const int iw = iwb + j;
                    if ((unsigned) iw >= (unsigned) p.W) continue;
                    acc += (int) wc[i * p.kw + j] * (int) tp[(ih - ih_lo) * p.W + iw];
                }
            }
            if (acc32) acc32[oidx] = acc;
            // conv.c:739 and :746-752: acc * s + bias32, then * (aux / 127): three separately rounded operations
            float f = __fadd_rn(__fmul_rn((float) acc, p.in_scale), (float) reinterpret_cast<const int32_t *>(bv)[c]);
            const float v = apply_act(__fmul_rn(f, __fdiv_rn(weight_aux[c], 127.0f)), ep);
            if (p.out_s8) reinterpret_cast<int8_t *>(y)[oidx] = (int8_t) quant_s8(v, p.out_inv_scale);
            else reinterpret_cast<float *>(y)[oidx] = v;
        } else {
            const float *wc = reinterpret_cast<const float *>(wv) + (long long) c * khkw;
            float acc = 0.0f;
            for (int i = 0; i < p.kh; ++i) {
                const int ih = ihb + i;
                if ((unsigned) ih >= (unsigned) p.H) continue;
                for (int j = 0; j < p.kw; ++j) {
                    const int iw = iwb + j;
                    if ((unsigned) iw >= (unsigned) p.W) continue;
                    acc = __fadd_rn(acc, __fmul_rn(wc[i * p.kw + j], tp[(ih - ih_lo) * p.W + iw]));
                }
            }
            acc = __fadd_rn(acc, reinterpret_cast<const float *>(bv)[c]);
            reinterpret_cast<float *>(y)[oidx] = apply_act(acc, ep);
        }
    }
}

// 3x3 with equal strides 1 or 2 takes the unrolled kernel
static int dw_specialisation(const onhip_conv_desc_t &d) {
    if (d.kh == 3 && d.kw == 3 && d.stride_h == d.stride_w && (d.stride_h == 1 || d.stride_h == 2)) return d.stride_h;
    return 0;
}

static int dw_plan(const onhip_conv_desc_t &d, int OH, int OW, DwParams *p) {
    p->C = d.cout; p->H = d.h; p->W = d.w; p->OH = OH; p->OW = OW;
    p->kh = d.kh; p->kw = d.kw; p->sh = d.stride_h; p->sw = d.stride_w; p->pt = d.pad_t; p->pl = d.pad_l;
    p->planes = d.n * d.cout;
    const int plane = d.h * d.w;
    if (plane <= DW_LDS_FLOATS) {
        // whole planes; keep at least a few hundred outputs per workgroup but leave enough workgroups for 256 CUs
        int ppw = DW_LDS_FLOATS / plane;
        const int want_wgs = 256 * 8;
        const int cap = (p->planes + want_wgs - 1) / want_wgs;
        if (ppw > cap) ppw = cap < 1 ? 1 : cap;
        while (ppw > 1 && ppw * OH * OW > 4096) --ppw;
        p->planes_per_wg = ppw;
        p->bands = 1;
        p->band_rows = OH;
        // strips of rows per thread: long enough to amortise the set-up, short enough to keep 256 threads busy
        int sr = (ppw * OH * OW) / (2 * DW_THREADS);
        p->strip_rows = sr < 1 ? 1 : sr > 8 ? 8 : sr;
        if (p->strip_rows > OH) p->strip_rows = OH;
        return (p->planes + ppw - 1) / ppw;
    }
    // bands of output rows: (band_rows - 1) * sh + kh input rows must fit
    int max_in_rows = DW_LDS_FLOATS / d.w;
    int band = (max_in_rows - d.kh) / d.stride_h + 1;
    if (band < 1) return -1;
    if (band > OH) band = OH;
    p->planes_per_wg = 0;
    p->band_rows = band;
    p->bands = (OH + band - 1) / band;
    int sr = (band * OW) / (2 * DW_THREADS);
    p->strip_rows = sr < 1 ? 1 : sr > 8 ? 8 : sr;
    return p->planes * p->bands;
}

int depthwise_f32_launch(const onhip_conv_desc_t &d, int OH, int OW, const float *x, const float *w,
                         const float *bias, const Epilogue &ep, float *y, hipStream_t stream) {
    DwParams p;
    memset(&p, 0, sizeof(p));
    const long long wgs = dw_plan(d, OH, OW, &p);
    if (wgs < 1 || wgs > 0x7fffffffLL) return set_error(ONHIP_ERR_ARG, "depthwise: image row of %d elements too wide", d.w);
    const int s3 = dw_specialisation(d);
    if (s3 == 1)
        hipLaunchKernelGGL((depthwise_tiled_kernel<false, 1>), dim3((unsigned) wgs), dim3(DW_THREADS), 0, stream, p, x, w,
                           bias, nullptr, ep, y, nullptr);
    else if (s3 == 2)
        hipLaunchKernelGGL((depthwise_tiled_kernel<false, 2>), dim3((unsigned) wgs), dim3(DW_THREADS), 0, stream, p, x, w,
                           bias, nullptr, ep, y, nullptr);
    else
        hipLaunchKernelGGL((depthwise_tiled_kernel<false, 0>), dim3((unsigned) wgs), dim3(DW_THREADS), 0, stream, p, x, w,
                           bias, nullptr, ep, y, nullptr);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int depthwise_w8a32_launch(const onhip_conv_desc_t &d, int OH, int OW, const float *x, const int8_t *w8,
                           const int32_t *bias32, const float *weight_aux, const Epilogue &ep, void *y,
                           int32_t *acc32, hipStream_t stream) {
    DwParams p;
    memset(&p, 0, sizeof(p));
    const long long wgs = dw_plan(d, OH, OW, &p);
    if (wgs < 1 || wgs > 0x7fffffffLL) return set_error(ONHIP_ERR_ARG, "depthwise: image row of %d elements too wide", d.w);
    p.in_scale = d.input_scale;
    p.inv_in_scale = 1.0f / d.input_scale;
    p.out_s8 = d.out_s8;
    p.out_inv_scale = d.out_s8 ? 1.0f / d.output_scale : 0.0f;
    const int s3 = dw_specialisation(d);
    if (s3 == 1)
        hipLaunchKernelGGL((depthwise_tiled_kernel<true, 1>), dim3((unsigned) wgs), dim3(DW_THREADS), 0, stream, p, x, w8,
                           bias32, weight_aux, ep, y, acc32);
    else if (s3 == 2)
        hipLaunchKernelGGL((depthwise_tiled_kernel<true, 2>), dim3((unsigned) wgs), dim3(DW_THREADS), 0, stream, p, x, w8,
                           bias32, weight_aux, ep, y, acc32);
    else
        hipLaunchKernelGGL((depthwise_tiled_kernel<true, 0>), dim3((unsigned) wgs), dim3(DW_THREADS), 0, stream, p, x, w8,
                           bias32, weight_aux, ep, y, acc32);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

}  // namespace onhip
