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
constexpr int DW_LDS_FLOATS = 8192;   // at most 32 KiB of LDS per workgroup (five per CU); the launch asks for what the chunk needs
constexpr int DW_RT = 4;              // 3x3 specialisation: output rows per thread

struct DwParams {
    int C, H, W, OH, OW, kh, kw, sh, sw, pt, pl;
    int planes;          // batch * C
    int planes_per_wg;   // >= 1 when whole planes fit in LDS, else 0
    int band_rows;       // output rows per workgroup when a plane is split into bands
    int bands;           // bands per plane (1 when planes_per_wg >= 1)
    int pitch;           // LDS row pitch: the padded columns the windows reach, and at least left padding + W
    int tile_rows;       // whole planes: tile rows per plane (the rows the windows reach, at least top padding + H)
    int flat_stage;      // small whole planes: stage by flat index
    int lds_floats;      // LDS cells of one workgroup's chunk (a multiple of 4)
    unsigned magic_hw, magic_w;   // floor(2^32 / d) + 1 for d = H*W and d = W (d >= 2)
    Div31 div_ow, div_c;          // exact division by OW and by C
    Div31 div_unit;               // whole-plane mode: by the work units (strips or outputs) of one plane
    float in_scale, inv_in_scale, out_inv_scale;
    int out_s8;
};

__device__ __forceinline__ int dw_div(int x, const Div31 &d) {
    return (int) ((__umulhi((unsigned) x, d.magic) >> d.shift) + ((unsigned) x & d.pass));
}

// The LDS tile holds, for each plane of the chunk, every input row and column the chunk's outputs
// touch, padding included and zero-filled, so the compute phase reads it without predicates:
// tile row = ih - (oh0 * sh - pt), tile column = iw + pl.
//
// S3 > 0: 3x3 filter with stride S3, fully unrolled: a thread computes DW_RT vertically adjacent
// outputs from a (DW_RT - 1) * S3 + 3 by 3 register window.  S3 == 0: any filter, one output at a time.
template <bool INT8, int S3, int EPI>
__global__ __launch_bounds__(DW_THREADS) void depthwise_tiled_kernel(DwParams p, const float *__restrict__ x,
                                                                     const void *__restrict__ wv,
                                                                     const void *__restrict__ bv,
                                                                     const float *__restrict__ weight_aux, Epilogue ep,
                                                                     void *__restrict__ y, int32_t *__restrict__ acc32) {
    // sized by the launch to the chunk (at most DW_LDS_FLOATS): a small chunk leaves LDS for more resident workgroups,
    // which is what hides the stage -> compute dependency of each one
    extern __shared__ __align__(16) float tile[];
    const int tid = threadIdx.x;
    int plane0, nplanes, oh0, oh1;
    if (p.planes_per_wg >= 1) {
        plane0 = blockIdx.x * p.planes_per_wg;
        nplanes = min(p.planes_per_wg, p.planes - plane0);
        oh0 = 0; oh1 = p.OH;
    } else {
        plane0 = blockIdx.x / p.bands;
        nplanes = 1;
        const int band = blockIdx.x - plane0 * p.bands;
        oh0 = band * p.band_rows;
        oh1 = min(p.OH, oh0 + p.band_rows);
    }
    const int ih_first = oh0 * p.sh - p.pt;                      // input row of tile row 0 (may be negative)
    // tile rows per plane: what the band's windows reach, or (whole planes) at least every row of the image, so that
    // the flat copy below has a cell for each input even where a stride above 1 leaves the last rows unread
    const int trows = p.planes_per_wg >= 1 ? p.tile_rows : (oh1 - 1 - oh0) * p.sh + p.kh;
    const int pitch = p.pitch;
    const int plane_cells = trows * pitch;
    // ---- stage -----------------------------------------------------------------------------------------
    // 1. clear the cells of the chunk (padding stays zero), 2. copy the rows that exist: a thread keeps its
    // group of four columns and walks down the rows, 128-bit loads when rows are 16-byte aligned.
    {
        const int cells = nplanes * plane_cells;
        float4 *t4 = reinterpret_cast<float4 *>(tile);
        for (int i = tid; i < (cells + 3) / 4; i += DW_THREADS) t4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        __syncthreads();
        if (p.flat_stage) {
            // small planes: the chunk is one contiguous run of nplanes * H * W inputs; walk it flat and scatter
            // into the padded tile (flat index -> plane, row, column by multiply-high division)
            const int hw = p.H * p.W;
            const int total = nplanes * hw;
            const float *src = x + (long long) plane0 * hw;
            for (int i = tid; i < total; i += DW_THREADS) {
                const int pl = (int) __umulhi((unsigned) i, p.magic_hw);
                const int rem = i - pl * hw;
                const int r = (int) __umulhi((unsigned) rem, p.magic_w);
                const int c = rem - r * p.W;
                const float v = src[i];
                tile[pl * plane_cells + (r - ih_first) * pitch + c + p.pl] = INT8 ? (float) quant_s8(v, p.inv_in_scale) : v;
            }
            __syncthreads();
        } else {
        const int r_lo = max(0, -ih_first);                       // first tile row that exists in the image
        const int r_hi = min(trows, p.H - ih_first);              // one past the last
        const bool vec = (p.W & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
        const int groups = vec ? p.W / 4 : p.W;                   // column groups per row
        const int gpp = groups < DW_THREADS ? groups : DW_THREADS;  // groups handled per pass
        const int rows_per_pass = DW_THREADS / gpp;
        const int ry = tid / gpp, gx = tid - ry * gpp;
        if (ry < rows_per_pass) {
            for (int pl = 0; pl < nplanes; ++pl) {
                const float *src = x + ((long long) (plane0 + pl) * p.H + ih_first) * p.W;   // tile row 0 of this plane
                float *dst = tile + pl * plane_cells + p.pl;
                for (int g = gx; g < groups; g += gpp) {
                    for (int tr = r_lo + ry; tr < r_hi; tr += rows_per_pass) {
                        if (vec) {
                            float4 v = *reinterpret_cast<const float4 *>(src + tr * p.W + 4 * g);
                            if (INT8) { v.x = (float) quant_s8(v.x, p.inv_in_scale); v.y = (float) quant_s8(v.y, p.inv_in_scale);
                                        v.z = (float) quant_s8(v.z, p.inv_in_scale); v.w = (float) quant_s8(v.w, p.inv_in_scale); }
                            float *o = dst + tr * pitch + 4 * g;
                            o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
                        } else {
                            const float v = src[tr * p.W + g];
                            dst[tr * pitch + g] = INT8 ? (float) quant_s8(v, p.inv_in_scale) : v;
                        }
                    }
                }
            }
        }
        __syncthreads();
        }
    }
    // ---- compute --------------------------------------------------------------------------------------
    const int out_rows = oh1 - oh0;
    const int khkw = p.kh * p.kw;
    if constexpr (S3 > 0) {
        constexpr int WR = (DW_RT - 1) * S3 + 3;                  // window rows
        const int nsr = (out_rows + DW_RT - 1) / DW_RT;
        const int strips_per_plane = nsr * p.OW;
        const int strips = nplanes * strips_per_plane;
        for (int sidx = tid; sidx < strips; sidx += DW_THREADS) {
            // a band has one plane; whole planes have the host's divisor (no integer division in the loop)
            const int pl = p.planes_per_wg >= 1 ? dw_div(sidx, p.div_unit) : 0;
            const int rem = sidx - pl * strips_per_plane;
            const int sr = dw_div(rem, p.div_ow);
            const int ow = rem - sr * p.OW;
            const int plane = plane0 + pl;
            const int c = plane - dw_div(plane, p.div_c) * p.C;
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
            const int r0 = sr * DW_RT;                             // first output row of the strip, band-relative
            const float *tp = tile + pl * plane_cells + ow * S3;
            float win[WR][3];
#pragma unroll
            for (int r = 0; r < WR; ++r) {
                // rows past the end of the band belong to outputs that are not stored: stay inside the tile
                const int tr = min(r0 * S3 + r, trows - 1);
#pragma unroll
                for (int j = 0; j < 3; ++j) win[r][j] = tp[tr * pitch + j];
            }
            const long long obase = ((long long) plane * p.OH + oh0 + r0) * p.OW + ow;
            float *yf = reinterpret_cast<float *>(y) + obase;
            int8_t *y8 = reinterpret_cast<int8_t *>(y) + obase;
            int32_t *ya = acc32 ? acc32 + obase : nullptr;
#pragma unroll
            for (int q = 0; q < DW_RT; ++q) {
                if (r0 + q >= out_rows) break;
                const int oidx = q * p.OW;
                float v;
                if (INT8) {
                    int acc = 0;
#pragma unroll
                    for (int i = 0; i < 3; ++i)
#pragma unroll
                        for (int j = 0; j < 3; ++j) acc += (int) wreg[i * 3 + j] * (int) win[q * S3 + i][j];
                    if (ya) ya[oidx] = acc;
                    // conv.c:739 and :746-752: acc * s + bias32, then * (aux / 127): separately rounded
                    const float f = __fadd_rn(__fmul_rn((float) acc, p.in_scale), bias_f);
                    v = act_fast<EPI>(__fmul_rn(f, coeff), ep);
                } else {
                    float acc = 0.0f;
#pragma unroll
                    for (int i = 0; i < 3; ++i)
#pragma unroll
                        for (int j = 0; j < 3; ++j) acc = __fadd_rn(acc, __fmul_rn(wreg[i * 3 + j], win[q * S3 + i][j]));
                    v = act_fast<EPI>(__fadd_rn(acc, bias_f), ep);
                }
                if (INT8 && p.out_s8) y8[oidx] = (int8_t) quant_s8(v, p.out_inv_scale);
                else yf[oidx] = v;
            }
        }
        return;
    }
    const int per_plane = out_rows * p.OW;
    const int total_out = nplanes * per_plane;
    for (int o = tid; o < total_out; o += DW_THREADS) {
        const int pl = p.planes_per_wg >= 1 ? dw_div(o, p.div_unit) : 0;
        const int rem = o - pl * per_plane;
        const int r = dw_div(rem, p.div_ow);
        const int ow = rem - r * p.OW;
        const int plane = plane0 + pl;
        const int c = plane - dw_div(plane, p.div_c) * p.C;
        const float *tp = tile + pl * plane_cells + (r * p.sh) * pitch + ow * p.sw;
        const long long oidx = ((long long) plane * p.OH + oh0 + r) * p.OW + ow;
        float v;
        if (INT8) {
            const int8_t *wc = reinterpret_cast<const int8_t *>(wv) + (long long) c * khkw;
            int acc = 0;
            for (int i = 0; i < p.kh; ++i)
                for (int j = 0; j < p.kw; ++j) acc += (int) wc[i * p.kw + j] * (int) tp[i * pitch + j];
            if (acc32) acc32[oidx] = acc;
            const float f = __fadd_rn(__fmul_rn((float) acc, p.in_scale), (float) reinterpret_cast<const int32_t *>(bv)[c]);
            v = act_fast<EPI>(__fmul_rn(f, __fdiv_rn(weight_aux[c], 127.0f)), ep);
        } else {
            const float *wc = reinterpret_cast<const float *>(wv) + (long long) c * khkw;
            float acc = 0.0f;
            for (int i = 0; i < p.kh; ++i)
                for (int j = 0; j < p.kw; ++j) acc = __fadd_rn(acc, __fmul_rn(wc[i * p.kw + j], tp[i * pitch + j]));
            v = act_fast<EPI>(__fadd_rn(acc, reinterpret_cast<const float *>(bv)[c]), ep);
        }
        if (INT8 && p.out_s8) reinterpret_cast<int8_t *>(y)[oidx] = (int8_t) quant_s8(v, p.out_inv_scale);
        else reinterpret_cast<float *>(y)[oidx] = v;
    }
}

// 3x3 with equal strides 1 or 2 takes the unrolled kernel
static int dw_specialisation(const onhip_conv_desc_t &d) {
    if (d.kh == 3 && d.kw == 3 && d.stride_h == d.stride_w && (d.stride_h == 1 || d.stride_h == 2)) return d.stride_h;
    return 0;
}

static int dw_specialisation(const onhip_conv_desc_t &d);

static int dw_plan(const onhip_conv_desc_t &d, int OH, int OW, DwParams *p) {
    p->C = d.cout; p->H = d.h; p->W = d.w; p->OH = OH; p->OW = OW;
    p->div_ow = make_div31((unsigned) OW);
    p->div_c = make_div31((unsigned) d.cout);
    // work units of one whole plane: strips of DW_RT rows in the 3x3 kernels, single outputs otherwise
    p->div_unit = make_div31((unsigned) (dw_specialisation(d) ? ((OH + DW_RT - 1) / DW_RT) * OW : OH * OW));
    p->kh = d.kh; p->kw = d.kw; p->sh = d.stride_h; p->sw = d.stride_w; p->pt = d.pad_t; p->pl = d.pad_l;
    p->planes = d.n * d.cout;
    // columns 0 .. (OW-1)*sw + kw - 1 of the padded row are read; the copy into the tile writes every column of the
    // image, so the pitch also covers those a stride above 1 leaves unread at the right edge (same for the rows of a
    // whole plane)
    const int reach_w = (OW - 1) * d.stride_w + d.kw, reach_h = (OH - 1) * d.stride_h + d.kh;
    p->pitch = reach_w > d.w + d.pad_l ? reach_w : d.w + d.pad_l;
    const int full_rows = reach_h > d.h + d.pad_t ? reach_h : d.h + d.pad_t;
    p->tile_rows = full_rows;
    const int plane_cells = full_rows * p->pitch;
    if (plane_cells <= DW_LDS_FLOATS) {
        // whole planes: as many as fit, but leave enough workgroups to fill 256 CUs several times over
        int ppw = DW_LDS_FLOATS / plane_cells;
        const int want_wgs = 256 * 8;
        const int cap = (p->planes + want_wgs - 1) / want_wgs;
        if (ppw > cap) ppw = cap < 1 ? 1 : cap;
        p->planes_per_wg = ppw;
        p->bands = 1;
        p->band_rows = OH;
        // rows shorter than a wavefront: the row-walking copy would leave most lanes idle
        p->flat_stage = d.w < 32 && d.w >= 2 && d.h * d.w >= 2 && (long long) ppw * d.h * d.w * d.h * d.w < (1LL << 32);
        p->magic_hw = (unsigned) (0x100000000ULL / (unsigned) (d.h * d.w)) + 1u;
        p->magic_w = (unsigned) (0x100000000ULL / (unsigned) d.w) + 1u;
        p->lds_floats = (ppw * plane_cells + 3) / 4 * 4;
        return (p->planes + ppw - 1) / ppw;
    }
    // bands of output rows: (band_rows - 1) * sh + kh tile rows must fit
    const int max_rows = DW_LDS_FLOATS / p->pitch;
    int band = (max_rows - d.kh) / d.stride_h + 1;
    if (max_rows < d.kh || band < 1) return -1;
    if (band > OH) band = OH;
    // equal bands, a multiple of the per-thread strip where possible
    const int nb = (OH + band - 1) / band;
    band = (OH + nb - 1) / nb;
    if (band % DW_RT && (band / DW_RT + 1) * DW_RT <= (max_rows - d.kh) / d.stride_h + 1) band = (band / DW_RT + 1) * DW_RT;
    p->planes_per_wg = 0;
    p->band_rows = band;
    p->bands = (OH + band - 1) / band;
    p->lds_floats = (((band - 1) * d.stride_h + d.kh) * p->pitch + 3) / 4 * 4;
    return p->planes * p->bands;
}

template <bool INT8>
static void dw_dispatch(int s3, int epi, unsigned wgs, hipStream_t stream, const DwParams &p, const float *x, const void *w,
                        const void *b, const float *aux, const Epilogue &ep, void *y, int32_t *acc32) {
#define ONHIP_DW_CASE(S, E)                                                                                             \
    if (s3 == S && epi == E) {                                                                                          \
        hipLaunchKernelGGL((depthwise_tiled_kernel<INT8, S, E>), dim3(wgs), dim3(DW_THREADS), (size_t) p.lds_floats * 4, stream, p, x, w, b, aux, \
                           ep, y, acc32);                                                                               \
        return;                                                                                                         \
    }
#define ONHIP_DW_ROW(S) ONHIP_DW_CASE(S, EPI_NONE) ONHIP_DW_CASE(S, EPI_RELU) ONHIP_DW_CASE(S, EPI_CLIP) ONHIP_DW_CASE(S, EPI_GENERIC)
    ONHIP_DW_ROW(0) ONHIP_DW_ROW(1) ONHIP_DW_ROW(2)
#undef ONHIP_DW_ROW
#undef ONHIP_DW_CASE
}

int depthwise_f32_launch(const onhip_conv_desc_t &d, int OH, int OW, const float *x, const float *w,
                         const float *bias, const Epilogue &ep, float *y, hipStream_t stream) {
    DwParams p;
    memset(&p, 0, sizeof(p));
    const long long wgs = dw_plan(d, OH, OW, &p);
    if (wgs < 1 || wgs > 0x7fffffffLL) return set_error(ONHIP_ERR_ARG, "depthwise: image row of %d elements too wide", d.w);
    dw_dispatch<false>(dw_specialisation(d), epi_of_act(ep.act), (unsigned) wgs, stream, p, x, w, bias, nullptr, ep, y, nullptr);
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
    dw_dispatch<true>(dw_specialisation(d), epi_of_act(ep.act), (unsigned) wgs, stream, p, x, w8, bias32, weight_aux, ep, y,
                      acc32);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

}  // namespace onhip
