// Depthwise convolution of the int8 chain form for gfx950: int8 NHWC activations in (channels padded to 16), int8
// weights [C][1][kh][kw] as the reference holds them, int8 NHWC (or fp32 NCHW) out.  The arithmetic is the reference's
// W8A32 depthwise path, device/x86/Conv/conv.c:617-755: int32 sum of int8 products (:727-739), then
// (float) acc * input_scale + (float) bias32 and the product with weight_aux / 127, each separately rounded (:746-752),
// the activation, and for an int8 result the consumer's own quantiser (:961-973) on that fp32 value.
//
// A depthwise layer has 2 * kh * kw operations per output byte and no reduction over channels, so the matrix cores have
// nothing to do; the kernel is sized by its vector arithmetic and by how its loads meet the cache.
//   * A wavefront works on ONE group of 16 channels (the 16 bytes of a pixel one 128-bit load brings) and its lanes run
//     along output pixels; the four wavefronts of a workgroup take different groups of the same pixels at the same
//     time, so the cache lines of those pixels are fetched once per workgroup.
//   * With the group uniform in the wavefront, the weights are the same for every lane: the workgroup converts the
//     weights of its (up to four) groups to float once into LDS ([group][quad of channels][tap][4]) and a lane reads
//     four of them per 128-bit broadcast read.  Pixels and chunks of four channel groups both spread over the grid, so
//     a 7 x 7 plane with 960 channels still makes hundreds of workgroups.
//   * The products are formed in fp32: v_cvt_f32_ubyte{0..3} turns a byte into a float in one instruction, but only an
//     unsigned one, so the input is biased by 128 (one xor per dword) and the sum starts at -128 * sum(w).  Every
//     product and partial sum is an integer below 2^24, so the fp32 sum equals the int32 sum exactly, in any order.
//   * 3x3 with stride 1 / 2: a lane computes 4 / 2 vertically adjacent outputs from a register window of 6 / 5 input
//     rows, so a loaded pixel feeds up to three outputs.  Padding and the ragged end of the grid are buffer offsets
//     outside the descriptor (the load returns 0, which the bias turns into the integer 0).
#include <string.h>

#include "igemm_kernel.hpp"

namespace onhip {

#ifndef DWS8_R1
#define DWS8_R1 2
#endif

struct DwS8Params {
    int C, Cp, G, N, H, W, OH, OW, kh, kw, taps, sh, sw, pad;
    int strips;            // strips of R output rows per image
    int items;             // N * strips * OW lanes' worth of work per channel group
    int gw;                // wavefronts of a workgroup that take different channel groups (1, 2 or 4)
    int pchunks;           // chunks of 64 * (4 / gw) lanes' items; workgroup id = chunk of channel groups * pchunks + pixel chunk
    Div31 div_ow, div_strips, div_taps, div_pchunks;
    float in_scale, out_inv_scale;
    const int8_t *x;
    const int8_t *w;
    const int32_t *b32;
    const float *aux;
    void *y;
    unsigned x_bytes, y_bytes;
    Epilogue ep;
};

__device__ __forceinline__ int dws8_div(int x, const Div31 &d) {
    return (int) ((__umulhi((unsigned) x, d.magic) >> d.shift) + ((unsigned) x & d.pass));
}

// the four bytes of a dword, biased by 128, as floats
__device__ __forceinline__ void dws8_bytes(unsigned v, float f[4]) {
    v ^= 0x80808080u;
    f[0] = (float) (v & 0xffu);
    f[1] = (float) ((v >> 8) & 0xffu);
    f[2] = (float) ((v >> 16) & 0xffu);
    f[3] = (float) (v >> 24);
}

// S3 > 0: 3x3 filter with stride S3 in both directions; S3 == 0: any filter, one output per lane
template <int S3, int EPI, bool OUT_F32>
__global__ __launch_bounds__(256) void dw_s8_nhwc_kernel(const DwS8Params p) {
    // the weights and per-channel constants of the gw channel groups this workgroup's wavefronts take
    extern __shared__ __align__(16) float lds[];
    float *wl = lds;                              // [gw][4][taps][4]
    float *cst = lds + p.gw * 16 * p.taps;        // [gw][3][16]: -128 * sum of the channel's weights, bias, weight_aux / 127
    const int tid = threadIdx.x;
    // Workgroup id = chunk of channel groups * pchunks + pixel chunk.
    // Consecutive workgroup ids go round-robin over the 8 XCDs, each with an L2 of its own: every XCD gets a contiguous
    // run of the numbering, so that the chunks either side of a boundary (which may share a line, and share their halo
    // rows) meet in one L2.
    int lid;
    {
        const int nb = (int) gridDim.x, bid = (int) blockIdx.x;
        const int q = nb >> 3, rmd = nb & 7, xcd = bid & 7, idx = bid >> 3;
        lid = xcd * q + (xcd < rmd ? xcd : rmd) + idx;
    }
    const int gchunk = dws8_div(lid, p.div_pchunks), pchunk = lid - gchunk * p.pchunks;
    const int c_first = gchunk * p.gw * 16;       // first channel of the workgroup
    for (int i = tid; i < p.gw * 16 * p.taps; i += 256) {
        const int cl = dws8_div(i, p.div_taps), t = i - cl * p.taps, c = c_first + cl;
        const float w = c < p.C ? (float) p.w[(long long) c * p.taps + t] : 0.0f;
        wl[(((cl >> 4) * 4 + ((cl & 15) >> 2)) * p.taps + t) * 4 + (cl & 3)] = w;
    }
    for (int cl = tid; cl < p.gw * 16; cl += 256) {
        const int c = c_first + cl;
        int sum = 0;
        float bias = 0.0f, coeff = 0.0f;
        if (c < p.C) {
            for (int t = 0; t < p.taps; ++t) sum += (int) p.w[(long long) c * p.taps + t];
            bias = (float) p.b32[c];
            coeff = __fdiv_rn(p.aux[c], 127.0f);
        }
        float *cc = cst + (cl >> 4) * 48 + (cl & 15);
        cc[0] = -128.0f * (float) sum;
        cc[16] = bias;
        cc[32] = coeff;
    }
    __syncthreads();

    constexpr int R = S3 == 1 ? DWS8_R1 : S3 == 2 ? 2 : 1;
    constexpr int ROWS = S3 > 0 ? (R - 1) * S3 + 3 : 1;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int gsub = wave % p.gw, psub = wave / p.gw;
    const int g = gchunk * p.gw + gsub;           // the wavefront's channel group; gsub indexes the tables in LDS
    if (g >= p.G) return;
    const int per_wg = 64 * (4 / p.gw);
    const int item = pchunk * per_wg + psub * 64 + lane;
    const bool live = item < p.items;
    const int it = live ? item : 0;
    const int ns = dws8_div(it, p.div_ow), ow = it - ns * p.OW;
    const int n = dws8_div(ns, p.div_strips), oh0 = (ns - n * p.strips) * R;
    const rsrc_t rx = make_rsrc(p.x, p.x_bytes);
    const rsrc_t ry = make_rsrc(p.y, p.y_bytes);
    const int sh = S3 > 0 ? S3 : p.sh, sw = S3 > 0 ? S3 : p.sw;
    const int ih0 = oh0 * sh - p.pad, iw0 = ow * sw - p.pad;

    if constexpr (S3 > 0) {
        unsigned voff[ROWS][3];
#pragma unroll
        for (int r = 0; r < ROWS; ++r)
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                const int ih = ih0 + r, iw = iw0 + j;
                const bool ok = live && ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
                voff[r][j] = ok ? (unsigned) (((n * p.H + ih) * p.W + iw) * p.Cp + g * 16) : OOB;
            }
        {
            uint4 px[ROWS][3];
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
#pragma unroll
                for (int j = 0; j < 3; ++j) px[r][j] = buf_load_b128(rx, voff[r][j], 0u);
            unsigned outw[R][4];
#pragma unroll
            for (int cq = 0; cq < 4; ++cq) {
                const float4 *wq = reinterpret_cast<const float4 *>(wl + (gsub * 4 + cq) * 9 * 4);
                const float4 *cq4 = reinterpret_cast<const float4 *>(cst + gsub * 48 + cq * 4);
                const float4 init = cq4[0], bias = cq4[4], coeff = cq4[8];
                float w[9][4];
#pragma unroll
                for (int t = 0; t < 9; ++t) {
                    const float4 v = wq[t];
                    w[t][0] = v.x; w[t][1] = v.y; w[t][2] = v.z; w[t][3] = v.w;
                }
                float acc[R][4];
#pragma unroll
                for (int q = 0; q < R; ++q) { acc[q][0] = init.x; acc[q][1] = init.y; acc[q][2] = init.z; acc[q][3] = init.w; }
#pragma unroll
                for (int r = 0; r < ROWS; ++r)
#pragma unroll
                    for (int j = 0; j < 3; ++j) {
                        const uint4 v = px[r][j];
                        float f[4];
                        dws8_bytes(cq == 0 ? v.x : cq == 1 ? v.y : cq == 2 ? v.z : v.w, f);
#pragma unroll
                        for (int q = 0; q < R; ++q) {
                            const int i = r - q * S3;   // filter row this input row is for output q
                            if (i < 0 || i > 2) continue;
#pragma unroll
                            for (int k = 0; k < 4; ++k) acc[q][k] = __fmaf_rn(f[k], w[i * 3 + j][k], acc[q][k]);
                        }
                    }
                const float bs[4] = {bias.x, bias.y, bias.z, bias.w}, cf[4] = {coeff.x, coeff.y, coeff.z, coeff.w};
#pragma unroll
                for (int q = 0; q < R; ++q) {
                    unsigned word = 0;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        // conv.c:739 and :746-752: acc * s + bias32, then * (aux / 127): separately rounded
                        const float fl = __fadd_rn(__fmul_rn(acc[q][k], p.in_scale), bs[k]);
                        const float v = act_fast<EPI>(__fmul_rn(fl, cf[k]), p.ep);
                        const int c = g * 16 + cq * 4 + k;
                        if constexpr (OUT_F32) {
                            const int oh = oh0 + q;
                            const bool ok = live && oh < p.OH && c < p.C;
                            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), ry,
                                                                  ok ? (unsigned) ((((n * p.C + c) * p.OH + oh) * p.OW + ow) * 4) : OOB, 0, 0);
                        } else {
                            const unsigned b = c < p.C ? (unsigned) quant_s8(v, p.out_inv_scale) & 0xffu : 0u;
                            word |= b << (8 * k);
                        }
                    }
                    outw[q][cq] = word;
                }
            }
            if constexpr (!OUT_F32) {
#pragma unroll
                for (int q = 0; q < R; ++q) {
                    const int oh = oh0 + q;
                    const bool ok = live && oh < p.OH;
                    // The group's offset goes into the vector offset, the scalar offset stays the constant 0: after a 128-bit
                    // buffer store whose scalar offset is a REGISTER the compiler leaves no gap before the next instruction
                    // that writes one of the data registers, and on this GPU that instruction then changes what some lanes
                    // store (seen here as the first dword of a pixel's 16 bytes holding the next row's index, now and then).
                    __builtin_amdgcn_raw_buffer_store_b128(u32x4{outw[q][0], outw[q][1], outw[q][2], outw[q][3]}, ry,
                                                           ok ? (unsigned) (((n * p.OH + oh) * p.OW + ow) * p.Cp + g * 16) : OOB, 0, 0);
                }
            }
        }
    } else {
        {
            float acc[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) acc[k] = cst[gsub * 48 + k];
            for (int i = 0; i < p.kh; ++i)
                for (int j = 0; j < p.kw; ++j) {
                    const int ih = ih0 + i, iw = iw0 + j;
                    const bool ok = live && ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
                    const uint4 v = buf_load_b128(rx, ok ? (unsigned) (((n * p.H + ih) * p.W + iw) * p.Cp) : OOB, (unsigned) g * 16u);
                    const int t = i * p.kw + j;
#pragma unroll
                    for (int cq = 0; cq < 4; ++cq) {
                        float f[4];
                        dws8_bytes(cq == 0 ? v.x : cq == 1 ? v.y : cq == 2 ? v.z : v.w, f);
                        const float4 w = *reinterpret_cast<const float4 *>(wl + ((gsub * 4 + cq) * p.taps + t) * 4);
                        acc[cq * 4 + 0] = __fmaf_rn(f[0], w.x, acc[cq * 4 + 0]);
                        acc[cq * 4 + 1] = __fmaf_rn(f[1], w.y, acc[cq * 4 + 1]);
                        acc[cq * 4 + 2] = __fmaf_rn(f[2], w.z, acc[cq * 4 + 2]);
                        acc[cq * 4 + 3] = __fmaf_rn(f[3], w.w, acc[cq * 4 + 3]);
                    }
                }
            unsigned outw[4] = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                const float fl = __fadd_rn(__fmul_rn(acc[k], p.in_scale), cst[gsub * 48 + 16 + k]);
                const float v = act_fast<EPI>(__fmul_rn(fl, cst[gsub * 48 + 32 + k]), p.ep);
                const int c = g * 16 + k;
                if constexpr (OUT_F32) {
                    const bool ok = live && c < p.C;
                    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), ry,
                                                          ok ? (unsigned) ((((n * p.C + c) * p.OH + oh0) * p.OW + ow) * 4) : OOB, 0, 0);
                } else {
                    const unsigned b = c < p.C ? (unsigned) quant_s8(v, p.out_inv_scale) & 0xffu : 0u;
                    outw[k >> 2] |= b << (8 * (k & 3));
                }
            }
            if constexpr (!OUT_F32)
                __builtin_amdgcn_raw_buffer_store_b128(u32x4{outw[0], outw[1], outw[2], outw[3]}, ry,
                                                       live ? (unsigned) (((n * p.OH + oh0) * p.OW + ow) * p.Cp + g * 16) : OOB, 0, 0);
        }
    }
}


// the shapes the kernel takes: what fits its LDS table of weights and its 32-bit offsets
bool dw_s8_ok(const onhip_conv_desc_t &d, int OH, int OW) {
    const long long cp = (d.cout + 15) / 16 * 16;
    const long long taps = (long long) d.kh * d.kw;
    if (d.group == 1 || d.cout != d.cin || !d.has_bias) return false;
    if (taps > 225) return false;   // the table of four channel groups' weights stays within 64 KiB of LDS
    if ((long long) d.n * d.h * d.w * cp >= (1LL << 31) || (long long) d.n * OH * OW * cp >= (1LL << 31)) return false;
    if ((long long) d.n * d.cout * OH * OW * 4 >= (1LL << 31)) return false;
    return true;
}

template <int S3, bool OUT_F32>
static void dw_s8_dispatch(int epi, unsigned wgs, size_t lds_bytes, hipStream_t st, const DwS8Params &p) {
    switch (epi) {
        case EPI_NONE: hipLaunchKernelGGL((dw_s8_nhwc_kernel<S3, EPI_NONE, OUT_F32>), dim3(wgs), dim3(256), lds_bytes, st, p); break;
        case EPI_RELU: hipLaunchKernelGGL((dw_s8_nhwc_kernel<S3, EPI_RELU, OUT_F32>), dim3(wgs), dim3(256), lds_bytes, st, p); break;
        case EPI_CLIP: hipLaunchKernelGGL((dw_s8_nhwc_kernel<S3, EPI_CLIP, OUT_F32>), dim3(wgs), dim3(256), lds_bytes, st, p); break;
        default: hipLaunchKernelGGL((dw_s8_nhwc_kernel<S3, EPI_GENERIC, OUT_F32>), dim3(wgs), dim3(256), lds_bytes, st, p); break;
    }
}

// xq: int8 NHWC, channels padded to 16 (padding channels zero); w8 [C][kh * kw]; y: int8 NHWC like xq when d.out_s8, else
// fp32 NCHW.  Uniform padding (checked by the caller, like every W8A32 form).
int dw_s8_launch(const onhip_conv_desc_t &d, int OH, int OW, const int8_t *xq, const int8_t *w8, const int32_t *bias32,
                 const float *weight_aux, const Epilogue &ep, void *y, hipStream_t stream) {
    if (!dw_s8_ok(d, OH, OW)) return set_error(ONHIP_ERR_ARG, "depthwise int8 NHWC: %d channels with a %dx%d filter are beyond this kernel", d.cout, d.kh, d.kw);
    DwS8Params p;
    memset(&p, 0, sizeof(p));
    p.C = d.cout; p.Cp = (d.cout + 15) / 16 * 16; p.G = p.Cp / 16;
    p.N = d.n; p.H = d.h; p.W = d.w; p.OH = OH; p.OW = OW;
    p.kh = d.kh; p.kw = d.kw; p.taps = d.kh * d.kw; p.sh = d.stride_h; p.sw = d.stride_w; p.pad = d.pad_t;
    const int s3 = (d.kh == 3 && d.kw == 3 && d.stride_h == d.stride_w && (d.stride_h == 1 || d.stride_h == 2)) ? d.stride_h : 0;
    const int R = s3 == 1 ? DWS8_R1 : s3 == 2 ? 2 : 1;
    p.strips = (OH + R - 1) / R;
    const long long items = (long long) d.n * p.strips * OW;
    if (items >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "depthwise int8 NHWC: too many outputs");
    p.items = (int) items;
    p.gw = p.G >= 4 ? 4 : p.G >= 2 ? 2 : 1;
    p.div_ow = make_div31((unsigned) OW);
    p.div_strips = make_div31((unsigned) p.strips);
    p.div_taps = make_div31((unsigned) p.taps);
    p.in_scale = d.input_scale;
    p.out_inv_scale = d.out_s8 ? 1.0f / d.output_scale : 0.0f;
    p.x = xq; p.w = w8; p.b32 = bias32; p.aux = weight_aux; p.y = y;
    p.x_bytes = (unsigned) ((long long) d.n * d.h * d.w * p.Cp);
    p.y_bytes = d.out_s8 ? (unsigned) ((long long) d.n * OH * OW * p.Cp) : (unsigned) ((long long) d.n * d.cout * OH * OW * 4);
    p.ep = ep;
    const int per_wg = 64 * (4 / p.gw);
    const int gchunks = (p.G + p.gw - 1) / p.gw;
    p.pchunks = (int) ((items + per_wg - 1) / per_wg);
    p.div_pchunks = make_div31((unsigned) p.pchunks);
    const long long wgs = (long long) p.pchunks * gchunks;
    if (wgs > 0x7fffffffLL) return set_error(ONHIP_ERR_ARG, "depthwise int8 NHWC: too many workgroups");
    const size_t lds_bytes = ((size_t) p.gw * 16 * p.taps + (size_t) p.gw * 48) * 4;
    const int epi = epi_of_act(ep.act);
    if (d.out_s8) {
        if (s3 == 1) dw_s8_dispatch<1, false>(epi, (unsigned) wgs, lds_bytes, stream, p);
        else if (s3 == 2) dw_s8_dispatch<2, false>(epi, (unsigned) wgs, lds_bytes, stream, p);
        else dw_s8_dispatch<0, false>(epi, (unsigned) wgs, lds_bytes, stream, p);
    } else {
        if (s3 == 1) dw_s8_dispatch<1, true>(epi, (unsigned) wgs, lds_bytes, stream, p);
        else if (s3 == 2) dw_s8_dispatch<2, true>(epi, (unsigned) wgs, lds_bytes, stream, p);
        else dw_s8_dispatch<0, true>(epi, (unsigned) wgs, lds_bytes, stream, p);
    }
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

}  // namespace onhip
