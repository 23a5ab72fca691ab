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


// ---- 3x3 filters on the matrix cores ------------------------------------------------------------------------------------
// The kernel above needs about 47 vector instructions per output byte (byte -> float conversions, nine multiply-adds,
// the store's arithmetic) and is bound by them: counters put its vector pipes at 60 % busy and its memory pipes nearly
// idle.  The matrix cores do a depthwise filter tap as a product with a DIAGONAL matrix: for 32 channels and 32 pixels,
//     v_mfma_i32_32x32x32_i8:  D[m][n] += sum_k A[m][k] B[k][n],  A[m][k] = (m == k) ? w[channel m][tap] : 0,
//                                                                B[k][n] = x[pixel n under the tap][channel k]
// 31 of 32 products are with zero, and it is still a third of the vector instructions' time, on a pipe that runs beside
// them.  B is exactly what memory holds: a lane's operand, 16 consecutive reduction indices of one column, is the 16
// bytes of one channel group of one NHWC pixel; the nine taps are nine loads at shifted pixels (zeros outside the image
// from the buffer descriptor: int8 zero is the real zero, no bias trick).  The int32 sums are exact, so the bytes are
// those of the kernel above and of the reference (conv.c:727-752, :961-973).
//   * A workgroup owns a band of output rows of one image and up to 8 channel groups.  It copies the input rows the band
//     reads (halo included) into LDS with consecutive lanes on consecutive 16-byte units of memory, so memory is read once
//     and in runs; the nine shifted operands of a block of 32 output pixels are then nine ds_read_b128.  (Loaded straight
//     from memory they are nine loads of 32 useful bytes per cache line, the L1 does not hold the lines of the wavefronts
//     of a compute unit, and the layer is bound by refetching them: 57 us for 144 channels on 56 x 56 x 64 either way.)
//   * A wavefront owns one block of 32 channels (two 16-channel groups) and walks the band's blocks of 32 output pixels;
//     its nine diagonal matrices (36 registers) and its lanes' 16 biases and 16 factors are set up once.
//   * The accumulator gives a lane one pixel and the channels 8 q + 4 (lane / 32) + k: for the int8 NHWC store the two lane
//     halves exchange two dwords, after which each holds the 16 consecutive bytes of one channel group (one 128-bit
//     store); for the fp32 NCHW store the layout is already right (32 consecutive pixels of a channel per store).
struct DwMfmaParams {
    DwS8Params b;
    int gc;                // channel groups (16 channels) per workgroup: 2, 4 or 8, i.e. one block of 32 channels per wavefront
    int gchunks;           // chunks of gc groups
    int pitch_u;           // 16-byte units a pixel takes in LDS: gc + 1, odd, so that neighbouring pixels start in different banks
    int brows;             // output rows of a band
    int bands;             // bands per image
    int rows, lw;          // input rows and columns of a band, halo included
    int gc_last;           // groups of the last chunk (G - (gchunks - 1) * gc)
    int gsh, gsh_last;     // log2 of gc, and of gc_last rounded up to a power of two
    int consts_at;         // byte offset of the per-wavefront channel constants in LDS
    Div31 div_row, div_rowl;   // by the units of a staged row, lw << gsh, and the same for the last chunk
    Div31 div_gchunks, div_bands;
};

// a 16-byte LDS read the compiler neither delays to its use nor waits for on its own: the nine operand reads of a pixel
// block are issued together and waited for once (left to the compiler, each read sits right before its MFMA with a wait
// in between: nine LDS latencies per block)
__device__ __forceinline__ i32x4 dws8_lds_read(unsigned addr) {
    i32x4 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
    return v;
}

template <int EPI, bool OUT_F32>
__global__ __launch_bounds__(256) void dw_s8_mfma_kernel(const DwMfmaParams mp) {
    constexpr int UNR = 4;
    const DwS8Params &p = mp.b;
    extern __shared__ __align__(16) unsigned char tile[];          // [rows][lw][pitch_u][16 bytes], then [4 wavefronts][2][32] floats
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    int lid;
    {
        const int nb = (int) gridDim.x, bid = (int) blockIdx.x;
        const int q = nb >> 3, rmd = nb & 7, xcd = bid & 7, idx = bid >> 3;
        lid = xcd * q + (xcd < rmd ? xcd : rmd) + idx;
    }
    // chunks of the same pixels next to each other (they share cache lines), then the bands of an image (they share rows)
    const int nbnd = dws8_div(lid, mp.div_gchunks), gchunk = lid - nbnd * mp.gchunks;
    const int n = dws8_div(nbnd, mp.div_bands), band = nbnd - n * mp.bands;
    const int g_first = gchunk * mp.gc;
    const rsrc_t rx = make_rsrc(p.x, p.x_bytes);
    const rsrc_t ry = make_rsrc(p.y, p.y_bytes);

    // the band's input rows into LDS: consecutive lanes on consecutive 16-byte units of memory (runs of 16 gc bytes per
    // pixel); everything outside the image, and groups past the last, as zeros from the buffer descriptor
    const int ih_base = band * mp.brows * p.sh - p.pad;
    const bool last_chunk = gchunk == mp.gchunks - 1;                // uniform
    const int groups_here = last_chunk ? mp.gc_last : mp.gc;
    // units are numbered (row, column, group) with the groups of a pixel rounded up to a power of two (gc is one; the
    // last chunk may have fewer): one division per unit, the rest is shifts
    const int gsh = last_chunk ? mp.gsh_last : mp.gsh;
    const Div31 drow = last_chunk ? mp.div_rowl : mp.div_row;
    const int row_units = mp.lw << gsh, units = mp.rows * row_units;
    for (int base = 0; base < units; base += 256 * UNR) {
        uint4 v[UNR];
        unsigned dst[UNR];
#pragma unroll
        for (int k = 0; k < UNR; ++k) {
            const int u = base + k * 256 + tid;
            const int row = dws8_div(u, drow), rem = u - row * row_units;
            const int col = rem >> gsh, unit = rem & ((1 << gsh) - 1);
            const int ih = ih_base + row, iw = col - p.pad;
            const bool ok = u < units && unit < groups_here && (unsigned) ih < (unsigned) p.H && (unsigned) iw < (unsigned) p.W;
            v[k] = buf_load_b128(rx, ok ? (unsigned) (((n * p.H + ih) * p.W + iw) * p.Cp + (g_first + unit) * 16) : OOB, 0u);
            dst[k] = u < units ? (unsigned) (((row * mp.lw + col) * mp.pitch_u + unit) * 16) : 0xffffffffu;
        }
#pragma unroll
        for (int k = 0; k < UNR; ++k)
            if (dst[k] != 0xffffffffu) *reinterpret_cast<uint4 *>(tile + dst[k]) = v[k];
    }

    // The wavefront's block of 32 channels: with fewer than four blocks in the chunk the wavefronts share them and split
    // the pixels (three blocks: the fourth wavefront only helps with the copy).
    const int nbl = (groups_here + 1) >> 1;
    const int wave_c = nbl >= 3 ? 4 : nbl, cbl = wave % wave_c, psub = wave / wave_c, pstep = 4 / wave_c;
    const int cb0 = g_first * 16 + cbl * 32;                        // first channel of the block
    const bool group_ok = g_first + cbl * 2 + lh < p.G;             // the lane half's channel group exists
    // the nine diagonal matrices: row li, reduction indices 16 lh .. 16 lh + 15; the diagonal passes through this lane
    // when li / 16 == lh, at byte li % 16
    i32x4 amat[9];
    {
        const int c = cb0 + li;
        const bool on = cbl < nbl && (li >> 4) == lh && c < p.C;
        const rsrc_t rw = make_rsrc(p.w, (unsigned) (p.C * 9));
        unsigned wb[9];
#pragma unroll
        for (int t = 0; t < 9; ++t)
            wb[t] = (unsigned) __builtin_amdgcn_raw_buffer_load_b8(rw, on ? (unsigned) (c * 9 + t) : OOB, 0, 0) & 0xffu;
        const int dw = (li & 15) >> 2, sh = 8 * (li & 3);
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const int v = (int) (wb[t] << sh);
            amat[t] = i32x4{dw == 0 ? v : 0, dw == 1 ? v : 0, dw == 2 ? v : 0, dw == 3 ? v : 0};
        }
    }
    // bias (as a float) and factor weight_aux / 127 of the block's 32 channels: lane li of the lower half fetches and divides
    // for channel li, the lanes pick their 16 channels 8 q + 4 lh + k up from LDS after the barrier
    float *wconst = reinterpret_cast<float *>(tile + mp.consts_at) + wave * 64;
    if (lh == 0) {
        const rsrc_t rb = make_rsrc(p.b32, (unsigned) (p.C * 4)), ra = make_rsrc(p.aux, (unsigned) (p.C * 4));
        const unsigned off = (unsigned) (cb0 + li) * 4u;               // past C: zeros
        wconst[li] = (float) (int) __builtin_amdgcn_raw_buffer_load_b32(rb, off, 0, 0);
        wconst[32 + li] = __fdiv_rn(buf_load_f32(ra, off, 0), 127.0f);
    }
    // which bytes of the lane's four output words are channels of the tensor (the rest are written as zero)
    unsigned keep[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        keep[q] = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) keep[q] |= cb0 + 8 * q + 4 * lh + k < p.C ? 0xffu << (8 * k) : 0u;
    }
    __syncthreads();
    if (cbl >= nbl) return;
    const unsigned lds0 = (unsigned) (size_t) (__attribute__((address_space(3))) unsigned char *) tile;
    float bias[16], coeff[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 b4 = *reinterpret_cast<const float4 *>(wconst + 8 * q + 4 * lh);
        const float4 c4 = *reinterpret_cast<const float4 *>(wconst + 32 + 8 * q + 4 * lh);
        bias[4 * q] = b4.x; bias[4 * q + 1] = b4.y; bias[4 * q + 2] = b4.z; bias[4 * q + 3] = b4.w;
        coeff[4 * q] = c4.x; coeff[4 * q + 1] = c4.y; coeff[4 * q + 2] = c4.z; coeff[4 * q + 3] = c4.w;
    }
    // int8 output behind no activation, Relu or Clip: activation, the product with 1 / output_scale and the quantiser's
    // clamp are one median of three on v / output_scale.  The product is monotonic and so is its rounding, so clamping
    // before it to [a, b] and after it to [fl(a / s), fl(b / s)] give the same float; two nested clamps are one.  (A NaN
    // comes out as the lower bound here and as 0 from the separate steps; no finite scale or weight produces one.)
    float q_lo = -128.0f, q_hi = 127.0f;
    if constexpr (EPI == EPI_RELU) q_lo = 0.0f;
    if constexpr (EPI == EPI_CLIP) {
        q_lo = fmaxf(__fmul_rn(p.ep.clip_min, p.out_inv_scale), -128.0f);
        q_hi = fminf(__fmul_rn(p.ep.clip_max, p.out_inv_scale), 127.0f);
    }

    const int oh_first = band * mp.brows;
    const int band_pix = min(mp.brows, p.OH - oh_first) * p.OW;     // output pixels of this band
    const int pblocks = (band_pix + 31) >> 5;
    for (int pb = psub; pb < pblocks; pb += pstep) {
        const int pi = pb * 32 + li;
        const bool live = pi < band_pix;
        const int pc = live ? pi : 0;
        const int orow = dws8_div(pc, p.div_ow), ow = pc - orow * p.OW;
        const int oh = oh_first + orow;
        const unsigned in0 = (unsigned) (((orow * p.sh) * mp.lw + ow * p.sw) * mp.pitch_u + cbl * 2 + lh) * 16u;
        i32x4 xv[9];
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
            for (int j = 0; j < 3; ++j) xv[i * 3 + j] = dws8_lds_read(lds0 + in0 + (unsigned) ((i * mp.lw + j) * mp.pitch_u) * 16u);
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(xv[0]), "+v"(xv[1]), "+v"(xv[2]), "+v"(xv[3]), "+v"(xv[4]), "+v"(xv[5]), "+v"(xv[6]), "+v"(xv[7]), "+v"(xv[8])
                     :: "memory");
        i32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0;
#pragma unroll
        for (int t = 0; t < 9; ++t) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(amat[t], xv[t], acc, 0, 0, 0);

        unsigned word[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            int b8[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int r = 4 * q + k, c = cb0 + 8 * q + 4 * lh + k;
                // conv.c:739 and :746-752: acc * s + bias32, then * (aux / 127): separately rounded
                const float fl = __fadd_rn(__fmul_rn((float) acc[r], p.in_scale), bias[r]);
                const float pre = __fmul_rn(fl, coeff[r]);
                if constexpr (OUT_F32) {
                    const bool ok = live && c < p.C;
                    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(act_fast<EPI>(pre, p.ep)), ry,
                                                          ok ? (unsigned) (((n * p.C + c) * p.OH + oh) * p.OW + ow) * 4u : OOB, 0, 0);
                } else if constexpr (EPI == EPI_GENERIC) {
                    b8[k] = quant_s8(act_fast<EPI>(pre, p.ep), p.out_inv_scale);
                } else {
                    b8[k] = round_half_away_small(__builtin_amdgcn_fmed3f(__fmul_rn(pre, p.out_inv_scale), q_lo, q_hi));
                }
            }
            if constexpr (!OUT_F32) {
                // the low bytes of four integers into one word: three byte permutes
                const unsigned p01 = __builtin_amdgcn_perm((unsigned) b8[1], (unsigned) b8[0], 0x0c0c0400u);
                const unsigned p23 = __builtin_amdgcn_perm((unsigned) b8[3], (unsigned) b8[2], 0x0c0c0400u);
                word[q] = __builtin_amdgcn_perm(p23, p01, 0x05040100u) & keep[q];
            }
        }
        if constexpr (!OUT_F32) {
            // word[q] = channels 8 q + 4 lh .. + 3.  Lane half 0 stores channels 0..15 = {own 0, partner 0, own 1, partner 1},
            // half 1 channels 16..31 = {partner 2, own 2, partner 3, own 3}: each half sends the two words the other needs
            const unsigned r0 = (unsigned) __shfl_xor((int) (lh ? word[0] : word[2]), 32, 64);
            const unsigned r1 = (unsigned) __shfl_xor((int) (lh ? word[1] : word[3]), 32, 64);
            const u32x4 out = lh ? u32x4{r0, word[2], r1, word[3]} : u32x4{word[0], r0, word[1], r1};
            // the whole offset in the vector offset, scalar offset the constant 0: see the store of the kernel above
            __builtin_amdgcn_raw_buffer_store_b128(out, ry, live && group_ok ? (unsigned) (((n * p.OH + oh) * p.OW + ow) * p.Cp + cb0 + lh * 16) : OOB,
                                                   0, 0);
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

template <bool OUT_F32>
static void dw_s8_mfma_dispatch(int epi, unsigned wgs, size_t lds, hipStream_t st, const DwMfmaParams &p) {
    switch (epi) {
        case EPI_NONE: hipLaunchKernelGGL((dw_s8_mfma_kernel<EPI_NONE, OUT_F32>), dim3(wgs), dim3(256), lds, st, p); break;
        case EPI_RELU: hipLaunchKernelGGL((dw_s8_mfma_kernel<EPI_RELU, OUT_F32>), dim3(wgs), dim3(256), lds, st, p); break;
        case EPI_CLIP: hipLaunchKernelGGL((dw_s8_mfma_kernel<EPI_CLIP, OUT_F32>), dim3(wgs), dim3(256), lds, st, p); break;
        default: hipLaunchKernelGGL((dw_s8_mfma_kernel<EPI_GENERIC, OUT_F32>), dim3(wgs), dim3(256), lds, st, p); break;
    }
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
    const int epi = epi_of_act(ep.act);
    if (d.kh == 3 && d.kw == 3 && !getenv("ONHIP_DW_NO_MFMA")) {   // 3x3, any stride: the matrix-core kernel
        DwMfmaParams mp;
        memset(&mp, 0, sizeof(mp));
        mp.b = p;
        mp.gc = p.G >= 8 ? 8 : p.G > 2 ? (p.G + 1) / 2 * 2 : 2;
        if (mp.gc == 6) mp.gc = 4;                                 // blocks of 32 channels in ones, twos or fours per workgroup
        // 9 or 10 groups in chunks of 8 leave a chunk of one or two whose workgroups copy as many rows as the full ones; in
        // chunks of 4, with the smaller tiles five workgroups fit a compute unit (144 channels on 56 x 56 x 64: 39 -> 30 us)
        long long lds_cap = 48 * 1024;
        if (p.G == 9 || p.G == 10) { mp.gc = 4; lds_cap = 32 * 1024; }
        mp.gchunks = (p.G + mp.gc - 1) / mp.gc;
        mp.pitch_u = mp.gc + 1;
        mp.lw = (OW - 1) * d.stride_w + 3;
        const long long row_bytes = (long long) mp.lw * mp.pitch_u * 16;
        auto rows_of = [&](int brows) { return (brows - 1) * d.stride_h + 3; };
        // the tallest band whose input fits 48 KiB of LDS (three workgroups per compute unit), shortened while that leaves
        // the chip fewer than 1024 workgroups.  (Measured and not kept: two pixel blocks per trip with their MFMA chains
        // interleaved, 10 to 25 % slower for its registers; bands down to 16 KiB for more workgroups per unit, slower.)
        int brows = OH;
        while (brows > 1 && (rows_of(brows) * row_bytes > lds_cap || (long long) d.n * ((OH + brows - 1) / brows) * mp.gchunks < 1024)) --brows;
        if (rows_of(brows) * row_bytes <= 64 * 1024) {
            mp.brows = brows;
            mp.bands = (OH + brows - 1) / brows;
            mp.rows = rows_of(brows);
            mp.gc_last = p.G - (mp.gchunks - 1) * mp.gc;
            mp.gsh = mp.gc == 8 ? 3 : mp.gc == 4 ? 2 : 1;
            mp.gsh_last = mp.gc_last > 4 ? 3 : mp.gc_last > 2 ? 2 : mp.gc_last > 1 ? 1 : 0;
            mp.div_row = make_div31((unsigned) (mp.lw << mp.gsh));
            mp.div_rowl = make_div31((unsigned) (mp.lw << mp.gsh_last));
            mp.consts_at = (int) (mp.rows * row_bytes);
            mp.div_gchunks = make_div31((unsigned) mp.gchunks);
            mp.div_bands = make_div31((unsigned) mp.bands);
            const long long wgs = (long long) d.n * mp.bands * mp.gchunks;
            if (wgs > 0x7fffffffLL) return set_error(ONHIP_ERR_ARG, "depthwise int8 NHWC: too many workgroups");
            const size_t lds = (size_t) mp.rows * row_bytes + 4 * 64 * sizeof(float);
            if (d.out_s8) dw_s8_mfma_dispatch<false>(epi, (unsigned) wgs, lds, stream, mp);
            else dw_s8_mfma_dispatch<true>(epi, (unsigned) wgs, lds, stream, mp);
            ONHIP_CHECK_HIP(hipGetLastError());
            return ONHIP_OK;
        }
    }
    const int per_wg = 64 * (4 / p.gw);
    const int gchunks = (p.G + p.gw - 1) / p.gw;
    p.pchunks = (int) ((items + per_wg - 1) / per_wg);
    p.div_pchunks = make_div31((unsigned) p.pchunks);
    const long long wgs = (long long) p.pchunks * gchunks;
    if (wgs > 0x7fffffffLL) return set_error(ONHIP_ERR_ARG, "depthwise int8 NHWC: too many workgroups");
    const size_t lds_bytes = ((size_t) p.gw * 16 * p.taps + (size_t) p.gw * 48) * 4;
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
